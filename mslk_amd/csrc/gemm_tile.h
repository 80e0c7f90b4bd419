// LDS-tiled FP8 x FP8 -> fp32 MFMA main loop and fused rowwise-scale epilogue for gfx950.
//
// One workgroup (4 wavefronts in a 2 x 2 grid by default; 2 x 4 and 4 x 2 grids of 8 wavefronts compile
// too but measured no faster) produces a BM x BN tile of
//   Y[m, n] = bf16( (sum_k XQ[m, k] * WQ[n, k]) * x_scale[m] * w_scale[n] + bias[n] )
// (reference math: csrc/gemm/ck/fp8_rowwise/kernels/fp8_rowwise_common.h:54-82,168-204; bias:
//  csrc/gemm/cutlass/f8f8bf16_rowwise/f8f8bf16_rowwise_common.cuh:150-198).
//
// Data movement
//   * K is consumed in steps of 128 bytes.  Each step's XQ tile (BM rows x 128 B) and WQ tile
//     (BN rows x 128 B) are copied global -> LDS by the DMA form of the 128-bit global load
//     (no VGPR staging).  One wave-level load fills 1024 contiguous LDS bytes = 8 tile rows.
//   * Inside a 128-byte LDS row the eight 16-byte chunks are XOR-permuted with
//     swz(row) = (row & 7) ^ ((row >> 3) & 1), so that the 16 lanes of an MFMA operand read
//     (16 consecutive rows, same logical chunk) touch 16 different 16-byte bank groups.  The DMA
//     cannot scatter inside a wave, so the permutation is applied on the GLOBAL side: lane l of a
//     load fetches logical chunk (l & 7) ^ swz(row) of its row.
//   * Two XQ buffers and three WQ buffers: while step k is multiplied, the XQ tile of step k+1 and the
//     WQ tiles of steps k+1 and k+2 are in flight (the weights are the cold, read-once stream).
// Rows
//   * A wave row owns BM / WM consecutive rows of a tile.  With ROWSKIP (the grouped kernels) a tile with at most three
//     quarters of its rows valid is multiplied differently: its 16-row m fragments are dealt to the wave rows round-robin
//     (wave row wm owns fragments wm, wm + WM, ...), the K loop is one compiled for a quarter, half or three quarters of
//     the m fragments per wave, and the XQ loads and the epilogue work of fragments without valid rows are left out: the
//     cost of a ragged tile (the last row tile of an MoE group) follows its row count in steps of BM / 4 rows, down to
//     what the weight stream alone costs.  (Dealing the fragments of FULL tiles round-robin as well cost 2 % on them.)
// Math
//   * v_mfma_f32_16x16x128_f8f6f4 (both operands e4m3, unit block scales).  WQ rows are the first
//     operand and XQ rows the second, so a lane ends up holding 4 consecutive n for one m.
//   * Both operands give lane (i = l & 15, g = l >> 4) the 32 bytes k in [32 g, 32 g + 32) of
//     row i; any k permutation would do as long as both operands share it.
// Epilogue
//   * A wave has its SIMD to itself, so every instruction and every memory wait of the epilogue is exposed.  Scales
//     and bias are fetched before the first store (a load waited for between stores waits for the stores too); each
//     16-row fragment row is scaled, converted and transposed through a wave-private LDS buffer, and the read-back
//     and the stores of one fragment row are interleaved with the arithmetic of the next.
#pragma once
#include "common.h"

namespace mslk_amd {

constexpr int kBK = 128;  // bytes (= fp8 elements) of K per main-loop step

// RING = 0: two XQ buffers and three WQ buffers (weights two steps ahead, activations one).
// RING = n: n buffers for each operand, both streams n - 1 steps ahead -- for small tiles, whose step is much
// shorter than a memory round trip.
template <int BM, int BN, int WAVES_M = 2, int WAVES_N = 2, int RING_STAGES = 0>
struct TileShape {
  static constexpr int RING = RING_STAGES;
  static constexpr int kBM = BM, kBN = BN;
  static constexpr int WM = WAVES_M, WN = WAVES_N;   // wave grid over the tile
  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NTHREADS = NW * 64;
  static constexpr int FM = BM / WAVES_M / 16;  // 16-row m fragments per wave
  static constexpr int FN = BN / WAVES_N / 16;  // 16-row n fragments per wave
  static constexpr int A_BYTES = BM * kBK;
  static constexpr int B_BYTES = BN * kBK;
  static constexpr int A_STAGES = RING_STAGES ? RING_STAGES : 2;   // XQ tiles: the one being read and the one in flight
  static constexpr int B_STAGES = RING_STAGES ? RING_STAGES : 3;   // WQ tiles: one being read, two in flight
  static constexpr int LDS_BYTES = A_STAGES * A_BYTES + B_STAGES * B_BYTES;
  static constexpr int LA = BM / 8 / NW;        // wave-level loads of the A tile per wave per step
  static constexpr int LB = BN / 8 / NW;
};

MSLK_AMD_DEVINL int lds_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

MSLK_AMD_DEVINL void wait_vmcnt0() { __builtin_amdgcn_s_waitcnt(0x0F70); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// The output is written once and not re-read by this kernel: a streaming (non-temporal) store keeps
// it from displacing the operand tiles in L2 and from piling up as dirty lines to flush at kernel end.
// Written as an instruction with vector-register operands: given the choice, the register allocator parks the
// read-back values in accumulator registers, all of which hold the tile, and spills part of it.  The compiler does
// not see a store here, so the wait states the hardware needs between a store of more than 8 bytes and a vector
// instruction that overwrites its data registers (the allocator reuses them at once) are part of the statement.
//
// Rules for the statements in this file that the compiler cannot look into (each was learnt from a wrong result or a fault):
//   1. An instruction written by hand gets the wait states the hardware asks for INSIDE its statement (the s_nop 1 below,
//      the s_nop 0 between the M0 write and the load in dma16): the hazard pass does not see through it.
//   2. A memory READ written by hand must keep its destination registers live until a wait inside the same statement:
//      the allocator otherwise hands them out again while the load is in flight, and the late write-back lands in a live
//      value (an address, once: a memory fault).  This file has no such read -- dma16 has no register destination.
//   3. What the compiler does not know to be in flight it does not wait for: every read of bytes copied by dma16 sits
//      behind an explicit s_waitcnt vmcnt in wait_and_barrier() / wait_vmcnt0().
//   4. Accumulator registers read by hand (v_accvgpr_read_b32 in the epilogue) follow a fixed 48 wait states behind the
//      last MFMA of the K loop.
// Which test fails when a rule is broken (all compare integer-valued products bit for bit): store16_stream and the
// accumulator reads -- tests/test_gemm_gpu.py::test_exact_on_full_256_tiles (one tile per workgroup, fused and plain
// epilogue, both output types, both bias types), tests/test_exact_paths_gpu.py::test_persistent_workgroups_exact (epilogue
// behind the next tile's first loads), ::test_tensorlist_grouped_exact / ::test_stacked_and_offsets_over_m_exact (ragged and
// interleaved epilogues); dma16 and the load waits -- every test of tests/test_exact_paths_gpu.py (each tile shape and
// ring depth has a case) and tests/test_preshuffle_gpu.py; graph replays that must repeat the eager bits --
// tests/test_gemm_gpu.py::test_hip_graph_capture_and_replay, tests/test_grouped_mm_gpu.py::test_graph_replay_follows_device_side_group_sizes.
MSLK_AMD_DEVINL void store16_stream(uint16_t* dst, uint4 val) {
  const v4i v = {(int)val.x, (int)val.y, (int)val.z, (int)val.w};
  asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
}

// Global -> LDS copy of 16 bytes per lane (1 KiB per wave, contiguous in LDS from `lds_wave_base`), addressed as
// wave-uniform base + 32-bit lane offset.  Written as an instruction instead of the compiler's builtin for two reasons:
//   * while a load the compiler knows of as "writes LDS through the vector memory path" is in flight, every wait it
//     inserts for an LDS read becomes lgkmcnt(0) -- all reads, not the one whose value is needed.  The K loop always has
//     loads in flight, and its fragment re-loads (sixteen reads behind the barrier, the first MFMA of the next step needs
//     the first four) waited for the last of them.  With the load opaque the compiler counts its LDS reads exactly;
//   * the address stays "scalar base + 32-bit vector offset" (the builtin's address was kept as sixteen 64-bit vector
//     pairs and advanced by a vector instruction per load).
// Consequences the callers carry: the compiler sees neither the LDS write nor the outstanding load, so every read of
// the copied bytes sits behind an explicit s_waitcnt vmcnt (wait_and_barrier / wait_vmcnt0) -- none relies on a wait the
// compiler would have inserted -- and the "memory" clobber keeps LDS accesses from moving across the statement.  No
// register receives data, so there is nothing the register allocator could reuse too early.  M0 (the LDS address of
// the copy) is written inside the statement and declared clobbered; nothing else in these kernels uses M0.  One wait
// state separates the M0 write from the load.  A violation shows in the bit-exact tests of tests/test_exact_paths_gpu.py
// and tests/test_gemm_gpu.py::test_exact_on_full_256_tiles (stale or missing operand bytes change integer sums).
MSLK_AMD_DEVINL const uint8_t* uniform_ptr(const uint8_t* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)v), hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
}
// STREAM: the bytes are read once by this launch (a weight tile that no other row tile of its XCD shares): the load is
// marked non-temporal, so the line does not displace what the L2 is asked for again.
template <bool STREAM = false>
MSLK_AMD_DEVINL void dma16(const uint8_t* base, uint32_t off, char* lds_wave_base) {
  const uint32_t dst = (uint32_t)(uintptr_t)(lds_ptr_t)lds_wave_base;
  if constexpr (STREAM)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" : : "v"(off), "s"(base), "s"(dst) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(base), "s"(dst) : "memory", "m0");
}


// PS (pre-shuffled weights): WQ arrives in the blocked layout [N/16][K/64][4][16][16 B] -- each
// 16-row x 64-byte block stored as (k chunk, row, 16 bytes), the order in which the 64 lanes of an
// MFMA operand read it (reference: mslk/quantize/shuffle.py:182-246).  One DMA then moves one block
// (1 KiB contiguous in HBM and in LDS), the WQ fragment read is lane-linear, and both operands give
// lane (i, g) the k bytes [16 g, 16 g + 16) and [64 + 16 g, 64 + 16 g + 16) of row i.
// XQ_EARLY: how many of the LA loads of an XQ tile are issued two K steps ahead instead of one (two-plus-three buffers;
// see step()).
// STAMPS: the wave notes the constant-rate counter (s_memrealtime, 100 MHz) when its first operands are behind the first
// barrier and when the K loop hands the last step to the fused epilogue -- the measuring build of the dense kernel
// (mslk_amd_debug_gemm_phases) writes them out beside its own entry and exit times; no other kernel carries them.
// W_STREAM: the weight tile is fetched with non-temporal loads (dma16<true>): for tiles whose weight block at most two row
// tiles share.
template <typename TS, int BIAS, bool PS = false, bool ROWSKIP = false, int XQ_EARLY = TS::LA / 2, bool STAMPS = false,
          bool W_STREAM = false>
struct GemmTile {
  // Per-lane state that is constant over the K loop.
  uint32_t a_off[TS::LA];   // byte offset of this lane's 16-byte chunk relative to a_base, k = 0
  uint32_t b_off[TS::LB];
  int out_f16 = 0;          // output element type: 0 bf16, 1 fp16 (set by the caller before run())
  uint64_t stamp_first_operands = 0, stamp_k_loop_end = 0;   // STAMPS only
  int a_rows = TS::kBM;     // valid rows of the XQ tile (wave-uniform)
  const uint8_t* a_base;    // XQ + m0 * K   (wave-uniform)
  const uint8_t* b_base;    // WQ + n0 * K

  // xq/wq point at row m0 / n0 of the operands; rows_a / rows_b = valid rows from there (>= 1).
  // `ld` = bytes between consecutive rows of XQ and of WQ (equal to K unless the operands are K slices).
  MSLK_AMD_DEVINL void init(const uint8_t* xq_tile, const uint8_t* wq_tile, int rows_a, int rows_b, uint32_t ld) {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));   // recompute the row / chunk of each load per tile instead of keeping 32 values live
    const int wave = wave_id();
    // the tile pointers are the same in every lane; say so, so that the DMA loads get their base in scalar registers
    a_base = uniform_ptr(xq_tile);
    b_base = uniform_ptr(wq_tile);
    a_rows = rows_a;
#pragma unroll
    for (int i = 0; i < TS::LA; ++i) {
      const int row = (wave * TS::LA + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      const int rc = row < rows_a ? row : rows_a - 1;   // clamp: edge tiles re-read the last row
      a_off[i] = (uint32_t)rc * ld + chunk * 16;
    }
#pragma unroll
    for (int i = 0; i < TS::LB; ++i) {
      if constexpr (PS) {
        // load q of the stage = block (16-row group q / 2, 64-byte half q % 2); edge tiles re-read the last group
        const int q = wave * TS::LB + i;
        const int groups = rows_b >> 4;
        const int nb = (q >> 1) < groups ? (q >> 1) : groups - 1;
        b_off[i] = (uint32_t)nb * 16u * ld + (q & 1) * 1024 + lane * 16;
      } else {
        const int row = (wave * TS::LB + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ lds_swz(row);
        const int rc = row < rows_b ? row : rows_b - 1;
        b_off[i] = (uint32_t)rc * ld + chunk * 16;
      }
    }
  }

  // Wave index as a scalar, so that LDS destinations of the DMA are formed in SGPRs.
  MSLK_AMD_DEVINL static int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

  // DMA load number i (0 .. LA-1 for the XQ tile, 0 .. LB-1 for the WQ tile) of the K step at byte k0.
  // `abuf` / `bbuf` are the LDS buffers that receive the XQ / WQ tile of the K step at byte k0.
  MSLK_AMD_DEVINL void issue_a(char* abuf, int k0, int i) {
    dma16(a_base + k0, a_off[i], abuf + (wave_id() * TS::LA + i) * 1024);
  }
  MSLK_AMD_DEVINL void issue_b(char* bbuf, int k0, int i) {
    // pre-shuffled: the K step at byte k0 starts 16 rows x k0 bytes into the row group
    dma16<W_STREAM>(b_base + (PS ? k0 * 16 : k0), b_off[i], bbuf + (wave_id() * TS::LB + i) * 1024);
  }
  MSLK_AMD_DEVINL void issue_a_all(char* abuf, int k0) {
#pragma unroll
    for (int i = 0; i < TS::LA; ++i) issue_a(abuf, k0, i);
  }
  // Ragged tiles: a wave whose share of the XQ tile (8 * LA consecutive rows) starts beyond the valid rows fetches
  // nothing -- nobody multiplies those rows (one wave-uniform branch for the wave's loads of a step).
  MSLK_AMD_DEVINL void issue_a_live(char* abuf, int k0, int lo = 0, int hi = TS::LA) {
    if (wave_id() * TS::LA * 8 < a_rows) {
#pragma unroll
      for (int i = 0; i < TS::LA; ++i)
        if (i >= lo && i < hi) issue_a(abuf, k0, i);
    }
  }
  MSLK_AMD_DEVINL void issue_b_all(char* bbuf, int k0) {
#pragma unroll
    for (int i = 0; i < TS::LB; ++i) issue_b(bbuf, k0, i);
  }

  // K tail (K % 128 != 0, K % 16 == 0): only `k_valid` bytes of each row remain.  Chunks at or
  // beyond K are zero-filled with a plain LDS store by the lane that would have fetched them.
  MSLK_AMD_DEVINL void issue_loads_tail(char* abuf, char* bbuf, int k0, int k_valid) {
    const int lane = threadIdx.x & 63, wave = wave_id();
#pragma unroll
    for (int i = 0; i < TS::LA; ++i) {
      const int row = (wave * TS::LA + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      char* dst = abuf + (wave * TS::LA + i) * 1024;
      if (chunk * 16 < k_valid) dma16(a_base + k0, a_off[i], dst);
      else *reinterpret_cast<uint4*>(dst + lane * 16) = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < TS::LB; ++i) {
      const int row = (wave * TS::LB + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      char* dst = bbuf + (wave * TS::LB + i) * 1024;
      const bool valid = PS ? ((wave * TS::LB + i) & 1) * 64 < k_valid : chunk * 16 < k_valid;
      if (valid) dma16<W_STREAM>(b_base + (PS ? k0 * 16 : k0), b_off[i], dst);
      else *reinterpret_cast<uint4*>(dst + lane * 16) = make_uint4(0, 0, 0, 0);
    }
  }

  // LDS byte offsets of this lane's two 16-byte halves of an MFMA operand fragment, relative to the
  // first row of the fragment: lane (i = l & 15, g = l >> 4) reads logical chunks 2g and 2g + 1 of row i
  // (chunks g and g + 4 when the weights are pre-shuffled, whose blocks fix that k assignment).
  struct FragOff { int off0, off1; };
  MSLK_AMD_DEVINL static FragOff frag_off() {
    const int lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int s = lds_swz(i);
    const int c0 = PS ? g : 2 * g, c1 = PS ? g + 4 : 2 * g + 1;
    return FragOff{i * kBK + ((c0 ^ s) << 4), i * kBK + ((c1 ^ s) << 4)};
  }
  // Fragment t of a wave: STRIDE bytes after fragment t - 1 (consecutive 16-row blocks for WQ; every WM-th for XQ).
  template <int STRIDE = 16 * kBK>
  MSLK_AMD_DEVINL static v8i load_frag(const char* tile, int t, FragOff fo) {
    const v4i lo = *reinterpret_cast<const v4i*>(tile + t * STRIDE + fo.off0);
    const v4i hi = *reinterpret_cast<const v4i*>(tile + t * STRIDE + fo.off1);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
  // ILV (ragged tiles): wave row wm owns the m fragments wm, wm + WM, ...; otherwise the fragments wm * FM ... wm * FM + FM - 1
  template <bool ILV>
  MSLK_AMD_DEVINL static v8i load_frag_a(const char* tile, int t, FragOff fo) {
    return load_frag<(ILV ? TS::WM : 1) * 16 * kBK>(tile, t, fo);
  }
  // WQ fragment t of the wave: as load_frag, or lane-linear out of the two 1 KiB blocks of row group t.
  MSLK_AMD_DEVINL static v8i load_frag_b(const char* tile, int t, FragOff fo) {
    if constexpr (PS) {
      const char* blk = tile + t * 2048 + (threadIdx.x & 63) * 16;
      const v4i lo = *reinterpret_cast<const v4i*>(blk);
      const v4i hi = *reinterpret_cast<const v4i*>(blk + 1024);
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
      return load_frag(tile, t, fo);
    }
  }
  // The part of an XQ / WQ buffer this wave multiplies.
  template <bool ILV = false>
  MSLK_AMD_DEVINL static const char* a_tile_of(const char* abuf) {
    return abuf + (wave_id() / TS::WN) * (ILV ? 16 : TS::kBM / TS::WM) * kBK;
  }
  MSLK_AMD_DEVINL static const char* b_tile_of(const char* bbuf) {
    return bbuf + (wave_id() % TS::WN) * (TS::kBN / TS::WN) * kBK;
  }
  // First fragments of a K step: all XQ fragments and WQ fragment 0.
  template <int FMV = TS::FM>
  MSLK_AMD_DEVINL void load_first_frags(const char* abuf, const char* bbuf, v8i (&xf)[TS::FM], v8i& wf0) {
    const FragOff fo = frag_off();
    wf0 = load_frag_b(b_tile_of(bbuf), 0, fo);
#pragma unroll
    for (int tm = 0; tm < FMV; ++tm) xf[tm] = load_frag_a<(FMV < TS::FM)>(a_tile_of<(FMV < TS::FM)>(abuf), tm, fo);
  }

  // Waits until at most `pending` of this wave's DMA loads (the youngest ones) are still in flight and
  // all its LDS reads have returned, then passes the workgroup barrier.
  template <int PENDING>
  MSLK_AMD_DEVINL static void wait_and_barrier() {
    static_assert(PENDING >= 0 && PENDING < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");                  // no LDS access moves across the barrier at compile time
    // vmcnt(PENDING) lgkmcnt(0), expcnt untouched; vmcnt is split into bits [3:0] and [15:14] of the immediate
    __builtin_amdgcn_s_waitcnt(0x0070 | (PENDING & 15) | ((PENDING >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }

  // One K step of MFMAs on the WQ tile in `b_cur`; xf / wf0 (the step's XQ fragments and WQ fragment 0)
  // are already in registers.  The step is software-pipelined across the workgroup barrier; the weight
  // stream runs two steps ahead, the activation stream one to two:
  //   * DMA_B: the global -> LDS loads of the WQ tile two steps on (byte offset k_b, buffer `b_far`) are
  //     issued between the MFMA groups in front of the barrier, so that their issue cost hides under
  //     matrix work.
  //   * NEXT: before the last MFMA group the wave waits for everything but the WQ loads it issued in this
  //     step, and for all its LDS reads, and passes the barrier (after which `a_nxt` and `b_nxt` are
  //     complete and nobody reads `b_cur` any more).  The operands of the last group are in registers;
  //     each XQ fragment is re-loaded from `a_nxt` right after the MFMA that used it last, so the barrier
  //     and the LDS latency overlap with matrix work and the following step starts with its first
  //     fragments already on their way.
  //   * NA_TAIL (two-plus-three buffers): the first NA_TAIL loads of the XQ tile two steps on (byte offset
  //     k_a_tail) go into `a_tail_dst`, the buffer THIS step's XQ fragments came from: they have been in
  //     registers since the previous step, and once the barrier of this step is passed every wave has them,
  //     so the loads follow the barrier, spread over the MFMAs of the last group.  They are then a whole step
  //     old at the barrier that needs them; a load issued in front of the barrier, as the WQ loads are, has
  //     to go to the other buffer and is less than a step old when it is needed -- less than the latency of
  //     a line that misses the L2, which is what a tile sees whose XQ rows few other tiles of its XCD share.
  //     All loads behind the barrier is too many: the four waves pass it together and their loads then queue
  //     in front of the MFMAs (measured: 2 - 4 % slower on large shapes); half and half costs nothing there.
  //   * NA_HEAD: the last NA_HEAD loads of the XQ tile ONE step on (byte offset k_a) go into `a_dst` in front
  //     of the WQ loads.
  //   * Symmetric ring (TileShape::RING): NA_HEAD = LA, all XQ loads go with the WQ loads in front of the barrier
  //     into `a_dst` != `a_nxt`, and PENDING, the number of this wave's youngest loads that may still be in
  //     flight at the barrier, covers RING - 2 steps.
  // FMV < FM: a ragged tile, only the first FMV m fragments of every wave hold valid rows -- see step_rows().
  template <int NA_HEAD, bool DMA_B, bool NEXT, int PENDING, int FMV = TS::FM, int NA_TAIL = 0>
  MSLK_AMD_DEVINL void step(const char* b_cur, char* a_dst, const char* a_nxt, const char* b_nxt, char* b_far, int k_a,
                            int k_b, v4f (&acc)[TS::FN][TS::FM], v8i (&xf)[TS::FM], v8i& wf0, char* a_tail_dst = nullptr,
                            int k_a_tail = 0) {
    static_assert(NA_HEAD >= 0 && NA_TAIL >= 0 && NA_HEAD <= TS::LA && NA_TAIL <= TS::LA && (NA_TAIL == 0 || NEXT), "XQ loads of a step");
    if constexpr (FMV < TS::FM) {
      step_rows<NA_HEAD, DMA_B, NEXT, PENDING, FMV, NA_TAIL>(b_cur, a_dst, a_nxt, b_nxt, b_far, k_a, k_b, acc, xf, wf0, a_tail_dst, k_a_tail);
      return;
    }
    v8i wf_last;
    step_head<NA_HEAD, DMA_B>(b_cur, a_dst, b_far, k_a, k_b, acc, xf, wf0, wf_last);
    step_tail<NEXT, PENDING, NA_TAIL>(a_nxt, b_nxt, acc, xf, wf0, wf_last, a_tail_dst, k_a_tail);
  }

  // The part of a full-tile K step in front of its barrier: every n fragment but the last, with the step's DMA loads.
  // Leaves the last WQ fragment of the step in `wf_last`.
  template <int NA_HEAD, bool DMA_B>
  MSLK_AMD_DEVINL void step_head(const char* b_cur, char* a_dst, char* b_far, int k_a, int k_b, v4f (&acc)[TS::FN][TS::FM],
                                 v8i (&xf)[TS::FM], const v8i& wf0, v8i& wf_last) {
    constexpr int HALF = TS::FN / 2;
    constexpr int NA = NA_HEAD, NB = DMA_B ? TS::LB : 0;   // the step's loads: the last NA of the XQ tile's first, then WQ
    constexpr int ND = NA + NB, GD = TS::FN - 1;
    constexpr int NDMA = (ND + HALF - 1) / HALF;                      // DMA loads per MFMA group (first half only)
    constexpr int PER_SLOT = (NDMA + TS::FM - 1) / TS::FM;            // 1 unless the tile has few MFMAs per group
    constexpr int SLOTS = PER_SLOT > 0 ? (NDMA + PER_SLOT - 1) / PER_SLOT : 0;   // MFMA slots of a group that carry loads
    constexpr bool SPREAD = (PER_SLOT <= 1 || ND % HALF != 0) && ND <= GD * TS::FM;   // also: a load count the halves cannot share evenly
    static_assert(SPREAD || ND % HALF == 0, "DMA loads spread evenly over the first half");
    const FragOff fo = frag_off();
    const char* b_tile = b_tile_of(b_cur);
    v8i wf = wf0;
    auto issue = [&](int q) {
      if (q < NA) {
        if constexpr (NA > 0) issue_a(a_dst, k_a, TS::LA - NA + q);
      } else {
        if constexpr (DMA_B) issue_b(b_far, k_b, q - NA);
      }
    };
#pragma unroll
    for (int tn = 0; tn < TS::FN - 1; ++tn) {
      // Issue order inside a group: the read of the next WQ fragment follows the first MFMA, the DMA
      // loads follow the last MFMAs, one each, so that every DMA is issued in the shadow of an MFMA.
      v8i wf_next;
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm) {
        acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
        if (tm == 0) wf_next = load_frag_b(b_tile, tn + 1, fo);
        if constexpr (SPREAD) {
          // Large tiles (at most one load per MFMA): the loads of a step are spread over ALL groups in front of the
          // barrier, so that the load path sees them at an even rate.
          const int first = (tn * ND + GD - 1) / GD, next = ((tn + 1) * ND + GD - 1) / GD;   // group tn issues loads [first, next)
          const int ds = tm - (TS::FM - (next - first));
          if (ds >= 0) issue(first + ds);
        } else {
          const int d = tm - (TS::FM - SLOTS);
          if (tn < HALF && d >= 0) {
#pragma unroll
            for (int j = 0; j < PER_SLOT; ++j)
              if (d * PER_SLOT + j < NDMA) issue(tn * NDMA + d * PER_SLOT + j);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      wf = wf_next;
      __builtin_amdgcn_sched_barrier(0);
    }
    wf_last = wf;
  }

  // The rest of the step: the barrier (NEXT), then the last n fragment, whose XQ fragments are replaced by those of the
  // next step as they retire; A_TAIL: the XQ tile at byte k_a goes into `a_free`, one load behind each MFMA.
  template <bool NEXT, int PENDING, int NA_TAIL = 0>
  MSLK_AMD_DEVINL void step_tail(const char* a_nxt, const char* b_nxt, v4f (&acc)[TS::FN][TS::FM], v8i (&xf)[TS::FM], v8i& wf0,
                                 const v8i& wf_last, char* a_free = nullptr, int k_a = 0) {
    const FragOff fo = frag_off();
    if constexpr (NEXT) {
      wait_and_barrier<PENDING>();
      wf0 = load_frag_b(b_tile_of(b_nxt), 0, fo);
    }
    const char* a_next = a_tile_of<false>(a_nxt);
#pragma unroll
    for (int tm = 0; tm < TS::FM; ++tm) {
      acc[TS::FN - 1][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf_last, xf[tm], acc[TS::FN - 1][tm], 0, 0, 0, 0, 0, 0);
      if constexpr (NA_TAIL > 0) {   // the first NA_TAIL loads of the XQ tile, spread over the MFMAs
#pragma unroll
        for (int q = (tm * NA_TAIL + TS::FM - 1) / TS::FM; q < ((tm + 1) * NA_TAIL + TS::FM - 1) / TS::FM; ++q) issue_a(a_free, k_a, q);
      }
      if constexpr (NEXT) {
        xf[tm] = load_frag_a<false>(a_next, tm, fo);
        __builtin_amdgcn_sched_barrier(0);  // keep the re-load right behind its MFMA
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // One K step of a ragged tile: as step(), but every n fragment multiplies only the first FMV m fragments of the wave,
  // the WQ loads follow the first MFMA group as one block and the XQ loads (left out by waves whose rows are all beyond
  // the valid ones) the first MFMA behind the barrier.  Such a step is short: it waits for memory rather than for the
  // matrix cores, so the fine interleave of step() would buy nothing.
  template <int NA_HEAD, bool DMA_B, bool NEXT, int PENDING, int FMV, int NA_TAIL>
  MSLK_AMD_DEVINL void step_rows(const char* b_cur, char* a_dst, const char* a_nxt, const char* b_nxt, char* b_far, int k_a,
                                 int k_b, v4f (&acc)[TS::FN][TS::FM], v8i (&xf)[TS::FM], v8i& wf0, char* a_tail_dst, int k_a_tail) {
    static_assert(TS::FN >= 3 && FMV >= 1 && FMV < TS::FM, "ragged step");
    const FragOff fo = frag_off();
    const char* b_tile = b_tile_of(b_cur);
    v8i wf = wf0;
#pragma unroll
    for (int tn = 0; tn < TS::FN - 1; ++tn) {
      const v8i wf_next = load_frag_b(b_tile, tn + 1, fo);
#pragma unroll
      for (int tm = 0; tm < FMV; ++tm)
        acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
      if (tn == 0) {
        if constexpr (NA_HEAD > 0) issue_a_live(a_dst, k_a, TS::LA - NA_HEAD, TS::LA);   // older than the WQ loads of the step
        if constexpr (DMA_B) issue_b_all(b_far, k_b);
      }
      wf = wf_next;
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (NEXT) {
      wait_and_barrier<PENDING>();
      wf0 = load_frag_b(b_tile_of(b_nxt), 0, fo);
    }
    const char* a_next = a_tile_of<true>(a_nxt);
#pragma unroll
    for (int tm = 0; tm < FMV; ++tm) {
      acc[TS::FN - 1][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[tm], acc[TS::FN - 1][tm], 0, 0, 0, 0, 0, 0);
      if constexpr (NA_TAIL > 0) {
        if (tm == 0) issue_a_live(a_tail_dst, k_a_tail, 0, NA_TAIL);
      }
      if constexpr (NEXT) {
        xf[tm] = load_frag_a<true>(a_next, tm, fo);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // Whole tile: K loop + epilogue.  m_rem / n_rem = valid rows / columns of this tile (>= 1).
  // xq_tile / wq_tile / xs / ws / bias / y are already offset to the tile's first row and column.
  // N = elements between consecutive rows of Y; K = bytes of each operand row to consume;
  // ld = bytes between consecutive operand rows.
  MSLK_AMD_DEVINL void run(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, const float* xs,
                           const float* ws, const void* bias, uint16_t* y, int m_rem, int n_rem, int N, int K) {
    run(lds, xq_tile, wq_tile, xs, ws, bias, y, m_rem, n_rem, N, K, (uint32_t)K);
  }
  MSLK_AMD_DEVINL void run(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, const float* xs,
                           const float* ws, const void* bias, uint16_t* y, int m_rem, int n_rem, int N, int K,
                           uint32_t ld) {
    v4f acc[TS::FN][TS::FM];
    accumulate_rows(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
    epilogue(lds, acc, xs, ws, bias, y, m_rem, n_rem, N);
  }

  // K loop over K bytes of the operand rows, then the raw fp32 sums of the tile to `part` (row pitch ldp floats, already
  // offset to the tile's first row and column): one slice of a K-split product, scaled and converted by a later pass.
  // A lane holds 4 consecutive columns of one row per fragment, so full tiles with 16-byte aligned rows store 16 bytes.
  MSLK_AMD_DEVINL void run_partial(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, float* part, int m_rem,
                                   int n_rem, int ldp, int K, uint32_t ld) {
    static_assert(TS::FM * TS::FN * 4 < 256, "tiles whose sums live in vector registers");
    v4f acc[TS::FN][TS::FM];
    accumulate_rows(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int row0 = (wave / TS::WN) * (TS::kBM / TS::WM) + (lane & 15);
    const int col0 = (wave % TS::WN) * (TS::kBN / TS::WN) + 4 * (lane >> 4);
    const bool vec = (ldp & 3) == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0;
#pragma unroll
    for (int tm = 0; tm < TS::FM; ++tm) {
      const int m = row0 + tm * 16;
      if (m >= m_rem) continue;
#pragma unroll
      for (int tn = 0; tn < TS::FN; ++tn) {
        const int n = col0 + tn * 16;
        float* dst = part + (int64_t)m * ldp + n;
        if (vec && n + 3 < n_rem) {
          *reinterpret_cast<float4*>(dst) = make_float4(acc[tn][tm][0], acc[tn][tm][1], acc[tn][tm][2], acc[tn][tm][3]);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < n_rem) dst[r] = acc[tn][tm][r];
        }
      }
    }
  }

  // Whether run_interior() may take the tile: every row and column valid, 16-byte aligned rows of Y and scale / bias
  // vectors, K a positive multiple of the K step.
  MSLK_AMD_DEVINL static bool interior_ok(const float* ws, const void* bias, const uint16_t* y, int m_rem, int n_rem, int N, int K) {
    // (without bias: its 32 values per lane on top of both operands of the step do not fit the registers)
    return BIAS == 0 && TS::RING == 0 && TS::FM * TS::FN * 4 >= 256 && m_rem >= TS::kBM && n_rem >= TS::kBN && K >= kBK && K % kBK == 0 &&
           (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 && (reinterpret_cast<uintptr_t>(ws) & 15) == 0 &&
           (BIAS == 0 || (reinterpret_cast<uintptr_t>(bias) & (BIAS == 1 ? 15 : 7)) == 0);
  }
  // run() for such a tile: the epilogue starts inside the last K step.  That step issues no loads, and once the eight
  // MFMAs of a fragment row are issued its accumulators are final while the rows after it are still being multiplied;
  // so the step runs fragment row by fragment row, and the scaling, conversion and transpose of row tm - 1 and the
  // stores of row tm - 2 are issued between the MFMAs of row tm -- the matrix pipe works under the vector
  // instructions of the epilogue instead of in front of them.  Same arithmetic, same bits.
  MSLK_AMD_DEVINL void run_interior(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, const float* xs,
                                    const float* ws, const void* bias, uint16_t* y, int N, int K) {
    v4f acc[TS::FN][TS::FM];
    LastStep last;
    prologue<false>(lds, xq_tile, wq_tile, TS::kBM, TS::kBN, K, (uint32_t)K);
    accumulate_issued<false, TS::FM, true>(lds, K, acc, &last);
    // the transposes go into the two WQ buffers that are dead: waves 0, 1 into the first, waves 2, 3 into the second
    static_assert(TS::NW == 4 && 2 * EPI_WAVE_BYTES <= TS::B_BYTES, "two transpose buffers per free WQ buffer");
    const int wave = wave_id();
    char* buf = (wave >> 1 ? last.b_free1 : last.b_free0) + (wave & 1) * EPI_WAVE_BYTES;
    if (out_f16) epilogue_impl<true, true, true, false, true>(buf, acc, xs, ws, bias, y, TS::kBM, TS::kBN, N, &last);
    else epilogue_impl<true, false, true, false, true>(buf, acc, xs, ws, bias, y, TS::kBM, TS::kBN, N, &last);
  }

  // K loop of a tile with m_rem valid rows.
  MSLK_AMD_DEVINL void accumulate_rows(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, int m_rem, int n_rem, int K,
                                       uint32_t ld, v4f (&acc)[TS::FN][TS::FM]) {
    // A tile with at most three quarters of its rows takes a K loop compiled for fewer m fragments per wave: the
    // fragments are dealt to the wave rows round-robin, so m_rem rows need ceil(ceil(m_rem / 16) / WM) of them.
    if constexpr (ROWSKIP && TS::RING == 0 && TS::FM % 4 == 0) {
      constexpr int Q = TS::kBM / 4;
      if (m_rem > 3 * Q) accumulate<TS::FM>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
      else if (m_rem > 2 * Q) accumulate<3 * TS::FM / 4>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
      else if (m_rem > Q) accumulate<TS::FM / 2>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
      else accumulate<TS::FM / 4>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
    } else {
      accumulate<TS::FM>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld, acc);
    }
  }

  // K loop only: acc = sum over the K bytes of the operand rows starting at xq_tile / wq_tile.  Ends with a
  // workgroup barrier, after which the LDS buffers are dead.
  template <int FMV = TS::FM>
  MSLK_AMD_DEVINL void accumulate(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, int m_rem, int n_rem, int K,
                                  uint32_t ld, v4f (&acc)[TS::FN][TS::FM]) {
    if constexpr (TS::RING == 0) {
      prologue<(FMV < TS::FM)>(lds, xq_tile, wq_tile, m_rem, n_rem, K, ld);
    } else {
      init(xq_tile, wq_tile, m_rem < TS::kBM ? m_rem : TS::kBM, n_rem < TS::kBN ? n_rem : TS::kBN, ld);
    }
    accumulate_issued<false, FMV>(lds, K, acc);
  }

  // Two-plus-three buffers only: per-lane addresses of a tile and the first DMA loads of its K loop (step 0 of both
  // operands, step 1 of WQ) into the buffers the loop starts from.  A persistent workgroup calls this for its next
  // tile before the epilogue of the current one, which must then stay out of those three buffers.
  template <bool LIVE_ROWS_ONLY = false>
  MSLK_AMD_DEVINL void prologue(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, int m_rem, int n_rem, int K,
                                uint32_t ld) {
    static_assert(TS::RING == 0, "the symmetric ring issues its own prologue");
    init(xq_tile, wq_tile, m_rem < TS::kBM ? m_rem : TS::kBM, n_rem < TS::kBN ? n_rem : TS::kBN, ld);
    const int KT = K / kBK;
    if (KT > 0) {
      if constexpr (LIVE_ROWS_ONLY) issue_a_live(lds, 0);
      else issue_a_all(lds, 0);
      issue_b_all(lds + 2 * TS::A_BYTES, 0);
      if (KT > 1) issue_b_all(lds + 2 * TS::A_BYTES + TS::B_BYTES, kBK);
    }
  }

  // K loop after prologue() (or, for the symmetric ring, after init()).  DRAIN: the wave has other memory
  // operations in flight behind the prologue loads (the stores of the previous tile's epilogue), so the first wait
  // is for all of them instead of "all but the youngest WQ loads".
  // What accumulate_issued<..., HOLD_LAST = true> leaves to the caller: the last full K step (its XQ fragments and WQ
  // fragment 0 in registers, its WQ tile in `b_cur`) and the two WQ buffers nobody touches any more.
  struct LastStep {
    v8i xf[TS::FM];
    v8i wf0;
    const char* b_cur;
    char* b_free0;
    char* b_free1;
  };
  // HOLD_LAST (K a positive multiple of the K step, two-plus-three buffers): the last step is not multiplied and the
  // final barrier is not passed; `last` describes it (see run_interior()).
  template <bool DRAIN, int FMV = TS::FM, bool HOLD_LAST = false>
  MSLK_AMD_DEVINL void accumulate_issued(char* lds, int K, v4f (&acc)[TS::FN][TS::FM], LastStep* last = nullptr) {
    static_assert(FMV == TS::FM || TS::RING == 0, "row skipping is built for the two-plus-three buffer tiles");
    static_assert(!HOLD_LAST || (TS::RING == 0 && FMV == TS::FM), "the held last step belongs to full two-plus-three buffer tiles");
#pragma unroll
    for (int tn = 0; tn < TS::FN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    const int KT = K / kBK;           // full steps
    const int k_tail = K - KT * kBK;  // 0 or a multiple of 16
    v8i xf[TS::FM], wf0;
    char* a_tail = lds;               // buffers the K tail may use once the full steps are done
    char* b_tail = lds + TS::A_STAGES * TS::A_BYTES;
    if constexpr (TS::RING == 0) {
      char* a_cur = lds;
      char* a_nxt = lds + TS::A_BYTES;
      char* b_cur = lds + 2 * TS::A_BYTES;
      char* b_nxt = b_cur + TS::B_BYTES;
      char* b_far = b_nxt + TS::B_BYTES;
      if (KT > 0) {
        if (KT > 1 && !DRAIN) wait_and_barrier<TS::LB>();
        else wait_and_barrier<0>();
        if constexpr (STAMPS) stamp_first_operands = __builtin_amdgcn_s_memrealtime();
        load_first_frags<FMV>(a_cur, b_cur, xf, wf0);
        // The prologue fetched XQ 0, WQ 0, WQ 1.  Step kt multiplies (the fragments of a_cur, b_cur) and fetches WQ of step
        // kt + 2 into b_far.  Of every XQ tile the first XT loads are issued two steps ahead (step kt: those of step kt + 2,
        // behind its barrier, into a_cur), the others one step ahead (step kt: those of step kt + 1, with the WQ loads, into
        // a_nxt).  Order of issue as a wave sees it: ... XQ(kt+1)[0,XT) | XQ(kt+1)[XT,LA) WQ(kt+2) | barrier kt | XQ(kt+2)[0,XT) ...:
        // at barrier kt only the LB loads of WQ(kt+2) may be pending.
        constexpr int XT = XQ_EARLY, XH = TS::LA - XT;
        if (KT > 1) {
          if constexpr (FMV < TS::FM) issue_a_live(a_nxt, kBK, 0, XT);
          else {
#pragma unroll
            for (int i = 0; i < XT; ++i) issue_a(a_nxt, kBK, i);
          }
        }
        for (int kt = 0; kt < KT - 2; ++kt) {
          step<XH, true, true, TS::LB, FMV, XT>(b_cur, a_nxt, a_nxt, b_nxt, b_far, (kt + 1) * kBK, (kt + 2) * kBK, acc, xf, wf0, a_cur, (kt + 2) * kBK);
          { char* t = a_cur; a_cur = a_nxt; a_nxt = t; }
          { char* t = b_cur; b_cur = b_nxt; b_nxt = b_far; b_far = t; }
        }
        if (KT > 1) {
          step<XH, false, true, 0, FMV>(b_cur, a_nxt, a_nxt, b_nxt, b_far, (KT - 1) * kBK, 0, acc, xf, wf0);
          { char* t = a_cur; a_cur = a_nxt; a_nxt = t; }
          { char* t = b_cur; b_cur = b_nxt; b_nxt = b_far; b_far = t; }
        }
        if constexpr (HOLD_LAST) {
          if constexpr (STAMPS) stamp_k_loop_end = __builtin_amdgcn_s_memrealtime();
#pragma unroll
          for (int tm = 0; tm < TS::FM; ++tm) last->xf[tm] = xf[tm];
          last->wf0 = wf0;
          last->b_cur = b_cur;
          last->b_free0 = b_nxt;
          last->b_free1 = b_far;
          return;
        }
        step<0, false, false, 0, FMV>(b_cur, a_nxt, a_nxt, b_nxt, b_far, 0, 0, acc, xf, wf0);
      }
    } else {
      // Symmetric ring: buffer i % RING holds step i; step kt fetches step kt + RING - 1 into the buffers step
      // kt - 1 used (free since the barrier of that step), and at its barrier everything but the loads of the
      // last RING - 2 steps has to be there.
      constexpr int NS = TS::RING;
      constexpr int PER_STEP = TS::LA + TS::LB;
      static_assert(NS >= 3 && (NS - 2) * PER_STEP < 64, "vmcnt is a 6-bit counter");
      char* const a0 = lds;
      char* const b0 = lds + NS * TS::A_BYTES;
      auto abuf = [&](int i) { return a0 + i * TS::A_BYTES; };
      auto bbuf = [&](int i) { return b0 + i * TS::B_BYTES; };
      if (KT > 0) {
        const int pre = KT < NS - 1 ? KT : NS - 1;
        for (int i = 0; i < pre; ++i) {
          issue_a_all(abuf(i), i * kBK);
          issue_b_all(bbuf(i), i * kBK);
        }
        if (pre == NS - 1) wait_and_barrier<(NS - 2) * PER_STEP>();
        else wait_and_barrier<0>();
        load_first_frags(abuf(0), bbuf(0), xf, wf0);
        int cur = 0;   // kt % NS
        int kt = 0;
        for (; kt + NS - 1 < KT; ++kt) {
          const int nxt = cur + 1 == NS ? 0 : cur + 1, far = cur == 0 ? NS - 1 : cur - 1;
          step<TS::LA, true, true, (NS - 2) * PER_STEP>(bbuf(cur), abuf(far), abuf(nxt), bbuf(nxt), bbuf(far),
                                                       (kt + NS - 1) * kBK, (kt + NS - 1) * kBK, acc, xf, wf0);
          cur = nxt;
        }
        for (; kt + 1 < KT; ++kt) {   // nothing left to fetch: the first of these steps waits for all that is in flight
          const int nxt = cur + 1 == NS ? 0 : cur + 1;
          step<0, false, true, 0>(bbuf(cur), abuf(nxt), abuf(nxt), bbuf(nxt), bbuf(nxt), 0, 0, acc, xf, wf0);
          cur = nxt;
        }
        step<0, false, false, 0>(bbuf(cur), abuf(cur), abuf(cur), bbuf(cur), bbuf(cur), 0, 0, acc, xf, wf0);
      }
    }
    if (k_tail > 0) {
      __syncthreads();   // everybody is done with the buffers of the full steps before one pair is refilled
      issue_loads_tail(a_tail, b_tail, KT * kBK, k_tail);
      wait_vmcnt0();    // the DMA loads are not visible to the compiler: the wait is explicit
      __syncthreads();
      load_first_frags<FMV>(a_tail, b_tail, xf, wf0);
      step<0, false, false, 0, FMV>(b_tail, a_tail, a_tail, b_tail, b_tail, 0, 0, acc, xf, wf0);
    }
    __syncthreads();  // the stages are dead from here on: the epilogue reuses LDS as a transpose buffer
  }

  // Epilogue.  A lane's accumulators of one 16-row m fragment are 4 consecutive n in each of the
  // FN n fragments; storing them directly would write 32-byte pieces of 16 different rows per
  // instruction.  Instead each wave scales, converts to bf16 and parks the 16 x (BN/2) block in a
  // private LDS buffer (row pitch BN + 16 bytes keeps the 8-byte writes and 16-byte reads off shared
  // banks), then reads it back row-major so that one store instruction writes 4 full rows of
  // BN/2 bf16 (16 lanes x 16 bytes each).
  // LDS the epilogue of one wave uses: two transpose buffers and the row scales of the wave's rows
  static constexpr int EPI_WAVE_BYTES = 2 * 16 * ((TS::kBN / TS::WN) * 2 + 16) + (TS::kBM / TS::WM) * 4;
  MSLK_AMD_DEVINL void epilogue(char* lds, v4f (&acc)[TS::FN][TS::FM], const float* xs, const float* ws,
                                const void* bias, uint16_t* y, int m_rem, int n_rem, int N) {
    static_assert((TS::NTHREADS / 64) * EPI_WAVE_BYTES <= TS::LDS_BYTES && EPI_WAVE_BYTES % 16 == 0, "epilogue buffers fit");
    epilogue_at(lds + wave_id() * EPI_WAVE_BYTES, acc, xs, ws, bias, y, m_rem, n_rem, N);
  }
  // As epilogue(), with the wave's private transpose buffer (EPI_WAVE_BYTES) placed by the caller.
  MSLK_AMD_DEVINL void epilogue_at(char* buf, v4f (&acc)[TS::FN][TS::FM], const float* xs, const float* ws,
                                   const void* bias, uint16_t* y, int m_rem, int n_rem, int N) {
    // Tiles whose columns are all valid (the common case, also for the ragged last row tile of an MoE
    // group) take a path whose only bounds logic is one row test per store instruction.
    // 16-byte accesses need 16-byte aligned rows of Y and aligned scale / bias vectors (a tile that
    // starts at a column offset inside a wider output may have neither).
    const bool vec16 = (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const bool full = n_rem >= TS::kBN && vec16 && (reinterpret_cast<uintptr_t>(ws) & 15) == 0 &&
                      (BIAS == 0 || (reinterpret_cast<uintptr_t>(bias) & (BIAS == 1 ? 15 : 7)) == 0);
    const bool interior = full && m_rem >= TS::kBM;   // no bounds logic at all
    if constexpr (ROWSKIP && TS::RING == 0 && TS::FM % 4 == 0) {
      // a tile multiplied by one of the reduced K loops has its m fragments dealt to the wave rows round-robin
      if (m_rem <= 3 * (TS::kBM / 4)) {
        if (out_f16) {
          if (full) epilogue_impl<true, true, false, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
          else epilogue_impl<false, true, false, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
        } else {
          if (full) epilogue_impl<true, false, false, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
          else epilogue_impl<false, false, false, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
        }
        return;
      }
    }
    if (out_f16) {
      if (interior) epilogue_impl<true, true, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
      else if (full) epilogue_impl<true, true, false>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
      else epilogue_impl<false, true, false>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
    } else {
      if (interior) epilogue_impl<true, false, true>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
      else if (full) epilogue_impl<true, false, false>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
      else epilogue_impl<false, false, false>(buf, acc, xs, ws, bias, y, m_rem, n_rem, N);
    }
  }

  // FULL: every column of the tile is valid and rows of Y are 16-byte aligned; rows may still be ragged unless
  // ALL_ROWS says that the tile has all its rows too.
  // ILV: the m fragments of the tile were dealt to the wave rows round-robin (ragged tiles of the grouped kernels).
  // FUSED: `last` holds the last K step, still to be multiplied; it is multiplied here, fragment row by fragment row,
  // with the epilogue of the rows that are final issued between its MFMAs (run_interior()).
  template <bool FULL, bool F16, bool ALL_ROWS, bool ILV = false, bool FUSED = false>
  MSLK_AMD_DEVINL void epilogue_impl(char* buf, v4f (&acc)[TS::FN][TS::FM], const float* xs, const float* ws,
                                     const void* bias, uint16_t* y, int m_rem, int n_rem, int N, LastStep* last = nullptr) {
    static_assert(!FUSED || (FULL && ALL_ROWS && !ILV && TS::RING == 0), "the fused last step is for interior tiles");
    constexpr int WN = TS::kBN / TS::WN;         // columns per wave
    constexpr int PITCH = WN * 2 + 16;           // bytes per staged row
    constexpr int BUF = 16 * PITCH;
    constexpr int CH = WN / 8;                   // 16-byte chunks per row (16 for BN = 256)
    constexpr int RPI = 64 / CH;                 // rows written per store instruction
    int lane = threadIdx.x & 63;
    // Everything derived from the lane id below is recomputed per call: inside a loop over tiles the compiler would
    // otherwise keep these values live across the K loop, where registers are scarce, and spill them.
    asm volatile("" : "+v"(lane));
    const int wave = wave_id();
    const int wm = wave / TS::WN, wn = wave % TS::WN;
    const int j = lane & 15, q = lane >> 4;
    constexpr int ROWS_W = TS::kBM / TS::WM;     // rows per wave
    static_assert(2 * BUF + ROWS_W * 4 == EPI_WAVE_BYTES, "epilogue buffer size");
    const int n_base = wn * WN;
    // tile row of row 0 of this wave's m fragment tm
    auto frag_row = [&](int tm) { return ILV ? (tm * TS::WM + wm) * 16 : wm * (TS::kBM / TS::WM) + tm * 16; };
    // fragments of this wave with at least one valid row (formed from m_rem: a persistent workgroup has already run
    // init() for its next tile when the epilogue of the current one starts)
    int fm_live = TS::FM;
    if constexpr (!ALL_ROWS) {
      const int nf = ((m_rem < TS::kBM ? m_rem : TS::kBM) + 15) >> 4;
      const int mine = ILV ? (nf - wm + TS::WM - 1) / TS::WM : nf - wm * TS::FM;
      fm_live = mine < 0 ? 0 : (mine > TS::FM ? TS::FM : mine);
    }
    const bool vec_store = (N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const bool pair_store = (N & 1) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;

    float wsv[TS::FN][4], bv[TS::FN][4];
#pragma unroll
    for (int tn = 0; tn < TS::FN; ++tn) {
      const int n = n_base + tn * 16 + 4 * q;
      if constexpr (FULL) {
        const float4 w4 = *reinterpret_cast<const float4*>(ws + n);
        wsv[tn][0] = w4.x; wsv[tn][1] = w4.y; wsv[tn][2] = w4.z; wsv[tn][3] = w4.w;
        if constexpr (BIAS == 1) {
          const float4 b4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(bias) + n);
          bv[tn][0] = b4.x; bv[tn][1] = b4.y; bv[tn][2] = b4.z; bv[tn][3] = b4.w;
        } else if constexpr (BIAS == 2) {
          const uint2 b2 = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(bias) + n);
          bv[tn][0] = bf16_bits_to_f32(b2.x & 0xFFFFu); bv[tn][1] = bf16_bits_to_f32(b2.x >> 16);
          bv[tn][2] = bf16_bits_to_f32(b2.y & 0xFFFFu); bv[tn][3] = bf16_bits_to_f32(b2.y >> 16);
        } else {
          bv[tn][0] = bv[tn][1] = bv[tn][2] = bv[tn][3] = 0.f;
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool ok = n + r < n_rem;
          wsv[tn][r] = ok ? ws[n + r] : 0.f;
          if constexpr (BIAS == 1) bv[tn][r] = ok ? reinterpret_cast<const float*>(bias)[n + r] : 0.f;
          else if constexpr (BIAS == 2) bv[tn][r] = ok ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(bias)[n + r]) : 0.f;
          else bv[tn][r] = 0.f;
        }
      }
    }

    const int rd_row = lane / CH, rd_chunk = lane % CH;
    const uint32_t lane_off = ((uint32_t)rd_row * (uint32_t)N + (uint32_t)(n_base + rd_chunk * 8)) * 2u;   // bytes; 16 N < 2^31
    constexpr int NP = 16 / RPI;                 // store instructions per 16-row fragment
    constexpr bool ACC_IN_AGPRS = TS::FM * TS::FN * 4 >= 256;
    static_assert(!FUSED || ACC_IN_AGPRS, "the fused last step reads accumulator registers");
    if constexpr (ACC_IN_AGPRS && !FUSED) {
      // The reads below are opaque to the compiler's hazard handling: 48 wait states let the last MFMA of the K loop
      // (32 cycles) retire before its result is read.
      asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15");
    }

    // The row scales go through LDS (one global load per row instead of one per lane and fragment row, and no
    // registers held for the whole epilogue).  All global loads of the epilogue are issued before its first store: the
    // wait for a load issued between stores would also wait for every older store to be acknowledged by memory.
    float* xs_lds = reinterpret_cast<float*>(buf + 2 * BUF);
#pragma unroll
    for (int i = 0; i < (ROWS_W + 63) / 64; ++i) {
      const int r = lane + i * 64;
      const int row = frag_row(r >> 4) + (r & 15);
      if (ROWS_W % 64 == 0 || r < ROWS_W) xs_lds[r] = (ALL_ROWS || row < m_rem) ? xs[row] : 0.f;
    }

    // Scale, convert and park n fragments [tn0, tn1) of fragment row tm in transpose buffer tm & 1.
    auto park = [&](int tm, int tn0, int tn1, float xsv) {
      char* b = buf + (tm & 1) * BUF;
#pragma unroll
      for (int tn = tn0; tn < tn1; ++tn) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // A tile of 256 accumulators per lane stays in accumulator registers until this point: left to itself
          // the register allocator moves part of it to vector registers ahead of time, runs out of them and spills,
          // and a reload between the stores waits for all of them.  (Smaller tiles live in vector registers.)
          float a;
          if constexpr (ACC_IN_AGPRS && !FUSED) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a) : "a"(acc[tn][tm][r]));   // volatile: stays behind the s_nop
          else a = acc[tn][tm][r];
          v[r] = (a * wsv[tn][r]) * xsv;   // w_scale first, then x_scale: the order of the reference's epilogue (fp8_rowwise_common.h:66)
          if constexpr (BIAS != 0) v[r] += bv[tn][r];
        }
        uint2 pk;
        pk.x = pack_out_x2<F16>(v[0], v[1]);
        pk.y = pack_out_x2<F16>(v[2], v[3]);
        *reinterpret_cast<uint2*>(b + j * PITCH + (tn * 16 + 4 * q) * 2) = pk;
      }
    };
    // Row-major read-back of fragment row tm (the buffer is private to the wave and LDS operations of one wave
    // complete in order, so no barrier separates it from park(tm)).
    auto fetch = [&](int tm, uint4 (&val)[NP]) {
      const char* b = buf + (tm & 1) * BUF;
#pragma unroll
      for (int pass = 0; pass < NP; ++pass)
        val[pass] = *reinterpret_cast<const uint4*>(b + (pass * RPI + rd_row) * PITCH + rd_chunk * 16);
    };
    // Wave-uniform 64-bit row base + one 32-bit lane offset that is the same for every store of the tile.
    auto dst_of = [&](int tm, int pass) {
      return reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(y + (int64_t)(frag_row(tm) + pass * RPI) * N) + lane_off);
    };

    if constexpr (FUSED) {
      static_assert(TS::FN % NP == 0, "whole n fragments per store");
      constexpr int TPP = TS::FN / NP;   // n fragments (and MFMAs of a fragment row) per store instruction
      const FragOff fo = frag_off();
      const char* b_tile = b_tile_of(last->b_cur);
      v8i wf[TS::FN];
      wf[0] = last->wf0;
#pragma unroll
      for (int tn = 1; tn < TS::FN; ++tn) wf[tn] = load_frag_b(b_tile, tn, fo);
      uint4 val[NP];
      char* dst = reinterpret_cast<char*>(y + (int64_t)frag_row(0) * N) + lane_off;
      const int64_t dst_step = (int64_t)RPI * N * 2;
      float xsv = 0.f;
      __builtin_amdgcn_sched_barrier(0);
      // iteration t: MFMAs of fragment row t, park of row t - 1 (its MFMAs were issued a whole row, 8 x 32 cycles, ago),
      // stores of row t - 2
#pragma unroll
      for (int t = 0; t < TS::FM + 2; ++t) {
        if (t >= 2) fetch(t - 2, val);
        if (t >= 1 && t - 1 < TS::FM) xsv = xs_lds[(t - 1) * 16 + j];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pass = 0; pass < NP; ++pass) {
          if (t < TS::FM) {
#pragma unroll
            for (int tn = pass * TPP; tn < (pass + 1) * TPP; ++tn)
              acc[tn][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[tn], last->xf[t], acc[tn][t], 0, 0, 0, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
          }
          if (t >= 1 && t - 1 < TS::FM) {
            park(t - 1, pass * TPP, (pass + 1) * TPP, xsv);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (t >= 2) {
            store16_stream(reinterpret_cast<uint16_t*>(dst), val[pass]);
            dst += dst_step;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else if constexpr (FULL) {
      // With one wave per SIMD nothing else hides the LDS round trip between parking a fragment row and
      // storing it, so the rows are pipelined by hand: the read-back of row tm - 1 is issued before the
      // arithmetic of row tm and its stores follow that arithmetic.
      // The stores of row tm - 1 are spread between the pieces of that arithmetic, so the store path and the
      // vector ALU work side by side.
      static_assert(TS::FN % NP == 0, "whole n fragments per store");
      uint4 val[NP];
      // consecutive store instructions of a fragment are RPI rows apart, consecutive fragments of a wave 16 * WM rows:
      // one 64-bit add per store
      char* dst = reinterpret_cast<char*>(y + (int64_t)frag_row(0) * N) + lane_off;
      const int64_t dst_step = (int64_t)RPI * N * 2;
      const int64_t frag_step = ILV ? (int64_t)(TS::WM - 1) * 16 * N * 2 : 0;
      float xsv = xs_lds[j];
#pragma unroll
      for (int tm = 0; tm <= TS::FM; ++tm) {
        // ragged tiles: fragments without a valid row are neither scaled nor stored (wave-uniform tests)
        const bool do_park = tm < TS::FM && (ALL_ROWS || tm < fm_live);
        const bool do_store = tm > 0 && (ALL_ROWS || tm - 1 < fm_live);
        if (do_store) fetch(tm - 1, val);
        const float xsv_next = tm + 1 < TS::FM ? xs_lds[(tm + 1) * 16 + j] : 0.f;   // read one fragment row ahead
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pass = 0; pass < NP; ++pass) {
          if (do_park) park(tm, pass * (TS::FN / NP), (pass + 1) * (TS::FN / NP), xsv);
          __builtin_amdgcn_sched_barrier(0);
          if (tm > 0) {
            const int r0 = frag_row(tm - 1) + pass * RPI;   // first of the RPI rows this instruction writes
            if (ALL_ROWS || r0 + RPI <= m_rem) store16_stream(reinterpret_cast<uint16_t*>(dst), val[pass]);   // wave-uniform test
            else if (do_store && r0 + rd_row < m_rem) store16_stream(reinterpret_cast<uint16_t*>(dst), val[pass]);    // ragged last rows
            dst += dst_step;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if (ILV && tm > 0 && TS::WM > 1) dst += frag_step;
        xsv = xsv_next;
      }
    } else {
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm) {
        if (tm >= fm_live) continue;   // no valid row in this fragment (wave-uniform)
        park(tm, 0, TS::FN, xs_lds[tm * 16 + j]);
        uint4 vals[NP];
        fetch(tm, vals);
#pragma unroll
        for (int pass = 0; pass < NP; ++pass) {
          const uint4 val = vals[pass];
          const int mm = frag_row(tm) + pass * RPI + rd_row;
          const int nn = n_base + rd_chunk * 8;
          uint16_t* dst = dst_of(tm, pass);
          if (mm >= m_rem || nn >= n_rem) continue;
          if (vec_store && nn + 7 < n_rem) {
            store16_stream(dst, val);
          } else if (nn + 7 < n_rem) {
            // all eight columns valid, but rows of Y are only 2- or 4-byte aligned (N % 8 != 0): a 16-byte copy with
            // no alignment promise, for which the compiler picks the widest store the target allows
            __builtin_memcpy(dst, &val, 16);
          } else if (pair_store) {   // rows are 4-byte aligned: store bf16 pairs
            const uint32_t w[4] = {val.x, val.y, val.z, val.w};
            uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (nn + 2 * e + 1 < n_rem) d32[e] = w[e];
              else if (nn + 2 * e < n_rem) dst[2 * e] = (uint16_t)w[e];
            }
          } else {
            const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (nn + e < n_rem) dst[e] = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
          }
        }
      }
    }
  }
};

}  // namespace mslk_amd
