"""Benchmark of the FP8 rowwise quantized-linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras]

Prints ONE JSON line.  The headline (`value`) is the reference's own GEMM metric
(bench/gemm/gemm_bench.py:490: 2*M*N*K / t of the f8f8bf16_rowwise call, quantization outside the
timed region as in bench/gemm/gemm_ops.py:162-169) on BASELINE config 1: M=N=K=4096, x with 1 % outlier
channels, pre-quantized w.  A step is one f8f8bf16_rowwise call through the C ABI with all operands
resident in HBM; steps rotate over several operand sets so that consecutive calls do not find their
inputs in the 256 MB Infinity Cache.  Extras in the same line: the quantize pass (GB/s), quantize + GEMM
as one path, the decode sweep (M in 1,4,16,64 at N=K=8192, GB/s of algorithmic bytes), cfg0/cfg2/cfg4 GEMM
rates, the roofline object of the dominant kernel and the CPU baseline (the reference's CPU torch path
restated in oracle/, timed on this host's cores on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_FLOPS = 5.0e15     # MI355X dense FP8 MFMA
PEAK_FP8_FLOPS_REF = 4.6e15  # the figure the reference's bench uses for gfx950 (bench/gemm/gemm_bench.py:61-68)
PEAK_HBM_BPS = 8.0e12


TRAFFIC_SOURCE = "profiles/gemm_4096_traffic_pmc.txt"


def _measured_traffic_bytes():
    """HBM-side bytes per 4096^3 GEMM launch from the committed rocprofv3 FETCH_SIZE/WRITE_SIZE summary
    (counters cannot be read from inside this process); None when the summary is absent."""
    path = os.path.join(ROOT, *TRAFFIC_SOURCE.split("/"))
    try:
        for ln in open(path):
            if ln.startswith("traffic per launch ="):
                return float(ln.split("=")[1].split("MB")[0]) * 1e6
    except OSError:
        pass
    return None


def _events_ms(fn, iters):
    """Average duration of fn() in ms, HIP events on the current stream (the one kernels launch on)."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


SETTLE_MS = 50.0


def _settle(fn, min_ms=SETTLE_MS):
    """Clock-settling phase OUTSIDE every timed region: fn(i) is launched until at least `min_ms` of GPU time has passed
    (the shader clock, the power state and the caches reach the state a long-running job sees; a handful of warm-up
    steps does not get there).  Returns the number of launches."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    start.record()
    n = 0
    while True:
        for _ in range(32):
            fn(n)
            n += 1
        stop = torch.cuda.Event(enable_timing=True)
        stop.record()
        stop.synchronize()
        if start.elapsed_time(stop) >= min_ms:
            return n


def _parity(y, xq, wq, xs, ws, bias=None, block=2048):
    """The three accuracy figures of the path for one output, against the rowwise-dequantized fp32 product formed on the
    GPU with plain torch (a floating-point reference, not the product path): max|y-ref|/max|ref|, ||y-ref||_F/||ref||_F and
    the number of elements beyond |y-ref| <= 1e-2 |ref| + 1e-2 rms(ref) (the elementwise form of the reference's tests,
    test/gemm/gemm_test.py:493-505)."""
    import torch
    wd = wq.float() * ws.float()[:, None]
    M = xq.shape[0]
    max_abs_ref = 0.0
    max_abs_diff = 0.0
    sq_ref = 0.0
    sq_diff = 0.0
    refs = []
    for r0 in range(0, M, block):
        ref = (xq[r0:r0 + block].float() * xs[r0:r0 + block].float()[:, None]) @ wd.t()
        if bias is not None:
            ref += bias.float()[None, :]
        d = y[r0:r0 + block].float() - ref
        max_abs_ref = max(max_abs_ref, ref.abs().max().item())
        max_abs_diff = max(max_abs_diff, d.abs().max().item())
        sq_ref += ref.double().pow(2).sum().item()
        sq_diff += d.double().pow(2).sum().item()
        refs.append((r0, ref.abs(), d.abs()))
    n = float(M) * wq.shape[0]
    rms = (sq_ref / n) ** 0.5
    bad = sum(int((d > 1e-2 * a + 1e-2 * rms).sum().item()) for _, a, d in refs)
    return {"max_rel": max_abs_diff / max_abs_ref if max_abs_ref else 0.0, "normwise": (sq_diff / sq_ref) ** 0.5 if sq_ref else 0.0,
            "elementwise_violations": bad, "elements": int(n)}


def _median_events_ms(fn, iters, repeats=5):
    xs = sorted(_events_ms(fn, iters) for _ in range(repeats))
    return xs[len(xs) // 2]


def _graph_ms(fn, iters, repeats=5):
    """Per-call time of `iters` calls of fn(i) recorded into ONE HIP graph and replayed (the way the
    reference's bench times its ops: triton do_bench_cudagraph, bench/common/utils.py:55-63)."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(min(iters, 8)):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(iters):
            fn(i)
    # Capture is host work during which the GPU idles and its clocks fall; a replay of a short graph lasts about a
    # millisecond, so a few warm-up replays do not bring them back (decode GEMMs measured 0.5 - 2 us per node slower that
    # way than the same kernels launched one by one after a settling phase).  Replay for the same settling time instead.
    warm = torch.cuda.Event(enable_timing=True)
    warm.record()
    while True:
        for _ in range(3):
            graph.replay()
        now = torch.cuda.Event(enable_timing=True)
        now.record()
        now.synchronize()
        if warm.elapsed_time(now) >= 20.0:
            break
    times = []
    for _ in range(repeats):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop) / iters)
    return sorted(times)[len(times) // 2]


class CApi:
    """Direct C-ABI callers (a few microseconds of host time per launch)."""

    def __init__(self):
        import torch
        from mslk_amd import _lib
        self.L = _lib.lib()
        self.check = _lib.check

    @property
    def stream(self):
        import torch
        return torch.cuda.current_stream().cuda_stream

    def gemm(self, xq, wq, xs, ws, y, bias=None):
        M = xq.shape[0]
        N, K = wq.shape
        bcode = 0 if bias is None else (1 if bias.dtype.itemsize == 4 else 2)
        # the workspace the library asks for (K-split shapes), allocated once per size and outside every timed region,
        # as the caching allocator does for the operator
        need = self.L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
        wsp = None
        if need:
            import torch
            if getattr(self, "_wsp", None) is None or self._wsp.numel() < need:
                self._wsp = torch.empty(need, dtype=torch.uint8, device=xq.device)
            wsp = self._wsp.data_ptr()
        self.check(self.L.mslk_amd_f8f8bf16_rowwise(xq.data_ptr(), wq.data_ptr(), xs.data_ptr(), ws.data_ptr(),
                                                    None if bias is None else bias.data_ptr(), bcode, y.data_ptr(),
                                                    M, N, K, wsp, need, self.stream))

    def grouped_call(self, xq, wq, xs, ws, ys):
        """Pre-marshalled TensorList call: returns a closure that only crosses the C ABI."""
        import ctypes
        G = len(xq)
        P = ctypes.c_void_p * G
        I = ctypes.c_int64 * G
        args = (G, P(*[t.data_ptr() for t in xq]), P(*[t.data_ptr() for t in wq]), P(*[t.data_ptr() for t in xs]),
                P(*[t.data_ptr() for t in ws]), P(*[t.data_ptr() for t in ys]), I(*[t.shape[0] for t in xq]),
                I(*[t.shape[0] for t in wq]), I(*[t.shape[1] for t in wq]), self.stream)
        return lambda: self.check(self.L.mslk_amd_f8f8bf16_rowwise_grouped(*args))

    def quantize(self, x, xq, scale):
        rows, K = x.shape
        self.check(self.L.mslk_amd_quantize_fp8_row(x.data_ptr(), 0, rows, K, K, xq.data_ptr(), K, scale.data_ptr(),
                                                    None, self.stream))


def cpu_baseline(wl, budget_s=20.0):
    """Times the reference's CPU torch path (quantize torch branch + matmul_fp8_row CPU fallback, restated in
    oracle/) on a row sample of the same workload sized to about `budget_s` seconds of CPU work."""
    import torch
    from oracle import fp8_rowwise_oracle as O
    N, K = wl.w.shape
    wq, ws = O.quantize_fp8_row(wl.w)
    probe_rows = 64
    xq, xs = O.quantize_fp8_row(wl.x[:probe_rows])
    t0 = time.perf_counter()
    O.matmul_fp8_row_cpu(xq, wq, xs, ws)
    probe = max(time.perf_counter() - t0, 1e-4)
    rows = int(min(wl.x.shape[0], max(probe_rows, probe_rows * (budget_s / 3.0) / probe)))
    rows = max(64, rows // 64 * 64)
    x = wl.x[:rows]
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        q, s = O.quantize_fp8_row(x)
        O.matmul_fp8_row_cpu(q, wq, s, ws, wl.bias)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[1]
    return {"value": 2.0 * rows * N * K / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"first {rows} of {wl.x.shape[0]} rows of x (quantize_fp8_row torch branch + bf16 matmul CPU fallback), "
                      f"N={N}, K={K}, median of 3, {t * 1e3:.1f} ms; os.cpu_count()={os.cpu_count()}"}


def _vendor_sweep(api):
    """`--only vendor`: this library against the vendor library (hipBLASLt behind torch._scaled_mm, row-wise scales) on
    weight shapes of 8B / 70B-class models at M = 1 ... 16384; same operands, rotating sets larger than the caches,
    best of three event-timed loops.  Prints one line per shape and a summary line (JSON)."""
    import torch
    import mslk_amd
    dev = "cuda:0"
    ratios = []
    for (N, K) in [(8192, 8192), (10240, 8192), (57344, 8192), (8192, 28672), (4096, 4096), (6144, 4096), (28672, 4096), (4096, 14336)]:
        nsets = 6 if N * K < 2 ** 27 else 3
        g = torch.Generator(device=dev).manual_seed(N + K)
        weights = [mslk_amd.quantize_fp8_row(torch.randn(N, K, device=dev, generator=g).bfloat16(), use_triton=False) for _ in range(nsets)]
        for M in (1, 16, 64, 128, 256, 384, 512, 1024, 2048, 4096, 8192, 16384):
            acts = [mslk_amd.quantize_fp8_row(torch.randn(M, K, device=dev, generator=g).bfloat16(), use_triton=False) for _ in range(nsets)]
            ys = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nsets)]

            def ours(i):
                j = i % nsets
                api.gemm(acts[j][0], weights[j][0], acts[j][1], weights[j][1], ys[j])

            def vendor(i):
                j = i % nsets
                torch._scaled_mm(acts[j][0], weights[j][0].t(), scale_a=acts[j][1][:, None], scale_b=weights[j][1][None, :],
                                 out_dtype=torch.bfloat16)

            def best_us(fn):
                for i in range(8):
                    fn(i)
                torch.cuda.synchronize()
                return min(_events_ms(fn, 40) for _ in range(3)) * 1e3

            vendor(0)   # the first call picks the vendor kernel
            t_vendor, t_ours = best_us(vendor), best_us(ours)
            ratios.append(t_vendor / t_ours)
            print(f"M={M:6d} N={N:6d} K={K:6d}: ours {t_ours:8.1f} us {2.0 * M * N * K / t_ours / 1e9:5.2f} PFLOP/s | "
                  f"vendor {t_vendor:8.1f} us | vendor/ours {t_vendor / t_ours:4.2f}", flush=True)
            del acts, ys
        del weights
        torch.cuda.empty_cache()
    ratios.sort()
    print(json.dumps({"shapes": len(ratios), "ours_faster": sum(r > 1.0 for r in ratios), "median_ratio": round(ratios[len(ratios) // 2], 3),
                      "min_ratio": round(ratios[0], 3), "max_ratio": round(ratios[-1], 3)}))


def _vendor_random(api, seed, cases):
    """`--only vendor-random --seed S --cases N`: as `--only vendor`, on N shapes drawn with seed S -- M log-uniform in
    1 ... 23000 (40 %: a batch size from a fixed list), N and K from the dimensions of common models, capped at 2^41
    multiply-adds.  Prints one line per shape with the kernel the dispatch picks, then the shapes this library is behind on."""
    import random
    import torch
    import mslk_amd
    dev = "cuda:0"
    rnd = random.Random(seed)
    g = torch.Generator(device=dev).manual_seed(7)

    def q(r, c, s=1.0):
        return mslk_amd.quantize_fp8_row((torch.randn(r, c, device=dev, generator=g) * s).bfloat16(), use_triton=False)

    def best_us(fn):
        for i in range(6):
            fn(i)
        torch.cuda.synchronize()
        return min(_events_ms(fn, 30) for _ in range(3)) * 1e3

    res = []
    for _ in range(cases):
        N = rnd.choice([512, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192, 11008, 12288, 13824, 14336, 16384,
                        22016, 24576, 32768])
        K = rnd.choice([512, 1024, 2048, 2560, 3072, 4096, 5120, 6144, 7168, 8192, 11008, 13824, 14336, 16384])
        M = int(2 ** rnd.uniform(0, 14.5))
        if rnd.random() < 0.4:
            M = rnd.choice([8, 32, 48, 96, 192, 320, 768, 1536, 3072, 6144, 12288])
        while M * N * K > 2 ** 41:
            M //= 2
        M = max(M, 1)
        nsets = max(2, min(6, (400 << 20) // (N * K)))
        ws = [q(N, K, 0.02) for _ in range(nsets)]
        xs = [q(M, K) for _ in range(nsets)]
        y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

        def ours(i):
            j = i % nsets
            api.gemm(xs[j][0], ws[j][0], xs[j][1], ws[j][1], y)

        def vendor(i):
            j = i % nsets
            torch._scaled_mm(xs[j][0], ws[j][0].t(), scale_a=xs[j][1][:, None], scale_b=ws[j][1][None, :], out_dtype=torch.bfloat16)

        try:
            vendor(0)
            tv = best_us(vendor)
        except Exception:   # the vendor library may not take the shape
            tv = float("nan")
        to = best_us(ours)
        name = api.L.mslk_amd_debug_dispatch_name(M, N, K, 0, 0, 0, 1).decode()
        print(f"M={M:6d} N={N:6d} K={K:6d}: ours {to:8.1f} us  vendor {tv:8.1f} us  vendor/ours {tv / to:5.2f}  "
              f"{2.0 * M * N * K / to / 1e9:5.2f} PFLOP/s  {name}", flush=True)
        res.append((tv / to, M, N, K))
        del ws, xs, y
    ok = [r for r in res if r[0] == r[0]]
    ok.sort()
    print(json.dumps({"seed": seed, "shapes": len(res), "ours_faster": sum(1 for r in ok if r[0] >= 1.0),
                      "median_ratio": ok[len(ok) // 2][0] if ok else None,
                      "behind": [{"M": M, "N": N, "K": K, "vendor_over_ours": round(r, 3)} for (r, M, N, K) in ok if r < 1.0]}))


def _ksplit(api):
    """`--only ksplit`: shapes with few output tiles and a long K, timed with the workspace the library asks for (K split:
    two launches) and without it (the ordinary kernels), same operands, rotating weight sets.  One line per shape."""
    import torch
    import mslk_amd
    dev = "cuda:0"
    L = api.L
    g = torch.Generator(device=dev).manual_seed(3)

    def q(r, c, s=1.0):
        return mslk_amd.quantize_fp8_row((torch.randn(r, c, device=dev, generator=g) * s).bfloat16(), use_triton=False)

    rows = []
    for K in (6144, 8192, 14336):
        for N in (512, 1024, 2048, 4096):
            nsets = max(2, min(8, (300 << 20) // (N * K)))
            ws = [q(N, K, 0.02) for _ in range(nsets)]
            for M in (64, 96, 128, 256, 512):
                need = L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
                xq, xs = q(M, K)
                y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                wsp = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)

                def run(with_workspace):
                    def step(i):
                        w, sc = ws[i % nsets]
                        api.check(L.mslk_amd_f8f8bf16_rowwise(xq.data_ptr(), w.data_ptr(), xs.data_ptr(), sc.data_ptr(), None, 0, y.data_ptr(),
                                                              M, N, K, wsp.data_ptr() if with_workspace else None,
                                                              need if with_workspace else 0, api.stream))
                    for i in range(5):
                        step(i)
                    torch.cuda.synchronize()
                    return min(_median_events_ms(step, 40) for _ in range(2)) * 1e3

                unsplit = run(False)
                split = run(True) if need else None
                name = L.mslk_amd_debug_dispatch_name(M, N, K, 0, 0, 0, 1).decode()
                rows.append({"M": M, "N": N, "K": K, "unsplit_us": round(unsplit, 2), "with_workspace_us": None if split is None else round(split, 2),
                             "slices": need // (M * N * 4), "dispatch": name})
                print(f"M={M:4d} N={N:5d} K={K:6d}: unsplit {unsplit:6.1f} us | " +
                      (f"K split in {need // (M * N * 4)} slices {split:6.1f} us ({unsplit / split:4.2f}x)" if need else "not split"), flush=True)
            del ws
    done = [r for r in rows if r["with_workspace_us"]]
    print(json.dumps({"shapes": len(rows), "split": len(done),
                      "slower_than_unsplit_by_more_than_2_percent": sum(1 for r in done if r["with_workspace_us"] > 1.02 * r["unsplit_us"]),
                      "best_ratio": max(r["unsplit_us"] / r["with_workspace_us"] for r in done) if done else None}))


def _ceilings(api):
    """`--only ceilings`: what this GPU sustains on the two resources the roofline fractions are priced against, from
    kernels that live in the library (mslk_amd_debug_stream_read / mslk_amd_debug_mfma_loop): a pure read of HBM-resident
    buffers (register loads and the LDS-DMA loads of the GEMM kernels, the decode weight size and 1 GiB) and a
    register-only FP8 MFMA loop in both instruction forms on zeros, uniform random codes and the codes of the cfg1
    operands.  Prints one JSON line."""
    import torch
    import mslk_amd
    from mslk_amd import workloads as W
    dev = "cuda:0"
    L = api.L
    out = {}
    sink = torch.zeros(16, dtype=torch.int32, device=dev)
    # ---- streaming read: six distinct 64 MiB buffers (more than the 256 MB Infinity Cache) and one 1 GiB buffer
    small = [torch.randint(0, 255, (64 << 20,), dtype=torch.uint8, device=dev) for _ in range(6)]
    big = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device=dev)
    for mode, mname in ((0, "register_loads"), (1, "lds_dma_loads"), (2, "lds_dma_loads_nontemporal")):
        for label, bufs in (("64MiB", small), ("1GiB", [big])):
            best = None
            for wgs in (512, 1024, 2048, 4096):
                def step(i, bufs=bufs, wgs=wgs, mode=mode):
                    b = bufs[i % len(bufs)]
                    api.check(L.mslk_amd_debug_stream_read(b.data_ptr(), b.numel(), mode, wgs, sink.data_ptr(), api.stream))
                _settle(step, 10.0)
                ms = _median_events_ms(step, 30 if label == "64MiB" else 6)
                if best is None or ms < best[0]:
                    best = (ms, wgs)
            nbytes = bufs[0].numel()
            out[f"stream_read_{mname}_{label}"] = {"ms": best[0], "workgroups": best[1], "TBps": nbytes / (best[0] * 1e-3) / 1e12,
                                                   "frac_of_8TBps": nbytes / (best[0] * 1e-3) / PEAK_HBM_BPS}
    # ---- the operand streams of a medium-M shape alone: M = 256, N = K = 8192 on 128 x 64 tiles (256 workgroups, two row
    # tiles), activations from the L2, weights from HBM (the six 64 MiB buffers in turn), without LDS reads or multiplies;
    # beside them the GEMM itself on the same bytes
    Mt, Nt, Kt = 256, 8192, 8192
    xbuf = small[0][: Mt * Kt].clone()
    ones_m, ones_n = torch.ones(Mt, device=dev), torch.ones(Nt, device=dev)
    yt = torch.empty(Mt, Nt, dtype=torch.bfloat16, device=dev)
    for b in small + [xbuf]:
        b &= 0x77                                            # no NaN codes, so that the GEMM beside the probe multiplies finite values
    streams = {}
    for which, wname in ((1, "activations_only"), (2, "weights_only"), (3, "both")):
        def step(i, which=which):
            b = small[i % len(small)]
            api.check(L.mslk_amd_debug_tile_streams(xbuf.data_ptr(), xbuf.numel(), b.data_ptr(), b.numel(), Kt, Mt // 128, Nt // 64,
                                                    which, api.stream))
        _settle(step, 10.0)
        streams[wname + "_us"] = _median_events_ms(step, 60) * 1e3
    f8 = torch.float8_e4m3fn
    def gemm_step(i):
        api.gemm(xbuf.view(f8).view(Mt, Kt), small[i % len(small)].view(f8).view(Nt, Kt), ones_m, ones_n, yt)
    _settle(gemm_step, 10.0)
    streams["gemm_us"] = _median_events_ms(gemm_step, 60) * 1e3
    streams["gemm_kernel"] = L.mslk_amd_debug_dispatch_name(Mt, Nt, Kt, 0, 0, 0, 1).decode()
    streams["MB_activations_per_launch_from_L2"] = (Mt // 128) * (Nt // 64) * 128 * Kt / 1e6
    streams["MB_weights_per_launch_from_HBM"] = Nt * Kt / 1e6
    out["tile_streams_M256_N8192_K8192"] = streams
    del small, big
    # the launch itself: the same kernel on 16 bytes
    tiny = torch.zeros(1024, dtype=torch.uint8, device=dev)
    out["empty_launch_us"] = _median_events_ms(
        lambda i: api.check(L.mslk_amd_debug_stream_read(tiny.data_ptr(), 1024, 0, 256, sink.data_ptr(), api.stream)), 200) * 1e3
    # ---- register-only MFMA loops: 256 workgroups x 4 waves x iters x 2 * 128^3 FLOP
    wl = W.cfg1()
    xq, _ = mslk_amd.quantize_fp8_row(wl.x[:64].to(dev), use_triton=False)
    wq, _ = mslk_amd.quantize_fp8_row(wl.w[:64].to(dev), use_triton=False)
    cfg1_codes = torch.cat([xq.view(torch.uint8).reshape(-1)[:65536], wq.view(torch.uint8).reshape(-1)[:65536]]).contiguous()
    rnd = torch.randint(0, 255, (131072,), dtype=torch.uint8, device=dev)
    rnd[(rnd & 0x7F) == 0x7F] = 0x30                      # no NaN codes
    datas = (("zeros", torch.zeros(131072, dtype=torch.uint8, device=dev)), ("uniform_random_codes", rnd),
             ("cfg1_operand_codes", cfg1_codes))
    iters, wgs = 512, 256
    flops = wgs * 4 * iters * 2.0 * 128 ** 3
    fsink = torch.zeros(16, device=dev)
    for dname, data in datas:
        for form, fname in ((0, "16x16x128"), (1, "32x32x64")):
            def step(i, data=data, form=form):
                api.check(L.mslk_amd_debug_mfma_loop(data.data_ptr(), form, iters, wgs, fsink.data_ptr(), api.stream))
            _settle(step, 30.0)
            ms = _median_events_ms(step, 20)
            out[f"mfma_loop_{fname}_{dname}"] = {"ms": ms, "PFLOPs": flops / (ms * 1e-3) / 1e15,
                                                 "frac_of_5PF": flops / (ms * 1e-3) / PEAK_FP8_FLOPS,
                                                 "implied_clock_GHz": flops / (ms * 1e-3) / (256 * 4 * 2048.0) / 1e9}
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--only", default="",
                    help="helper: run only this piece (gemm|gemm-timed|power|phases|quantize|decode|decode-eager|decode-graph|cfg2|grouped|traffic|vendor|vendor-random|ksplit|ceilings) and exit")
    ap.add_argument("--seed", type=int, default=1, help="--only vendor-random: seed of the shape draw")
    ap.add_argument("--cases", type=int, default=80, help="--only vendor-random: number of shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives or sharding in the path); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import mslk_amd  # noqa: F401
    from mslk_amd import workloads as W

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    api = CApi()
    extras = {}
    if args.only == "vendor":
        _vendor_sweep(api)
        return
    if args.only == "ksplit":
        _ksplit(api)
        return
    if args.only == "vendor-random":
        _vendor_random(api, args.seed, args.cases)
        return
    if args.only == "ceilings":
        _ceilings(api)
        return

    # ---------------------------------------------------------------- cfg1: 4096^3
    wl = W.cfg1()
    M, K = wl.x.shape
    N = wl.w.shape[0]
    x_dev = wl.x.to(dev)
    wq0, ws0 = mslk_amd.quantize_fp8_row(wl.w.to(dev), use_triton=False)
    xq0, xs0 = mslk_amd.quantize_fp8_row(x_dev, use_triton=False)
    NSETS = 6  # 6 x (16 + 16 + 32 MiB) = 384 MiB of distinct operands > 256 MB Infinity Cache
    sets = [(xq0.clone(), wq0.clone(), xs0.clone(), ws0.clone(), torch.empty(M, N, dtype=torch.bfloat16, device=dev))
            for _ in range(NSETS)]

    def gemm_step(i):
        xq, wq, xs, ws, y = sets[i % NSETS]
        api.gemm(xq, wq, xs, ws, y)

    flops = 2.0 * M * N * K
    if args.only == "phases":
        # Where the time of the headline launch goes: the measuring build of the same kernel (four counter readings per
        # wave, mslk_amd_debug_gemm_phases) on the same operand rotation, on the cfg1 codes and on all-zero codes.
        stamps = torch.zeros(256 * 4 * 4, dtype=torch.int64, device=dev)
        out = {}
        for label in ("cfg1_codes", "zero_codes"):
            psets = sets if label == "cfg1_codes" else [(torch.zeros_like(xq0), torch.zeros_like(wq0), xs0, ws0, sets[j][4]) for j in range(NSETS)]

            def phase_step(i):
                xq, wq, xs, ws, y = psets[i % NSETS]
                api.check(api.L.mslk_amd_debug_gemm_phases(xq.data_ptr(), wq.data_ptr(), xs.data_ptr(), ws.data_ptr(), y.data_ptr(),
                                                           M, N, K, stamps.data_ptr(), api.stream))

            _settle(phase_step)
            period_ms = _median_events_ms(phase_step, 200)
            torch.cuda.synchronize()
            t = stamps.view(256, 4, 4).cpu().double() * 1e-2   # 100 MHz counter -> microseconds
            t = t - t[..., 0].min()
            entry, first, k_end, end = (t[..., i].flatten() for i in range(4))

            def mmm(v):
                return {"min": round(float(v.min()), 2), "median": round(float(v.median()), 2), "max": round(float(v.max()), 2)}

            xcd_last = [round(float(t[torch.arange(256) % 8 == c][..., 3].max()), 2) for c in range(8)]
            out[label] = {"us_per_launch_events": round(period_ms * 1e3, 2),
                          "wave_entry_after_first_entry_us": mmm(entry),
                          "entry_to_first_operands_us": mmm(first - entry),
                          "k_loop_31_steps_us": mmm(k_end - first),
                          "k_loop_per_step_us": mmm((k_end - first) / (K // 128 - 1)),
                          "last_step_fused_with_epilogue_us": mmm(end - k_end),
                          "wave_end_after_first_entry_us": mmm(end),
                          "last_wave_end_per_xcd_us": xcd_last,
                          "launch_period_minus_last_wave_end_us": round(period_ms * 1e3 - float(end.max()), 2)}
        print(json.dumps({"gemm_phases_4096": out}))
        return
    if args.only == "traffic":
        # Counter calibration for `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`: a plain device copy of known
        # size (256 MiB read + 256 MiB written by one elementwise kernel) next to a few GEMM launches.
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        for i in range(12):
            gemm_step(i)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_each_way": 256 << 20, "gemm_launches": 12}))
        return
    settle_launches = 0
    if args.only in ("", "gemm", "gemm-timed", "power"):
        settle_launches = _settle(gemm_step)      # outside the timed region, named in config.workload
        for i in range(args.warmup):
            gemm_step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev_start = torch.cuda.Event(enable_timing=True)
        ev_stop = torch.cuda.Event(enable_timing=True)
        ev_start.record()
        for i in range(args.steps):
            gemm_step(i)
        ev_stop.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        kern_ms = ev_start.elapsed_time(ev_stop) / args.steps
        value = flops / (wall_ms * 1e-3) / 1e12
        achieved = flops / (kern_ms * 1e-3) / 1e12
        if args.only == "gemm-timed":   # for profiling: settle + warm-up + timed launches of the one kernel, nothing else
            print(json.dumps({"gemm_ms": kern_ms, "tflops": achieved, "settle_launches": settle_launches}))
            return
        extras["parity_cfg1"] = _parity(sets[0][4], xq0, wq0, xs0, ws0)
        graph_ms = _graph_ms(gemm_step, 120)
        extras["gemm_cfg1_graph_replay"] = {"ms": graph_ms, "TFLOPs": flops / (graph_ms * 1e-3) / 1e12,
                                            "frac_mfma": flops / (graph_ms * 1e-3) / PEAK_FP8_FLOPS,
                                            "note": "120 launches in one HIP graph, same operand rotation"}
        if (not args.no_extras and args.only == "") or args.only == "power":
            # The same launches on all-zero codes: the matrix cores then draw little power and the clock stays at its
            # maximum, so the difference to the timed run is what the power limit costs on this data (the schedule, the
            # bytes moved and the instruction stream are identical).  Not a performance claim.
            zsets = [(torch.zeros_like(xq0), torch.zeros_like(wq0), xs0, ws0, sets[j][4]) for j in range(NSETS)]

            def zero_step(i):
                xq, wq, xs, ws, y = zsets[i % NSETS]
                api.gemm(xq, wq, xs, ws, y)

            _settle(zero_step)
            z_ms = _median_events_ms(zero_step, 200)
            _settle(gemm_step)
            r_ms = _median_events_ms(gemm_step, 200)
            extras["gemm_cfg1_zero_operands"] = {"ms": z_ms, "TFLOPs": flops / (z_ms * 1e-3) / 1e12,
                                                 "frac_mfma": flops / (z_ms * 1e-3) / PEAK_FP8_FLOPS,
                                                 "ms_real_operands_same_loop": r_ms,
                                                 "note": "same kernel, same bytes, all-zero codes: what the launch costs when the "
                                                         "power limit does not bind (see bench.py --only ceilings)"}
            del zsets
            if args.only == "power":
                print(json.dumps(extras))
                return
        if not args.no_extras and args.only == "":
            # For scale only: the vendor library (hipBLASLt behind torch._scaled_mm, row-wise scales) on the same
            # operand rotation.  Not part of the product path and not a fallback.
            try:
                def vendor_step(i):
                    xq, wq, xs, ws, y = sets[i % NSETS]
                    torch._scaled_mm(xq, wq.t(), scale_a=xs[:, None], scale_b=ws[None, :], out_dtype=torch.bfloat16, out=y)
                for i in range(20):
                    vendor_step(i)
                v_ms = _median_events_ms(vendor_step, 100)
                extras["vendor_scaled_mm_rowwise_cfg1"] = {"ms": v_ms, "TFLOPs": flops / (v_ms * 1e-3) / 1e12,
                                                           "note": "torch._scaled_mm (hipBLASLt), same operands"}
            except Exception as e:  # the library may not offer row-wise scales for this shape
                extras["vendor_scaled_mm_rowwise_cfg1"] = {"error": str(e)[:160]}
        if args.only == "gemm":
            print(json.dumps({"gemm_ms": kern_ms, "tflops": achieved, "graph_ms": graph_ms,
                              "graph_tflops": flops / (graph_ms * 1e-3) / 1e12}))
            return
    # ---------------------------------------------------------------- quantize pass (cfg1 activations)
    xq_tmp = torch.empty(M, K, dtype=torch.float8_e4m3fn, device=dev)
    xs_tmp = torch.empty(M, dtype=torch.float32, device=dev)
    xsets = [x_dev.clone() for _ in range(10)]  # 10 x 32 MiB of distinct inputs

    def quant_step(i):
        api.quantize(xsets[i % len(xsets)], xq_tmp, xs_tmp)

    if (not args.no_extras and args.only == "") or args.only == "quantize":
        for i in range(10):
            quant_step(i)
        q_ms = _median_events_ms(quant_step, 50)
        q_bytes = 3.0 * M * K + 4.0 * M
        extras["quantize_cfg1"] = {"ms": q_ms, "GBps": q_bytes / (q_ms * 1e-3) / 1e9,
                                   "frac_hbm": q_bytes / (q_ms * 1e-3) / PEAK_HBM_BPS, "bytes": q_bytes,
                                   "note": "arithmetic of the reference's torch emulation (use_triton=False)"}

        def quant_triton_step(i):   # the arithmetic a GPU caller of the reference gets by default (IEEE divisions, saturating)
            api.check(api.L.mslk_amd_quantize_fp8_row_triton_arithmetic(
                xsets[i % len(xsets)].data_ptr(), 0, M, K, K, xq_tmp.data_ptr(), K, xs_tmp.data_ptr(), None, 1.0 / 512.0,
                None, 0, 1, api.stream))

        for i in range(10):
            quant_triton_step(i)
        qt_ms = _median_events_ms(quant_triton_step, 50)
        extras["quantize_cfg1_triton_arithmetic"] = {"ms": qt_ms, "GBps": q_bytes / (qt_ms * 1e-3) / 1e9,
                                                     "frac_hbm": q_bytes / (qt_ms * 1e-3) / PEAK_HBM_BPS}
        # dequantize_fp8_row on the same shape: 1 B in + 2 B out per element, rotating over 10 code sets
        qsets = [torch.randint(0, 120, (M, K), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn) for _ in range(10)]
        dq_out = [torch.empty(M, K, dtype=torch.bfloat16, device=dev) for _ in range(4)]

        def dequant_step(i):
            api.check(api.L.mslk_amd_dequantize_fp8_row(qsets[i % 10].data_ptr(), xs_tmp.data_ptr(), M, K,
                                                        dq_out[i % 4].data_ptr(), api.stream))

        for i in range(10):
            dequant_step(i)
        d_ms = _median_events_ms(dequant_step, 50)
        extras["dequantize_cfg1"] = {"ms": d_ms, "GBps": q_bytes / (d_ms * 1e-3) / 1e9,
                                     "frac_hbm": q_bytes / (d_ms * 1e-3) / PEAK_HBM_BPS, "bytes": q_bytes}
        del qsets, dq_out

        # fused producers of the MoE activations on cfg4's token count (8192 x 5120, bf16)
        from mslk_amd import moe
        Tm, Dm, Em = 8192, 5120, 16
        gen = torch.Generator(device="cpu").manual_seed(5)
        h = torch.randn(Tm, 2 * Dm, generator=gen).bfloat16().to(dev)
        hsets = [h.clone() for _ in range(3)]                       # 3 x 160 MiB
        fq = torch.empty(Tm, Dm, dtype=torch.float8_e4m3fn, device=dev)
        fs = torch.empty(Tm, dtype=torch.float32, device=dev)

        def silu_step(i):
            hh = hsets[i % 3]
            api.check(api.L.mslk_amd_silu_mul_quant(hh.data_ptr(), hh.data_ptr() + 2 * Dm, 0, Tm, Dm, 2 * Dm, 2 * Dm,
                                                    fq.data_ptr(), fs.data_ptr(), None, None, 0, api.stream))

        for i in range(6):
            silu_step(i)
        f_ms = _median_events_ms(silu_step, 30)
        f_bytes = 5.0 * Tm * Dm + 4.0 * Tm
        extras["silu_mul_quant_8192x5120"] = {"ms": f_ms, "GBps": f_bytes / (f_ms * 1e-3) / 1e9,
                                              "frac_hbm": f_bytes / (f_ms * 1e-3) / PEAK_HBM_BPS, "bytes": f_bytes}
        tok = torch.randperm(Tm, generator=gen).to(torch.int32).to(dev)
        exp = torch.randint(0, Em, (Tm,), generator=gen).to(dev)
        scores = torch.rand(Tm, Em, generator=gen).to(dev)
        xsrc = [hsets[j][:, :Dm].contiguous() for j in range(3)]

        def gather_step(i):
            api.check(api.L.mslk_amd_gather_scale_quant_dense_tokens(
                xsrc[i % 3].data_ptr(), 0, Tm, Dm, tok.data_ptr(), 1, exp.data_ptr(), 0, Tm, scores.data_ptr(), 2, Em, Em, 1,
                fq.data_ptr(), fs.data_ptr(), None, None, 0, api.stream))

        for i in range(6):
            gather_step(i)
        g_ms = _median_events_ms(gather_step, 30)
        g_bytes = 3.0 * Tm * Dm + 16.0 * Tm
        extras["gather_scale_quant_8192x5120"] = {"ms": g_ms, "GBps": g_bytes / (g_ms * 1e-3) / 1e9,
                                                  "frac_hbm": g_bytes / (g_ms * 1e-3) / PEAK_HBM_BPS, "bytes": g_bytes}
        del hsets, xsrc, h
        if args.only == "quantize":
            print(json.dumps(extras))
            return

        def path_step(i):
            xq, wq, xs, ws, y = sets[i % NSETS]
            api.quantize(xsets[i % len(xsets)], xq, xs)
            api.gemm(xq, wq, xs, ws, y)

        for i in range(10):
            path_step(i)
        p_ms = _median_events_ms(path_step, 50)
        extras["quantize_plus_gemm_cfg1"] = {"ms": p_ms, "TFLOPs": flops / (p_ms * 1e-3) / 1e12}
    del xsets

    # ---------------------------------------------------------------- decode, eager or graph launches only (for a kernel trace)
    if args.only in ("decode-eager", "decode-graph"):
        # The same decode GEMMs launched one by one or replayed from ONE HIP graph, and nothing else: under
        # `rocprofv3 --kernel-trace --stats` the two runs give each kernel's duration in either mode, to set beside the
        # per-launch times (M = 1, 16 and 64 run three different kernels, so the statistics keep them apart).
        wq3, ws3 = mslk_amd.quantize_fp8_row(W.cfg3_weight().to(dev), use_triton=False)
        wsets = [wq3.clone() for _ in range(6)]
        res = {}
        for Md in (1, 16, 64):
            xq3, xs3 = mslk_amd.quantize_fp8_row(W.cfg3_activations(Md).to(dev), use_triton=False)
            y3 = torch.empty(Md, 8192, dtype=torch.bfloat16, device=dev)

            def dec_step(i):
                api.gemm(xq3, wsets[i % len(wsets)], xs3, ws3, y3)

            if args.only == "decode-eager":
                _settle(dec_step, 20.0)
                res[f"M{Md}"] = {"ms_per_launch": _median_events_ms(dec_step, 60)}
            else:
                res[f"M{Md}"] = {"ms_per_launch": _graph_ms(dec_step, 60, repeats=12)}
        print(json.dumps({args.only: res}))
        return

    # ---------------------------------------------------------------- decode sweep (cfg3)
    if (not args.no_extras and args.only == "") or args.only == "decode":
        Nd = Kd = 8192
        wq3, ws3 = mslk_amd.quantize_fp8_row(W.cfg3_weight().to(dev), use_triton=False)
        wsets = [wq3.clone() for _ in range(6)]  # 6 x 64 MiB > Infinity Cache
        wshuf = [mslk_amd.preshuffle_b_mfma(w) for w in wsets]   # the same weights in the pre-shuffled (blocked) layout
        decode = {}
        for Md in (1, 4, 16, 64):
            xd = W.cfg3_activations(Md).to(dev)
            xq3, xs3 = mslk_amd.quantize_fp8_row(xd, use_triton=False)
            y3 = torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev)

            def dec_step(i):
                api.gemm(xq3, wsets[i % len(wsets)], xs3, ws3, y3)

            def dec_path_step(i):
                api.quantize(xd, xq3, xs3)
                api.gemm(xq3, wsets[i % len(wsets)], xs3, ws3, y3)

            def dec_fused_step(i):
                api.check(api.L.mslk_amd_quantize_f8f8bf16_rowwise(xd.data_ptr(), 0, Kd, wsets[i % len(wsets)].data_ptr(),
                                                                   ws3.data_ptr(), None, 0, y3.data_ptr(), Md, Nd, Kd,
                                                                   None, None, api.stream))

            def dec_ps_step(i):
                api.check(api.L.mslk_amd_f8f8_rowwise_preshuffle(xq3.data_ptr(), wshuf[i % len(wshuf)].data_ptr(), xs3.data_ptr(),
                                                                 ws3.data_ptr(), None, 0, y3.data_ptr(), 0, Md, Nd, Kd, api.stream))

            _settle(dec_step, 20.0)
            for i in range(12):
                dec_step(i)
                dec_ps_step(i)
            ms_ps = _median_events_ms(dec_ps_step, 60)
            ms = _median_events_ms(dec_step, 60)
            ms_path = _median_events_ms(dec_path_step, 60)
            ms_graph = _graph_ms(dec_step, 60)
            nbytes = Nd * Kd + Md * Kd + 2.0 * Md * Nd + 4.0 * (Md + Nd)
            fused = {}
            if api.L.mslk_amd_quantize_f8f8bf16_rowwise_supported(Md, Nd, Kd):
                for i in range(12):
                    dec_fused_step(i)
                ms_fused = _median_events_ms(dec_fused_step, 60)
                fbytes = Nd * Kd + 2.0 * Md * Kd + 2.0 * Md * Nd + 4.0 * Nd      # bf16 activations in, no codes or scales in HBM
                y1, q1, s1 = mslk_amd.quantize_f8f8bf16_rowwise(xd, wsets[0], ws3)
                fused = {"ms_fused_quantize": ms_fused, "GBps_fused_quantize": fbytes / (ms_fused * 1e-3) / 1e9,
                         "frac_hbm_fused_quantize": fbytes / (ms_fused * 1e-3) / PEAK_HBM_BPS,
                         "fused_codes_and_scales_equal_quantizer": bool(torch.equal(q1.view(torch.uint8), xq3.view(torch.uint8))
                                                                        and torch.equal(s1, xs3))}
            dec_step(0)
            par = _parity(y3, xq3, wsets[0], xs3, ws3)
            decode[f"M{Md}"] = {"ms": ms, "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_hbm": nbytes / (ms * 1e-3) / PEAK_HBM_BPS,
                                "ms_with_quantize": ms_path, "bytes": nbytes, "ms_graph_replay": ms_graph,
                                "GBps_graph_replay": nbytes / (ms_graph * 1e-3) / 1e9,
                                "ms_preshuffled_weights": ms_ps, "GBps_preshuffled_weights": nbytes / (ms_ps * 1e-3) / 1e9,
                                "frac_hbm_preshuffled_weights": nbytes / (ms_ps * 1e-3) / PEAK_HBM_BPS, **fused, "parity": par}
        for k, d in decode.items():
            # what a deployer gets per M after offline weight preparation: the faster of the row-major and the
            # pre-shuffled weight layout (both are operators of the path; the weights are re-laid out once, offline)
            best = min(d["ms"], d["ms_preshuffled_weights"])
            d["best_layout"] = "preshuffled" if d["ms_preshuffled_weights"] < d["ms"] else "row-major"
            d["ms_best_layout"] = best
            d["frac_hbm_best_layout"] = d["bytes"] / (best * 1e-3) / PEAK_HBM_BPS
        extras["decode_N8192_K8192"] = decode
        del wsets, wshuf
        if args.only == "decode":
            print(json.dumps(extras))
            return

    # ---------------------------------------------------------------- other configs (GEMM rate only)
    if not args.no_extras and args.only == "":
        wl0 = W.cfg0()
        a, sa = mslk_amd.quantize_fp8_row(wl0.x.to(dev), use_triton=False)
        b, sb = mslk_amd.quantize_fp8_row(wl0.w.to(dev), use_triton=False)
        y0 = torch.empty(1024, 1024, dtype=torch.bfloat16, device=dev)
        _settle(lambda i: api.gemm(a, b, sa, sb, y0), 20.0)
        ms = _median_events_ms(lambda i: api.gemm(a, b, sa, sb, y0), 100)
        extras["gemm_cfg0_1024"] = {"ms": ms, "TFLOPs": 2.0 * 1024**3 / (ms * 1e-3) / 1e12, "parity": _parity(y0, a, b, sa, sb)}

    if (not args.no_extras and args.only == "") or args.only == "cfg2":

        wl2 = W.cfg2()
        a, sa = mslk_amd.quantize_fp8_row(wl2.x.to(dev), use_triton=False)
        b, sb = mslk_amd.quantize_fp8_row(wl2.w.to(dev), use_triton=False)
        bias2 = wl2.bias.to(dev)
        y2 = torch.empty(8192, 28672, dtype=torch.bfloat16, device=dev)
        _settle(lambda i: api.gemm(a, b, sa, sb, y2, bias2))
        ms = _median_events_ms(lambda i: api.gemm(a, b, sa, sb, y2, bias2), 10)
        f2 = 2.0 * 8192 * 28672 * 4096
        extras["gemm_cfg2_8192x28672x4096_bias"] = {"ms": ms, "TFLOPs": f2 / (ms * 1e-3) / 1e12,
                                                     "frac_mfma": f2 / (ms * 1e-3) / PEAK_FP8_FLOPS,
                                                     "parity": _parity(y2, a, b, sa, sb, bias2)}
        del a, b, y2, wl2
        if args.only == "cfg2":
            print(json.dumps(extras))
            return

    if (not args.no_extras and args.only == "") or args.only == "grouped":

        wl4 = W.cfg4()
        xq4, xs4 = mslk_amd.quantize_fp8_row(wl4.x.to(dev), use_triton=False)
        wq4, ws4 = [], []
        for w in wl4.w:
            q, s = mslk_amd.quantize_fp8_row(w.to(dev), use_triton=False)
            wq4.append(q)
            ws4.append(s)
        xl, sl = list(xq4.split(wl4.counts)), list(xs4.split(wl4.counts))
        ys4 = torch.ops.mslk.f8f8bf16_rowwise_grouped(xl, wq4, sl, ws4)
        call4 = api.grouped_call(xl, wq4, sl, ws4, ys4)
        _settle(lambda i: call4())   # the first few dozen launches on freshly allocated 640 MiB of weights run up to 25 % slower
        ms = _median_events_ms(lambda i: call4(), 10)
        f4 = 2.0 * 8192 * 8192 * 5120
        # the same call through the operator (argument checks, output allocation and marshalling of 80 pointers in Python)
        ms_op = _median_events_ms(lambda i: torch.ops.mslk.f8f8bf16_rowwise_grouped(xl, wq4, sl, ws4), 10)
        t0 = time.perf_counter()
        for _ in range(20):
            torch.ops.mslk.f8f8bf16_rowwise_grouped(xl, wq4, sl, ws4)
        host_us = (time.perf_counter() - t0) / 20 * 1e6   # launches are asynchronous: this is host time per call
        torch.cuda.synchronize()
        par4 = [_parity(ys4[e], xl[e], wq4[e], sl[e], ws4[e]) for e in range(16) if wl4.counts[e]]
        extras["grouped_cfg4_16x8192x5120"] = {"ms": ms, "TFLOPs": f4 / (ms * 1e-3) / 1e12,
                                                "frac_mfma": f4 / (ms * 1e-3) / PEAK_FP8_FLOPS, "counts": wl4.counts,
                                                "ms_through_torch_ops": ms_op, "host_us_per_torch_ops_call": host_us,
                                                "parity": {"max_rel": max(p["max_rel"] for p in par4),
                                                           "normwise": max(p["normwise"] for p in par4),
                                                           "elementwise_violations": sum(p["elementwise_violations"] for p in par4),
                                                           "elements": sum(p["elements"] for p in par4)}}
        # the same experts through the device-resident group layouts (no host knowledge of the sizes),
        # and as a uniform batch of 16 x [512 x 8192 x 5120] (same FLOPs, no ragged tiles)
        WQ4, WS4 = torch.stack(wq4), torch.stack(ws4)
        del wq4, ws4, call4
        y4 = torch.empty(8192, 8192, dtype=torch.bfloat16, device=dev)
        sizes = torch.tensor(wl4.counts, dtype=torch.int64, device=dev)
        ends = sizes.cumsum(0).to(torch.int32)
        L = api.L

        def stacked_call():
            api.check(L.mslk_amd_f8f8bf16_rowwise_grouped_stacked(xq4.data_ptr(), WQ4.data_ptr(), xs4.data_ptr(), WS4.data_ptr(),
                                                                  sizes.data_ptr(), 16, 8192, 8192, 5120, y4.data_ptr(), api.stream))

        def offsets_call():
            api.check(L.mslk_amd_f8f8bf16_rowwise_grouped_mm(xq4.data_ptr(), WQ4.data_ptr(), xs4.data_ptr(), WS4.data_ptr(),
                                                             ends.data_ptr(), 1, 16, 8192, 8192, 5120, y4.data_ptr(), api.stream))

        def batched_call():
            api.check(L.mslk_amd_f8f8bf16_rowwise_batched(xq4.data_ptr(), WQ4.data_ptr(), xs4.data_ptr(), WS4.data_ptr(),
                                                          None, 0, 16, 512, 8192, 5120, y4.data_ptr(), api.stream))

        one = torch.tensor([8192], dtype=torch.int64, device=dev)

        def single_group_call():   # one expert takes all 8192 rows: its 40 MiB of weights stay in the Infinity Cache
            api.check(L.mslk_amd_f8f8bf16_rowwise_grouped_stacked(xq4.data_ptr(), WQ4.data_ptr(), xs4.data_ptr(), WS4.data_ptr(),
                                                                  one.data_ptr(), 1, 8192, 8192, 5120, y4.data_ptr(), api.stream))

        # cfg4's sizes come sorted (largest expert first), the worst order for the equal-count XCD slices of the
        # device-extent layouts: the same sizes in a fixed shuffled order, as a router would produce them
        import random
        shuffled = list(wl4.counts)
        random.Random(1).shuffle(shuffled)
        sizes_shuffled = torch.tensor(shuffled, dtype=torch.int64, device=dev)

        def stacked_shuffled_call():
            api.check(L.mslk_amd_f8f8bf16_rowwise_grouped_stacked(xq4.data_ptr(), WQ4.data_ptr(), xs4.data_ptr(), WS4.data_ptr(),
                                                                  sizes_shuffled.data_ptr(), 16, 8192, 8192, 5120, y4.data_ptr(), api.stream))

        for name, call in (("grouped_stacked_cfg4", stacked_call), ("grouped_mm_2d3d_cfg4", offsets_call),
                           ("grouped_stacked_cfg4_sizes_shuffled", stacked_shuffled_call),
                           ("batched_16x512x8192x5120", batched_call), ("grouped_one_warm_group_8192x8192x5120", single_group_call)):
            _settle(lambda i: call(), 20.0)
            ms = _median_events_ms(lambda i: call(), 10)
            extras[name] = {"ms": ms, "TFLOPs": f4 / (ms * 1e-3) / 1e12, "frac_mfma": f4 / (ms * 1e-3) / PEAK_FP8_FLOPS}
        del WQ4, wl4
        if args.only == "grouped":
            print(json.dumps(extras))
            return

    # ---------------------------------------------------------------- CPU baseline
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(wl)

    line = {
        "metric": "FP8 rowwise GEMM TFLOP/s @M=N=K=4096 (% FP8 peak); decode-shape HBM GB/s",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> fp32 accumulate -> bf16", "data": "synthetic",
        "config": {"workload": "cfg1: f8f8bf16_rowwise M=N=K=4096, x ~ N(0,1) with 1% K-channels x20 quantized by "
                               "quantize_fp8_row, w ~ N(0,0.02) pre-quantized; one step = one GEMM call via the C ABI, "
                               f"rotating over {NSETS} operand sets ({NSETS * 64} MiB); quantize timed separately (see extras); "
                               f"before the --warmup steps an untimed clock-settling phase of the same launches runs until "
                               f"{SETTLE_MS:.0f} ms of GPU time have passed ({settle_launches} launches in this run)"},
        "pct_of_fp8_peak_5.0PF": 100.0 * value * 1e12 / PEAK_FP8_FLOPS,
        "pct_of_reference_peak_4.6PF": 100.0 * value * 1e12 / PEAK_FP8_FLOPS_REF,
        "roofline": {"kernel": "dense_tiled_kernel<256,256> (f8f8bf16_rowwise 4096^3)", "bound": "mfma",
                     "achieved": achieved, "peak": PEAK_FP8_FLOPS / 1e12, "unit": "TFLOP/s",
                     "frac": achieved * 1e12 / PEAK_FP8_FLOPS, "traffic": _measured_traffic_bytes(),
                     "traffic_source": f"{TRAFFIC_SOURCE} (rocprofv3 counters of an earlier run of this command, not measured in this run)",
                     "kernel_ms": kern_ms,
                     "flops_per_launch": flops},
        "cpu_baseline": cpu,
        "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
