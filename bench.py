#!/usr/bin/env python3
"""Benchmark of the W8A8 block-FP8 linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--table PATH]

One step = one pass of the hot path over one batch of synthetic input: per-token-group FP8
quantisation of the activation (bf16 [M,K], groups of 128, column-major scales) followed by the
block-scaled FP8 GEMM against a 128x128-block-quantised weight, bf16 out - what
Fp8LinearMethod.apply runs for one projection.  The headline workload is a DeepSeek-V3 projection
from BASELINE.json configs[2] at M=4096.  Inputs are generated on the GPU before the timed region
and rotated over enough buffers that weights and activations come from HBM, not from the 256 MB
last-level cache.  100 untimed priming steps run first (the chip's clocks settle over about 50 ms of
load), then the W warm-up steps, then exactly K timed steps between two device synchronisations.

Prints ONE JSON line.  `value` is the whole step in TFLOP/s (2*M*N*K per step); `roofline`
prices the dominant kernel (the GEMM) against the published dense-FP8 MFMA peak, with its
duration measured by HIP events around the GEMM launches only; `roofline_quant` does the same for
the group-quant kernel at the largest configs[1] size against the HBM peak; `cpu_baseline` times
the C restatement of the reference arithmetic (oracle/, OpenMP) on a bounded sample of the same
workload on this machine's host cores.

--table PATH additionally writes a per-shape report (configs[1], [2] and [3]) as markdown.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X published dense FP8 MFMA peak
PEAK_HBM_GBS = 8000.0  # MI355X published HBM3E peak

METRIC = "FP8 block GEMM TFLOPS (% MFMA peak) + group-quant GB/s at DeepSeek-V3 shapes"
HEADLINE = dict(M=4096, N=18432, K=7168, name="DeepSeek-V3 gate_up (TP2) projection")
QUANT_SHAPE = dict(M=16384, K=7168)
PRIME_STEPS = 100  # untimed steps ahead of the warm-up steps (clock settling, see run_headline)

DSV3_NK = [(24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304), (18432, 7168), (7168, 18432)]
LLAMA_NK = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]


def _activation(torch, M, K, seed, dev):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32)
    mask = torch.rand((M, K), generator=g, device=dev) < 1e-3
    return torch.where(mask, x * 50.0, x).to(torch.bfloat16)


def _block_quant_weight(torch, N, K, seed, dev):
    """N(0,0.02) bf16 weight -> e4m3fn + float32 scale per 128x128 block (scale = blockamax/448)."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 1000003)
    w = (torch.randn((N, K), generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16).float()
    nt, kt = (N + 127) // 128, (K + 127) // 128
    wp = torch.zeros((nt * 128, kt * 128), device=dev)
    wp[:N, :K] = w
    blk = wp.view(nt, 128, kt, 128)
    s = blk.abs().amax(dim=(1, 3)) / 448.0
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (blk / s[:, None, :, None]).clamp(-448.0, 448.0).view(nt * 128, kt * 128)[:N, :K]
    return q.contiguous().to(torch.float8_e4m3fn), s.contiguous()


def _events(torch, n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _time_calls(torch, fn, iters, warm=3):
    """Average device time of fn(i) in microseconds, HIP events on the current stream."""
    for i in range(warm):
        fn(i)
    torch.cuda.synchronize()
    a, b = _events(torch, 2)
    a.record()
    for i in range(iters):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / iters


def _time_graph(torch, fn, iters, replays=3, warm_launches=0):
    """Average device time of fn(i) in microseconds with the launches replayed from one HIP graph, so
    that host-side launch cost (Python, ctypes, allocator) does not show up in small-shape timings.
    Every entry point of the library is capture-legal (no allocation, no sync, no memset)."""
    for i in range(max(2, warm_launches)):  # a cold chip clocks memory-bound kernels up to 15 % slower
        fn(i)
    torch.cuda.synchronize()
    # after host-side work (the CPU legs of the report) the chip has idled: keep it under this load for about 60 ms so
    # that its clocks have settled when the timed replays start
    t_settle = time.perf_counter()
    i = 0
    while time.perf_counter() - t_settle < 0.06:
        fn(i)
        i += 1
        if i % 16 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(iters):
            fn(i)
    g.replay()
    torch.cuda.synchronize()
    a, b = _events(torch, 2)
    a.record()
    for _ in range(replays):
        g.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / (iters * replays)


QUANT_LAYOUTS = (("row_major_f32", {}), ("col_major_f32", dict(column_major_scales=True)),
                 ("ue8m0_packed", dict(column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)))


def _quant_launcher(torch, xs, kw):
    """fn(i) that quantises xs[i % n] into output buffers allocated once per input (rotating with it), the way a
    serving loop meets them: the caching allocator hands the same blocks back every step.  Allocating inside the
    timed graph instead gives every captured launch its own 120 MB of output and measures about 10 % slower."""
    from sglang_amd import sgl_kernel as ops
    from sglang_amd.fp8_kernel import create_per_token_group_quant_fp8_output_scale, fp8_dtype, fp8_max, fp8_min

    n = len(xs)
    qs = [torch.empty(x.shape, device=x.device, dtype=fp8_dtype) for x in xs]
    ss = [create_per_token_group_quant_fp8_output_scale(
        x_shape=x.shape, device=x.device, group_size=128, column_major_scales=kw.get("column_major_scales", False),
        scale_tma_aligned=kw.get("scale_tma_aligned", False), scale_ue8m0=kw.get("scale_ue8m0", False)) for x in xs]
    ue = kw.get("scale_ue8m0", False)
    return lambda i: ops.sgl_per_token_group_quant_8bit(xs[i % n], qs[i % n], ss[i % n], 128, 1e-10, fp8_min, fp8_max, ue)


def quant_bytes(M, K, ue8m0=False):
    return M * K * 3 + (M * K // 128) * (1 if ue8m0 else 4)


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` on the headline workload, as derived from rocprofv3 FETCH_SIZE / WRITE_SIZE
    counter runs of this script (the summary under profiles/ carries one `TRAFFIC_BYTES <kernel> <bytes>` line per
    kernel); None when no such summary is present."""
    path = os.path.join(ROOT, "profiles", "bench_headline_hbm_traffic_pmc.md")
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "TRAFFIC_BYTES" and parts[1] == kernel:
                    return int(parts[2])
    except OSError:
        pass
    return None


def gemm_bytes(M, N, K):
    return M * K + N * K + 2 * M * N + 4 * (M * K // 128 + (N // 128) * (K // 128))


def run_headline(torch, dev, steps, warmup):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul

    M, N, K = HEADLINE["M"], HEADLINE["N"], HEADLINE["K"]
    nbuf = 3
    xs = [_activation(torch, M, K, s, dev) for s in range(nbuf)]
    ws = [_block_quant_weight(torch, N, K, s, dev) for s in range(nbuf)]

    def step(i):
        x = xs[i % nbuf]
        wq, wsc = ws[i % nbuf]
        q, s = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
        return w8a8_block_fp8_matmul(q, wq, s, wsc, [128, 128], torch.bfloat16)

    # The chip needs about 50 ms of sustained load before its clocks settle: timed right after a cold start the same
    # 30 steps measure 538 us each after 5 warm-up steps, 511 after 30 and 499 after 100.  PRIME_STEPS untimed steps
    # therefore run before the W warm-up steps whatever W is (reported as config.priming_steps).
    for i in range(PRIME_STEPS):
        step(i)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps

    # dominant kernel alone: events bracket only the GEMM launches (same stream), quantised inputs prepared before
    qs = [sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True) for x in xs]
    torch.cuda.synchronize()
    gemm_us = _time_calls(
        torch, lambda i: w8a8_block_fp8_matmul(qs[i % nbuf][0], ws[i % nbuf][0], qs[i % nbuf][1], ws[i % nbuf][1],
                                               [128, 128], torch.bfloat16), max(steps, 10))
    return ms_per_step, gemm_us


def run_quant_roofline(torch, dev, iters=30):
    M, K = QUANT_SHAPE["M"], QUANT_SHAPE["K"]
    nbuf = 3  # 3 x (235 + 117 MB) > last-level cache
    xs = [_activation(torch, M, K, s, dev) for s in range(nbuf)]
    out = {}
    # the GEMM leg before this one leaves the chip in a different power state: settle on this kernel first
    settle = _quant_launcher(torch, xs, {})
    for i in range(1500):
        settle(i)
    torch.cuda.synchronize()
    for name, kw in QUANT_LAYOUTS:
        us = _time_graph(torch, _quant_launcher(torch, xs, kw), iters, replays=5, warm_launches=300)
        out[name] = (us, quant_bytes(M, K, name == "ue8m0_packed") / us / 1e3)
    return out


def hbm_stream_read_gbs(torch, dev, gib=4, runs=5):
    """Read rate (GB/s) of the library's LDS-staged load path on a plain contiguous buffer of `gib` GiB - the ceiling
    the weight-streaming kernels can reach on this machine (fp8k_tune_stream_read, timed with HIP events; best of
    `runs`, each run reads the whole buffer once, far more than the 256 MB last-level cache holds)."""
    from sglang_amd._lib import check, lib, stream_ptr

    buf = torch.empty(gib << 30, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).random_(0, 1 << 30)
    best = float("inf")
    for _ in range(runs + 1):
        a, b = _events(torch, 2)
        a.record()
        check(lib.fp8k_tune_stream_read(buf.data_ptr(), buf.numel(), stream_ptr(dev)))
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b))
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    read = buf.numel() // ncu // 65536 * 65536 * ncu
    del buf
    return read / best / 1e6


def hbm_tile_read_gbs(torch, dev, pitch, gib=4, runs=5):
    """Read rate (GB/s) of the same load path when the buffer is fetched the way a GEMM fetches an un-shuffled weight
    [rows, pitch]: 256-row tiles, one 128-byte K block of every row per stage (fp8k_tune_stream_read_tiles)."""
    from sglang_amd._lib import check, lib, stream_ptr

    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    rows = (gib << 30) // pitch // (256 * ncu) * (256 * ncu)
    buf = torch.empty(rows * pitch, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).random_(0, 1 << 30)
    best = float("inf")
    for _ in range(runs + 1):
        a, b = _events(torch, 2)
        a.record()
        check(lib.fp8k_tune_stream_read_tiles(buf.data_ptr(), rows, pitch, stream_ptr(dev)))
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b))
    del buf
    return rows * pitch / best / 1e6


def mfma_ceiling_tflops(torch, dev, iters=40000, runs=3):
    """Rate of a bare v_mfma_f32_32x32x64 (e4m3) loop on this machine (fp8k_tune_mfma_peak: 8 waves per CU, operands in
    registers, nothing else in the loop) on operand bytes taken from a quantised headline weight ("random") and on
    all-zero bytes ("zeros"); best of `runs` after a settling launch.  The power management clocks the chip by what the
    data toggles: the random-data figure is the practical ceiling of any FP8 GEMM on real data here, and its ratio to
    the zero-data figure separates that limit from kernel quality."""
    import ctypes

    from sglang_amd._lib import check, lib, stream_ptr

    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    wq, _ = _block_quant_weight(torch, 4096, 4096, 0, dev)
    sink = torch.empty(ncu * 512, dtype=torch.float32, device=dev)
    out = {}
    for name, ops in (("random", wq.view(torch.uint8)), ("zeros", torch.zeros_like(wq.view(torch.uint8)))):
        out[name] = _mfma_probe(torch, dev, ops, sink, 0, iters, runs)
    return out


def _mfma_probe(torch, dev, ops, sink, form, iters, runs):
    """TFLOP/s of one form of the MFMA probes (0: fp8k_tune_mfma_peak, 1..4: fp8k_tune_mfma_loop), best of `runs`."""
    import ctypes

    from sglang_amd._lib import check, lib, stream_ptr

    flops = ctypes.c_int64(0)
    best = float("inf")
    for r in range(runs + 1):
        a, b = _events(torch, 2)
        a.record()
        if form == 0:
            check(lib.fp8k_tune_mfma_peak(ops.data_ptr(), ops.numel(), iters, sink.data_ptr(), sink.numel(),
                                          ctypes.byref(flops), stream_ptr(dev)))
        else:
            check(lib.fp8k_tune_mfma_loop(ops.data_ptr(), ops.numel(), iters // 2, form, sink.data_ptr(), sink.numel(),
                                          ctypes.byref(flops), stream_ptr(dev)))
        b.record()
        torch.cuda.synchronize()
        if r:
            best = min(best, a.elapsed_time(b))
    return round(flops.value / best / 1e9, 1)


MFMA_LOOP_FORMS = ("bare MFMA loop", "+ block-scaled product form (16 scale FMAs per two MFMAs)",
                   "+ operand fragments refilled from LDS", "+ one workgroup barrier per K block",
                   "+ eight 1 KB stage loads per wave and K block",
                   "the complete loop without the scale FMAs (products accumulate in place)",
                   "the same with 16 multiplies per tile and K block (accumulators rescaled between K blocks)")


def mfma_loop_lines(torch, dev, iters=40000, runs=3):
    """The tile kernel's K loop built up from the bare MFMA loop one ingredient at a time (fp8k_tune_mfma_loop), on
    quantised-weight bytes and on zeros: what each ingredient costs the matrix cores on this machine."""
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    wq, _ = _block_quant_weight(torch, 4096, 4096, 0, dev)
    sink = torch.empty(ncu * 512, dtype=torch.float32, device=dev)
    rnd, zer = wq.view(torch.uint8), torch.zeros_like(wq.view(torch.uint8))
    lines = ["| form | TFLOP/s on quantised-weight bytes | of 5 PFLOP/s | TFLOP/s on zeros | of 5 PFLOP/s |", "|---|---|---|---|---|"]
    for form, name in enumerate(MFMA_LOOP_FORMS):
        a = _mfma_probe(torch, dev, rnd, sink, form, iters, runs)
        b = _mfma_probe(torch, dev, zer, sink, form, iters, runs)
        lines.append("| %d: %s | %.0f | %.2f | %.0f | %.2f |" % (form, name, a, a / PEAK_FP8_TFLOPS, b, b / PEAK_FP8_TFLOPS))
    # the stage loads above walk 16 MiB (more than one XCD's 4 MB L2: most come from the memory-side cache); the same with
    # a 2 MiB range, every load an L2 hit
    a = _mfma_probe(torch, dev, rnd[:2 << 20], sink, 4, iters, runs)
    b = _mfma_probe(torch, dev, zer[:2 << 20], sink, 4, iters, runs)
    lines.append("| 4 with every stage load an L2 hit | %.0f | %.2f | %.0f | %.2f |" % (a, a / PEAK_FP8_TFLOPS, b, b / PEAK_FP8_TFLOPS))
    return lines


def headline_zero_data_us(torch, dev):
    """The headline GEMM launch on all-zero operands and unit scales: the same instructions and memory traffic with no
    bit toggling in the matrix cores.  Reported next to the random-data time so that a slower box (or a lower power
    cap) can be told from a slower kernel."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    M, N, K = HEADLINE["M"], HEADLINE["N"], HEADLINE["K"]
    nbuf = 3
    ws = [(torch.zeros((N, K), device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn),
           torch.ones((N // 128, K // 128), device=dev)) for _ in range(nbuf)]
    qs = [(torch.zeros((M, K), device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn),
           torch.ones((K // 128, M), device=dev).t()) for _ in range(nbuf)]
    return _time_graph(torch, lambda i: w8a8_block_fp8_matmul(qs[i % nbuf][0], ws[i % nbuf][0], qs[i % nbuf][1],
                                                              ws[i % nbuf][1], [128, 128], torch.bfloat16), 12)


def stream_mix_lines(torch, dev, gib=4):
    """What stores inside a read stream cost on this machine: fp8k_tune_stream_read_write (one workgroup per CU reads its
    share in 32 KB stages, two in flight, and after every `tile` of stages writes 8 KB x n to a place of its own) against
    the same stream without stores, next to a plain fill and a plain copy (torch kernels) of the same size."""
    from sglang_amd._lib import check, lib, stream_ptr

    def best_ms(fn, runs=4):
        best = float("inf")
        for _ in range(runs + 1):
            a, b = _events(torch, 2)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            best = min(best, a.elapsed_time(b))
        return best

    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    src = torch.empty(gib << 30, dtype=torch.uint8, device=dev)
    src.view(torch.int32).random_(0, 1 << 30)
    dst = torch.empty(gib << 29, dtype=torch.uint8, device=dev)
    lines = ["| stages of 32 KB per tile | stores per tile and CU | us | read GB/s | us added per tile | time of a stored byte / time of a read byte |",
             "|---|---|---|---|---|---|"]
    for spt in (56, 16):
        share = src.numel() // ncu // (32768 * spt) * (32768 * spt)
        tiles = share // (32768 * spt)
        base = None
        for spw in (0, 1, 2, 4, 8, 16):
            ms = best_ms(lambda: check(lib.fp8k_tune_stream_read_write(src.data_ptr(), src.numel(), dst.data_ptr(), dst.numel(),
                                                                        spt, spw, stream_ptr(dev))))
            if spw == 0:
                base = ms
            added = (ms - base) * 1e3 / tiles
            rel = "" if spw == 0 else "%.1f" % ((ms - base) / base * (spt * 32768) / (spw * 8192))
            lines.append("| %d | %d KB | %.0f | %.0f | %.1f | %s |" % (spt, spw * 8, ms * 1e3, share * ncu / ms / 1e6, added, rel))
    n = dst.numel()
    ms = best_ms(lambda: dst.fill_(1))
    lines += ["", "plain fill of %.1f GiB (torch): %.0f us = %.0f GB/s written" % (n / 2**30, ms * 1e3, n / ms / 1e6)]
    ms = best_ms(lambda: dst.copy_(src[:n]))
    lines.append("plain copy of %.1f GiB (torch): %.0f us = %.0f GB/s read + the same written" % (n / 2**30, ms * 1e3, n / ms / 1e6))
    del src, dst
    return lines


def run_cpu_baseline(seconds_target=12.0):
    """C restatement of quant + block GEMM (oracle/, OpenMP) on M_cpu rows of the headline workload."""
    import numpy as np

    from oracle import c_oracle, fp8_oracle as O

    lib = c_oracle.load()
    cores = lib.oracle_num_threads()
    N, K = HEADLINE["N"], HEADLINE["K"]
    rng = np.random.default_rng(0)
    wq = rng.integers(0, 0x77, (N, K), dtype=np.uint8) | (rng.integers(0, 2, (N, K), dtype=np.uint8) << 7)
    wsc = rng.uniform(1e-4, 2e-4, (N // 128, K // 128)).astype(np.float32)
    eps = float(O.clamp_eps(1e-10, "bf16"))

    def once(M):
        x = O.bf16_bits(O.make_activation(M, K, 0))
        t0 = time.perf_counter()
        q, s = c_oracle.group_quant_bf16(lib, x, 128, eps)
        c_oracle.block_gemm(lib, q, wq, s, wsc)
        return time.perf_counter() - t0

    # size the sample to about `seconds_target` of CPU work: rows of the headline batch, whole batches if fast
    t_probe = once(64)
    rows = 64 * seconds_target / max(t_probe, 1e-3)
    M = int(min(HEADLINE["M"], max(64, rows // 64 * 64)))
    reps = int(max(1, min(8, rows // HEADLINE["M"])))
    dt = sum(once(M) for _ in range(reps))
    # the algorithm of the reference's own CPU kernel (fp8_scaled_mm_cpu: W8A16 - bf16 activations, weight blocks
    # dequantised to bf16), restated in C/OpenMP, on a quarter of the same sample
    Mt = max(64, M // 4 // 64 * 64)
    xt = O.bf16_bits(O.make_activation(Mt, K, 0))
    t0 = time.perf_counter()
    c_oracle.w8a16_block_gemm(lib, xt, wq, wsc)
    dtt = time.perf_counter() - t0
    return dict(value=2.0 * M * reps * N * K / dt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                sample="C/OpenMP restatement of per-token-group quant + block-FP8 matmul, %d pass(es) over M=%d rows "
                       "of the headline workload (N=%d, K=%d), %.1f s of CPU time on %d threads"
                       % (reps, M, N, K, dt, cores),
                w8a16_twin=dict(value=2.0 * Mt * N * K / dtt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                                sample="C/OpenMP restatement of the algorithm of the reference's CPU kernel "
                                       "fp8_scaled_mm_cpu (W8A16: bf16 activations, weight blocks dequantised to bf16, "
                                       "float accumulation), M=%d rows of the same workload, %.1f s" % (Mt, dtt)))


def _rand_fp8(torch, shape, gen, dev):
    b = torch.randint(0, 256, shape, generator=gen, device=dev, dtype=torch.uint8)
    return torch.where((b & 0x7F) == 0x7F, b & 0xFE, b).view(torch.float8_e4m3fn)  # no NaN codes


# ---------------------------------------------------------------------------------------------------------------
# CPU column of the per-shape report: this build's own torch-CPU restatement of the reference's torch-native path
# (per-token-group quant formula of python/sglang/test/test_block_fp8.py:23-48, block-tile matmul loop of :273-325:
# k_tiles x n_tiles float32 matmuls with the scale applied per tile), timed on this machine's host cores.  It belongs
# to the cpu_baseline leg; its result on the same tensors is also what the GPU output is compared with in the report.
# ---------------------------------------------------------------------------------------------------------------
CPU_ROW_CAP = 128  # rows of a shape that the interpreter-bound CPU loop is timed on (stated in the report)


def _median_time(fn, runs=5):
    fn()
    ts = []
    for _ in range(runs):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def cpu_group_quant(torch, x):
    g = x.reshape(-1, 128)
    amax = g.abs().amax(dim=-1, keepdim=True).clamp(min=1e-10).to(torch.float32)
    s = amax / 448.0
    q = (g / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.reshape(x.shape), s.reshape(x.shape[0], -1)


def cpu_block_matmul(torch, q, s, wq, ws):
    """C[:, j-block] += (A_i @ B_ji^T) * As[:, i] * Bs[j, i], tile by tile in float32, bf16 out."""
    M, K = q.shape
    N = wq.shape[0]
    A = q.to(torch.float32)
    B = wq.to(torch.float32)
    C = torch.zeros((M, N), dtype=torch.float32)
    for i in range(K // 128):
        a = A[:, i * 128:(i + 1) * 128]
        for j in range((N + 127) // 128):
            C[:, j * 128:(j + 1) * 128] += (a @ B[j * 128:(j + 1) * 128, i * 128:(i + 1) * 128].t()) * s[:, i:i + 1] * ws[j, i]
    return C.to(torch.bfloat16)


def _rel_err(torch, got, ref):
    """'a / b': a = max |got - ref| / max |ref|; b = the largest element-wise relative error over the elements above 1 % of
    max |ref| (for a 16-bit output b cannot be below the output rounding, 2^-8 for bf16)."""
    g, r = got.double(), ref.double()
    top = r.abs().max().clamp(min=1e-30)
    d = (g - r).abs()
    big = r.abs() > 1e-2 * top
    elem = float((d[big] / r.abs()[big]).max()) if bool(big.any()) else 0.0
    return "%.1e / %.1e" % (float(d.max() / top), elem)


def moe_table(torch, dev, token_counts=(1, 32, 256, 1024, 4096, 16384), cpu=False):
    """BASELINE configs[4]: 256 experts, hidden 7168, intermediate 2048, top-8 grouped-sigmoid routing."""
    from sglang_amd.fused_moe import biased_grouped_topk, fused_experts_impl

    E, H, I, topk = 256, 7168, 2048, 8
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    w1 = _rand_fp8(torch, (E, 2 * I, H), g, dev)
    w2 = _rand_fp8(torch, (E, H, I), g, dev)
    w1s = torch.rand((E, 2 * I // 128, H // 128), generator=g, device=dev) * 2e-4 + 1e-4
    w2s = torch.rand((E, H // 128, I // 128), generator=g, device=dev) * 2e-4 + 1e-4
    bias = torch.randn((E,), generator=g, device=dev) * 0.01  # near-balanced routing, as a trained router gives
    lines = ["", "## configs[4] block-FP8 fused MoE layer (E=256, H=7168, I=2048, top-8 of 8 groups / top-4 groups)", "",
             "whole layer: align + quant + grouped GEMM w13 + silu_and_mul + quant + grouped GEMM w2 + top-k sum; "
             "bytes = fp8 weights of the experts hit (44.04 MB each); roofline = the binding one of those bytes at 8 TB/s and the "
             "layer's FLOPs (2 x M x 8 x 3 I H) at the 5 PFLOP/s dense-FP8 peak;",
             "CPU: the same layer in torch-CPU ops, expert by expert, on the first token only (8 experts) - us per token", "",
             "| M | experts hit | us | TFLOP/s | weight GB/s | bound | frac | max rel err vs CPU (token 0) | CPU us / token |",
             "|---|---|---|---|---|---|---|---|---|"]
    for M in token_counts:
        print("[table] configs[4] M=%d" % M, file=sys.stderr, flush=True)
        x = _activation(torch, M, H, M, dev)
        logits = torch.randn((M, E), generator=g, device=dev)
        tw, ids = biased_grouped_topk(x, logits, bias, topk, True, 8, 4)
        hit = int(torch.unique(ids).numel())
        kw = dict(use_fp8_w8a8=True, w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128], routed_scaling_factor=2.5)
        us = _time_graph(torch, lambda i: fused_experts_impl(x, w1, w2, tw, ids, **kw), 10 if M < 4096 else 5)
        flops = 2.0 * M * topk * 3 * I * H
        wbytes = hit * 3 * I * H
        err, cpu_us = "", ""
        if cpu and M in (1, 32, 256, 4096):
            out = fused_experts_impl(x, w1, w2, tw, ids, **kw)[0].cpu()
            x0 = x[:1].cpu()

            def layer_cpu():
                xq, xs = cpu_group_quant(torch, x0)
                acc = torch.zeros((1, H), dtype=torch.float32)
                for k in range(topk):
                    e = int(ids[0, k])
                    h1 = cpu_block_matmul(torch, xq, xs, w1[e].cpu(), w1s[e].cpu())
                    act = torch.nn.functional.silu(h1[:, :I].float()).to(torch.bfloat16) * h1[:, I:]
                    aq, a_s = cpu_group_quant(torch, act)
                    h2 = cpu_block_matmul(torch, aq, a_s, w2[e].cpu(), w2s[e].cpu()).float()
                    acc = acc + (h2 * float(tw[0, k])).to(torch.bfloat16).float()
                return (acc * 2.5).to(torch.bfloat16)

            t = _median_time(layer_cpu, runs=1)
            err = _rel_err(torch, out, layer_cpu()[0])
            cpu_us = "%.0f" % (t * 1e6)
        t_hbm, t_mfma = wbytes / (PEAK_HBM_GBS * 1e3), flops / (PEAK_FP8_TFLOPS * 1e6)  # microseconds
        lines.append("| %d | %d | %.1f | %.1f | %.0f | %s | %.2f | %s | %s |" % (
            M, hit, us, flops / us / 1e6, wbytes / us / 1e3, "hbm" if t_hbm >= t_mfma else "mfma", max(t_hbm, t_mfma) / us,
            err, cpu_us))
    return lines


def grouped_lines(torch, dev, shapes):
    """The masked grouped GEMM of the DeepGEMM-shaped entry points (G groups of m rows each, [G, N, K] weights) with
    power-of-two scales: once handed over as float32 tensors (float-scale grouped kernel) and once as packed UE8M0 words
    (256-row blocks: the matrix cores apply the exponents)."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_masked

    def pack(e):  # exponent bytes [.., kb] -> int32 words [.., ceil(kb / 4)], K block 4 j + i in byte i of word j
        kb = e.shape[-1]
        pad = (-kb) % 4
        if pad:
            e = torch.cat([e, torch.zeros(e.shape[:-1] + (pad,), dtype=e.dtype, device=e.device)], dim=-1)
        e = e.view(e.shape[:-1] + (-1, 4))
        return (e[..., 0] | (e[..., 1] << 8) | (e[..., 2] << 16) | (e[..., 3] << 24)).contiguous()

    lines = ["| groups | rows / group | N | K | float scales us | packed UE8M0 us | TFLOP/s (packed) |", "|---|---|---|---|---|---|---|"]
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    for (G, m, N, K) in shapes:
        a = _rand_fp8(torch, (G, m, K), g, dev)
        b = _rand_fp8(torch, (G, N, K), g, dev)
        ea = torch.randint(115, 125, (G, m, K // 128), device=dev, dtype=torch.int32, generator=g)
        eb = torch.randint(115, 125, (G, N // 128, K // 128), device=dev, dtype=torch.int32, generator=g)
        a_s, b_s = (ea << 23).view(torch.float32), (eb << 23).view(torch.float32)
        a_p, b_p = pack(ea), pack(eb.repeat_interleave(128, dim=1))
        masked = torch.full((G,), m, device=dev, dtype=torch.int32)
        out = torch.empty((G, m, N), device=dev, dtype=torch.bfloat16)
        t_f = _time_graph(torch, lambda i: grouped_gemm_nt_f8f8bf16_masked((a, a_s), (b, b_s), out, masked, m), 5)
        t_p = _time_graph(torch, lambda i: grouped_gemm_nt_f8f8bf16_masked((a, a_p), (b, b_p), out, masked, m), 5)
        lines.append("| %d | %d | %d | %d | %.0f | %.0f | %.0f |" % (G, m, N, K, t_f, t_p, 2.0 * G * m * N * K / t_p / 1e6))
    return lines


def gemm_lines(torch, dev, shapes, data="random"):
    """Block-FP8 GEMM alone at the given (M, N, K): device time, TFLOP/s and algorithmic GB/s.  data = "zeros" runs
    the same launches on all-zero operands (and unit scales): the same instructions and memory traffic, but no bit of
    the matrix-core data paths toggles - the time difference against "random" is what the chip's power management
    takes (it lowers the clock under the random-data load)."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul

    lines = ["| M | N | K | us | TFLOP/s | % of 5 PFLOP/s | GB/s (algorithmic) |", "|---|---|---|---|---|---|---|"]
    for (M, N, K) in shapes:
        # enough weights in rotation that none is still in the 256 MB memory-side cache when its turn comes again
        nbuf = max(3, min(64, int(600e6 // (N * K)) + 1))
        ws = [_block_quant_weight(torch, N, K, s % 3, dev) if s < 3 else None for s in range(nbuf)]
        for s in range(3, nbuf):
            ws[s] = (ws[s % 3][0].clone(), ws[s % 3][1].clone())
        qs = [sglang_per_token_group_quant_fp8(_activation(torch, M, K, s % 3, dev), 128, column_major_scales=True)
              for s in range(nbuf)]
        if data == "zeros":
            for q, sc in ws + qs:
                q.view(torch.uint8).zero_()
                sc.fill_(1.0)
        us = _time_graph(torch, lambda i: w8a8_block_fp8_matmul(qs[i % nbuf][0], ws[i % nbuf][0], qs[i % nbuf][1],
                                                                ws[i % nbuf][1], [128, 128], torch.bfloat16), max(20, nbuf))
        tf = 2.0 * M * N * K / us / 1e6
        lines.append("| %d | %d | %d | %.1f | %.1f | %.1f | %.0f |" % (M, N, K, us, tf, tf / PEAK_FP8_TFLOPS * 100,
                                                                      gemm_bytes(M, N, K) / us / 1e3))
    return lines


def _bound(flops, nbytes):
    """(name, floor in us) of the binding roofline: dense-FP8 MFMA peak or HBM peak, whichever takes longer."""
    t_mfma, t_hbm = flops / (PEAK_FP8_TFLOPS * 1e6), nbytes / (PEAK_HBM_GBS * 1e3)
    return ("mfma", t_mfma) if t_mfma >= t_hbm else ("hbm", t_hbm)


def write_table(torch, dev, path, cpu=True):
    """Per-shape report of configs[0]..[4]: GPU time, throughput, fraction of the binding roofline, and next to it the
    torch-native restatement on this machine's host cores (rows capped at CPU_ROW_CAP) with the GPU result's maximum
    relative error against it on those rows."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.fp8_utils import w8a8_block_fp8_linear
    from sglang_amd.sgl_kernel import fp8_scaled_mm, mark_ue8m0

    stream_gbs = hbm_stream_read_gbs(torch, dev)
    lines = ["# Per-shape report (one MI355X, synthetic data, rotating buffers)", "",
             "GPU: device time by HIP events around a HIP graph that replays the launches back to back (host launch cost excluded).",
             "Roofline: the binding one of dense-FP8 MFMA peak (5 PFLOP/s) and HBM peak (8 TB/s) for the shape's algorithmic",
             "FLOPs (2 M N K) and bytes (operands + output + scales); `frac` = that floor / measured time.",
             "CPU: this build's torch-CPU restatement of the reference's torch-native path (group quant formula + k_tiles x",
             "n_tiles block-tile float32 matmul loop), median of 5 runs after one warm-up, at most %d rows of the shape" % CPU_ROW_CAP,
             "(the loop is interpreter-bound); host: torch.get_num_threads() = %d, os.cpu_count() = %d." % (
                 torch.get_num_threads(), os.cpu_count()),
             "`err` = max |gpu - cpu| / max |cpu| on the rows the CPU computed, then the largest element-wise |gpu - cpu| / |cpu| over "
             "the elements above 1 % of max |cpu| (bounded below by the bf16 output rounding, 2^-8 = 3.9e-3); quant: bytes and scales "
             "compared for equality.",
             "HBM read rate that the library's LDS-staged load path reaches on a plain 4 GiB buffer on this machine "
             "(fp8k_tune_stream_read): %.0f GB/s = %.2f of the 8 TB/s that `frac` is priced against." % (stream_gbs, stream_gbs / PEAK_HBM_GBS), ""]

    # ---- configs[0]
    lines += ["## configs[0] single W8A8 block-FP8 linear (x bf16 [32,4096], W [4096,4096], seed 0), quant + GEMM", "",
              "| M | N | K | GPU us | TFLOP/s | bound | frac | err | CPU us | CPU GFLOP/s |", "|---|---|---|---|---|---|---|---|---|---|"]
    M, N, K = 32, 4096, 4096
    x = _activation(torch, M, K, 0, dev)
    wq, wsc = _block_quant_weight(torch, N, K, 0, dev)
    us = _time_graph(torch, lambda i: w8a8_block_fp8_linear(x, wq, [128, 128], wsc), 20)
    bname, floor = _bound(2.0 * M * N * K, 2 * M * K + N * K + 2 * M * N)
    err, cpu_us, cpu_gf = "", "", ""
    if cpu:
        xc, wqc, wsc_c = x.cpu(), wq.cpu(), wsc.cpu()
        t = _median_time(lambda: cpu_block_matmul(torch, *cpu_group_quant(torch, xc), wqc, wsc_c))
        ref = cpu_block_matmul(torch, *cpu_group_quant(torch, xc), wqc, wsc_c)
        err = _rel_err(torch, w8a8_block_fp8_linear(x, wq, [128, 128], wsc).cpu(), ref)
        cpu_us, cpu_gf = "%.0f" % (t * 1e6), "%.1f" % (2.0 * M * N * K / t / 1e9)
    lines.append("| %d | %d | %d | %.1f | %.1f | %s | %.3f | %s | %s | %s |" % (M, N, K, us, 2.0 * M * N * K / us / 1e6, bname, floor / us,
                                                                              err, cpu_us, cpu_gf))

    # ---- configs[1]
    lines += ["", "## configs[1] per-token-group quant, K=7168, group 128 (bound: HBM)", "",
              "| M | layout | GPU us | GB/s | frac of 8 TB/s | bytes+scales equal to CPU | CPU us | CPU GB/s |", "|---|---|---|---|---|---|---|---|"]
    for M in (1, 64, 512, 4096, 16384):
        print("[table] configs[1] M=%d" % M, file=sys.stderr, flush=True)
        nbuf = 3 if M >= 4096 else 8
        xs = [_activation(torch, M, 7168, s, dev) for s in range(nbuf)]
        cpu_us, cpu_gbs, ref = "", "", None
        if cpu:
            rows = min(M, 4096)
            xc = xs[0][:rows].cpu()
            t = _median_time(lambda: cpu_group_quant(torch, xc), runs=5 if rows <= 512 else 3)
            ref = cpu_group_quant(torch, xc)
            cpu_us, cpu_gbs = "%.0f" % (t * 1e6), "%.2f" % (quant_bytes(rows, 7168) / t / 1e9)
        for name, kw in QUANT_LAYOUTS:
            us = _time_graph(torch, _quant_launcher(torch, xs, kw), 30, warm_launches=100)
            gbs = quant_bytes(M, 7168, name == "ue8m0_packed") / us / 1e3
            same = ""
            if ref is not None and name != "ue8m0_packed":
                q, s = sglang_per_token_group_quant_fp8(xs[0], 128, **kw)
                rows = ref[0].shape[0]
                same = "yes" if (torch.equal(q[:rows].cpu().view(torch.uint8), ref[0].view(torch.uint8))
                                 and torch.equal(s[:rows].cpu().contiguous(), ref[1])) else "NO"
            lines.append("| %d | %s | %.1f | %.0f | %.3f | %s | %s | %s |" % (M, name, us, gbs, gbs / PEAK_HBM_GBS, same,
                                                                         cpu_us if name == "row_major_f32" else "",
                                                                         cpu_gbs if name == "row_major_f32" else ""))
        del xs

    # ---- configs[2]
    lines += ["", "## configs[2] block-FP8 GEMM, DeepSeek-V3 shapes", "",
              "`quant + GEMM us`: the whole linear (w8a8_block_fp8_linear on the bf16 activation: group quant launch, then the GEMM) - "
              "what a decode step pays per projection; the other columns are the GEMM alone on pre-quantised activations.", "",
              "| M | N | K | GPU us | TFLOP/s | GB/s (algorithmic) | bound | frac | quant + GEMM us | err | CPU us (rows) | CPU GFLOP/s |",
              "|---|---|---|---|---|---|---|---|---|---|---|---|"]
    for (N, K) in DSV3_NK:
        print("[table] configs[2] N=%d K=%d" % (N, K), file=sys.stderr, flush=True)
        nbuf = 3
        ws = [_block_quant_weight(torch, N, K, s, dev) for s in range(nbuf)]
        wq_c, ws_c = (ws[0][0].cpu(), ws[0][1].cpu()) if cpu else (None, None)
        for M in (1, 16, 128, 1024, 4096):
            qs = [sglang_per_token_group_quant_fp8(_activation(torch, M, K, s, dev), 128, column_major_scales=True)
                  for s in range(nbuf)]
            us = _time_graph(torch, lambda i: w8a8_block_fp8_matmul(qs[i % nbuf][0], ws[i % nbuf][0], qs[i % nbuf][1],
                                                                    ws[i % nbuf][1], [128, 128], torch.bfloat16), 20)
            tf = 2.0 * M * N * K / us / 1e6
            bname, floor = _bound(2.0 * M * N * K, gemm_bytes(M, N, K))
            xb = [_activation(torch, M, K, s, dev) for s in range(nbuf)]
            us_lin = _time_graph(torch, lambda i: w8a8_block_fp8_linear(xb[i % nbuf], ws[i % nbuf][0], [128, 128], ws[i % nbuf][1]), 20)
            del xb
            err, cpu_us, cpu_gf = "", "", ""
            if cpu:
                rows = min(M, CPU_ROW_CAP)
                qc, sc_ = qs[0][0][:rows].cpu(), qs[0][1][:rows].cpu().contiguous()
                t = _median_time(lambda: cpu_block_matmul(torch, qc, sc_, wq_c, ws_c), runs=3)
                ref = cpu_block_matmul(torch, qc, sc_, wq_c, ws_c)
                got = w8a8_block_fp8_matmul(qs[0][0], ws[0][0], qs[0][1], ws[0][1], [128, 128], torch.bfloat16)[:rows].cpu()
                err = _rel_err(torch, got, ref)
                cpu_us, cpu_gf = "%.0f (%d)" % (t * 1e6, rows), "%.1f" % (2.0 * rows * N * K / t / 1e9)
            lines.append("| %d | %d | %d | %.1f | %.1f | %.0f | %s | %.3f | %.1f | %s | %s | %s |" % (
                M, N, K, us, tf, gemm_bytes(M, N, K) / us / 1e3, bname, floor / us, us_lin, err, cpu_us, cpu_gf))
        del ws

    lines += ["", "## configs[2] shapes at M=4096 with UE8M0 scales (packed activation exponents, power-of-two weight scales:",
              "## the matrix core applies the block scales itself)", "",
              "| M | N | K | GPU us | TFLOP/s | frac of 5 PFLOP/s |", "|---|---|---|---|---|---|"]
    for (N, K) in DSV3_NK:
        nbuf, M = 3, 4096
        ws = [_block_quant_weight(torch, N, K, s, dev) for s in range(nbuf)]
        ws = [(w, mark_ue8m0(torch.exp2(torch.ceil(torch.log2(sc))))) for w, sc in ws]
        qs = [sglang_per_token_group_quant_fp8(_activation(torch, M, K, s, dev), 128, column_major_scales=True,
                                               scale_tma_aligned=True, scale_ue8m0=True) for s in range(nbuf)]
        us = _time_graph(torch, lambda i: w8a8_block_fp8_matmul(qs[i % nbuf][0], ws[i % nbuf][0], qs[i % nbuf][1],
                                                                ws[i % nbuf][1], [128, 128], torch.bfloat16), 20)
        tf = 2.0 * M * N * K / us / 1e6
        lines.append("| %d | %d | %d | %.1f | %.1f | %.3f |" % (M, N, K, us, tf, tf / PEAK_FP8_TFLOPS))
        del ws

    # ---- configs[3]
    lines += ["", "## configs[3] per-token fp8_scaled_mm, Llama-3-8B shapes (CPU: (A.float() @ B.float().T) * sa * sb in torch)", "",
              "| M | N | K | GPU us | TFLOP/s | bound | frac | err | CPU us (rows) | CPU GFLOP/s |", "|---|---|---|---|---|---|---|---|---|---|"]
    for (N, K) in LLAMA_NK:
        print("[table] configs[3] N=%d K=%d" % (N, K), file=sys.stderr, flush=True)
        nbuf = 3
        bs = [(torch.randn((N, K), device=dev) * 50).clamp(-448, 448).to(torch.float8_e4m3fn) for _ in range(nbuf)]
        sb = torch.rand(N, device=dev) * 1e-3
        b_c, sb_c = (bs[0].cpu().float(), sb.cpu()) if cpu else (None, None)
        for M in (1, 8, 64, 512, 2048, 8192):
            a = [(torch.randn((M, K), device=dev) * 50).clamp(-448, 448).to(torch.float8_e4m3fn) for _ in range(nbuf)]
            sa = torch.rand(M, device=dev)
            us = _time_graph(torch, lambda i: fp8_scaled_mm(a[i % nbuf], bs[i % nbuf].t(), sa, sb, torch.bfloat16), 20)
            tf = 2.0 * M * N * K / us / 1e6
            bname, floor = _bound(2.0 * M * N * K, M * K + N * K + 2 * M * N + 4 * (M + N))
            err, cpu_us, cpu_gf = "", "", ""
            if cpu:
                rows = min(M, CPU_ROW_CAP)
                a_c, sa_c = a[0][:rows].cpu(), sa[:rows].cpu()
                fn = lambda: ((a_c.float() @ b_c.t()) * sa_c[:, None] * sb_c[None, :]).to(torch.bfloat16)
                t = _median_time(fn, runs=3)
                got = fp8_scaled_mm(a[0], bs[0].t(), sa, sb, torch.bfloat16)[:rows].cpu()
                err = _rel_err(torch, got, fn())
                cpu_us, cpu_gf = "%.0f (%d)" % (t * 1e6, rows), "%.1f" % (2.0 * rows * N * K / t / 1e9)
            lines.append("| %d | %d | %d | %.1f | %.1f | %s | %.3f | %s | %s | %s |" % (M, N, K, us, tf, bname, floor / us, err, cpu_us, cpu_gf))
        del bs
    lines += moe_table(torch, dev, cpu=cpu)
    print("[table] masked grouped GEMM", file=sys.stderr, flush=True)
    lines += ["", "## masked grouped block-FP8 GEMM of the DeepGEMM-shaped entry points (align + scale sort + grouped GEMM; every row "
              "valid; power-of-two scales handed over as float32 tensors / as packed UE8M0 words)", ""]
    lines += grouped_lines(torch, dev, [(256, 128, 4096, 7168), (256, 128, 7168, 2048), (32, 1024, 4096, 7168), (32, 1024, 7168, 2048)])
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--table", type=str, default=None, help="also write the per-shape markdown report here")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB read + 256 MiB write elementwise kernel (reference point for "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--no-ceilings", action="store_true",
                    help="skip the machine-ceiling legs (stream read, bare MFMA loop, headline launch on all-zero data): "
                         "for counter runs, whose per-kernel averages should cover the random-data launches only")
    ap.add_argument("--moe", type=str, default=None,
                    help="only time the fused MoE layer at these token counts (comma separated) and print its table")
    ap.add_argument("--gemm", type=str, default=None,
                    help="only time the block-FP8 GEMM at these shapes (MxNxK, comma separated) and print its table")
    ap.add_argument("--gemm-data", choices=("random", "zeros"), default="random",
                    help="operands of the --gemm runs: synthetic random data (default) or all zeros (same work, no "
                         "toggling in the matrix cores: shows what the power management takes)")
    ap.add_argument("--gemm-plan", type=str, default=None,
                    help="kernel family of the --gemm runs as KIND or KIND:SPLITS (fp8k_tune_force_gemm_plan; e.g. 3 = the "
                         "direct kernel with float partials, 5 = the direct kernel that cuts K across a workgroup's waves)")
    ap.add_argument("--grouped", type=str, default=None,
                    help="only time the masked grouped GEMM (groups x rows x N x K, comma separated) with float and "
                         "with packed UE8M0 scales")
    ap.add_argument("--stream-read", action="store_true", help="only measure the HBM read rate of the LDS-staged load path")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="only measure the bare matrix-core rate on random and on all-zero FP8 operands")
    ap.add_argument("--mfma-loop", action="store_true",
                    help="only measure the tile kernel's K loop built up from the bare MFMA loop one ingredient at a time")
    ap.add_argument("--stream-mix", action="store_true",
                    help="only measure what small write-outs inside the read stream cost (read stream with stores, fill, copy)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no cross-GPU step); --gpus %d is not "
              "supported" % args.gpus, file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU fallback", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.moe:
        print("\n".join(moe_table(torch, dev, tuple(int(t) for t in args.moe.split(",")))))
        return 0
    if args.gemm:
        shapes = [tuple(int(v) for v in t.split("x")) for t in args.gemm.split(",")]
        if args.gemm_plan:
            from sglang_amd._lib import lib

            kind, _, splits = args.gemm_plan.partition(":")
            lib.fp8k_tune_force_gemm_plan(int(kind), int(splits or 0))
        print("\n".join(gemm_lines(torch, dev, shapes, args.gemm_data)))
        return 0
    if args.grouped:
        shapes = [tuple(int(v) for v in t.split("x")) for t in args.grouped.split(",")]
        print("\n".join(grouped_lines(torch, dev, shapes)))
        return 0
    if args.stream_mix:
        print("\n".join(stream_mix_lines(torch, dev)))
        return 0
    if args.mfma_loop:
        print("\n".join(mfma_loop_lines(torch, dev)))
        return 0
    if args.mfma_ceiling:
        c = mfma_ceiling_tflops(torch, dev)
        print("bare v_mfma_f32_32x32x64 e4m3 loop, 8 waves per CU: %.0f TFLOP/s on quantised-weight bytes (%.2f of 5 PFLOP/s), "
              "%.0f TFLOP/s on all-zero bytes (%.2f)" % (c["random"], c["random"] / PEAK_FP8_TFLOPS, c["zeros"],
                                                        c["zeros"] / PEAK_FP8_TFLOPS))
        return 0
    if args.stream_read:
        print("HBM stream read (4 GiB buffer, LDS-staged loads, one workgroup per CU): %.0f GB/s" % hbm_stream_read_gbs(torch, dev))
        for pitch in (2048, 7168, 16384):
            print("the same buffer read as 256-row tiles of a [rows, %d] matrix, one 128-byte K block of each row per stage: "
                  "%.0f GB/s" % (pitch, hbm_tile_read_gbs(torch, dev, pitch)))
        return 0
    ms_per_step, gemm_us = run_headline(torch, dev, args.steps, args.warmup)
    M, N, K = HEADLINE["M"], HEADLINE["N"], HEADLINE["K"]
    flops = 2.0 * M * N * K
    value = flops / (ms_per_step * 1e-3) / 1e12
    gemm_tf = flops / gemm_us / 1e6
    quant = run_quant_roofline(torch, dev)
    q_us, q_gbs = quant["row_major_f32"]
    if args.table:
        write_table(torch, dev, args.table, cpu=not args.no_cpu)
    if args.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
    cpu = None if args.no_cpu else run_cpu_baseline()

    out = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> f32 accumulate, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": "w8a8 block-FP8 linear = per-token-group quant (bf16 [%d,%d], group 128) + block-scaled FP8 "
                        "GEMM vs 128x128-block weight [%d,%d]; %s, BASELINE configs[2]" % (M, K, N, K, HEADLINE["name"]),
            "M": M, "N": N, "K": K, "weight_buffers_rotated": 3, "priming_steps": PRIME_STEPS,
        },
        "roofline": {
            "kernel": "gemm_tile256_kernel (block-scaled FP8 MFMA GEMM)",
            "bound": "mfma",
            "achieved": round(gemm_tf, 2),
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm_tf / PEAK_FP8_TFLOPS, 4),
            "traffic": measured_traffic("gemm_tile256_kernel"),
            "avg_launch_us": round(gemm_us, 2),
        },
        "roofline_quant": {
            "kernel": "group_quant_kernel, bf16 [%d,%d], row-major f32 scales" % (QUANT_SHAPE["M"], QUANT_SHAPE["K"]),
            "bound": "hbm",
            "achieved": round(q_gbs, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(q_gbs / PEAK_HBM_GBS, 4),
            "traffic": measured_traffic("group_quant_kernel"),
            "avg_launch_us": round(q_us, 2),
            "other_layouts_GBps": {k: round(v[1], 1) for k, v in quant.items()},
        },
        "hbm_stream_read_GBps": None if args.no_ceilings else round(hbm_stream_read_gbs(torch, dev), 1),
        "mfma_ceiling_TFLOPs": None if args.no_ceilings else mfma_ceiling_tflops(torch, dev),
        "headline_zero_data_us": None if args.no_ceilings else round(headline_zero_data_us(torch, dev), 2),
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
