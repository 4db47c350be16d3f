#!/usr/bin/env python3
"""Benchmark of the BGEMM / BWTA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all]

A step is one pass of the hot path over one batch of synthetic input: one 8192^3
{-1,1}x{-1,1} BGEMM on prepacked operands (benchmark configuration 5, the compute-bound case the
metric's target is quoted on), int32 output, operands resident in HBM before the timed
region.  One JSON line goes to stdout; `value` is effective binary TOPS = 2*M*N*K / t
(the reference drivers' own op count, lowbit_kernel/csrc/benchmark.cu:291).  With --all the
line also carries the other benchmark configurations (MLP forward, batched attention A x V,
decode-shape BWTA) under "all_configs".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "bgemm-cuda_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

INT8_MFMA_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published
FP4_MFMA_PEAK_TOPS = 10100.0      # MI355X dense fp4 MFMA, published
HBM_PEAK_GBS = 8000.0             # MI355X HBM3E, published
MEASURED_TRAFFIC_BYTES_C5_FP4 = int((96.5 + 257.0) * 2 ** 20)   # fetched + written, rocprofv3 --pmc


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_gpu(fn, warmup, steps):
    """Average milliseconds per call of fn(i), timed with events on the launch stream."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_gpu_graph(fn, n_launch, warmup, replays):
    """Average milliseconds per launch with the CPU launch cost removed: n_launch calls of fn(i)
    are captured into one HIP graph, which is replayed `replays` times between two events."""
    import torch
    for i in range(min(n_launch, max(warmup, 1))):
        fn(i)                                   # also grows any cached buffers before capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for i in range(n_launch):
            fn(i)                               # warm the side stream's buffers eagerly
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            for i in range(n_launch):
                fn(i)
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (replays * n_launch)


def pm1_f16(shape, seed, device):
    import torch
    g = torch.Generator(device=device).manual_seed(seed)
    bits = torch.randint(0, 2, shape, generator=g, device=device, dtype=torch.int8)
    return (1 - 2 * bits).to(torch.half)


def check_sampled(out, w16, x16, n_rows=64, n_cols=64):
    """Spot parity check of an [N,M] XOR result against the fp32 closed form on sampled rows."""
    import torch
    N, M = out.shape
    g = torch.Generator().manual_seed(7)
    rs = torch.randperm(M, generator=g)[:n_rows].to(out.device)
    cs = torch.randperm(N, generator=g)[:n_cols].to(out.device)
    want = (x16[cs].float().cpu() @ w16[rs].float().cpu().T).to(torch.int32)
    return bool(torch.equal(out[cs][:, rs].cpu(), want))


def bench_c5(steps, warmup, M=8192, N=8192, K=8192, splitK=1, variant=0):
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    w16, x16 = pm1_f16((M, K), 5001, dev), pm1_f16((N, K), 5002, dev)
    wp, xp = lk.pack_sign(w16), lk.pack_sign(x16)
    out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(wp, xp, lk.MODE_XOR, torch.int32, splitK, variant, out=out)
    ms = time_gpu(fn, warmup, steps)
    ok = check_sampled(out[0], w16, x16)
    ops = 2.0 * M * N * K
    bytes_alg = M * K / 8 + N * K / 8 + 4.0 * M * N
    pack_ms = time_gpu(lambda i: lk.pack_sign(x16), 2, 10)
    return {"name": "C5 BGEMM %dx%dx%d xor int32 splitK=%d" % (M, N, K, splitK), "ms": ms,
            "tops": ops / ms / 1e9, "gbs": bytes_alg / ms / 1e6, "ops": ops, "bytes": bytes_alg,
            "bit_exact": ok, "act_pack_ms": pack_ms}, (w16, x16)


def bench_c5_dropin(steps, warmup, M=8192, N=8192, K=8192):
    """The same GEMM through the reference's own entry point, `bgemm_linear_forward_cuda(in_feats, weights)`:
    fp16 operands in, both sign-packed on every call (one launch), fp16 out."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    w16, x16 = pm1_f16((M, K), 5001, dev), pm1_f16((N, K), 5002, dev)
    out = [None]

    def fn(i):
        out[0] = lk.bgemm_linear_forward_cuda(x16, w16, 1, 1)
    ms = time_gpu(fn, warmup, steps)
    g = torch.Generator().manual_seed(7)
    rs, cs = torch.randperm(M, generator=g)[:64].to(dev), torch.randperm(N, generator=g)[:64].to(dev)
    want = (x16[cs].float() @ w16[rs].float().T).half()
    ok = bool(torch.equal(out[0][cs][:, rs], want))
    ops = 2.0 * M * N * K
    return {"name": "C5 through the fp16 drop-in call %dx%dx%d (packs both operands per call, fp16 out)" % (M, N, K),
            "ms": ms, "tops": ops / ms / 1e9, "ops": ops, "bit_exact": ok}


def cpu_baseline_c5(w16, x16, budget_s=12.0):
    """Reference CPU path (torch matmul on +-1 fp32 tensors) on a bounded column slice."""
    import torch
    from oracle import oracle
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, 16)))
    M, K = w16.shape
    wf = w16.float().cpu()
    n = 64
    xf = x16[:n].float().cpu()
    t0 = time.perf_counter()
    oracle.cpu_path_linear(xf, wf)
    dt = max(time.perf_counter() - t0, 1e-4)
    n = int(min(x16.shape[0], max(64, n * budget_s / dt / 3)))
    xf = x16[:n].float().cpu()
    oracle.cpu_path_linear(xf, wf)                       # warm-up at the timed size
    reps, t0 = 0, time.perf_counter()
    while reps < 2 or time.perf_counter() - t0 < budget_s / 2:
        oracle.cpu_path_linear(xf, wf)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": 2.0 * M * n * K / dt / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "torch.matmul fp32 on +-1 tensors, W[%d,%d] x X[%d,%d] (%d of %d activation rows), %d reps"
                      % (M, K, n, K, n, x16.shape[0], reps)}


def bench_c4(steps, warmup, N, splitK, variant=0, copies=64):
    """Decode-shape BWTA linear: W[11008,4096] prepacked, ternary activations, weights rotated
    over `copies` buffers (> 256 MB in total) so no launch finds its weights in cache."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    M, K = 11008, 4096
    g = torch.Generator(device=dev).manual_seed(4000 + N)
    t = torch.randint(0, 4, (N, K), generator=g, device=dev)
    x16 = torch.where(t == 0, -1.0, torch.where(t == 3, 1.0, 0.0)).to(torch.half)      # p(0) = 0.5
    xt = lk.pack_ternary(x16)
    w16 = pm1_f16((M, K), 4001, dev)
    base = lk.pack_sign(w16)
    wps = [lk.PackedBits(base.data.clone(), None, 1, M, K) for _ in range(copies)]
    out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(wps[i % copies], xt, lk.MODE_BWTA, torch.int32, splitK, variant, out=out)
    ms_eager = time_gpu(fn, warmup, steps)
    ms = time_gpu_graph(fn, copies, 4, max(2, steps // copies))
    want = (torch.sign(x16.float()).cpu() @ w16.float().cpu().T).to(torch.int32)
    ok = bool(torch.equal(out[0].cpu(), want))
    ops = 2.0 * M * N * K
    bytes_alg = M * K / 8 + 2 * N * K / 8 + 4.0 * M * N
    return {"name": "C4 BWTA W[11008,4096] N=%d splitK=%d" % (N, splitK), "ms": ms, "tops": ops / ms / 1e9,
            "ms_eager_launch": ms_eager, "gbs": bytes_alg / ms / 1e6, "ops": ops, "bytes": bytes_alg, "bit_exact": ok}


def bench_c4_batched(steps, N, B=64):
    """The same decode-shape BWTA linear over B weight matrices in ONE launch (the layers of a model,
    a set of experts): 361 MB of weights stream through once, so the launch is long enough to show the
    bandwidth the kernel sustains rather than the latency of one 5.6 MB launch."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    M, K = 11008, 4096
    g = torch.Generator(device=dev).manual_seed(4100 + N)
    t = torch.randint(0, 4, (N, K), generator=g, device=dev)
    x16 = torch.where(t == 0, -1.0, torch.where(t == 3, 1.0, 0.0)).to(torch.half)
    xt = lk.pack_ternary(x16)
    words = M * K // 32
    wdata = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, words), generator=g, device=dev, dtype=torch.int32)
    wb = lk.PackedBits(wdata, None, B, M, K)
    out = torch.empty((B, N, M), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(wb, xt, lk.MODE_BWTA, torch.int32, 1, 0, out=out)
    ms = time_gpu_graph(fn, 4, 2, max(5, steps // 40))
    # parity of three of the matrices against the fp32 closed form on unpacked bits
    ok = True
    for b in (0, B // 2, B - 1):
        w_logical = lk.logical_from_tiled(lk.PackedBits(wdata[b:b + 1], None, 1, M, K))
        shifts = torch.arange(31, -1, -1, device=dev, dtype=torch.int32)
        bits = ((w_logical.unsqueeze(-1) >> shifts) & 1).reshape(M, K)
        want = (torch.sign(x16.float()) @ (1 - 2 * bits).float().T).to(torch.int32)
        ok = ok and bool(torch.equal(out[b], want))
    ops = 2.0 * B * M * N * K
    bytes_alg = B * (M * K / 8 + 4.0 * M * N) + 2 * N * K / 8
    return {"name": "C4 batched: %d x BWTA W[11008,4096] N=%d in one launch" % (B, N), "ms": ms, "tops": ops / ms / 1e9,
            "gbs": bytes_alg / ms / 1e6, "ops": ops, "bytes": bytes_alg, "bit_exact": ok}


def bench_c4_from_fp16(steps, N, copies=64):
    """A decode step as a model runs it: fp16 activations in, prepacked W[11008,4096], int32 out.  Timed as two
    launches (ternary pack, then the packed GEMM) and as the one launch that packs its activations itself; weights
    rotate over `copies` buffers as in bench_c4."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    M, K = 11008, 4096
    g = torch.Generator(device=dev).manual_seed(4200 + N)
    t = torch.randint(0, 4, (N, K), generator=g, device=dev)
    x16 = torch.where(t == 0, -1.0, torch.where(t == 3, 1.0, 0.0)).to(torch.half)
    base = lk.pack_sign(pm1_f16((M, K), 4001, dev))
    wps = [lk.PackedBits(base.data.clone(), None, 1, M, K) for _ in range(copies)]
    two = lambda i: lk.bgemm_packed_forward(wps[i % copies], lk.pack_ternary(x16), lk.MODE_BWTA, torch.int32)
    one = lambda i: lk.bgemm_packed_weight_forward(wps[i % copies], x16, lk.MODE_BWTA, torch.int32)
    ok = bool(torch.equal(two(0)[0], one(0)))
    ms_two = time_gpu_graph(two, copies, 2, max(2, steps // copies))
    ms_one = time_gpu_graph(one, copies, 2, max(2, steps // copies))
    ms_one_eager, ms_two_eager = time_gpu(one, 20, steps), time_gpu(two, 20, steps)
    ops = 2.0 * M * N * K
    bytes_alg = M * K / 8 + 2.0 * N * K + 4.0 * M * N
    return {"name": "C4 decode step from fp16 activations, W[11008,4096] N=%d (one launch: the kernel packs x itself)" % N,
            "ms": ms_one, "ms_pack_then_gemm": ms_two, "ms_eager_launch": ms_one_eager, "ms_pack_then_gemm_eager": ms_two_eager,
            "tops": ops / ms_one / 1e9, "gbs": bytes_alg / ms_one / 1e6, "ops": ops, "bytes": bytes_alg, "bit_exact": ok}


def bench_floor():
    """What the hardware allows a kernel of the decode path's shape: the cost of launching an empty kernel,
    of reading one cold 5.6 MB buffer (the packed W[11008,4096]), and the bandwidth a plain read sustains."""
    import ctypes
    import torch
    so = os.path.join(ROOT, "bgemm-cuda_amd", "libbgemm_membench.so")
    L = ctypes.CDLL(so)
    p, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.bgemm_membench_empty.argtypes = [ci, ci, p, p]
    L.bgemm_membench_read.argtypes = [p, i64, ci, ci, p, p]
    dev = torch.device("cuda:0")
    nbytes, copies = 11008 * 4096 // 8, 64
    buf = torch.ones(copies * nbytes // 4, dtype=torch.int32, device=dev)
    scratch = torch.zeros(64, dtype=torch.int32, device=dev)
    st = lambda: torch.cuda.current_stream().cuda_stream
    res = {}
    res["empty_kernel_us"] = 1e3 * time_gpu_graph(
        lambda i: L.bgemm_membench_empty(344, 512, scratch.data_ptr(), st()), 64, 2, 20)
    best = None
    for blocks, threads in ((512, 512), (1024, 256), (1024, 512), (2048, 256)):
        us = 1e3 * time_gpu_graph(lambda i: L.bgemm_membench_read(buf.data_ptr() + (i % copies) * nbytes, nbytes, blocks,
                                                                  threads, scratch.data_ptr(), st()), copies, 2, 20)
        best = us if best is None else min(best, us)
    res["cold_read_5p6MB_us"] = best
    res["cold_read_5p6MB_gbs"] = nbytes / best / 1e3
    best = None
    for blocks, threads in ((2048, 512), (4096, 512), (8192, 512)):
        us = 1e3 * time_gpu_graph(lambda i: L.bgemm_membench_read(buf.data_ptr(), copies * nbytes, blocks, threads,
                                                                  scratch.data_ptr(), st()), 4, 2, 10)
        best = us if best is None else min(best, us)
    res["sustained_read_361MB_us"] = best
    res["sustained_read_gbs"] = copies * nbytes / best / 1e3
    res["sustained_read_frac_of_8TBs"] = res["sustained_read_gbs"] / HBM_PEAK_GBS
    return res


def bench_c3(steps, warmup, variant=0):
    """192 x ([512,512] {0,1} x [512,64] {-1,1}) -> int32 [192,512,64]."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    B, S, D = 192, 512, 64
    attn16 = pm1_f16((B, S, S), 3001, dev)                 # sign bit clear = 1
    v16 = pm1_f16((B, S, D), 3002, dev)
    ap, vp = lk.pack_sign(attn16), lk.pack_sign(v16.transpose(1, 2).contiguous())
    out = torch.empty((B, S, D), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(vp, ap, lk.MODE_ATTN_X, torch.int32, 1, variant, out=out)
    ms_eager = time_gpu(fn, warmup, steps)
    ms = time_gpu_graph(fn, 20, 4, max(2, steps // 20))
    want = torch.bmm((attn16[:4] > 0).float(), v16[:4].float()).to(torch.int32)
    ok = bool(torch.equal(out[:4], want))
    ops = 2.0 * B * S * S * D
    bytes_alg = B * (S * S / 8 + S * D / 8 + 4.0 * S * D)
    return {"name": "C3 attention AxV 192x[512,512]x[512,64]", "ms": ms, "ms_eager_launch": ms_eager,
            "tops": ops / ms / 1e9,
            "gbs": bytes_alg / ms / 1e6, "ops": ops, "bytes": bytes_alg, "bit_exact": ok}


def bench_c2(steps, warmup):
    """3-layer binarised MLP forward 784->4096->4096->10, batch 128, fp16 activations and per-output-channel
    fp16 scales.  Timed twice: op by op through the fp16 drop-in call (weights packed on every call, scaling as
    separate torch kernels, as the reference layer does), and fused (weights prepacked once, activations
    sign-packed in one pass, scaling applied in the GEMM's store)."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(2001)
    dims = [784, 4096, 4096, 10]
    x = torch.randn(128, 784, generator=g, device=dev).half()
    Ws = [torch.randn(dims[i + 1], dims[i], generator=g, device=dev).half() for i in range(3)]
    sws = [(W.float().norm(1, 1) / W.numel()).half() for W in Ws]
    sa = torch.tensor([1.0], device=dev).half()
    Wps = [lk.pack_sign(W) for W in Ws]

    def fwd_ops(i):
        h = x
        for W, sw in zip(Ws, sws):
            h = lk.bgemm_linear_forward_cuda(h, W, 1, 1) * sw * sa
        return h

    def fwd_fused(i):
        h = x
        for Wp, sw in zip(Wps, sws):
            h = lk.bgemm_packed_forward(Wp, lk.pack_sign(h), lk.MODE_XOR, splitK=8, scale=(sw, sa, None))[0]
        return h
    N = x.shape[0]
    hidden = [lk.zeros_packed(N, dims[1], 1, dev), lk.zeros_packed(N, dims[2], 1, dev)]

    def fwd_bits(i, inp=None):                  # hidden activations never stored: 4 launches
        hp = lk.pack_sign(x if inp is None else inp)
        for l in range(2):
            hp = lk.bgemm_packed_forward(Wps[l], hp, lk.MODE_XOR, splitK=8, scale=(sws[l], sa, None), bits_out=hidden[l])
        return lk.bgemm_packed_forward(Wps[2], hp, lk.MODE_XOR, splitK=8, scale=(sws[2], sa, None))[0]
    same = bool(torch.equal(fwd_ops(0), fwd_fused(0))) and bool(torch.equal(fwd_ops(0), fwd_bits(0)))
    ms_ops = time_gpu(fwd_ops, warmup, steps)
    ms_fused = time_gpu(fwd_fused, warmup, steps)
    ms_graph = time_gpu_graph(fwd_fused, 4, 2, max(2, steps // 4))
    ms_bits = time_gpu_graph(fwd_bits, 4, 2, max(2, steps // 4))
    # what a Python caller sees per forward when the four launches are replayed as one captured graph
    import bgemm_linear as bl
    fast = bl.GraphedInference(lambda t: fwd_bits(0, t), x)
    same = same and bool(torch.equal(fast(x), fwd_bits(0)))
    ms_call = time_gpu(lambda i: fast(x), warmup, steps)
    ops = 2.0 * 128 * (784 * 4096 + 4096 * 4096 + 4096 * 10)
    return {"name": "C2 MLP 784-4096-4096-10 batch 128, fp16 in/out, bits between layers (4 launches, graph replay)",
            "ms": ms_bits, "ms_fused_6_launches": ms_graph, "ms_graph_call_from_python": ms_call,
            "ms_eager_launch": ms_fused, "ms_op_by_op": ms_ops,
            "tops": ops / ms_bits / 1e9, "ops": ops, "bit_exact": same}


def run_extra(which, quick=False, variant=0):
    """The non-headline benchmark configurations: 'c4' decode BWTA, 'c3' attention, 'c2' MLP, 'sweep'.
    quick: a tenth of the launches (for counter collection, where every dispatch is serialised)."""
    extra = []
    div = 10 if quick else 1
    if which in ("c4", "all"):
        for N in (1, 4, 16):
            for sk in (1, 8):
                extra.append(bench_c4(2000 // div, 200 // div, N, sk, variant))
                log(json.dumps(extra[-1]))
        for N in (32, 64, 128):             # a batch of decode steps, beyond the configuration's row counts
            extra.append(bench_c4(1000 // div, 100 // div, N, 1, variant))
            log(json.dumps(extra[-1]))
        for N in (1, 4, 16):
            extra.append(bench_c4_batched(400 // div, N))
            log(json.dumps(extra[-1]))
        for N in (1, 4):
            extra.append(bench_c4_from_fp16(2000 // div, N))
            log(json.dumps(extra[-1]))
    if which in ("c3", "all"):
        extra.append(bench_c3(200 // div, 20 // div + 1, variant))
        log(json.dumps(extra[-1]))
    if which in ("c2", "all"):
        extra.append(bench_c2(200 // div, 20 // div + 1))
        log(json.dumps(extra[-1]))
    if which in ("sweep", "all"):
        extra.append(bench_c5_dropin(50 // div + 2, 5))
        log(json.dumps(extra[-1]))
        for (K, N) in [(4096, 256), (4096, 2048), (16384, 256), (16384, 2048)]:
            for sk in (1, 2, 4):
                r, _ = bench_c5(20, 3, 8192, N, K, sk)
                extra.append(r)
                log(json.dumps(r))
    for r in extra:
        r["frac_int8_mfma"] = r["tops"] / INT8_MFMA_PEAK_TOPS
        if "gbs" in r:
            r["frac_hbm"] = r["gbs"] / HBM_PEAK_GBS
    return extra


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--all", action="store_true", help="also time the other benchmark configurations")
    ap.add_argument("--only", choices=["c2", "c3", "c4", "sweep"], help="time just that configuration (for profiling)")
    ap.add_argument("--variant", type=int, default=0, help="0 auto, 1 VALU, 2 MFMA int8, 3 MFMA fp4")
    ap.add_argument("--split-k", type=int, default=1,
                    help="splitK of the headline launch: the most K ranges a tile may be computed in (same bits for any value)")
    ap.add_argument("--quick", action="store_true", help="with --only: a tenth of the launches (counter collection)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--floor", action="store_true",
                    help="print the hardware floors for the decode shape (empty launch, cold 5.6 MB read, sustained read)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a 256 MiB device-to-device copy (known traffic, for scaling rocprof counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU (its boxes have one); run with --gpus 1")

    import torch
    import _lib
    _lib.lib()          # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    if args.calib_copy:
        src = torch.empty(64 << 20, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        ms = time_gpu(lambda i: dst.copy_(src), 2, 5)
        log("calibration copy: 256 MiB read + 256 MiB written per launch, %.4f ms" % ms)
    if args.floor:
        print(json.dumps({"floor": bench_floor()}), flush=True)
        return
    if args.only:
        print(json.dumps({"configs": run_extra(args.only, args.quick, args.variant)}), flush=True)
        return

    c5, (w16, x16) = bench_c5(args.steps, args.warmup, splitK=args.split_k, variant=args.variant)
    log("C5:", json.dumps(c5))
    cpu = None if args.no_cpu else cpu_baseline_c5(w16, x16)
    del w16, x16
    extra = run_extra("all") if args.all else []
    fp4 = args.variant in (0, 3)
    peak = FP4_MFMA_PEAK_TOPS if fp4 else INT8_MFMA_PEAK_TOPS
    # HBM bytes per launch of the dominant kernel, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
    # profiles/gemm_mfma_f4_bgemm_8192x8192x8192.txt (scaled by the same counters on a 256 MiB device copy)
    traffic = MEASURED_TRAFFIC_BYTES_C5_FP4 if fp4 else None

    line = {
        "metric": "effective binary TOPS (2*M*N*K/t), bit-exact int32",
        "value": c5["tops"], "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": c5["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp4" if fp4 else "int8",
        "data": "synthetic",
        "config": {"workload": "BASELINE.json config 5: BGEMM M=N=K=8192, {-1,+1}x{-1,+1}, weights and activations "
                               "prepacked (tiled bit layout), int32 output, splitK=%d" % args.split_k,
                   "arithmetic": ("1-bit operands expanded in registers to E2M1 (fp4) MFMA operands, fp32 accumulation "
                                  "of exact integers" if fp4 else
                                  "1-bit operands expanded in registers to int8 MFMA operands, int32 accumulation"),
                   "op_count": "2*M*N*K binary multiply-accumulate ops per launch, the convention of the reference's "
                               "drivers (lowbit_kernel/csrc/benchmark.cu:291 prints it as TFLOPs)",
                   "bit_exact_sampled": c5["bit_exact"], "hbm_gbs_algorithmic": c5["gbs"],
                   "activation_pack_ms": c5["act_pack_ms"],
                   "frac_of_int8_mfma_peak": c5["tops"] / INT8_MFMA_PEAK_TOPS},
        "roofline": {"bound": "mfma", "achieved": c5["tops"], "peak": peak, "unit": "TFLOP/s",
                     "frac": c5["tops"] / peak, "traffic": traffic},
        "cpu_baseline": cpu,
    }
    if extra:
        line["all_configs"] = extra
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
