#!/usr/bin/env python3
"""Benchmark of the BGEMM / BWTA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--headline-only] [--only SECTION]

A step is one pass of the hot path over one batch of synthetic input: one 8192^3
{-1,1}x{-1,1} BGEMM on prepacked operands (benchmark configuration 5, the compute-bound case the
metric's target is quoted on), int32 output, operands resident in HBM before the timed
region.  One JSON line goes to stdout; `value` is effective binary TOPS = 2*M*N*K / t
(the reference drivers' own op count, lowbit_kernel/csrc/benchmark.cu:291).

Beside the headline the line carries, under "all_configs", one compact row per other benchmark
configuration (MLP forward, batched attention A x V, decode-shape BWTA: one launch, 64 matrices in one
launch, and the GEMMs a Llama-7B decode step issues; the sweep around 8192^3), each with its kernel, its time,
TOPS, GB/s, bit-exactness and the roofline that bounds it; under "floor" what the hardware allows a
decode-size launch (empty launch, cold read); under "mfma_peak_measured" the rate of the two MFMA
instructions the library issues with nothing else going on (the reference's protocol: warm-up launches,
then timed launches between two events, lowbit_kernel/csrc/kernel_test.h:10-11, csrc/benchmark.cu:275-291).
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "bgemm-cuda_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

INT8_MFMA_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published
FP4_MFMA_PEAK_TOPS = 10100.0      # MI355X dense fp4 MFMA, published
HBM_PEAK_GBS = 8000.0             # MI355X HBM3E, published
PRE_ROLL = 300                    # untimed launches of the headline GEMM before its warm-up steps (see bench_c5)
C5_PROFILE = os.path.join(ROOT, "profiles", "gemm_mfma_f4_bgemm_8192x8192x8192.txt")
PROBES_SO = os.path.join(ROOT, "libbench_probes.so")

KERNEL_NAMES = {0: "mfma 256x256", 1: "mfma 128x128", 2: "mfma 64x128", 3: "mfma 32x128", 4: "mfma 256x128", 5: "mfma 32x256",
                6: "mfma 64x64", 7: "mfma 128x64", 8: "mfma 128x256 signed", 16: "decode stream", 17: "decode split-K in the block",
                18: "decode four pieces a block", 19: "decode AND-popcount (vector ALU)", 32: "VALU popcount GEMM"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def log_row(r):
    """Progress on stderr: the row's id, time and whether it was bit-exact (the whole row is in the final line)."""
    log("%s: %s us%s" % (r.get("id", r.get("shape", "")), r.get("us", ""), "" if r.get("ok", True) else "  NOT BIT-EXACT"))


def measured_traffic_bytes():
    """HBM bytes per launch of the headline kernel as the tracked profile summary states them (a line
    `traffic_bytes_per_launch = N` under the FETCH_SIZE / WRITE_SIZE counter runs), or None."""
    try:
        m = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)", open(C5_PROFILE).read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


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


def time_gpu_repeats(fn, warmup, steps, repeats=5):
    """The reference's protocol with repeats: warm-up once, then `repeats` timed regions of exactly `steps` calls each;
    returns (median, min, max) milliseconds per call."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    ts = sorted(time_gpu(fn, 0, steps) for _ in range(repeats))
    return ts[len(ts) // 2], ts[0], ts[-1]


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


def ternary_f16(shape, seed, device):
    """{-1, 0, +1} with p(0) = 0.5."""
    import torch
    g = torch.Generator(device=device).manual_seed(seed)
    t = torch.randint(0, 4, shape, generator=g, device=device)
    return torch.where(t == 0, -1.0, torch.where(t == 3, 1.0, 0.0)).to(torch.half)


def random_packed(rows, K, batch, seed, device):
    """A packed operand of random bits (rows a multiple of 32, K of 256: no padding to keep zero)."""
    import torch
    import lowbit_kernel as lk
    assert rows % 32 == 0 and K % 256 == 0
    g = torch.Generator(device=device).manual_seed(seed)
    data = torch.randint(-2 ** 31, 2 ** 31 - 1, (batch, rows * K // 32), generator=g, device=device, dtype=torch.int32)
    return lk.PackedBits(data, None, batch, rows, K)


def unpacked_pm1(packed, b=0):
    """The +-1 fp32 matrix [rows, K] behind matrix b of a packed operand."""
    import torch
    import lowbit_kernel as lk
    one = lk.PackedBits(packed.data[b:b + 1], None, 1, packed.rows, packed.K)
    logical = lk.logical_from_tiled(one)
    shifts = torch.arange(31, -1, -1, device=logical.device, dtype=torch.int32)
    bits = ((logical.unsqueeze(-1) >> shifts) & 1).reshape(packed.rows, -1)[:, :packed.K]
    return (1 - 2 * bits).float()


def check_sampled(out, w16, x16, n_rows=64, n_cols=64):
    """Spot parity check of an [N,M] XOR result against the fp32 closed form on sampled rows."""
    import torch
    N, M = out.shape
    g = torch.Generator().manual_seed(7)
    rs = torch.randperm(M, generator=g)[:n_rows].to(out.device)
    cs = torch.randperm(N, generator=g)[:n_cols].to(out.device)
    want = (x16[cs].float().cpu() @ w16[rs].float().cpu().T).to(torch.int32)
    return bool(torch.equal(out[cs][:, rs].cpu(), want))


def kernel_of(w, x, mode, splitK=1, variant=0, out_dtype=None):
    import torch
    import lowbit_kernel as lk
    return KERNEL_NAMES.get(lk.packed_kernel_id(w, x, mode, splitK, variant, out_dtype or torch.int32), "?")


KERNEL_IDS = {"mfma 256x256": "m256x256", "mfma 128x128": "m128x128", "mfma 64x128": "m64x128", "mfma 32x128": "m32x128",
              "mfma 256x128": "m256x128", "mfma 32x256": "m32x256", "mfma 64x64": "m64x64", "mfma 128x64": "m128x64",
              "mfma 128x256 signed": "m128x256t",
              "decode stream": "stream", "decode split-K in the block": "splitk", "decode four pieces a block": "quad",
              "decode AND-popcount (vector ALU)": "popc", "VALU popcount GEMM": "valu"}


def row(name, ms, ops, bytes_alg, ok, kernel, bound, **more):
    """One compact all_configs row (the whole line has to fit the tail a driver keeps): id, k = kernel, us, tops,
    gbs = algorithmic GB/s, ok = bit-exact against the closed form computed in the same run, frac of the roofline that
    bounds it (b: "mfma" = fp4 dense peak the kernels issue against, "hbm" = 8 TB/s)."""
    tops, gbs = ops / ms / 1e9, bytes_alg / ms / 1e6
    r = {"id": name, "k": KERNEL_IDS.get(kernel, kernel), "us": round(ms * 1e3, 2), "tops": round(tops, 1), "gbs": round(gbs, 1),
         "ok": ok, "b": bound, "frac": round(tops / FP4_MFMA_PEAK_TOPS if bound == "mfma" else gbs / HBM_PEAK_GBS, 4)}
    r.update(more)
    return r


# ---------------------------------------------------------------- configuration 5: 8192^3 and its sweep
def bench_c5(steps, warmup, M=8192, N=8192, K=8192, splitK=1, variant=0, pre_roll=0, counted=False):
    """pre_roll: launches of the same GEMM issued (and waited for) before the warm-up steps, untimed: the GPU's
    clocks take some tens of milliseconds of matrix-core load to settle (the launch runs at 0.19 ms for the first
    hundred launches, 0.174 for the next and 0.171 from about 250 on), which five warm-up steps of 0.2 ms do not
    give them.  The reference's drivers warm up with 100 launches and time 10 000
    (lowbit_kernel/csrc/kernel_test.h:10-11): a steady-state figure, which is what the pre-roll makes of the
    few timed steps here."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    w16, x16 = pm1_f16((M, K), 5001, dev), pm1_f16((N, K), 5002, dev)
    # prepacked operands: the tiled bits.  `counted`: with their row popcounts as well (the large tiles then count
    # nothing in their main loop); the headline is timed without, and with them beside it.
    wp, xp = lk.pack_sign(w16), lk.pack_sign(x16)
    if counted and (variant & 0xff) != 1:
        lk.row_popcounts(wp), lk.row_popcounts(xp)
    out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(wp, xp, lk.MODE_XOR, torch.int32, splitK, variant, out=out)
    for i in range(pre_roll):
        fn(i)
    torch.cuda.synchronize()
    ms, ms_min, ms_max = time_gpu_repeats(fn, warmup, steps) if pre_roll else (time_gpu(fn, warmup, steps),) * 3
    ok = check_sampled(out[0], w16, x16)
    ms_counted = count_ms = None
    if pre_roll and xp.counts is None and (variant & 0xff) != 1:
        # beside the headline row: the same launches on operands that bring their row popcounts along
        lk.row_popcounts(wp), lk.row_popcounts(xp)
        for i in range(pre_roll):          # the check above left the GPU idle: its clocks have to settle again
            fn(i)
        torch.cuda.synchronize()
        ms_counted = time_gpu_repeats(fn, warmup, steps)[0]
        ok = ok and check_sampled(out[0], w16, x16)

        def count_again(i):
            xp.counts = None
            lk.row_popcounts(xp)
        count_ms = time_gpu(count_again, 2, 10)
    ops = 2.0 * M * N * K
    bytes_alg = M * K / 8 + N * K / 8 + 4.0 * M * N
    pack_ms = time_gpu(lambda i: lk.pack_sign(x16), 2, 10)
    return {"name": "C5 BGEMM %dx%dx%d xor int32 splitK=%d" % (M, N, K, splitK), "ms": ms, "ms_min": ms_min, "ms_max": ms_max,
            "tops": ops / ms / 1e9, "gbs": bytes_alg / ms / 1e6, "ops": ops, "bytes": bytes_alg,
            "bit_exact": ok, "act_pack_ms": pack_ms, "act_popcount_ms": count_ms, "ms_counted": ms_counted,
            "kernel": kernel_of(wp, xp, lk.MODE_XOR, splitK, variant)}, (w16, x16)


def bench_sweep(steps=40, warmup=5):
    """The sweep of configuration 5: K in {4096, 16384} x N in {256, 2048}, M = 8192.  One row per point: the
    library does not split these shapes across blocks, so split-K 1, 2 and 4 run the same kernel (timed at 1 and 4)."""
    rows = []
    for (K, N) in [(4096, 256), (4096, 2048), (16384, 256), (16384, 2048)]:
        r1, _ = bench_c5(steps, warmup, 8192, N, K, 1)
        r4, _ = bench_c5(steps, warmup, 8192, N, K, 4)
        rows.append(row("C5 sweep 8192x%dx%d" % (N, K), r1["ms"], r1["ops"], r1["bytes"],
                        r1["bit_exact"] and r4["bit_exact"], r1["kernel"], "mfma", us_splitK4=round(r4["ms"] * 1e3, 2)))
        log_row(rows[-1])
    return rows


def _lib_kernel_id(M, N, K):
    """The kernel the library runs for an [N,K] x [M,K] sign product with fp16 output."""
    import _lib
    return _lib.lib().bgemm_packed_kernel_id(_lib.MODE_XOR, _lib.OUT_F16, 1, M, N, K, 1, _lib.VARIANT_AUTO)


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
    return row("C5 fp16 drop-in call %dx%dx%d (packs both operands)" % (M, N, K),
               ms, 2.0 * M * N * K, 2.0 * (M * K + N * K + M * N), ok,
               "pack + " + KERNEL_NAMES.get(_lib_kernel_id(M, N, K), "?"), "mfma")


def cpu_baseline_c5(w16, x16, budget_s=12.0):
    """Reference CPU path (torch matmul on +-1 fp32 tensors) on a bounded column slice."""
    import torch
    from oracle import oracle
    # every host thread this process may use: the boxes give a one-GPU job 16 of the host's cores and set OMP_NUM_THREADS
    # to match (torch's default follows it); os.cpu_count() there counts the whole machine
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    torch.set_num_threads(max(1, min(avail, int(os.environ.get("OMP_NUM_THREADS", avail)))))
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
    return {"value": 2.0 * M * n * K / dt / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": "torch.matmul fp32 on +-1 tensors, W[%d,%d] x X[%d,%d] (%d of %d activation rows), %d reps"
                      % (M, K, n, K, n, x16.shape[0], reps)}


# ---------------------------------------------------------------- hardware floors and measured peaks
def probes():
    if not os.path.exists(PROBES_SO):
        raise ImportError("%s is missing: build it with `python __graft_entry__.py`" % PROBES_SO)
    L = ctypes.CDLL(PROBES_SO)
    p, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.bench_probe_empty.argtypes = [ci, ci, p, p]
    L.bench_probe_read.argtypes = [p, i64, ci, ci, p, p]
    L.bench_probe_mfma.argtypes = [ci, ci, ci, ci, p, p]
    L.bench_probe_exchange.argtypes = [p, ci, ci, ci, ci, ctypes.c_uint, p, ci, p]
    return L


class ColdRead:
    """Time of a plain read (no compute, no store) of `nbytes` that no cache holds: the probe walks a pool larger
    than the 256 MB Infinity Cache, one piece per launch."""

    def __init__(self):
        import torch
        self.L = probes()
        self.pool = torch.ones((384 << 20) // 4, dtype=torch.int32, device="cuda:0")
        self.scratch = torch.zeros(64, dtype=torch.int32, device="cuda:0")
        self.cache = {}

    def us(self, nbytes):
        import torch
        nbytes = int(nbytes) // 16 * 16
        if nbytes not in self.cache:
            copies = max(1, min(64, self.pool.numel() * 4 // nbytes))
            st = lambda: torch.cuda.current_stream().cuda_stream
            best = None
            for blocks, threads in ((512, 512), (1024, 256), (1024, 512), (2048, 256)):
                t = 1e3 * time_gpu_graph(lambda i: self.L.bench_probe_read(self.pool.data_ptr() + (i % copies) * nbytes, nbytes,
                                                                           blocks, threads, self.scratch.data_ptr(), st()),
                                         copies, 2, max(4, 256 // copies))
                best = t if best is None else min(best, t)
            self.cache[nbytes] = best
        return self.cache[nbytes]


def bench_floor(cold):
    """What the hardware allows a kernel of the decode path's shape: the cost of launching an empty kernel,
    of reading one cold 5.6 MB buffer (the packed W[11008,4096]), and the bandwidth a plain read sustains."""
    import torch
    L = cold.L
    st = lambda: torch.cuda.current_stream().cuda_stream
    nbytes = 11008 * 4096 // 8
    res = {"empty_kernel_us": round(1e3 * time_gpu_graph(lambda i: L.bench_probe_empty(344, 512, cold.scratch.data_ptr(), st()), 64, 2, 20), 3)}
    res["cold_read_5p6MB_us"] = round(cold.us(nbytes), 3)
    res["cold_read_5p6MB_gbs"] = round(nbytes / cold.us(nbytes) / 1e3, 1)
    total = 64 * nbytes
    best = None
    for blocks, threads in ((2048, 512), (4096, 512), (8192, 512)):
        us = 1e3 * time_gpu_graph(lambda i: L.bench_probe_read(cold.pool.data_ptr(), total, blocks, threads, cold.scratch.data_ptr(), st()), 4, 2, 10)
        best = us if best is None else min(best, us)
    res["sustained_read_361MB_us"] = round(best, 2)
    res["sustained_read_gbs"] = round(total / best / 1e3, 1)
    res["sustained_read_frac_of_8TBs"] = round(res["sustained_read_gbs"] / HBM_PEAK_GBS, 4)
    # one all-to-all exchange among resident blocks (one per compute unit), the floor under a layer of the chain kernel:
    # 3 units a block (a ternary row against two weight row tiles, less one), one replica and one replica per XCD
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stride, rounds, epoch = cus * 8, 200, 1
    buf = torch.zeros(2 * 8 * stride, dtype=torch.int64, device="cuda:0")
    err = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    for copies in (1, 8):
        best = None
        for rep in range(3):
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            L.bench_probe_exchange(buf.data_ptr(), cus, 3, copies, rounds, epoch, err.data_ptr(), stride, st())
            e1.record()
            torch.cuda.synchronize()
            epoch += rounds
            us = 1e3 * e0.elapsed_time(e1) / rounds
            best = us if best is None else min(best, us)
        res["all_to_all_exchange_%d_blocks_%s_us" % (cus, "1_replica" if copies == 1 else "8_replicas")] = round(best, 3)
    res["all_to_all_exchange_ok"] = bool((err == 0).all())
    return res


def bench_mfma_peak(cold):
    """The matrix cores alone: v_mfma_f32_32x32x64_f8f6f4 (E2M1 operands) and v_mfma_i32_32x32x32_i8 from two waves
    per SIMD with eight independent accumulators each, no memory traffic; then with a number of independent vector-ALU
    instructions after every MFMA (what the bit expansion adds to the issue stream: the probe's loop holds exactly that
    many v_and_b32 per MFMA).  20 warm-up + 100 timed launches."""
    import torch
    L = cold.L
    out = torch.empty(512 * 256, dtype=torch.int32, device="cuda:0")
    st = lambda: torch.cuda.current_stream().cuda_stream
    iters, blocks = 2000, 512
    res = {}

    def probe(fp4, valu):
        rc = L.bench_probe_mfma(fp4, valu, blocks, iters, out.data_ptr(), st())
        if rc != 0:
            raise RuntimeError("bench_probe_mfma(%d, %d) -> %d: libbench_probes.so is older than bench_probes.hip?" % (fp4, valu, rc))

    for fp4 in (1, 0):
        for valu in ((0, 1, 2, 3, 4, 5, 6, 8) if fp4 else (0, 4, 8)):
            ms = time_gpu(lambda i: probe(fp4, valu), 20, 100)
            ops = 2.0 * 32 * 32 * (64 if fp4 else 32) * 8 * iters * 4 * blocks
            key = ("fp4" if fp4 else "int8") + ("_tops" if valu == 0 else "_tops_with_%d_valu_per_mfma" % valu)
            res[key] = round(ops / ms / 1e9, 1)
    # the same with an instruction that reads two vector registers (v_perm_b32) instead of one (v_and_b32)
    for valu in (2, 4):
        ms = time_gpu(lambda i: probe(1, 100 + valu), 20, 100)
        res["fp4_tops_with_%d_two_register_valu_per_mfma" % valu] = round(2.0 * 32 * 32 * 64 * 8 * iters * 4 * blocks / ms / 1e9, 1)
    # expansions shared between the waves of a block through LDS: the loop with two v_and_b32 per MFMA plus the LDS traffic
    ms = time_gpu(lambda i: probe(1, -1), 20, 100)
    res["fp4_tops_with_2_valu_and_shared_fragments_through_lds"] = round(2.0 * 32 * 32 * 64 * 8 * iters * 4 * blocks / ms / 1e9, 1)
    res["fp4_frac_of_datasheet"] = round(res["fp4_tops"] / FP4_MFMA_PEAK_TOPS, 4)
    res["int8_frac_of_datasheet"] = round(res["int8_tops"] / INT8_MFMA_PEAK_TOPS, 4)
    return res


# ---------------------------------------------------------------- configuration 4: decode-shape BWTA
def bench_decode(cold, name, M, K, Ns, steps=640, total_mb=361):
    """One launch per matrix: prepacked W[M,K] x ternary activations [N,K] -> int32, weights rotated over enough
    copies (> 256 MB in total) that no launch finds them in a cache; launches replayed from a HIP graph.  Every row
    states its fraction of 8 TB/s and its ratio to a plain cold read of the same number of bytes."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    wbytes = M * K // 8
    copies = max(8, min(64, int(total_mb * 1e6 // wbytes)))
    pool = random_packed(M, K, copies, 4001, dev)
    wps = [lk.PackedBits(pool.data[c:c + 1], None, 1, M, K) for c in range(copies)]
    w_pm1 = unpacked_pm1(pool, 0)
    rows = []
    for N in Ns:
        x16 = ternary_f16((N, K), 4000 + N, dev)
        xt = lk.pack_ternary(x16)
        out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
        fn = lambda i: lk.bgemm_packed_forward(wps[i % copies], xt, lk.MODE_BWTA, torch.int32, 8, 0, out=out)
        fn(0)
        ok = bool(torch.equal(out[0], (torch.sign(x16.float()) @ w_pm1.T).to(torch.int32)))
        ms = time_gpu_graph(fn, copies, 4, max(2, steps // copies))
        bytes_alg = wbytes + 2 * N * K / 8 + 4.0 * M * N
        floor_us = cold.us(bytes_alg)
        rows.append(row("%s W[%d,%d] N=%d 1 launch cold" % (name, M, K, N), ms, 2.0 * M * N * K, bytes_alg, ok,
                        kernel_of(wps[0], xt, lk.MODE_BWTA, 8), "hbm", cold_read_us=round(floor_us, 2),
                        x_cold_read=round(ms * 1e3 / floor_us, 2)))
        log_row(rows[-1])
    return rows


def bench_decode_batched(N, B=64, replays=10):
    """The same decode-shape BWTA linear over B weight matrices in ONE launch (the layers of a model,
    a set of experts): 361 MB of weights stream through once, so the launch is long enough to show the
    bandwidth the kernel sustains rather than the latency of one 5.6 MB launch."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    M, K = 11008, 4096
    x16 = ternary_f16((N, K), 4100 + N, dev)
    xt = lk.pack_ternary(x16)
    wb = random_packed(M, K, B, 4101, dev)
    out = torch.empty((B, N, M), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(wb, xt, lk.MODE_BWTA, torch.int32, 1, 0, out=out)
    ms = time_gpu_graph(fn, 4, 2, replays)
    ok = True
    for b in (0, B // 2, B - 1):       # parity of three of the matrices against the fp32 closed form on unpacked bits
        ok = ok and bool(torch.equal(out[b], (torch.sign(x16.float()) @ unpacked_pm1(wb, b).T).to(torch.int32)))
    bytes_alg = B * (M * K / 8 + 4.0 * M * N) + 2 * N * K / 8
    return row("C4 %d matrices W[11008,4096] N=%d in 1 launch" % (B, N), ms, 2.0 * B * M * N * K, bytes_alg, ok,
               kernel_of(wb, xt, lk.MODE_BWTA), "hbm")


def bench_decode_from_fp16(N, steps=640, copies=64):
    """A decode step as a model runs it: fp16 activations in, prepacked W[11008,4096], int32 out.  Timed as two
    launches (ternary pack, then the packed GEMM) and as the one launch that packs its activations itself."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    M, K = 11008, 4096
    x16 = ternary_f16((N, K), 4200 + N, dev)
    pool = random_packed(M, K, copies, 4001, dev)
    wps = [lk.PackedBits(pool.data[c:c + 1], None, 1, M, K) for c in range(copies)]
    two = lambda i: lk.bgemm_packed_forward(wps[i % copies], lk.pack_ternary(x16), lk.MODE_BWTA, torch.int32)
    one = lambda i: lk.bgemm_packed_weight_forward(wps[i % copies], x16, lk.MODE_BWTA, torch.int32)
    ok = bool(torch.equal(two(0)[0], one(0)))
    ms_two = time_gpu_graph(two, copies, 2, max(2, steps // copies))
    ms_one = time_gpu_graph(one, copies, 2, max(2, steps // copies))
    ms_one_eager = time_gpu(one, 20, steps)
    bytes_alg = M * K / 8 + 2.0 * N * K + 4.0 * M * N
    return row("C4 from fp16 x, W[11008,4096] N=%d, kernel packs x" % N, ms_one,
               2.0 * M * N * K, bytes_alg, ok, "fusex", "hbm",
               us_pack_then_gemm=round(ms_two * 1e3, 2), us_from_python=round(ms_one_eager * 1e3, 2))


def bench_chain(cold, Ns=(1, 4, 16), blocks=32, replays=6):
    """Configuration 4 as the layers of a model see it: a chain of dependent decode-shaped layers, up W[11008,4096] ->
    down W[4096,11008] -> up -> ..., 2 * blocks layers with distinct weights (361 MB for 32 blocks: more than the
    Infinity Cache holds, so every replay reads them from HBM), ternary activations between the layers, in ONE launch
    (bgemm_chain_forward).  us per layer against 8 TB/s and against a plain cold read of a layer's bytes; bit-exact
    against the same chain evaluated layer by layer with torch on the de-binarised operands."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(4300)
    dims = [4096, 11008] * blocks + [4096]
    L = len(dims) - 1
    pools = {(11008, 4096): random_packed(11008, 4096, blocks, 4301, dev), (4096, 11008): random_packed(4096, 11008, blocks, 4302, dev)}
    layers = []
    for l in range(L):
        K, M = dims[l], dims[l + 1]
        w = lk.PackedBits(pools[(M, K)].data[l // 2:l // 2 + 1], None, 1, M, K)
        sw = ((0.5 + torch.rand(M, generator=g, device=dev)) / K ** 0.5).half()
        layers.append((w, sw, torch.tensor([1.0], device=dev).half(), None, torch.tensor([0.02], device=dev).half()))
    chain = lk.DecodeChain(layers, lk.MODE_BWTA, torch.int32)
    wbytes = 11008 * 4096 // 8
    rows = []
    for N in Ns:
        x16 = ternary_f16((N, 4096), 4310 + N, dev)
        xt = lk.pack_ternary(x16)
        out = torch.empty((N, 4096), dtype=torch.int32, device=dev)
        chain(xt, out=out)
        chain.check(N)
        # the same chain, layer by layer, in torch
        h = torch.sign(x16.float())
        for l, (w, sw, sa, bias, zp) in enumerate(layers):
            acc = (h @ unpacked_pm1(pools[(w.rows, w.K)], l // 2).T)
            if l + 1 < L:
                h = torch.sign(((acc.half() * sw * sa) - zp).float())
        ok = bool(torch.equal(out, acc.to(torch.int32)))
        ms = time_gpu_graph(lambda i: chain(xt, out=out), 1, 1, replays) / L
        chain.check(N)
        bytes_alg = wbytes + 2 * N * 7552 / 8 + 0.0          # a layer's weights + its ternary operand (mean K of up and down)
        floor_us = cold.us(wbytes)
        rows.append(row("C4 chain of %d dependent layers up/down W[11008,4096] N=%d, per layer" % (L, N), ms, 2.0 * 11008 * 4096 * N, bytes_alg, ok,
                        "chain", "hbm", cold_read_us=round(floor_us, 2), x_cold_read=round(ms * 1e3 / floor_us, 2), us_whole_chain=round(ms * L * 1e3, 1)))
        log_row(rows[-1])
    return rows


# ---------------------------------------------------------------- configurations 3 and 2
def bench_c3(steps=200, warmup=20, variant=0):
    """192 x ([512,512] {0,1} x [512,64] {-1,1}) -> int32 [192,512,64]."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    B, S, D = 192, 512, 64
    attn16 = pm1_f16((B, S, S), 3001, dev)                 # sign bit clear = 1
    v16 = pm1_f16((B, S, D), 3002, dev)
    ap, vp = lk.pack_sign(attn16), lk.pack_sign_transposed(v16)
    out = torch.empty((B, S, D), dtype=torch.int32, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(vp, ap, lk.MODE_ATTN_X, torch.int32, 1, variant, out=out)
    ms_eager = time_gpu(fn, warmup, steps)
    ms = time_gpu_graph(fn, 20, 4, max(2, steps // 20))
    ok = bool(torch.equal(out, torch.bmm((attn16 > 0).float(), v16.float()).to(torch.int32)))      # every head
    ops = 2.0 * B * S * S * D
    bytes_alg = B * (S * S / 8 + S * D / 8 + 4.0 * S * D)
    return row("C3 AxV 192x[512,512]x[512,64] int32", ms, ops, bytes_alg, ok, kernel_of(vp, ap, lk.MODE_ATTN_X), "hbm",
               us_from_python=round(ms_eager * 1e3, 2))


def bench_qk(steps=100):
    """The other half of the attention pair: Q.K^T, 192 x ([512,64] x [64,512]) -> fp16 scores [192,512,512]."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    B, S, D = 192, 512, 64
    q16, k16 = pm1_f16((B, S, D), 3003, dev), pm1_f16((B, S, D), 3004, dev)
    qp, kp = lk.pack_sign(q16), lk.pack_sign(k16)
    out = torch.empty((B, S, S), dtype=torch.half, device=dev)
    fn = lambda i: lk.bgemm_packed_forward(kp, qp, lk.MODE_XOR, torch.half, 1, 0, out=out)
    ms = time_gpu_graph(fn, 10, 2, max(2, steps // 10))
    ok = bool(torch.equal(out, torch.bmm(q16.float(), k16.float().transpose(1, 2)).half()))
    bytes_alg = B * (2 * S * D / 8 + 2.0 * S * S)
    return row("QK^T 192x[512,64]x[64,512] fp16", ms, 2.0 * B * S * S * D, bytes_alg, ok, kernel_of(kp, qp, lk.MODE_XOR, out_dtype=torch.half), "hbm")


def bench_c2(steps=200, warmup=20):
    """3-layer binarised MLP forward 784->4096->4096->10, batch 128, fp16 activations and per-output-channel
    fp16 scales.  Timed op by op through the fp16 drop-in call (weights packed on every call, scaling as
    separate torch kernels, as the reference layer does), fused (weights prepacked once, activations
    sign-packed in one pass, scaling applied in the GEMM's store), and with nothing but bits between the layers."""
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
    # the fp16 reference: torch matmul on the de-binarised tensors, scaled op by op
    h = x
    for W, sw in zip(Ws, sws):
        sx = torch.where(h.view(torch.int16) < 0, -1.0, 1.0)
        sw_ = torch.where(W.view(torch.int16) < 0, -1.0, 1.0)
        h = (sx @ sw_.T).half() * sw * sa
    same = bool(torch.equal(fwd_ops(0), h)) and bool(torch.equal(fwd_fused(0), h)) and bool(torch.equal(fwd_bits(0), h))
    ms_ops = time_gpu(fwd_ops, warmup, steps)
    ms_fused = time_gpu(fwd_fused, warmup, steps)
    ms_graph = time_gpu_graph(fwd_fused, 4, 2, max(2, steps // 4))
    ms_bits = time_gpu_graph(fwd_bits, 4, 2, max(2, steps // 4))
    ops = 2.0 * 128 * (784 * 4096 + 4096 * 4096 + 4096 * 10)
    bytes_alg = sum(W.numel() for W in Ws) / 8 + 2.0 * 128 * (784 + 10)
    return row("C2 MLP 784-4096-4096-10 b128, bits between layers, 4 launches (graph)", ms_bits, ops,
               bytes_alg, same, "pack+3 gemm", "mfma", us_6_launches=round(ms_graph * 1e3, 2),
               us_from_python=round(ms_fused * 1e3, 2), us_op_by_op=round(ms_ops * 1e3, 2))


# ---------------------------------------------------------------- thresholds behind the dispatch
THRESHOLD_SHAPES = [
    # (planes, batch, M, N, K): around the choices of pick_cfg (general kernel tiles) and of the decode kernels' ranges
    (1, 1, 8192, 8192, 2048), (1, 1, 8192, 8192, 4096), (1, 1, 8192, 8192, 8192), (1, 1, 8192, 8192, 16384),
    (1, 1, 8192, 2048, 4096), (1, 1, 8192, 2048, 16384), (1, 1, 11008, 768, 4096), (1, 1, 4096, 2048, 4096),
    (1, 1, 8192, 256, 4096), (1, 1, 8192, 256, 8192), (1, 1, 8192, 256, 16384), (1, 1, 8192, 512, 8192),
    (1, 1, 8192, 768, 16384), (1, 1, 8192, 1024, 16384), (1, 1, 1024, 1024, 16384), (1, 1, 4096, 256, 11008),
    # under one 256 x 128 block a unit, and a few more than one
    (1, 1, 8192, 768, 8192), (1, 1, 8192, 768, 4096), (1, 1, 11008, 512, 8192), (1, 1, 5120, 1024, 8192), (1, 1, 11008, 640, 8192),
    (1, 1, 4096, 1024, 4096), (1, 1, 8192, 512, 16384),
    # a short K into int32 rows of a power of two in bytes, and the same beside a power of two
    (1, 1, 2048, 4096, 1024), (1, 1, 2000, 4000, 1024), (1, 1, 4096, 2048, 1024), (1, 1, 8192, 1024, 1024),
    (1, 1, 4096, 256, 4096), (1, 1, 11008, 128, 4096), (1, 1, 4096, 384, 4096), (1, 1, 2048, 256, 16384),
    (1, 1, 256, 256, 16384), (1, 1, 4096, 128, 4096), (1, 192, 512, 512, 64), (1, 192, 64, 512, 512),
    (2, 1, 11008, 32, 4096), (2, 1, 11008, 64, 4096), (2, 1, 11008, 128, 4096), (2, 1, 4096, 128, 11008),
    (2, 1, 4096, 256, 11008), (2, 1, 4096, 512, 11008), (2, 1, 8192, 128, 8192), (2, 1, 8192, 256, 8192),
    # two planes past one round of the four-pieces kernel's blocks, and between one and two 128 x 128 blocks a unit
    (2, 1, 8192, 160, 8192), (2, 1, 11008, 96, 4096), (2, 1, 8192, 640, 8192), (2, 1, 11008, 576, 8192),
    # 144 blocks of 128 x 128; partly filled tiles; four to seven K-tiles
    (1, 1, 9216, 256, 4096), (1, 1, 9216, 256, 2048), (1, 1, 10240, 160, 8192), (1, 1, 12288, 160, 8192),
    (1, 1, 11008, 40, 1792), (1, 1, 1024, 384, 1024),
]


# the shapes of the default run's `dispatch` block: the two sides of the most contested choices
DISPATCH_SHAPES = [(1, 1, 8192, 8192, 2048), (1, 1, 8192, 2048, 4096), (1, 1, 11008, 768, 4096), (1, 1, 8192, 256, 4096), (1, 1, 8192, 256, 8192),
                   (1, 1, 8192, 512, 8192), (1, 1, 8192, 768, 8192), (1, 1, 11008, 640, 8192), (1, 1, 2000, 4000, 1024), (1, 1, 4096, 256, 4096),
                   (1, 1, 2048, 256, 16384), (2, 1, 11008, 128, 4096), (2, 1, 4096, 256, 11008), (2, 1, 8192, 256, 8192), (2, 1, 11008, 576, 8192),
                   (1, 1, 12288, 160, 8192)]


def dispatch_summary(rows):
    """How far the library's own choice is from the fastest kernel that can take each shape (cold weights): the
    largest and the 90th-percentile ratio and the three worst shapes."""
    rs = sorted((r["auto_vs_fastest_cold"], r["shape"], r["auto"], r["fastest_cold"]) for r in rows if r.get("auto_vs_fastest_cold"))
    if not rs:
        return None
    return {"shapes": len(rs), "regret_max": rs[-1][0], "regret_p90": rs[min(len(rs) - 1, int(0.9 * len(rs)))][0],
            "worst": [{"shape": x[1], "auto": KERNEL_IDS.get(x[2], x[2]), "fastest": KERNEL_IDS.get(x[3], x[3]), "x": x[0]} for x in rs[-3:][::-1]],
            "mismatch": [r["shape"] for r in rows if "mismatch" in r]}


def bench_thresholds(steps=60, shapes=None, warm=True):
    """Every shape above under every kernel that can take it (BGEMM_FORCE_KERNEL), weights from HBM (rotating copies
    beyond the Infinity Cache) and from a warm cache: the timings the dispatch thresholds of the library rest on."""
    import torch
    import lowbit_kernel as lk
    import _lib as B
    dev = torch.device("cuda:0")
    general = [B.KERNEL_MFMA_256x256, B.KERNEL_MFMA_256x128, B.KERNEL_MFMA_128x128, B.KERNEL_MFMA_64x128, B.KERNEL_MFMA_32x128,
               B.KERNEL_MFMA_32x256, B.KERNEL_MFMA_128x64, B.KERNEL_MFMA_64x64]
    rows = []
    for planes, batch, M, N, K in (shapes or THRESHOLD_SHAPES):
        mode = lk.MODE_BWTA if planes == 2 else lk.MODE_XOR
        wbytes = batch * M * K // 8
        copies = max(2, min(40, int(300e6 // wbytes)))
        pool = lk.pack_sign(pm1_f16((copies * batch, M, K), 11, dev))
        wps = [lk.PackedBits(pool.data[c * batch:(c + 1) * batch], None, batch, M, K) for c in range(copies)]
        if planes == 2:
            xp = lk.pack_ternary(ternary_f16((batch, N, K) if batch > 1 else (N, K), 12, dev))
        else:
            xp = lk.pack_sign(pm1_f16((batch, N, K) if batch > 1 else (N, K), 12, dev))
        out = torch.empty((batch, N, M), dtype=torch.int32, device=dev)
        auto = lk.packed_kernel_id(wps[0], xp, mode, 8)
        res = {"shape": "%d planes, batch %d, M=%d N=%d K=%d" % (planes, batch, M, N, K), "auto": KERNEL_NAMES[auto], "us_cold": {}, "us_warm": {}}
        ref = None
        # the first timings on a new shape come out a few percent slow (pool and output pages touched for the first
        # time): an untimed pass of the library's own choice first, so that no kernel in the list pays for it
        warm = lambda i: lk.bgemm_packed_forward(wps[i % copies], xp, mode, torch.int32, 8, 0, out=out)
        warm(0)
        time_gpu_graph(warm, copies, 2, 2)
        for kid in general + [B.KERNEL_MFMA_128x256T, B.KERNEL_SKINNY_SPLITK, B.KERNEL_SKINNY_QUAD]:
            if planes == 2 and kid in (B.KERNEL_MFMA_256x256, B.KERNEL_MFMA_256x128):
                continue
            if planes == 1 and kid == B.KERNEL_MFMA_128x256T:
                continue
            if kid in (B.KERNEL_MFMA_128x64, B.KERNEL_MFMA_64x64) and M > 64:
                continue
            if kid >= B.KERNEL_SKINNY_STREAM and -(-M // 32) * -(-N // 32) * batch > 8192:
                continue
            v = B.force_kernel(kid)
            fn = lambda i: lk.bgemm_packed_forward(wps[i % copies], xp, mode, torch.int32, 8, v, out=out)
            try:
                fn(0)
            except ValueError:
                continue
            if ref is None:
                ref = out.clone()
            elif not torch.equal(out, ref):
                res["mismatch"] = KERNEL_NAMES[kid]
            res["us_cold"][KERNEL_NAMES[kid]] = round(1e3 * time_gpu_graph(fn, copies, 2, max(2, steps // copies)), 2)
            if warm:
                res["us_warm"][KERNEL_NAMES[kid]] = round(1e3 * time_gpu_graph(lambda i: fn(0), 8, 2, max(2, steps // 8)), 2)
        res["fastest_cold"] = min(res["us_cold"], key=res["us_cold"].get)
        res["auto_vs_fastest_cold"] = round(res["us_cold"][res["auto"]] / res["us_cold"][res["fastest_cold"]], 3) if res["auto"] in res["us_cold"] else None
        rows.append(res)
        if shapes is None:
            log(json.dumps(res))
        del pool, wps, xp, out
    return rows


# ---------------------------------------------------------------- sections
def section_decode(cold):
    rows = bench_decode(cold, "C4", 11008, 4096, (1, 4, 16))
    for N in (1, 4, 16):
        rows.append(bench_decode_batched(N))
        log_row(rows[-1])
    # the GEMMs a Llama-7B decode step issues against one set of activations: QKV fused, gate + up fused, down
    rows += bench_decode(cold, "QKV", 12288, 4096, (1, 4, 16))
    rows += bench_decode(cold, "gate+up", 22016, 4096, (1, 4, 16))
    rows += bench_decode(cold, "down", 4096, 11008, (1, 4, 16))
    for N in (1, 4):
        rows.append(bench_decode_from_fp16(N))
        log_row(rows[-1])
    rows += bench_chain(cold)
    return rows


def bench_prefill(steps=20, warmup=5):
    """Binary weights x a batch of ternary rows (a prefill step, or a batch of decode steps).  On the signed tile (fp4 operands
    that carry the ternary values themselves) the matrix cores do the 2*M*N*K operations that `tops` counts; on the two-plane
    kernels the activations' bit planes are two products against one expansion of the weights, 4*M*N*K of matrix-core work;
    `frac` is the matrix-core work against the fp4 peak either way."""
    import torch
    import lowbit_kernel as lk
    dev = torch.device("cuda:0")
    rows = []
    for name, M, N, K in (("gate+up", 22016, 2048, 4096), ("down", 4096, 2048, 11008), ("square", 8192, 8192, 8192)):
        w16, x16 = pm1_f16((M, K), 6001, dev), ternary_f16((N, K), 6002, dev)
        wp, xt = lk.pack_sign(w16), lk.pack_ternary(x16)
        out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
        fn = lambda i: lk.bgemm_packed_forward(wp, xt, lk.MODE_BWTA, torch.int32, 1, 0, out=out)
        for i in range(50):
            fn(i)
        ms = time_gpu(fn, warmup, steps)
        ok = check_sampled(out[0], w16, x16)
        r = row("BWTA %s W[%d,%d] x %d rows" % (name, M, K, N), ms, 2.0 * M * N * K,
                M * K / 8 + 2 * N * K / 8 + 4.0 * M * N, ok, kernel_of(wp, xt, lk.MODE_BWTA), "mfma")
        r["frac"] = round((1 if r["k"] == "m128x256t" else 2) * r["tops"] / FP4_MFMA_PEAK_TOPS, 4)
        rows.append(r)
        log_row(r)
        del w16, x16, wp, xt, out
    # batches of decode steps: a few hundred ternary rows against one layer, weights rotating through HBM as a model's do
    for name, M, N, K in (("up", 11008, 128, 4096), ("gate+up", 22016, 128, 4096), ("down", 4096, 128, 11008), ("up", 11008, 512, 4096)):
        copies = max(2, min(40, int(300e6 // (M * K // 8))))
        w16, x16 = pm1_f16((M, K), 6003, dev), ternary_f16((N, K), 6004, dev)
        xt = lk.pack_ternary(x16)
        wps = [lk.pack_sign(w16 if c == 0 else pm1_f16((M, K), 6100 + c, dev)) for c in range(copies)]
        out = torch.empty((1, N, M), dtype=torch.int32, device=dev)
        fn = lambda i: lk.bgemm_packed_forward(wps[i % copies], xt, lk.MODE_BWTA, torch.int32, 1, 0, out=out)
        fn(0)
        ok = check_sampled(out[0], w16, x16)
        ms = min(time_gpu_graph(fn, copies, 2, 5) for _ in range(3))
        r = row("BWTA %s W[%d,%d] x %d rows cold" % (name, M, K, N), ms, 2.0 * M * N * K,
                M * K / 8 + 2 * N * K / 8 + 4.0 * M * N, ok, kernel_of(wps[0], xt, lk.MODE_BWTA), "mfma")
        r["frac"] = round((1 if r["k"] == "m128x256t" else 2) * r["tops"] / FP4_MFMA_PEAK_TOPS, 4)
        r["frac_hbm"] = round(r["gbs"] / HBM_PEAK_GBS, 4)
        rows.append(r)
        log_row(r)
        del w16, x16, wps, xt, out
    return rows


def all_configs(cold):
    rows = [bench_c2()]
    log_row(rows[-1])
    rows.append(bench_c3())
    log_row(rows[-1])
    rows.append(bench_qk())
    log_row(rows[-1])
    rows += section_decode(cold)
    rows += bench_sweep()
    rows += bench_prefill()
    rows.append(bench_c5_dropin(20, 3))
    log_row(rows[-1])
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--headline-only", action="store_true", help="time the 8192^3 launch only (profiling runs)")
    ap.add_argument("--only", choices=["c2", "c3", "c4", "chain", "sweep", "prefill", "floor", "peak", "thresholds"],
                    help="time just that section and print it (for profiling and for re-deriving the dispatch thresholds)")
    ap.add_argument("--variant", type=int, default=0, help="0 auto, 1 VALU, 2 MFMA int8, 3 MFMA fp4")
    ap.add_argument("--split-k", type=int, default=1,
                    help="splitK of the headline launch: the most K ranges a tile may be computed in (same bits for any value)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--pre-roll", type=int, default=PRE_ROLL,
                    help="untimed launches of the headline GEMM before the warm-up steps (clock ramp)")
    ap.add_argument("--counted", action="store_true",
                    help="time the headline on operands that bring their row popcounts (bgemm_packed_forward_counted)")
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
        del src, dst
    if args.only:
        cold = ColdRead() if args.only in ("c4", "chain", "floor", "peak") else None
        res = {"chain": lambda: bench_chain(cold), "c2": lambda: [bench_c2()], "c3": lambda: [bench_c3(), bench_qk()], "c4": lambda: section_decode(cold), "prefill": bench_prefill,
               "sweep": bench_sweep, "floor": lambda: bench_floor(cold), "peak": lambda: bench_mfma_peak(cold),
               "thresholds": bench_thresholds}[args.only]()
        out = {args.only: res}
        if args.only == "thresholds":
            out["dispatch"] = dispatch_summary(res)
        print(json.dumps(out), flush=True)
        return

    extra = floor = peak_measured = dispatch = None
    if not args.headline_only:
        cold = ColdRead()
        floor = bench_floor(cold)
        log("floor done")
        peak_measured = bench_mfma_peak(cold)
        log("mfma peak done")
        extra = all_configs(cold)
        dispatch = dispatch_summary(bench_thresholds(40, DISPATCH_SHAPES, warm=False))
        log("dispatch done")
        del cold
        torch.cuda.empty_cache()

    c5, (w16, x16) = bench_c5(args.steps, args.warmup, splitK=args.split_k, variant=args.variant, pre_roll=args.pre_roll,
                                  counted=args.counted)
    log("C5: %.5f ms" % c5["ms"])
    cpu = None if args.no_cpu else cpu_baseline_c5(w16, x16)
    del w16, x16
    fp4 = args.variant in (0, 3)
    peak = FP4_MFMA_PEAK_TOPS if fp4 else INT8_MFMA_PEAK_TOPS
    ok = bool(c5["bit_exact"]) and all(r["ok"] for r in (extra or []))

    roofline = {"bound": "mfma", "achieved": c5["tops"], "peak": peak, "unit": "TFLOP/s", "frac": c5["tops"] / peak,
                # HBM bytes per launch of this kernel from the FETCH_SIZE / WRITE_SIZE counter runs, as the tracked
                # profile summary of the same command states them (null when it holds no such line)
                "traffic": measured_traffic_bytes() if fp4 else None}
    if peak_measured:
        mp = peak_measured["fp4_tops" if fp4 else "int8_tops"]
        roofline["peak_measured"] = mp
        roofline["frac_of_measured_peak"] = round(c5["tops"] / mp, 4)
    line = {
        "metric": "effective binary TOPS (2*M*N*K/t), bit-exact int32",
        "value": c5["tops"] if c5["bit_exact"] else None, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": c5["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp4" if fp4 else "int8",
        "data": "synthetic",
        "config": {"workload": "BASELINE.json config 5: BGEMM M=N=K=8192, {-1,+1}x{-1,+1}, weights and activations "
                               "prepacked (tiled bit layout), int32 output, splitK=%d" % args.split_k,
                   "kernel": c5["kernel"],
                   "arithmetic": ("1-bit operands expanded in registers to E2M1 (fp4) MFMA operands, fp32 accumulation "
                                  "of exact integers" if fp4 else
                                  "1-bit operands expanded in registers to int8 MFMA operands, int32 accumulation"),
                   "op_count": "2*M*N*K binary multiply-accumulate ops per launch, the convention of the reference's "
                               "drivers (lowbit_kernel/csrc/benchmark.cu:291 prints it as TFLOPs)",
                   "pre_roll": "%d untimed launches of the same GEMM before the %d warm-up steps (clock ramp; the reference's "
                               "drivers warm up with 100 launches and time 10 000, lowbit_kernel/csrc/kernel_test.h:10-11)" % (args.pre_roll, args.warmup),
                   "timing": "median of 5 repeats of %d launches; ms_per_step min %.5f max %.5f" % (args.steps, c5["ms_min"], c5["ms_max"]),
                   "bit_exact_sampled": c5["bit_exact"], "hbm_gbs_algorithmic": c5["gbs"],
                   "activation_pack_ms": c5["act_pack_ms"], "activation_popcount_ms": c5["act_popcount_ms"],
                   "ms_per_step_with_row_popcounts_prepacked": c5["ms_counted"],
                   "frac_of_int8_mfma_peak": c5["tops"] / INT8_MFMA_PEAK_TOPS},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if extra is not None:
        # configuration 4's target (>= 70 % of HBM bandwidth) where a driver that keeps only the head of the line sees it
        line["config"]["c4_single_launch_frac_hbm"] = {r["id"].split(" N=")[1].split(" ")[0]: r["frac"] for r in extra if r["id"].startswith("C4 W[11008,4096] N=")}
        line["config"]["c4_chain_frac_hbm"] = {r["id"].split(" N=")[1].split(",")[0]: r["frac"] for r in extra if r["id"].startswith("C4 chain")}
        line["config"]["c4_chain_us_per_layer"] = {r["id"].split(" N=")[1].split(",")[0]: r["us"] for r in extra if r["id"].startswith("C4 chain")}
        line["all_configs"] = extra
        line["dispatch"] = dispatch
        line["floor"] = floor
        line["mfma_peak_measured"] = peak_measured
    print(json.dumps(line), flush=True)
    if not ok:
        sys.exit("bench.py: a timed configuration did NOT match its closed form bit for bit (see bit_exact in the line above)")


if __name__ == "__main__":
    main()
