"""Benchmark of the TBIK hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--table] [--no-ceiling]

A step is one tree-ordered matmul (`matmul_tp_persistent`) over the headline batch: X[2048,12288]
(SiLU-gated synthetic activations, bf16) times the down_proj weight W[4096,12288] (N(0,0.02), bf16,
stored [N,K] as nn.Linear does), inputs resident in HBM before the timed region.  Prints ONE JSON line.

Order of a run: the step is timed twice -- right after the host-side set-up (`value_after_idle`: W warm-up steps, K
timed steps, nothing else) and after `--settle-ms` of the same step run back to back (`value`: the settled rate);
then the context figures (the vendor library and this library's plain mm on the same operands, `context.ceiling`: what
the chip sustains on MFMAs alone and on a one-pass read, with the board power under each of these loops, and `context.table`:
the other shapes of the workload family, each with its algorithmic flops or bytes and the fraction of the stated
peak); the CPU baseline and the full-size parity check against it come last, so that they do not sit between the
set-up and the timed region.  `--table` prints the long form of the table to stderr as well.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

M_, K_, N_ = 2048, 12288, 4096
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_tree_deep_headline_counters.txt")


def traffic_from_profile():
    """HBM bytes one headline launch moves, read from the tracked rocprofv3 counter summary (FETCH_SIZE and WRITE_SIZE
    passes, each scaled by what the same counter reads for a plain copy of known size).  Counters need the profiler,
    so this is a figure of that profile, not of this run; None when the summary is missing."""
    import re
    try:
        with open(TRAFFIC_PROFILE) as f:
            m = re.search(r"traffic\s*=\s*([0-9.]+)\s*MB per launch", f.read())
        return float(m.group(1)) * 1e6 if m else None
    except OSError:
        return None


def hip_time_ms(fn, steps, warmup, settle_ms=0.0):
    """Average milliseconds per call, from HIP events on the stream the kernels are launched on.

    settle_ms > 0: the same call is first repeated for about that long.  After an idle period the chip's power
    management takes some 25 ms of continuous load to settle: the first ten headline launches run at 225 us, the next
    ten at 270-280 us, and only after about a hundred the rate is steady.  A handful of steps taken right after the
    host-side set-up measures that transient, not the kernel."""
    import torch
    if settle_ms > 0:
        t_end = time.perf_counter() + settle_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(8):
                fn()
            torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    s.record()
    for _ in range(steps):
        fn()
    e.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return s.elapsed_time(e) / steps, wall_ms / steps


def graph_time_ms(fn, calls, replays, settle_ms=0.0):
    """Average milliseconds per call with the host out of the way: `calls` calls are recorded into one HIP graph and the
    graph is replayed, so the kernels run back to back however long the Python operator around them takes (a decode
    kernel of 20 us sits behind 15-40 us of host work per call when launched one by one).  None where the calls cannot
    be recorded (an operator that synchronises); the caller then keeps its figure from one-by-one launches."""
    import torch
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(calls):
                fn()
    except Exception:                                   # noqa: BLE001 -- any refusal to record means "measure eagerly"
        torch.cuda.synchronize()
        return None
    t_end = time.perf_counter() + settle_ms * 1e-3
    g.replay()
    while time.perf_counter() < t_end:
        g.replay()
        torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(replays):
        g.replay()
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / (replays * calls)
    del g
    return ms


class PowerSampler:
    """Board power while a loop runs, read from the driver's hwmon file (microwatts, `power1_input` or `power1_average`
    of the first GPU) every 20 ms on a thread of its own; `mean_w()` drops the first quarter of the samples (ramp-up).
    None where the file does not exist."""

    def __init__(self):
        import glob
        import threading
        paths = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") +
                       glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
        self.path = paths[0] if paths else None
        self.samples, self._stop = [], False
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        while not self._stop:
            try:
                with open(self.path) as f:
                    self.samples.append(int(f.read().strip()) * 1e-6)
            except (OSError, ValueError):
                pass
            time.sleep(0.02)

    def __enter__(self):
        if self.path:
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self.path:
            self._thread.join()

    def mean_w(self):
        s = self.samples[len(self.samples) // 4:]
        return round(sum(s) / len(s), 1) if s else None


def power_of(fn, seconds=1.5):
    """(mean board power in W, microseconds per call) of `fn` run back to back for about `seconds`."""
    import torch
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    n, t0 = 0, time.perf_counter()
    with PowerSampler() as ps:
        while time.perf_counter() - t0 < seconds:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
            n += 50
        dt = time.perf_counter() - t0
    return ps.mean_w(), round(dt / n * 1e6, 1)


def _median_time(fn, budget_s, max_runs, min_runs=3):
    ts, spent = [], 0.0
    while (spent < budget_s or len(ts) < min_runs) and len(ts) < max_runs:
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
        spent += ts[-1]
    return statistics.median(ts), len(ts), spent


def cpu_baseline(budget_s=9.0, max_runs=30):
    """The CPU oracle (PyTorch restatement of the reference's tree order, the reference has no CPU path of its own) on
    the whole headline workload, all host threads: one warm-up, then repeated for about `budget_s` seconds, median.
    Beside it, bounded to a few seconds in all: the oracle on configuration 1 (A[256,4096] x W[4096,4096]) as a whole
    and cut into 2 / 4 / 8 shards with the shard tree, and the CPU library's plain bf16 `torch.matmul` on both shapes
    (order not fixed, no tree) for context.  Returns (record, oracle product of the headline workload)."""
    import torch
    from oracle import tbik_oracle as O
    X = O.silu_gated_bf16((M_, K_), 0)
    W = O.gaussian_bf16((N_, K_), 0.02, 1)
    Wt = W.t()
    O.matmul_tree(X[:256], Wt)
    t, n, spent = _median_time(lambda: O.matmul_tree(X, Wt), budget_s, max_runs)
    rec = {"value": round(2.0 * M_ * N_ * K_ / t / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
           "kind": "port",
           "sample": f"oracle matmul_tree on the full X[{M_},{K_}] and W[{N_},{K_}] of the headline workload, "
                     f"{n} runs in {spent:.1f} s, median {t:.2f} s each"}
    want = O.matmul_tree(X, Wt)
    A1 = O.gaussian_bf16((256, 4096), 1.0, 0)
    W1 = O.gaussian_bf16((4096, 4096), 0.02, 1).t()
    fl1 = 2.0 * 256 * 4096 * 4096
    c1 = {}
    for p in (1, 2, 4, 8):
        tp, _, _ = _median_time(lambda p=p: O.simulated_tp_matmul(A1, W1, p), 0.5, 10)
        c1[f"tp{p}_ms"] = round(tp * 1e3, 2)
    rec["config1_oracle_A256x4096_W4096x4096"] = dict(c1, GFLOPs_tp1=round(fl1 / (c1["tp1_ms"] * 1e-3) / 1e9, 1),
                                                      note="oracle per shard + shard tree, median")
    tm1, _, _ = _median_time(lambda: torch.matmul(A1, W1), 0.5, 10)
    tmh, _, _ = _median_time(lambda: torch.matmul(X, Wt), 2.0, 5, min_runs=2)
    rec["plain_cpu_torch_matmul_bf16"] = {"config1_ms": round(tm1 * 1e3, 2), "config1_GFLOPs": round(fl1 / tm1 / 1e9, 1),
                                          "headline_s": round(tmh, 3),
                                          "headline_TFLOPs": round(2.0 * M_ * N_ * K_ / tmh / 1e12, 4),
                                          "note": "CPU library matmul, bf16, order not fixed, no tree"}
    return rec, want


def ceiling(settle_ms, others=()):
    """What the chip sustains on bf16 MFMAs alone (register operands, one work-group per CU, 2 waves per SIMD: the wave
    shape of the tree kernel) for constant and for random operands, and on a one-pass read of 1 GiB (cold in the 256 MB
    memory-side cache).  Steady-state figures (same load phase as the headline).  `power_W`: the board power while each
    of these loops, and each (name, fn) of `others`, runs back to back for 1.5 s (the cap of this board is what
    `rocm-smi --showmaxpower` prints, 1400 W on MI355X): a kernel that sits at the cap is bound by energy per launch,
    not by a pipe."""
    import ctypes
    import torch
    from llm_reproducibility_amd import _lib
    from llm_reproducibility_amd.build import MEASURE_LIB_PATH
    if not os.path.exists(MEASURE_LIB_PATH):
        raise RuntimeError(f"{MEASURE_LIB_PATH} is missing: build it with `python -m llm_reproducibility_amd.build`")
    L = ctypes.CDLL(MEASURE_LIB_PATH)                      # the machine probes live outside the product library
    vp = ctypes.c_void_p
    L.tbik_probe_mfma_bf16.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp]
    L.tbik_probe_read.argtypes = [vp, ctypes.c_int64, vp, ctypes.c_int, vp]
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.empty(cus * 512, device=dev, dtype=torch.float32)
    res = {"work_groups": cus}
    iters = 800
    g = torch.Generator().manual_seed(0)
    ops_rand = torch.randn(32768, generator=g)
    ops_rand[:16384] *= 0.02                      # a operands like the weights, b operands like the activations
    for name, src in (("constant", torch.full((32768,), 1.0)), ("random", ops_rand)):
        buf = src.to(torch.bfloat16).to(dev)

        def run():
            _lib.check(L.tbik_probe_mfma_bf16(buf.data_ptr(), out.data_ptr(), cus, 8, -iters, stream), "tbik_probe_mfma_bf16")
        ms, _ = hip_time_ms(run, 30, 5, settle_ms)
        flop = float(cus) * 8 * iters * 16 * 16384
        res[f"mfma_only_{name}_operands_TFLOPs"] = round(flop / (ms * 1e-3) / 1e12, 1)
    nbytes = 1 << 30
    big = torch.empty(nbytes // 4, device=dev, dtype=torch.int32).random_()
    sink = torch.empty(cus * 16 * 256, device=dev, dtype=torch.int32)

    def read():
        _lib.check(L.tbik_probe_read(big.data_ptr(), nbytes, sink.data_ptr(), cus * 16, stream), "tbik_probe_read")
    ms, _ = hip_time_ms(read, 20, 3, settle_ms)
    res["one_pass_read_1GiB_GBps"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
    power = {}
    for name, src in (("mfma_only_constant", torch.full((32768,), 1.0)), ("mfma_only_random", ops_rand)):
        buf = src.to(torch.bfloat16).to(dev)
        power[name] = power_of(lambda: L.tbik_probe_mfma_bf16(buf.data_ptr(), out.data_ptr(), cus, 8, -iters, stream))
    for name, fn in others:
        power[name] = power_of(fn)
    time.sleep(2.0)
    with PowerSampler() as ps:
        time.sleep(1.0)
    power["idle"] = (ps.mean_w(), None)
    res["power_W_and_us_per_call"] = power
    res["note"] = ("MFMA-only loop on register operands and a plain grid-stride read: ceilings of any bf16 matmul kernel "
                   "on such data and of any one-pass kernel, measured in this run")
    return res


GRAPH_BELOW_MS = 0.15


def table(steps, warmup, hot=False, settle_ms=20.0, full=False, only=None, graphs=True):
    """Per-shape figures, each after `settle_ms` of the same call run back to back (the settled rate, as for the
    headline).  Unless `hot`, every case cycles through enough distinct input sets (more than 768 MB in all) that
    nothing it reads is still in the 256 MB memory-side cache from the previous call: the GB/s are HBM figures, as in
    a model whose every layer has its own weights.  With `graphs`, a case whose call takes less than 150 us is timed as
    replays of a HIP graph of about 32 such calls (`graph_time_ms`): the figure is then the kernels' own back-to-back time, not
    the Python operator's host time, which is longer than many of these kernels.

    Returns a list of rows {case, us, flop, bytes, TFLOPs, GBps, bound, frac}: `flop` and `bytes` are the algorithmic
    work of one call -- 2*M*N*K and 2*(M*K + K*N + M*N) for a matmul, the formulas of the reference's launch metadata
    (src/tbik/tree_based_matmul.py:23-24, src/bio/batch_invariant_ops.py:13-29); (p+1)*M*N*2 for the shard combine;
    rows*hidden*4 + hidden*2 for RMSNorm; 8 B per logit for the fp32 log_softmax; 4 B per element for the mean; K, V, q
    and the output once for attention -- `bound` names the roofline that applies to the case ("mfma": 2.5 PFLOP/s
    dense bf16, "hbm": 8 TB/s) and `frac` is the achieved share of it.  `full` adds the long list (vendor-library rows for
    context, the mm shapes of the decoder, prefill attention)."""
    import torch
    from llm_reproducibility_amd import ops
    from llm_reproducibility_amd.bio import batch_invariant_ops as bio
    from llm_reproducibility_amd.tbik import choose_leaf_k, matmul_tp_persistent, tree_combine
    dev = torch.device("cuda:0")
    rows = []

    def cycling(make, nbytes, fn):
        n = 1 if (hot or nbytes >= 768e6) else min(16, int(768e6 // nbytes) + 1)
        sets = [make() for _ in range(n)]
        state = [0]

        def call():
            args = sets[state[0] % n]
            state[0] += 1
            return fn(*args)
        return call, n

    def add(name, make, fn, flop, nbytes, bound, nsteps=None, short=None):
        """`short`: the key of the row in the JSON line; rows without one appear in the long form only."""
        if (short is None and not full) or (only and only not in name):
            return
        call, nsets = cycling(make, nbytes, fn)
        ms, _ = hip_time_ms(call, nsteps or steps, warmup, settle_ms)
        how = "eager"
        if graphs and ms < GRAPH_BELOW_MS:
            per_graph = nsets * max(1, 32 // nsets)      # whole turns through the input sets: every replay stays cold
            gms = graph_time_ms(call, per_graph, 3, settle_ms)
            if gms is not None:
                ms, how = gms, "graph"
        tf, gbs = flop / ms / 1e9, nbytes / ms / 1e6
        frac = tf / PEAK_BF16_TFLOPS if bound == "mfma" else gbs / PEAK_HBM_GBS
        rows.append({"case": name, "short": short, "us": round(ms * 1e3, 1), "flop": flop, "bytes": nbytes,
                     "TFLOPs": round(tf, 1), "GBps": round(gbs, 1), "bound": bound, "frac": round(frac, 4), "timed": how})

    def operands(M, K, N):
        return lambda: (torch.randn((M, K), device=dev).to(torch.bfloat16), (torch.randn((N, K), device=dev) * 0.02).to(torch.bfloat16))

    def gemm_row(name, M, K, N, leaf, fn=None, short=None):
        fl, by = 2.0 * M * N * K, 2.0 * (M * K + K * N + M * N)
        f = fn or (lambda X, W: matmul_tp_persistent(X, W.t(), leaf_k=leaf))
        # decode-sized batches stream the weights once (memory bound); from a few hundred rows on the matrix cores bound
        add(name, operands(M, K, N), f, fl, by, "hbm" if fl / by < 312 else "mfma", short=short)

    def library_row(M, K, N):
        # context only: the vendor library GEMM behind torch.matmul (no tree, reduction order not fixed) on like operands
        gemm_row(f"  [torch.matmul, not invariant] M={M} K={K} N={N}", M, K, N, 0, lambda X, W: torch.matmul(X, W.t()))

    for M in (1, 16, 128, 2048):
        gemm_row(f"tree matmul down_proj 8B M={M} K=12288 N=4096", M, 12288, 4096, 256, short=None if M == 2048 else f"tree dn8B M={M}")
    for M in (1, 128, 2048):
        library_row(M, 12288, 4096)
    # the same product with B handed over as a row-major [K,N] matrix (a plain `x @ B`): consumed in place by the tiled
    # kernels up to 1023 rows, repacked into the native [N,K] layout (inside the timed call) from 1024 rows on
    for M in (128, 2048):
        gemm_row(f"tree matmul down_proj 8B M={M}, B row-major [K,N] ({'repacked per call' if M >= 1024 else 'in place'})", M, 12288,
                 4096, 256, lambda X, W: matmul_tp_persistent(X, W.view(W.shape[1], W.shape[0])),
                 short=f"tree dn8B rowmajorB M={M}" if M == 2048 else None)
    for p in (2, 4, 8):
        gemm_row(f"tree matmul shard TP={p} M=2048 K={12288 // p} N=4096", 2048, 12288 // p, 4096, 256)
    for M in (1, 64, 512, 4096):
        gemm_row(f"tree matmul o_proj 32B M={M} K=8192 N=5120", M, 8192, 5120, 256, short=f"tree o32B M={M}")
    for M in (1, 64, 512, 4096):
        gemm_row(f"tree matmul down_proj 32B M={M} K=25600 N=5120 leaf128", M, 25600, 5120, choose_leaf_k(25600),
                 short=f"tree dn32B/128 M={M}")
    library_row(4096, 8192, 5120)
    library_row(4096, 25600, 5120)
    library_row(2048, 4096, 24576)
    library_row(8192, 4096, 24576)
    in_json = {("qkv", 1), ("qkv", 2048), ("gate_up", 1), ("gate_up", 2048), ("lm_head", 1), ("lm_head", 128)}
    for name, M, K, N in (("qkv", 1, 4096, 6144), ("qkv", 32, 4096, 6144), ("qkv", 128, 4096, 6144), ("qkv", 2048, 4096, 6144),
                          ("gate_up", 1, 4096, 24576), ("gate_up", 32, 4096, 24576), ("gate_up", 128, 4096, 24576),
                          ("gate_up", 2048, 4096, 24576), ("gate_up", 8192, 4096, 24576),
                          ("lm_head", 1, 4096, 151936), ("lm_head", 32, 4096, 151936), ("lm_head", 128, 4096, 151936)):
        gemm_row(f"batch-invariant mm {name} 8B M={M} K={K} N={N}", M, K, N, 0, lambda X, W: bio.matmul_persistent(X, W.t()),
                 short=f"mm {name} M={M}" if (name, M) in in_json else None)
    for p in (2, 4, 8):
        by = (p + 1) * 2048 * 4096 * 2
        add(f"tree_combine p={p} [2048,4096]", lambda p=p: ([torch.randn((2048, 4096), device=dev).to(torch.bfloat16) for _ in range(p)],),
            tree_combine, 0.0, by, "hbm", short=f"comb p={p}")
    w = torch.ones(4096, device=dev, dtype=torch.bfloat16)
    for r in (1, 7, 256, 4096):
        add(f"rmsnorm rows={r} hidden=4096", lambda r=r: (torch.randn((r, 4096), device=dev).to(torch.bfloat16),),
            lambda x: bio.rms_norm(x, w, 1e-6), 0.0, r * 4096 * 4 + 8192, "hbm", short=f"rms r={r}")
    for r in (1, 7, 256, 4096):
        add(f"log_softmax fp32 rows={r} vocab=151936 (8 B/elem)", lambda r=r: (torch.randn((r, 151936), device=dev),),
            bio.log_softmax, 0.0, r * 151936 * 8, "hbm", max(steps // 4, 3), short=f"lsm r={r}")
    for r in (256, 4096):
        add(f"log_softmax bf16 in/out rows={r} vocab=151936 (4 B/elem)",
            lambda r=r: (torch.randn((r, 151936), device=dev).to(torch.bfloat16),), bio.log_softmax, 0.0, r * 151936 * 4, "hbm",
            max(steps // 4, 3))
    for r in (1, 7, 256, 4096):
        add(f"mean rows={r} n=4096", lambda r=r: (torch.randn((r, 4096), device=dev),), lambda x: bio.mean_dim(x, -1), 0.0,
            r * 4096 * 4, "hbm", short=f"mean r={r}")
    for r in (1, 256, 4096):
        add(f"silu_mul rows={r} inter=12288 (6 B/elem)", lambda r=r: (torch.randn((r, 2 * 12288), device=dev).to(torch.bfloat16),),
            ops.bi_silu_mul, 0.0, r * 12288 * 6, "hbm", short="silu_mul r=4096" if r == 4096 else None)
    # decode-sized compositions: the producer inside the consuming matmul (one launch) against the two launches it
    # stands for (same bits); algorithmic bytes = the weights once
    for M in (1, 4):
        def make_norm(M=M):
            return (torch.randn((M, 4096), device=dev).to(torch.bfloat16), torch.randn((M, 4096), device=dev).to(torch.bfloat16),
                    (torch.randn((24576, 4096), device=dev) * 0.02).to(torch.bfloat16))
        by = 2.0 * 24576 * 4096
        add(f"RMSNorm(+residual) inside the mm, gate_up 8B M={M} (one launch)", make_norm,
            lambda x, r, W: ops.rmsnorm_gemm(x, w, 1e-6, r, W.t()), 2.0 * M * 24576 * 4096, by, "hbm", short=f"norm+mm gate_up M={M}")
        add(f"  the same as two launches (rms_norm, then mm) M={M}", make_norm,
            lambda x, r, W: bio.matmul_persistent(bio.rms_norm(x, w, 1e-6, residual=r)[0], W.t()), 2.0 * M * 24576 * 4096, by, "hbm",
            short=f"norm, mm gate_up M={M}")
    # (every work-group of the one-launch kernel forms all M * K activations itself: it takes up to 16384 of them, so one row
    # of the whole layer or four rows of a TP = 4 shard)
    for M, K, tag in ((1, 12288, "dn8B"), (4, 3072, "dn8B/TP4")):
        def make_gated(M=M, K=K):
            return (torch.randn((M, 2 * K), device=dev).to(torch.bfloat16), (torch.randn((4096, K), device=dev) * 0.02).to(torch.bfloat16))
        by = 2.0 * 4096 * K
        add(f"SiLU*up inside the tree matmul, down_proj 8B M={M} K={K} (one launch)", make_gated,
            lambda gu, W, K=K: ops.gemm_tree_silu_mul(gu[:, :K], gu[:, K:], W.t(), None, 256), 2.0 * M * 4096 * K, by, "hbm",
            short=f"silu+tree {tag} M={M}")
        add(f"  the same as two launches (silu_mul, then tree matmul) M={M} K={K}", make_gated,
            lambda gu, W: matmul_tp_persistent(ops.bi_silu_mul(gu), W.t()), 2.0 * M * 4096 * K, by, "hbm",
            short=f"silu, tree {tag} M={M}")
    # from five rows on the consumer runs inside the producer: the add-RMSNorm behind a row-split layer in the launch that
    # combines the layer's K shards, against the matmul followed by the norm (same bits)
    for M in (32, 128):
        def make_tn(M=M):
            return (torch.randn((M, 12288), device=dev).to(torch.bfloat16), torch.randn((M, 4096), device=dev).to(torch.bfloat16),
                    (torch.randn((4096, 12288), device=dev) * 0.02).to(torch.bfloat16))
        by = 2.0 * 4096 * 12288
        add(f"add-RMSNorm inside the shard combine of the tree matmul, down_proj 8B M={M}", make_tn,
            lambda x, r, W: ops.gemm_tree_add_rmsnorm(x, W.t(), None, 256, r, w, 1e-6), 2.0 * M * 4096 * 12288, by, "hbm",
            short=f"tree+norm dn8B M={M}")
        add(f"  the same as separate calls (tree matmul, then add-RMSNorm) M={M}", make_tn,
            lambda x, r, W: bio.rms_norm(matmul_tp_persistent(x, W.t()), w, 1e-6, residual=r), 2.0 * M * 4096 * 12288, by, "hbm",
            short=f"tree, norm dn8B M={M}")
    # ... and SiLU*up inside the merged gate/up projection (5 .. 64 rows), against the mm followed by the activation kernel
    def make_gu():
        return (torch.randn((32, 4096), device=dev).to(torch.bfloat16), (torch.randn((24576, 4096), device=dev) * 0.02).to(torch.bfloat16))
    add("SiLU*up inside the merged gate/up projection 8B M=32 (one launch)", make_gu, lambda x, W: ops.gemm_silu_mul(x, W),
        2.0 * 32 * 24576 * 4096, 2.0 * 24576 * 4096, "hbm", short="mm+silu gate_up M=32")
    add("  the same as two calls (mm, then silu_mul) M=32", make_gu, lambda x, W: ops.bi_silu_mul(bio.matmul_persistent(x, W.t())),
        2.0 * 32 * 24576 * 4096, 2.0 * 24576 * 4096, "hbm", short="mm, silu gate_up M=32")
    # fixed-order attention (Qwen3-8B heads: 32 query, 8 key/value, head_dim 128)
    Hq, Hkv, D = 32, 8, 128

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=dev)
    for name, short, B, qlen, ctx in (("decode 128 seqs ctx 768", "attn dec 128x768", 128, 1, 768),
                                      ("decode 8 seqs ctx 4096", "attn dec 8x4096", 8, 1, 4096),
                                      ("prefill 8 x 512", "attn pre 8x512", 8, 512, 512),
                                      ("prefill 1 x 4096", "attn pre 1x4096", 1, 4096, 4096)):
        L = ((ctx + 31) // 32) * 32
        qs, ql, cl = i32([b * qlen for b in range(B)]), i32([qlen] * B), i32([ctx] * B)
        pairs = B * Hq * (qlen * (2 * ctx - qlen + 1) // 2)          # causal (query, key) pairs
        byts = 2.0 * (2 * B * Hkv * ctx * D + 2 * B * qlen * Hq * D)   # K, V once; q and out

        def make(B=B, qlen=qlen, L=L):
            return (torch.randn((B * qlen, Hq, D), device=dev).to(torch.bfloat16),
                    torch.randn((B, Hkv, L, D), device=dev).to(torch.bfloat16),
                    torch.randn((B, Hkv, D, L), device=dev).to(torch.bfloat16))
        add(f"attention {name}", make, lambda q, kc, vt: ops.bi_attention_bf16(q, kc, vt, qs, ql, cl, qlen, D ** -0.5),
            4.0 * pairs * D, byts, "hbm" if qlen == 1 else "mfma", max(steps // 2, 3), short=short)
    return rows


def print_table(rows, hot):
    print("inputs " + ("reused by every call (hot in the memory-side cache)" if hot else
                       "cycled through more than 768 MB of distinct buffers (cold in the 256 MB memory-side cache)"), file=sys.stderr)
    print(f"{'case':66s} {'us':>10s} {'TFLOP/s':>9s} {'%MFMA':>6s} {'GB/s':>9s} {'%HBM':>6s} {'bound':>6s} {'timed':>6s}", file=sys.stderr)
    for r in rows:
        print(f"{r['case']:66s} {r['us']:10.1f} {r['TFLOPs']:9.1f} {100 * r['TFLOPs'] / PEAK_BF16_TFLOPS:6.1f} "
              f"{r['GBps']:9.1f} {100 * r['GBps'] / PEAK_HBM_GBS:6.1f} {r['bound']:>6s} {r['timed']:>6s}", file=sys.stderr)


def decode_step(layers=12, prompt_len=512, batches=(1, 32, 128)):
    """Wall time of a greedy decode step of the Qwen3-8B-architecture decoder (random weights, `layers` of its 36 layers,
    TP = 1), per layer: two generate() calls that differ only in the number of new tokens, so the prefill cancels.
    lm_head, the token choice and the embedding lookup run once per step and are in the figure (spread over `layers`)."""
    import torch
    from llm_reproducibility_amd.decoder import DecoderConfig, Qwen3Decoder
    cfg = DecoderConfig(num_layers=layers)
    t0 = time.perf_counter()
    model = Qwen3Decoder(cfg, tp_size=1, seed=0, init_on_device=True)
    g = torch.Generator().manual_seed(1)
    prompts = torch.randint(0, cfg.vocab_size, (max(batches), prompt_len), generator=g).tolist()
    out = {}
    short, long_ = 9, 41

    def run(bs, n):
        torch.cuda.synchronize()
        t = time.perf_counter()
        model.generate(prompts[:bs], n)
        torch.cuda.synchronize()
        return time.perf_counter() - t
    for bs in batches:
        row = {}
        for graphs, tag in ((False, ""), (True, "_graph")):
            model.use_graphs = graphs                    # the step recorded once into a HIP graph and replayed
            run(bs, short)                               # warm-up (first use of every kernel at this batch size)
            a = min(run(bs, short) for _ in range(2))
            b = min(run(bs, long_) for _ in range(2))
            step_us = (b - a) / (long_ - short) * 1e6
            row["us_per_step" + tag] = round(step_us, 1)
            row["us_per_layer" + tag] = round(step_us / layers, 1)
        out[f"batch_{bs}"] = row
    out["config"] = (f"{layers} layers of the 8B architecture (hidden 4096, 32/8 heads, intermediate 12288, vocabulary 151936), prompts of "
                     f"{prompt_len} tokens, wall time between the steps {short} and {long_} of greedy decoding, launched call by call (host launches included) "
                     f"and, _graph, as replays of the step recorded into one HIP graph; "
                     f"{time.perf_counter() - t0:.0f} s")
    del model
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--table", action="store_true", help="long form of the per-shape table, also printed to stderr")
    ap.add_argument("--table-hot", action="store_true", help="reuse one input set per table case (cache-hot figures)")
    ap.add_argument("--eager-table", action="store_true",
                    help="time every table case as one-by-one launches (no HIP-graph replays for the short ones)")
    ap.add_argument("--only", default=None, help="with --table: only the cases whose name contains this (for profiler runs)")
    ap.add_argument("--no-context-table", action="store_true", help="leave the per-shape table out of the JSON line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="continuous load (the step itself) in front of the warm-up steps of `value`, so that the timed "
                         "steps see the chip's settled state; `value_after_idle` is always measured without it")
    ap.add_argument("--ceiling", action="store_true", help="kept for older command lines: the ceilings are measured by default")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip `context.ceiling`: the MFMA-only and one-pass-read ceilings of this chip and the board power "
                         "while the headline step, this library's plain mm, the vendor GEMM and the probes run (10 s)")
    ap.add_argument("--no-decode-step", action="store_true", help="leave the decode-step timing of the 12-layer decoder out")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 5 plain device copies of X (50,331,648 B read + as many written each) so that a "
                         "counter run can scale FETCH_SIZE / WRITE_SIZE by what a copy of known size reads")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    from llm_reproducibility_amd import _lib
    from llm_reproducibility_amd.tbik import matmul_tp_persistent, tree_combine
    from oracle import tbik_oracle as O

    _lib.lib()
    dev = torch.device("cuda:0")
    X = O.silu_gated_bf16((M_, K_), 0).to(dev)
    W = O.gaussian_bf16((N_, K_), 0.02, 1).to(dev)      # [N,K], K contiguous
    Wt = W.t()
    step = lambda: matmul_tp_persistent(X, Wt)          # noqa: E731
    C = step()
    torch.cuda.synchronize()

    # ---- timed: W warm-up steps and K steps right after the set-up, then the same behind the load phase
    idle_ms, _ = hip_time_ms(step, args.steps, args.warmup)
    ms, wall_ms = hip_time_ms(step, args.steps, args.warmup, args.settle_ms)
    flops = 2.0 * M_ * N_ * K_
    algo_bytes = 2.0 * (M_ * K_ + K_ * N_ + M_ * N_)
    tflops = flops / (ms * 1e-3) / 1e12
    tflops_idle = flops / (idle_ms * 1e-3) / 1e12

    if args.calibrate_copy:
        Y = torch.empty_like(X)
        for _ in range(5):
            Y.copy_(X)
        torch.cuda.synchronize()
        del Y

    out = {
        "metric": "TBIK matmul TFLOP/s & % bf16 MFMA peak, M=2048 K=12288 N=4096",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Qwen3-8B down_proj tree matmul X[2048,12288] x W[12288,4096] (configs[1], M=2048), leaf 256, TP=1",
                   "M": M_, "K": K_, "N": N_, "leaf_k": 256},
        "value_after_idle": round(tflops_idle, 2),
        "protocol": f"value: {args.settle_ms:g} ms of the step back to back, then W warm-up + K timed steps (settled rate); "
                    "value_after_idle: W warm-up + K timed steps right after the set-up, no load phase",
        "pct_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        "algorithmic_GBps": round(algo_bytes / (ms * 1e-3) / 1e9, 1),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": traffic_from_profile(),
                     "traffic_source": "profiles/gemm_tree_deep_headline_counters.txt (a figure of that profile, not of this run)",
                     "kernel_avg_us": round(ms * 1e3, 2), "frac_after_idle": round(tflops_idle / PEAK_BF16_TFLOPS, 4)},
    }
    context = {}
    # the vendor library's plain GEMM on the same operands, measured the same way (reduction order not fixed, no tree;
    # not a code path of this library)
    lib_ms, _ = hip_time_ms(lambda: torch.matmul(X, Wt), args.steps, args.warmup, args.settle_ms)
    context["vendor_gemm_same_operands_TFLOPs"] = round(flops / (lib_ms * 1e-3) / 1e12, 2)
    context["note"] = "torch.matmul (vendor library), reduction order not fixed, no tree"
    # this library's own matmul without the tree (one fp32 accumulator over all of K, the batch-invariant mm) on the
    # same operands: the same ring and MFMA chain, so the difference to `value` is what the tree order costs
    from llm_reproducibility_amd.bio import batch_invariant_ops as bio
    mm_ms, _ = hip_time_ms(lambda: bio.matmul_persistent(X, Wt), args.steps, args.warmup, args.settle_ms)
    context["single_accumulator_mm_same_operands_TFLOPs"] = round(flops / (mm_ms * 1e-3) / 1e12, 2)
    if not args.no_ceiling and (args.ceiling or not args.only):
        from llm_reproducibility_amd.build import MEASURE_LIB_PATH
        if not os.path.exists(MEASURE_LIB_PATH):
            context["ceiling"] = {"skipped": "the measurement library is not built (python -m llm_reproducibility_amd.build)"}
        else:
            context["ceiling"] = ceiling(args.settle_ms, (("tree_matmul_headline", step),
                                                          ("single_accumulator_mm_same_operands", lambda: bio.matmul_persistent(X, Wt)),
                                                          ("vendor_gemm_same_operands", lambda: torch.matmul(X, Wt))))
    if args.table or not args.no_context_table:
        t0 = time.perf_counter()
        rows = table(12, 3, hot=args.table_hot, settle_ms=min(args.settle_ms, 10.0), full=args.table, only=args.only,
                     graphs=not args.eager_table)
        if args.table:
            print_table(rows, args.table_hot)
        # terse in the JSON line: case -> [us per call, algorithmic work of a call (flop when the bound is "m", bytes when
        # it is "h"), achieved share of the bound's peak, bound]
        context["table"] = {r["short"]: [r["us"], int(float(f"{(r['flop'] if r['bound'] == 'mfma' else r['bytes']):.4g}")),
                                         round(r["frac"], 3), r["bound"][0]] for r in rows if r["short"]}
        context["table_cols"] = ("[us per call (HIP events after 10 ms of load; "
                                 + ("12 calls of the Python operator" if args.eager_table else
                                    f"calls under {GRAPH_BELOW_MS * 1e3:g} us: 3 replays of a HIP graph of about 32 calls (whole turns through the input sets) of the Python "
                                    "operator, so no host time; longer ones: 12 calls one by one") + "; inputs "
                                 + ("reused" if args.table_hot else "cycled: cold") + "), algorithmic flop (m) or bytes (h), share of "
                                 f"{PEAK_BF16_TFLOPS:g} TFLOP/s (m) or {PEAK_HBM_GBS:g} GB/s (h), bound]; {time.perf_counter() - t0:.0f} s")

    # (with the compact per-shape table only: the profiler commands that switch the table off or ask for its long form stay
    # free of the decoder's kernels)
    if not args.no_decode_step and not args.no_context_table and not args.table and not args.only:
        context["decode_step"] = decode_step()

    # ---- not timed: what was timed equals the simulated TP=4 run bit for bit and agrees with the CPU oracle on the same
    # inputs within the stated tolerance (1 bf16 ulp, or 2^-8 of the output scale); the oracle run is also the CPU baseline
    parts = [matmul_tp_persistent(X[:, r * 3072:(r + 1) * 3072], W[:, r * 3072:(r + 1) * 3072].t()) for r in range(4)]
    assert torch.equal(tree_combine(parts), C), "TP=4 result differs from TP=1"
    assert torch.equal(step(), C), "the step is not reproducible from call to call"
    del parts
    parity = {"tp4_bitwise_equal": True}
    if not args.no_cpu_baseline:
        cpu, want = cpu_baseline()
        out["cpu_baseline"] = cpu
        bad = O.outside_tolerance(C, want)
        ulp = O.bf16_ulp_distance(C.cpu(), want)
        assert not bad.any(), f"{int(bad.sum())} elements outside the tolerance against the CPU oracle"
        scale = float(want.float().abs().max())
        parity.update({"vs_cpu_oracle_full_size": "every element within 1 bf16 ulp or 2^-8 of the output scale",
                       "bit_equal_fraction": round(float((ulp == 0).float().mean()), 5),
                       "within_1_ulp_fraction": round(float((ulp <= 1).float().mean()), 6),
                       "max_abs_diff_over_scale": float((C.cpu().float() - want.float()).abs().max()) / scale})
    context["parity"] = parity
    out["context"] = context
    print(json.dumps(out))


if __name__ == "__main__":
    main()
