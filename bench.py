"""Benchmark of the TBIK hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--table]

A step is one tree-ordered matmul (`matmul_tp_persistent`) over the headline batch: X[2048,12288]
(SiLU-gated synthetic activations, bf16) times the down_proj weight W[4096,12288] (N(0,0.02), bf16,
stored [N,K] as nn.Linear does), inputs resident in HBM before the timed region.  Prints ONE JSON line.
`--table` additionally prints (to stderr) the other shapes of the workload family: decode-sized M,
simulated TP shards + combine, and the batch-invariant reductions.
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
    ten at 270-280 us, and only after about a hundred the rate is steady (210-215 us).  A benchmark of a handful of
    steps taken right after the host-side set-up would measure that transient, not the kernel."""
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


def cpu_baseline(budget_s=12.0, max_runs=30):
    """The CPU oracle (PyTorch restatement of the reference's tree order) on the whole headline workload, all host
    threads: one warm-up, then repeated until about `budget_s` seconds of CPU work are spent; the median is reported."""
    import torch
    from oracle import tbik_oracle as O
    X = O.silu_gated_bf16((M_, K_), 0)
    W = O.gaussian_bf16((N_, K_), 0.02, 1)
    Wt = W.t()
    O.matmul_tree(X[:256], Wt)
    ts, spent = [], 0.0
    while spent < budget_s and len(ts) < max_runs:
        t0 = time.perf_counter()
        O.matmul_tree(X, Wt)
        ts.append(time.perf_counter() - t0)
        spent += ts[-1]
    t = statistics.median(ts)
    return {"value": round(2.0 * M_ * N_ * K_ / t / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"oracle matmul_tree on the full X[{M_},{K_}] and W[{N_},{K_}] of the headline workload, "
                      f"{len(ts)} runs in {spent:.1f} s, median {t:.2f} s each"}, O.matmul_tree(X, Wt)


def ceiling(settle_ms):
    """What the chip sustains on bf16 MFMAs alone (register operands, one work-group per CU, 2 waves per SIMD: the wave
    shape of the tree kernel) for constant and for random operands, and on a one-pass read of 1 GiB (cold in the 256 MB
    memory-side cache).  Steady-state figures (same load phase as the headline)."""
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
    iters = 800        # 800 x 16 MFMAs x 2 waves per SIMD = the MFMA count of one headline launch per SIMD on 256 CUs
    g = torch.Generator().manual_seed(0)
    ops_rand = torch.randn(32768, generator=g)
    ops_rand[:16384] *= 0.02                      # a operands like the weights, b operands like the activations
    for name, src in (("constant", torch.full((32768,), 1.0)), ("random", ops_rand)):
        buf = src.to(torch.bfloat16).to(dev)

        def run():
            _lib.check(L.tbik_probe_mfma_bf16(buf.data_ptr(), out.data_ptr(), cus, 8, iters, stream), "tbik_probe_mfma_bf16")
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
    res["note"] = ("MFMA-only loop on register operands and a plain grid-stride read: ceilings of any bf16 matmul kernel "
                   "on such data and of any one-pass kernel, measured in this run")
    return res


def table(steps, warmup, hot=False, settle_ms=20.0):
    """Per-shape figures, each after `settle_ms` of the same call run back to back (the settled rate, as for the
    headline).  Unless `hot`, every case cycles through enough distinct input sets (more than 768 MB in
    all) that nothing it reads is still in the 256 MB memory-side cache from the previous call: the GB/s are HBM
    figures, as in a model whose every layer has its own weights."""
    import torch
    from oracle import tbik_oracle as O
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
        return call

    def gemm_row(name, M, K, N, leaf):
        def make():
            return (torch.randn((M, K), device=dev).to(torch.bfloat16), (torch.randn((N, K), device=dev) * 0.02).to(torch.bfloat16))
        fl, by = 2.0 * M * N * K, 2.0 * (M * K + K * N + M * N)
        ms, _ = hip_time_ms(cycling(make, by, lambda X, W: matmul_tp_persistent(X, W.t(), leaf_k=leaf)), steps, warmup, settle_ms)
        rows.append((name, ms * 1e3, fl / ms / 1e9, by / ms / 1e6))

    for M in (1, 16, 128, 2048):
        gemm_row(f"down_proj 8B  M={M} K=12288 N=4096", M, 12288, 4096, 256)
    def library_row(M, K, N):
        # context only: the vendor library GEMM behind torch.matmul (no tree, reduction order not fixed) on like operands
        def make():
            return (torch.randn((M, K), device=dev).to(torch.bfloat16), (torch.randn((N, K), device=dev) * 0.02).to(torch.bfloat16))
        fl, by = 2.0 * M * N * K, 2.0 * (M * K + K * N + M * N)
        ms, _ = hip_time_ms(cycling(make, by, lambda X, W: torch.matmul(X, W.t())), steps, warmup, settle_ms)
        rows.append((f"  [torch.matmul, not invariant] M={M} K={K} N={N}", ms * 1e3, fl / ms / 1e9, by / ms / 1e6))

    for M in (1, 128, 2048):
        library_row(M, 12288, 4096)
    for p in (2, 4, 8):
        gemm_row(f"  shard TP={p}  M=2048 K={12288 // p} N=4096", 2048, 12288 // p, 4096, 256)
    for M in (1, 64, 512, 4096):
        gemm_row(f"o_proj 32B    M={M} K=8192 N=5120", M, 8192, 5120, 256)
    for M in (1, 64, 512, 4096):
        gemm_row(f"down_proj 32B M={M} K=25600 N=5120 leaf128", M, 25600, 5120, choose_leaf_k(25600))
    library_row(4096, 8192, 5120)
    library_row(4096, 25600, 5120)
    library_row(2048, 4096, 24576)
    library_row(8192, 4096, 24576)
    for name, M, K, N in (("qkv 8B", 2048, 4096, 6144), ("gate_up 8B", 2048, 4096, 24576), ("gate_up 8B", 8192, 4096, 24576),
                          ("lm_head 8B", 128, 4096, 151936),
                          ("qkv 8B", 1, 4096, 6144), ("qkv 8B", 32, 4096, 6144), ("qkv 8B", 128, 4096, 6144),
                          ("gate_up 8B", 1, 4096, 24576), ("gate_up 8B", 32, 4096, 24576), ("gate_up 8B", 128, 4096, 24576),
                          ("lm_head 8B", 1, 4096, 151936), ("lm_head 8B", 32, 4096, 151936)):
        def make(M=M, K=K, N=N):
            return (torch.randn((M, K), device=dev).to(torch.bfloat16), (torch.randn((N, K), device=dev) * 0.02).to(torch.bfloat16))
        by = 2.0 * (M * K + K * N + M * N)
        ms, _ = hip_time_ms(cycling(make, by, lambda X, W: bio.matmul_persistent(X, W.t())), steps, warmup, settle_ms)
        rows.append((f"batch-invariant mm {name} M={M} K={K} N={N}", ms * 1e3, 2.0 * M * N * K / ms / 1e9, by / ms / 1e6))
    for p in (2, 4, 8):
        by = (p + 1) * 2048 * 4096 * 2
        make = lambda p=p: ([torch.randn((2048, 4096), device=dev).to(torch.bfloat16) for _ in range(p)],)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, by, tree_combine), steps, warmup, settle_ms)
        rows.append((f"tree_combine p={p} [2048,4096]", ms * 1e3, 0.0, by / ms / 1e6))
    w = torch.ones(4096, device=dev, dtype=torch.bfloat16)
    for r in (1, 7, 256, 4096):
        by = r * 4096 * 4 + 8192
        make = lambda r=r: (torch.randn((r, 4096), device=dev).to(torch.bfloat16),)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, by, lambda x: bio.rms_norm(x, w, 1e-6)), steps, warmup, settle_ms)
        rows.append((f"rmsnorm rows={r} hidden=4096", ms * 1e3, 0.0, by / ms / 1e6))
    for r in (1, 7, 256, 4096):
        by = r * 151936 * 8
        make = lambda r=r: (torch.randn((r, 151936), device=dev),)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, by, bio.log_softmax), max(steps // 4, 3), warmup, settle_ms)
        rows.append((f"log_softmax rows={r} vocab=151936 (8 B/elem)", ms * 1e3, 0.0, by / ms / 1e6))
    for r in (256, 4096):
        by = r * 151936 * 4
        make = lambda r=r: (torch.randn((r, 151936), device=dev).to(torch.bfloat16),)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, by, bio.log_softmax), max(steps // 4, 3), warmup, settle_ms)
        rows.append((f"log_softmax bf16 in/out rows={r} vocab=151936 (4 B/elem)", ms * 1e3, 0.0, by / ms / 1e6))
    for r in (1, 7, 256, 4096):
        by = r * 4096 * 4
        make = lambda r=r: (torch.randn((r, 4096), device=dev),)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, 2 * by, lambda x: bio.mean_dim(x, -1)), steps, warmup, settle_ms)
        rows.append((f"mean rows={r} n=4096", ms * 1e3, 0.0, by / ms / 1e6))
    from llm_reproducibility_amd import ops
    for r in (1, 256, 4096):
        by = r * 12288 * 6
        make = lambda r=r: (torch.randn((r, 2 * 12288), device=dev).to(torch.bfloat16),)  # noqa: E731
        ms, _ = hip_time_ms(cycling(make, by, ops.bi_silu_mul), steps, warmup, settle_ms)
        rows.append((f"silu_mul rows={r} inter=12288 (6 B/elem)", ms * 1e3, 0.0, by / ms / 1e6))
    # fixed-order attention (Qwen3-8B heads: 32 query, 8 key/value, head_dim 128)
    Hq, Hkv, D = 32, 8, 128
    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=dev)
    for name, B, qlen, ctx in (("prefill 8 x 512", 8, 512, 512), ("prefill 1 x 4096", 1, 4096, 4096),
                               ("decode 128 seqs ctx 768", 128, 1, 768), ("decode 8 seqs ctx 4096", 8, 1, 4096)):
        L = ((ctx + 31) // 32) * 32
        qs, ql, cl = i32([b * qlen for b in range(B)]), i32([qlen] * B), i32([ctx] * B)
        pairs = B * Hq * (qlen * (2 * ctx - qlen + 1) // 2)          # causal (query, key) pairs
        byts = 2.0 * (2 * B * Hkv * ctx * D + 2 * B * qlen * Hq * D)   # K, V once; q and out

        def make(B=B, qlen=qlen, L=L):
            return (torch.randn((B * qlen, Hq, D), device=dev).to(torch.bfloat16),
                    torch.randn((B, Hkv, L, D), device=dev).to(torch.bfloat16),
                    torch.randn((B, Hkv, D, L), device=dev).to(torch.bfloat16))
        ms, _ = hip_time_ms(cycling(make, byts, lambda q, kc, vt: ops.bi_attention_bf16(q, kc, vt, qs, ql, cl, qlen, D ** -0.5)),
                            max(steps // 2, 3), warmup, settle_ms)
        rows.append((f"attention {name}", ms * 1e3, 4.0 * pairs * D / ms / 1e9, byts / ms / 1e6))
    print("inputs " + ("reused by every call (hot in the memory-side cache)" if hot else
                       "cycled through more than 768 MB of distinct buffers (cold in the 256 MB memory-side cache)"), file=sys.stderr)
    print(f"{'case':52s} {'us':>10s} {'TFLOP/s':>9s} {'%MFMA':>6s} {'GB/s':>9s} {'%HBM':>6s}", file=sys.stderr)
    for name, us, tf, gbs in rows:
        print(f"{name:52s} {us:10.1f} {tf:9.1f} {100 * tf / PEAK_BF16_TFLOPS:6.1f} {gbs:9.1f} {100 * gbs / PEAK_HBM_GBS:6.1f}",
              file=sys.stderr)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--table", action="store_true", help="also print the per-shape table to stderr")
    ap.add_argument("--table-hot", action="store_true", help="with --table: reuse one input set per case (cache-hot figures)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="continuous load (the step itself) in front of the warm-up steps, so that the timed steps see "
                         "the chip's settled state and not the transient that follows the host-side set-up; 0 disables")
    ap.add_argument("--ceiling", action="store_true",
                    help="also measure the MFMA-only and the one-pass-read ceilings of this chip (reported in `context`)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 5 plain device copies of X (50,331,648 B read + as many written each) so that a "
                         "counter run can scale FETCH_SIZE / WRITE_SIZE by what a copy of known size reads")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    from llm_reproducibility_amd import _lib
    from llm_reproducibility_amd.tbik import matmul_tp_persistent
    from oracle import tbik_oracle as O

    _lib.lib()
    dev = torch.device("cuda:0")
    # host-side work first (the GPU idles meanwhile): the CPU baseline, whose product is also the parity reference
    cpu, want = (None, None) if args.no_cpu_baseline else cpu_baseline()
    X = O.silu_gated_bf16((M_, K_), 0).to(dev)
    W = O.gaussian_bf16((N_, K_), 0.02, 1).to(dev)      # [N,K], K contiguous
    Wt = W.t()
    step = lambda: matmul_tp_persistent(X, Wt)          # noqa: E731
    C = step()
    # parity inside the bench (not timed): what is being timed equals the simulated TP=4 run bit for bit and agrees
    # with the CPU oracle on the same inputs within the stated tolerance (1 bf16 ulp, or 2^-8 of the output scale)
    from llm_reproducibility_amd.tbik import tree_combine
    parts = [matmul_tp_persistent(X[:, r * 3072:(r + 1) * 3072], W[:, r * 3072:(r + 1) * 3072].t()) for r in range(4)]
    assert torch.equal(tree_combine(parts), C), "TP=4 result differs from TP=1"
    del parts
    parity = None
    if want is not None:
        bad = O.outside_tolerance(C, want)
        ulp = O.bf16_ulp_distance(C.cpu(), want)
        assert not bad.any(), f"{int(bad.sum())} elements outside the tolerance against the CPU oracle"
        scale = float(want.float().abs().max())
        parity = {"vs_cpu_oracle_full_size": "every element within 1 bf16 ulp or 2^-8 of the output scale",
                  "bit_equal_fraction": round(float((ulp == 0).float().mean()), 5),
                  "within_1_ulp_fraction": round(float((ulp <= 1).float().mean()), 6),
                  "max_abs_diff_over_scale": float((C.cpu().float() - want.float()).abs().max()) / scale,
                  "tp4_bitwise_equal": True}

    if args.calibrate_copy:
        Y = torch.empty_like(X)
        for _ in range(5):
            Y.copy_(X)
        torch.cuda.synchronize()
        del Y

    # the figure right after the idle period (the transient), for the record; then the settled rate, which is `value`
    cold_ms, _ = hip_time_ms(step, args.steps, args.warmup)
    ms, wall_ms = hip_time_ms(step, args.steps, args.warmup, args.settle_ms)
    flops = 2.0 * M_ * N_ * K_
    algo_bytes = 2.0 * (M_ * K_ + K_ * N_ + M_ * N_)
    tflops = flops / (ms * 1e-3) / 1e12
    out = {
        "metric": "TBIK matmul TFLOP/s & % bf16 MFMA peak, M=2048 K=12288 N=4096",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Qwen3-8B down_proj tree matmul X[2048,12288] x W[12288,4096] (configs[1], M=2048), leaf 256, TP=1",
                   "M": M_, "K": K_, "N": N_, "leaf_k": 256},
        "pct_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        "algorithmic_GBps": round(algo_bytes / (ms * 1e-3) / 1e9, 1),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": traffic_from_profile(),
                     "traffic_source": "profiles/gemm_tree_deep_headline_counters.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                                       "scaled by a copy of known size; a figure of that profile, not of this run)",
                     "kernel_avg_us": round(ms * 1e3, 2)},
    }
    if cpu is not None:
        out["cpu_baseline"] = cpu
    context = {"settle_ms": args.settle_ms,
               "settle_note": "the timed steps follow settle_ms of the same step run back to back (then the warm-up steps): "
                              "after idling the chip needs about 25 ms of load to reach its steady rate",
               "first_steps_after_idle_TFLOPs": round(flops / (cold_ms * 1e-3) / 1e12, 2)}
    if parity is not None:
        context["parity"] = parity
    # the vendor library's plain GEMM on the same operands, measured the same way (reduction order not fixed, no tree;
    # not a code path of this library)
    lib_ms, _ = hip_time_ms(lambda: torch.matmul(X, Wt), args.steps, args.warmup, args.settle_ms)
    context["vendor_gemm_same_operands_TFLOPs"] = round(flops / (lib_ms * 1e-3) / 1e12, 2)
    context["note"] = "torch.matmul (vendor library), reduction order not fixed, no tree"
    # this library's own matmul without the tree (one fp32 accumulator over all of K, the batch-invariant mm) on the
    # same operands: the same tile, ring and MFMA chain, so the difference to `value` is what the tree order costs
    from llm_reproducibility_amd.bio import batch_invariant_ops as bio
    mm_ms, _ = hip_time_ms(lambda: bio.matmul_persistent(X, Wt), args.steps, args.warmup, args.settle_ms)
    context["single_accumulator_mm_same_operands_TFLOPs"] = round(flops / (mm_ms * 1e-3) / 1e12, 2)
    if args.ceiling:
        context["ceiling"] = ceiling(args.settle_ms)
    out["context"] = context
    if args.table:
        table(max(args.steps // 2, 5), max(args.warmup // 2, 2), hot=args.table_hot, settle_ms=min(args.settle_ms, 20.0))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
