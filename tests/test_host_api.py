"""Host-side contract of the plugin boundary and of the C ABI (no GPU, no compute calls)."""
import ctypes
import os
import re

import pytest
import torch

import llm_reproducibility_amd as pkg
from llm_reproducibility_amd import _lib, utils
from llm_reproducibility_amd.tbik import choose_leaf_k, matmul_tp_persistent, tree_combine

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FLAGS = ("VLLM_BATCH_INVARIANT", "VLLM_TP_INVARIANT", "ALIGN_TRAIN_INFERENCE", "TP_INVARIANT_MATMUL")


@pytest.fixture(autouse=True)
def clean_env(monkeypatch):
    for f in FLAGS:
        monkeypatch.delenv(f, raising=False)


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "tbik_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b((?:tbik|bi)_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    L = _lib.lib()
    for name in declared:
        assert hasattr(L, name), name
    assert L.tbik_abi_version() == _lib.ABI_VERSION
    assert L.tbik_error_string(0) == b"ok"
    assert b"leaves" in L.tbik_error_string(1)


def test_header_is_plain_c_and_a_c_host_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 on its own, and a host written in C (tests/c_host) builds
    with gcc against the library and the HIP runtime -- no C++, no Python in it."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no gcc on this machine")
    tu = tmp_path / "only_header.c"
    tu.write_text('#include "tbik_hip.h"\n#include "tbik_measure.h"\nint main(void) { return (int)sizeof(tbik_stream_t) == 0; }\n')
    r = subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(tu)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    _lib.lib()                                          # the library the host links against is built
    r = subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "tests", "c_host"), f"HOST_OUT={tmp_path / 'host'}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert (tmp_path / "host").exists()


def test_tree_params_through_the_c_abi():
    assert _lib.tree_params(12288, 256) == (48, 3, 5)
    assert _lib.tree_params(1536, 256) == (6, 3, 2)
    assert _lib.tree_params(3200, 128) == (25, 25, 1)
    with pytest.raises(ValueError):
        _lib.tree_params(3200, 256)


def test_workspace_query_and_plan_come_from_one_decision():
    """The workspace a caller is told to bring and the way the dispatcher runs the problem are one host-side decision
    (`tbik_gemm_plan_info` shows it): over a sweep of shapes the two agree on what each path needs -- nothing for the
    one-launch few-rows kernel, the K-shard partials for the 128x128 tiles, at least the partials of every K split
    otherwise -- and known shapes take the paths the design describes."""
    L = _lib.lib()
    out = (ctypes.c_int * 5)()

    def plan(M, N, K, leaf, f16=0, rowmajor=0):
        assert L.tbik_gemm_plan_info(M, N, K, leaf, f16, rowmajor, out) == _lib.TBIK_OK
        return list(out)

    seen = set()
    for M in (1, 2, 4, 5, 16, 17, 64, 65, 100, 128, 129, 256, 300, 512, 1000, 2048, 4096, 8192):
        for N in (64, 1000, 1024, 2048, 4096, 5120, 6144, 24576):
            for K, leaf in ((256, 256), (1024, 256), (4096, 256), (8192, 256), (12288, 256), (1536, 256), (25600, 128), (3200, 128)):
                path, split, na, split_b, pair = plan(M, N, K, leaf)
                ws = L.tbik_gemm_workspace_bytes(M, N, K, leaf)
                seen.add(path)
                if path == 0:
                    assert ws == 0 and M <= 16 and split in (2, 4, 8)
                elif path == 1:
                    assert 64 <= M <= 512 and leaf == 256 and ws == (0 if split == 1 else (split * M * N * 2 + 255) // 256 * 256)
                elif path == 2:
                    assert 0 < na < N and na % 256 == 0 and M >= 64
                    parts = [(sp, n) for sp, n in ((split, na), (split_b, N - na)) if sp > 1]
                    need = [sp * M * n * 2 for sp, n in parts]
                    assert ws >= (sum(need) if pair else max(need, default=0))
                else:
                    assert split >= 1 and (split & (split - 1)) == 0 and ws >= (split * M * N * 2 if split > 1 else 0)
                assert ws % 16 == 0
                # a row-major B runs on the tiled kernels only: one grid, partial results only
                rpath, rsplit, _, _, _ = plan(M, N, K, leaf, 0, 1)
                assert rpath == 3
                rws = L.tbik_gemm_workspace_bytes_rowmajor_b(M, N, K, leaf, 0)
                assert rws == (0 if rsplit == 1 else (rsplit * M * N * 2 + 255) // 256 * 256)
    assert seen == {0, 1, 2, 3}
    assert plan(1, 4096, 12288, 256)[0] == 0                                # decode: one launch
    assert plan(128, 4096, 12288, 256)[:2] == [1, 8]                        # down_proj 8B at 128 rows: 128x128 tiles, K in 8
    assert plan(2048, 4096, 12288, 256) == [3, 1, 0, 0, 0]                  # the benchmark shape: one round of 256 tiles, no cut
    p = plan(4096, 5120, 8192, 256)                                         # o_proj 32B: two regions in one launch
    assert p[0] == 2 and p[2] == 1024 and p[4] == 1
    assert L.tbik_gemm_plan_info(8, 8, 100, 256, 0, 0, out) == _lib.TBIK_ERR_INVALID   # K is not a whole number of leaves
    assert L.tbik_gemm_plan_info(8, 8, 256, 256, 0, 0, None) == _lib.TBIK_ERR_INVALID


def test_host_argument_checks_fire_before_any_launch():
    L = _lib.lib()
    # null pointers / bad sizes are rejected on the host, so these are safe without a GPU
    assert L.tbik_gemm_bf16(None, 0, None, 1, 0, None, 0, 4, 4, 256, 256, None, None, 0, None) == _lib.TBIK_ERR_INVALID
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert L.tbik_gemm_bf16(p16, 300, p16, 1, 300, p16, 8, 1, 8, 300, 256, None, None, 0, None) == _lib.TBIK_ERR_ALIGNMENT
    # B with neither dimension contiguous is not taken; a row-major B (ldb_n == 1) is, so its checks fire instead
    assert L.tbik_gemm_bf16(p16, 512, p16, 512, 2, p16, 8, 1, 8, 512, 256, None, None, 0, None) == _lib.TBIK_ERR_UNSUPPORTED
    assert L.tbik_gemm_bf16(p16, 512, p16, 4, 1, p16, 8, 1, 8, 512, 256, None, None, 0, None) == _lib.TBIK_ERR_INVALID      # ldb_k < N
    assert L.tbik_gemm_bf16(p16, 512, p16, 12, 1, p16, 8, 1, 8, 512, 256, None, None, 0, None) == _lib.TBIK_ERR_ALIGNMENT  # ldb_k % 8
    assert L.tbik_gemm_workspace_bytes_rowmajor_b(128, 4096, 12288, 256, 0) > 0
    assert L.tbik_gemm_bf16(p16 + 2, 512, p16, 1, 512, p16, 8, 1, 8, 512, 256, None, None, 0, None) == _lib.TBIK_ERR_ALIGNMENT
    assert L.tbik_gemm_bf16(p16, 384, p16, 1, 384, p16, 8, 1, 8, 384, 256, None, None, 0, None) == _lib.TBIK_ERR_INVALID
    arr = (ctypes.c_void_p * 3)(p16, p16, p16)
    assert L.tbik_tree_combine_bf16(arr, 3, p16, 8, None) == _lib.TBIK_ERR_INVALID
    assert L.bi_log_softmax_f32(p16, 8, p16, 8, 1, 8, None, 0, 0, None) == _lib.TBIK_ERR_WORKSPACE
    assert L.bi_log_softmax_workspace_bytes(7, 151936) == 7 * 38 * 8
    assert L.bi_rmsnorm_bf16(p16, 12, None, 0, None, p16, 12, None, 0, 1, 12, 1e-6, None) == _lib.TBIK_ERR_ALIGNMENT
    assert L.bi_mean_dim(p16, p16, 1, 4, 1, 7, None) == _lib.TBIK_ERR_UNSUPPORTED
    assert L.bi_silu_mul_bf16(p16, 24, p16, 12, 1, 12, None) == _lib.TBIK_ERR_ALIGNMENT
    assert L.bi_silu_mul_bf16(p16, 16, p16, 16, 1, 16, None) == _lib.TBIK_ERR_INVALID   # ld_in < 2 * inter
    with pytest.raises(_lib.TbikError):
        _lib.check(_lib.TBIK_ERR_ALIGNMENT, "x")


def test_env_flags(monkeypatch):
    assert not utils.batch_invariant_is_enabled() and not utils.tp_invariant_is_enabled()
    monkeypatch.setenv("VLLM_BATCH_INVARIANT", "1")
    assert utils.batch_invariant_is_enabled()
    monkeypatch.setenv("VLLM_BATCH_INVARIANT", "yes")      # does not parse -> off
    assert not utils.batch_invariant_is_enabled()
    monkeypatch.setenv("VLLM_TP_INVARIANT", "1")
    with pytest.raises(AssertionError):                     # TP invariance requires batch invariance
        utils.tp_invariant_is_enabled()
    monkeypatch.setenv("VLLM_BATCH_INVARIANT", "2")
    assert utils.tp_invariant_is_enabled() and utils.check_invariant_compat()
    monkeypatch.setenv("ALIGN_TRAIN_INFERENCE", "1")
    assert utils.compatible_mode_is_enabled()
    monkeypatch.setenv("TP_INVARIANT_MATMUL", "1")
    assert utils.tp_invariant_matmul_is_enabled()


def test_tp_invariant_matmul_flag_selects_the_product(monkeypatch):
    """TP_INVARIANT_MATMUL picks the product of the invariance check (the switch of the reference's smoke script,
    simple_matmul.py:8,14): off -> torch.matmul, on -> matmul_tp_persistent."""
    from llm_reproducibility_amd import check_matmul
    f, name = check_matmul.select_matmul()
    assert f is torch.matmul and name == "torch.matmul"
    monkeypatch.setenv("TP_INVARIANT_MATMUL", "1")
    f, name = check_matmul.select_matmul()
    assert f is matmul_tp_persistent and name == "matmul_tp_persistent"
    # the pairwise tree of the check: ((p0 + p1) + (p2 + p3)) with every add rounded to the parts' type -- on values
    # where a left-to-right sum rounds differently
    parts = [torch.tensor([v], dtype=torch.bfloat16) for v in (256.0, 1.0, 1.0, 1.0)]
    assert check_matmul.pairwise_tree_sum(parts).item() == 258.0      # (256+1 -> 256) + (1+1) = 258
    assert (((parts[0] + parts[1]) + parts[2]) + parts[3]).item() == 256.0
    with pytest.raises(ValueError):
        check_matmul.pairwise_tree_sum(parts[:3])
    # run on the CPU with the library product: the check itself works without a GPU (and without the kernels)
    monkeypatch.setenv("TP_INVARIANT_MATMUL", "0")
    name, batch_diff, shard_diff = check_matmul.run(64, 512, 32, 4, device="cpu", dtype=torch.float32)
    assert name == "torch.matmul" and batch_diff >= 0.0 and 0.0 <= shard_diff < 1e-3


def test_apply_patches_dispatch(monkeypatch, capsys):
    from llm_reproducibility_amd import layers, patch
    from llm_reproducibility_amd.bio import batch_invariant_ops as bio
    import importlib
    ptp = importlib.import_module("llm_reproducibility_amd.patch.patch_tp_invariant")
    calls = []
    monkeypatch.setattr(patch, "patch_batch_invariant", lambda: calls.append("bi"))
    monkeypatch.setattr(patch, "patch_tp_invariant", lambda: calls.append("tp"))
    monkeypatch.setattr(patch, "patch_align", lambda: calls.append("align"))
    monkeypatch.setattr(patch, "patch_training_baseline", lambda: calls.append("base"))
    pkg.apply_patches()
    assert calls == ["base"]
    calls.clear()
    monkeypatch.setenv("VLLM_BATCH_INVARIANT", "1")
    pkg.apply_patches()
    assert calls == ["bi"]
    calls.clear()
    monkeypatch.setenv("VLLM_TP_INVARIANT", "1")
    monkeypatch.setenv("ALIGN_TRAIN_INFERENCE", "1")
    pkg.apply_patches()
    assert calls == ["bi", "tp", "align"]
    calls.clear()
    monkeypatch.delenv("VLLM_BATCH_INVARIANT")
    monkeypatch.delenv("VLLM_TP_INVARIANT")
    pkg.apply_patches()
    assert calls == ["base"]
    monkeypatch.undo()
    # the real TP patch swaps the forward of the row-parallel layer and can be undone
    stock = layers.RowParallelLinear.forward
    ptp.patch_tp_invariant()
    assert layers.RowParallelLinear.forward is layers.tbik_row_parallel_forward
    ptp.unpatch_row_linear()
    assert layers.RowParallelLinear.forward is stock
    # mode switches are idempotent and restorable
    assert not bio.is_batch_invariant_mode_enabled()
    with bio.set_batch_invariant_mode(True):
        assert bio.is_batch_invariant_mode_enabled()
        bio.enable_batch_invariant_mode()
    assert not bio.is_batch_invariant_mode_enabled()
    capsys.readouterr()


def test_leaf_choice_is_a_property_of_the_layer():
    assert choose_leaf_k(12288) == 256 and choose_leaf_k(8192) == 256 and choose_leaf_k(4096) == 256
    assert choose_leaf_k(25600) == 128            # 25600 / 8 = 3200 = 25 * 128
    assert choose_leaf_k(25600, max_tp=4) == 256
    with pytest.raises(ValueError):
        choose_leaf_k(1000)


def test_operator_errors_match_the_reference_contract():
    a = torch.zeros((4, 512), dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="Dim doesn't match"):
        matmul_tp_persistent(a, torch.zeros((256, 8), dtype=torch.bfloat16))
    with pytest.raises(AssertionError):
        matmul_tp_persistent(torch.zeros((4, 384), dtype=torch.bfloat16), torch.zeros((384, 8), dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        matmul_tp_persistent(a.double(), torch.zeros((512, 8), dtype=torch.float64))
    with pytest.raises(ValueError):
        tree_combine([a, a, a])
    # there is no CPU path: CPU tensors fail loudly instead of falling back
    with pytest.raises((NotImplementedError, RuntimeError)):
        matmul_tp_persistent(a, torch.zeros((512, 8), dtype=torch.bfloat16))
    with pytest.raises((NotImplementedError, RuntimeError)):
        tree_combine([a, a])
    with pytest.raises(RuntimeError):
        tree_combine([a.float(), a.float()])
    with pytest.raises(RuntimeError):
        matmul_tp_persistent(a.float(), torch.zeros((512, 8)))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libtbik_hip.so"))
    with pytest.raises(RuntimeError, match="only implementation"):
        _lib.lib()


def test_tree_all_reduce_wrapper_contract(monkeypatch):
    """tree_all_reduce_sum[_native] without a process group: the world size comes from a stand-in, the gather from a
    stand-in that hands every rank's partial over, the adds from the CPU oracle.  Checks the ValueError of the reference
    (src/tbik/tree_based_all_reduce.py:26-27), that the input is not aliased, and that the wrapper's result is the
    adjacent-pair tree over the gathered partials in rank order."""
    import torch
    import torch.distributed as dist
    from oracle import tbik_oracle as O
    from llm_reproducibility_amd.tbik import tree_based_all_reduce as tar

    world = {"n": 3}
    monkeypatch.setattr(dist, "get_world_size", lambda group=None: world["n"])
    x = O.integer_bf16((4, 16), -300, 300, 0)
    for n in (3, 5, 6, 12):
        world["n"] = n
        with pytest.raises(ValueError):
            tar.tree_all_reduce_sum(x)
        with pytest.raises(ValueError):
            tar.tree_all_reduce_sum_native(x)
    partials = [O.integer_bf16((4, 16), -300, 300, 10 + r) for r in range(8)]
    calls = []

    def fake_all_gather(out_list, inp, group=None):
        calls.append((len(out_list), inp.is_contiguous(), group))
        for r, o in enumerate(out_list):
            o.copy_(partials[r])

    monkeypatch.setattr(dist, "all_gather", fake_all_gather)
    monkeypatch.setattr(tar, "tree_combine", lambda parts: O.tree_combine(list(parts)))
    for n in (1, 2, 4, 8):
        world["n"] = n
        calls.clear()
        before = partials[0].clone()
        got = tar.tree_all_reduce_sum(partials[0].t().contiguous().t(), device_group="grp")   # a non-contiguous view
        assert calls == [(n, True, "grp")]
        assert torch.equal(got, O.tree_combine(partials[:n]))
        assert got.data_ptr() != partials[0].data_ptr() and torch.equal(partials[0], before)
    # the tree, not a left-to-right sum: the two differ on these partials
    seq = partials[0].clone()
    for q in partials[1:8]:
        seq = seq + q
    assert not torch.equal(seq, O.tree_combine(partials))
