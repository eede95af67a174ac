"""tbik_gemm_bf16_static (the entry point that allocates nothing) against tbik_gemm_bf16 with a caller workspace,
through the C ABI: bit-equal outputs on two calls in a row (the second on a smaller input, so the fixed scratch array
still holds the first call's partials), the size limit, and no growth of the device memory in use."""
import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd import _lib

pytestmark = pytest.mark.gpu


def _both(L, dev, M, N, K, leaf, seed, with_bias):
    A = O.integer_bf16((M, K), -9, 9, seed).to(dev)
    W = O.integer_bf16((N, K), -7, 7, seed + 1).to(dev)
    bias = O.integer_bf16((N,), -300, 300, seed + 2).to(dev) if with_bias else None
    stream = torch.cuda.current_stream().cuda_stream
    nws = L.tbik_gemm_workspace_bytes(M, N, K, leaf)
    ws = torch.empty(max(nws, 1), device=dev, dtype=torch.uint8)
    want = torch.full((M, N), 7.0, device=dev, dtype=torch.bfloat16)
    got = torch.full((M, N), 9.0, device=dev, dtype=torch.bfloat16)
    bp = bias.data_ptr() if with_bias else None
    rc = L.tbik_gemm_bf16(A.data_ptr(), K, W.data_ptr(), 1, K, want.data_ptr(), N, M, N, K, leaf, bp,
                          ws.data_ptr() if nws else None, nws, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    used_before = torch.cuda.mem_get_info()[0]
    rc = L.tbik_gemm_bf16_static(A.data_ptr(), K, W.data_ptr(), 1, K, got.data_ptr(), N, M, N, K, leaf, bp, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return got, want, nws, used_before, (A, W, bias)


def test_static_scratch_entry_point_matches_the_workspace_entry_point(dev):
    L = _lib.lib()
    print("case first call 200x4096x12288", flush=True)
    got1, want1, nws1, _, keep = _both(L, dev, 200, 4096, 12288, 256, 1, True)     # K cut into shards: partials in scratch
    assert nws1 > 0
    assert torch.equal(got1.view(torch.int16), want1.view(torch.int16))
    cpu = O.matmul_tree(keep[0].cpu(), keep[1].cpu().t(), keep[2].cpu())
    assert torch.equal(got1.cpu().view(torch.int16), cpu.view(torch.int16))        # and both equal the oracle
    print("case second call 24x1024x4096 (smaller, same scratch)", flush=True)
    got2, want2, nws2, free_before, _ = _both(L, dev, 24, 1024, 4096, 256, 5, False)
    assert 0 < nws2 < nws1
    assert torch.equal(got2.view(torch.int16), want2.view(torch.int16))
    assert torch.cuda.mem_get_info()[0] >= free_before                           # the call took no device memory
    # a third call, leaf 128, another shape class
    print("case third call 96x5120x6400 leaf 128", flush=True)
    got3, want3, _, _, _ = _both(L, dev, 96, 5120, 6400, 128, 9, True)
    assert torch.equal(got3.view(torch.int16), want3.view(torch.int16))
    # the headline shape parks two tree levels of 16 MiB each, which fills the array (how much a shape needs is the
    # dispatcher's business and may shrink: the entry point only has to take whatever fits)
    print("case fourth call 2048x4096x12288 (fills the scratch array)", flush=True)
    got4, want4, nws4, _, _ = _both(L, dev, 2048, 4096, 12288, 256, 13, False)
    assert 0 < nws4 <= _lib.STATIC_SCRATCH_BYTES
    assert torch.equal(got4.view(torch.int16), want4.view(torch.int16))


def test_static_scratch_entry_point_rejects_what_does_not_fit(dev):
    L = _lib.lib()
    M, N, K = 4096, 5120, 8192
    assert L.tbik_gemm_workspace_bytes(M, N, K, 256) > _lib.STATIC_SCRATCH_BYTES
    C = torch.full((8,), 3.0, device=dev, dtype=torch.bfloat16)                 # never written: the call must not launch
    A = torch.zeros((8,), device=dev, dtype=torch.bfloat16)
    rc = L.tbik_gemm_bf16_static(A.data_ptr(), K, A.data_ptr(), 1, K, C.data_ptr(), N, M, N, K, 256, None,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.TBIK_ERR_SCRATCH_LIMIT
    assert "scratch" in L.tbik_error_string(rc).decode()
    torch.cuda.synchronize()
    assert bool((C == 3).all())
    # empty problems and invalid ones behave like the workspace entry point
    assert L.tbik_gemm_bf16_static(None, 8, None, 1, 8, None, 8, 0, 8, 256, 256, None, None) == 0
    assert L.tbik_gemm_bf16_static(None, 8, None, 1, 8, None, 8, 4, 8, 256, 256, None, None) == _lib.TBIK_ERR_INVALID
