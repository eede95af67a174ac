"""Fixed-order attention and the end-to-end greedy decode (the reference's simple_inference.py check: same prompts
under different (TP, batch) settings must give the same outputs), on a small random-init Qwen3-architecture model."""
import math

import pytest
import torch

from oracle import tbik_oracle as O
from llm_reproducibility_amd import ops
from llm_reproducibility_amd.decoder import DecoderConfig, Qwen3Decoder

pytestmark = pytest.mark.gpu


def _ref_attention(q, k, v, scale):
    """fp32 causal attention of one sequence: q [n, Hq, D] are the LAST n positions of k/v [L, Hkv, D]."""
    n, Hq, D = q.shape
    L, Hkv, _ = k.shape
    rep = Hq // Hkv
    kf = k.float().repeat_interleave(rep, dim=1)
    vf = v.float().repeat_interleave(rep, dim=1)
    s = torch.einsum("qhd,khd->hqk", q.float(), kf) * scale
    qpos = torch.arange(L - n, L, device=q.device)[:, None]
    kpos = torch.arange(L, device=q.device)[None, :]
    s = s.masked_fill(kpos > qpos, float("-inf"))
    return torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), vf)


def _make_cache(ks, vs, max_len, dev):
    B, Hkv, D = len(ks), ks[0].shape[1], ks[0].shape[2]
    kc = torch.zeros((B, Hkv, max_len, D), dtype=torch.bfloat16, device=dev)
    vt = torch.zeros((B, Hkv, D, max_len), dtype=torch.bfloat16, device=dev)
    for b, (k, v) in enumerate(zip(ks, vs)):
        kc[b, :, : k.shape[0]] = k.transpose(0, 1)
        vt[b, :, :, : v.shape[0]] = v.permute(1, 2, 0)
    return kc, vt


def test_attention_matches_fp32_reference_and_is_batch_and_phase_invariant(dev):
    torch.manual_seed(0)
    Hq, Hkv, D, scale = 8, 2, 128, 1.0 / math.sqrt(128)
    lens = [70, 33, 1, 128, 17]
    ks = [torch.randn((n, Hkv, D), device=dev).to(torch.bfloat16) for n in lens]
    vs = [torch.randn((n, Hkv, D), device=dev).to(torch.bfloat16) for n in lens]
    qs = [torch.randn((n, Hq, D), device=dev).to(torch.bfloat16) for n in lens]
    max_len = 160
    kc, vt = _make_cache(ks, vs, max_len, dev)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    starts = [sum(lens[:i]) for i in range(len(lens))]
    # prefill of the whole ragged batch
    out = ops.bi_attention_bf16(torch.cat(qs), kc, vt, i32(starts), i32(lens), i32(lens), max(lens), scale)
    for b, n in enumerate(lens):
        # the CPU oracle (float64 textbook attention); tolerance as stated for random inputs: within 1 bf16 ulp of the
        # oracle's value OR within 2^-8 of the output scale (the kernel rounds the probabilities to bf16 for the PV
        # product, the oracle does not)
        want = O.causal_attention(qs[b].cpu(), ks[b].cpu(), vs[b].cpu(), scale)
        got = out[starts[b]: starts[b] + n].cpu()
        bad = O.outside_tolerance(got, want.to(torch.bfloat16))
        assert not bad.any(), (b, int(bad.sum()), (got.double() - want).abs().max().item(), want.abs().max().item())
    # a sequence alone == the same sequence inside the batch (bitwise)
    for b in (0, 3):
        kc1, vt1 = _make_cache([ks[b]], [vs[b]], max_len, dev)
        alone = ops.bi_attention_bf16(qs[b], kc1, vt1, i32([0]), i32([lens[b]]), i32([lens[b]]), lens[b], scale)
        assert torch.equal(alone, out[starts[b]: starts[b] + lens[b]]), b
    # decode phase: the last token of every sequence as a single-query call == its prefill row (bitwise)
    q_last = torch.stack([q[-1] for q in qs])
    dec = ops.bi_attention_bf16(q_last, kc, vt, i32(list(range(len(lens)))), i32([1] * len(lens)), i32(lens), 1, scale)
    for b, n in enumerate(lens):
        assert torch.equal(dec[b], out[starts[b] + n - 1]), b
    # chunked prefill: the last 5 tokens of sequence 0 against the cache == the same rows of the full prefill
    tail = ops.bi_attention_bf16(qs[0][-5:], kc[:1], vt[:1], i32([0]), i32([5]), i32([lens[0]]), 5, scale)
    assert torch.equal(tail, out[starts[0] + lens[0] - 5: starts[0] + lens[0]])
    # a cache length that is not a whole number of 32-key tiles takes the one-wave-per-head kernel instead of the
    # grouped one (K/V tiles staged in LDS once per KV head): same per-row arithmetic, same bits
    kc2, vt2 = _make_cache(ks, vs, 164, dev)
    out2 = ops.bi_attention_bf16(torch.cat(qs), kc2, vt2, i32(starts), i32(lens), i32(lens), max(lens), scale)
    assert torch.equal(out2, out)
    # other group sizes (query heads per KV head): 1, 2, 8
    for hq, hkv in ((2, 2), (4, 2), (16, 2)):
        k1 = [torch.randn((n, hkv, D), device=dev).to(torch.bfloat16) for n in lens[:3]]
        v1 = [torch.randn((n, hkv, D), device=dev).to(torch.bfloat16) for n in lens[:3]]
        q1 = [torch.randn((n, hq, D), device=dev).to(torch.bfloat16) for n in lens[:3]]
        st = [sum(lens[:i]) for i in range(3)]
        ca, va = _make_cache(k1, v1, 96, dev)
        cb, vb = _make_cache(k1, v1, 100, dev)
        oa = ops.bi_attention_bf16(torch.cat(q1), ca, va, i32(st), i32(lens[:3]), i32(lens[:3]), max(lens[:3]), scale)
        ob = ops.bi_attention_bf16(torch.cat(q1), cb, vb, i32(st), i32(lens[:3]), i32(lens[:3]), max(lens[:3]), scale)
        assert torch.equal(oa, ob), (hq, hkv)
        # and against the oracle (a wrong query-head -> KV-head map would be the same mistake in both kernels), prefill
        # and the decode kernel of this group size
        dq = torch.stack([q[-1] for q in q1])
        od = ops.bi_attention_bf16(dq, ca, va, i32([0, 1, 2]), i32([1, 1, 1]), i32(lens[:3]), 1, scale)
        for b, n in enumerate(lens[:3]):
            want = O.causal_attention(q1[b].cpu(), k1[b].cpu(), v1[b].cpu(), scale).to(torch.bfloat16)
            assert not O.outside_tolerance(oa[st[b]: st[b] + n].cpu(), want).any(), (hq, hkv, b)
            assert torch.equal(od[b], oa[st[b] + n - 1]), (hq, hkv, b)


@pytest.mark.parametrize("hq,hkv,qlens,ctxs", [
    (8, 2, [4, 1, 3, 2, 4], [70, 33, 128, 17, 4]),        # four heads per KV head: up to four new queries fit one tile
    (16, 2, [2, 1, 2], [65, 1, 96]),                      # eight heads per KV head: two
    (4, 2, [8, 5, 1], [40, 64, 97]),                      # two heads per KV head: eight
    (2, 2, [16, 9, 1], [16, 100, 31]),                    # one head per KV head: sixteen
    (32, 8, [3, 4, 1], [2272, 2304, 2239]),               # the decoder's heads; 71, 72 and 70 key tiles
])
def test_a_few_new_queries_per_sequence_equal_their_prefill_rows(dev, hq, hkv, qlens, ctxs):
    """When the new queries of every sequence times the query heads of a KV head fit the 16 rows of one MFMA tile, a
    kernel of its own takes the call (rows = query x head of the group, the score tiles formed one tile ahead, the
    output channels split over the waves).  Its rows must be, bit for bit, the rows of the whole prefill of the same
    sequences (the grouped kernel), ragged batches included, whatever the other sequences of the batch bring; and the
    one-wave-per-head kernel (a cache length that is not a whole number of tiles) must agree as well."""
    torch.manual_seed(hq * 100 + len(qlens))
    D, scale = 128, 1.0 / math.sqrt(128)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    ks = [torch.randn((n, hkv, D), device=dev).to(torch.bfloat16) for n in ctxs]
    vs = [torch.randn((n, hkv, D), device=dev).to(torch.bfloat16) for n in ctxs]
    qs = [torch.randn((n, hq, D), device=dev).to(torch.bfloat16) for n in ctxs]
    max_len = (max(ctxs) + 31) // 32 * 32
    kc, vt = _make_cache(ks, vs, max_len, dev)
    starts = [sum(ctxs[:i]) for i in range(len(ctxs))]
    print("case few new queries", hq, hkv, qlens, ctxs, flush=True)
    full = ops.bi_attention_bf16(torch.cat(qs), kc, vt, i32(starts), i32(ctxs), i32(ctxs), max(ctxs), scale)
    tails = torch.cat([q[-n:] for q, n in zip(qs, qlens)])
    tstarts = [sum(qlens[:i]) for i in range(len(qlens))]
    got = ops.bi_attention_bf16(tails, kc, vt, i32(tstarts), i32(qlens), i32(ctxs), max(qlens), scale)
    for b, (n, c) in enumerate(zip(qlens, ctxs)):
        assert torch.equal(got[tstarts[b]: tstarts[b] + n], full[starts[b] + c - n: starts[b] + c]), (b, n, c)
    # a sequence on its own, and with a single new query where the batch had several
    for b in (0, len(qlens) - 1):
        kc1, vt1 = _make_cache([ks[b]], [vs[b]], max_len, dev)
        alone = ops.bi_attention_bf16(qs[b][-qlens[b]:], kc1, vt1, i32([0]), i32([qlens[b]]), i32([ctxs[b]]), qlens[b], scale)
        assert torch.equal(alone, got[tstarts[b]: tstarts[b] + qlens[b]]), b
        one = ops.bi_attention_bf16(qs[b][-1:], kc1, vt1, i32([0]), i32([1]), i32([ctxs[b]]), 1, scale)
        assert torch.equal(one[0], full[starts[b] + ctxs[b] - 1]), b
    # a sequence without new tokens in the batch leaves the others as they are and writes nothing
    q0 = list(qlens)
    q0[1] = 0
    t0 = [sum(q0[:i]) for i in range(len(q0))]
    tails0 = torch.cat([q[-n:] for q, n in zip(qs, q0) if n])
    out0 = ops.bi_attention_bf16(tails0, kc, vt, i32(t0), i32(q0), i32(ctxs), max(q0), scale)
    for b, n in enumerate(q0):
        assert torch.equal(out0[t0[b]: t0[b] + n], full[starts[b] + ctxs[b] - n: starts[b] + ctxs[b]]), b
    kc2, vt2 = _make_cache(ks, vs, max_len + 4, dev)
    assert torch.equal(ops.bi_attention_bf16(tails, kc2, vt2, i32(tstarts), i32(qlens), i32(ctxs), max(qlens), scale), got)
    # and a row of each sequence against the float64 oracle (a wrong row -> (query, head) map would be the same mistake
    # in nothing else: the prefill rows come from another kernel)
    for b in range(len(qlens)):
        if ctxs[b] > 300:
            continue
        want = O.causal_attention(qs[b].cpu(), ks[b].cpu(), vs[b].cpu(), scale).to(torch.bfloat16)
        assert not O.outside_tolerance(got[tstarts[b]: tstarts[b] + qlens[b]].cpu(), want[-qlens[b]:]).any(), b


def _oracle_heads(q, k, v, heads, rep, scale):
    """O.causal_attention for a subset of query heads (each with its own KV head), as [n, len(heads), D]."""
    outs = []
    for h in heads:
        kv = h // rep
        outs.append(O.causal_attention(q[:, h:h + 1], k[:, kv:kv + 1], v[:, kv:kv + 1], scale))
    return torch.cat(outs, dim=1)


def test_attention_matches_the_oracle_at_the_decoder_configuration(dev):
    """32 query heads over 8 KV heads of 128 channels (the grouped kernel with four waves per KV head), contexts of
    512-768 keys and one of 2304 (72 key tiles: the prefetch ring of the decode kernel wraps 18 times), prefill,
    chunked prefill and decode, against the float64 oracle; stated tolerance: within 1 bf16 ulp OR within 2^-8 of the
    output scale.  The one-wave-per-head kernel (a cache length that is not a whole number of tiles) must give the
    same bits."""
    torch.manual_seed(4)
    Hq, Hkv, D, scale = 32, 8, 128, 1.0 / math.sqrt(128)
    rep = Hq // Hkv
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    rnd = lambda *shape: torch.randn(shape, device=dev).to(torch.bfloat16)  # noqa: E731

    def check(got, q, k, v, heads, what):
        want = _oracle_heads(q.cpu(), k.cpu(), v.cpu(), heads, rep, scale).to(torch.bfloat16)
        bad = O.outside_tolerance(got[:, heads].cpu(), want)
        assert not bad.any(), (what, int(bad.sum()), O.bf16_ulp_distance(got[:, heads].cpu(), want).max().item())

    # ---- prefill of a ragged batch at 512 / 300 / 512 tokens: every head of the first sequence, one head of each
    # position inside a KV group for the others
    lens = [512, 300, 512]
    ks, vs, qs = [rnd(n, Hkv, D) for n in lens], [rnd(n, Hkv, D) for n in lens], [rnd(n, Hq, D) for n in lens]
    starts = [0, 512, 812]
    kc, vt = _make_cache(ks, vs, 768, dev)
    print("case prefill 32/8 heads", lens, flush=True)
    out = ops.bi_attention_bf16(torch.cat(qs), kc, vt, i32(starts), i32(lens), i32(lens), 512, scale)
    check(out[:512], qs[0], ks[0], vs[0], list(range(Hq)), "prefill seq 0")
    check(out[512:812], qs[1], ks[1], vs[1], [0, 5, 14, 31], "prefill seq 1")
    check(out[812:], qs[2], ks[2], vs[2], [3, 9, 22, 28], "prefill seq 2")
    kc2, vt2 = _make_cache(ks, vs, 772, dev)
    assert torch.equal(ops.bi_attention_bf16(torch.cat(qs), kc2, vt2, i32(starts), i32(lens), i32(lens), 512, scale), out)

    # ---- decode at contexts 768 / 768 / 700 / 513: the caches above grown by random keys, one query each
    ctx = [768, 768, 700, 513]
    kd, vd, qd = [rnd(n, Hkv, D) for n in ctx], [rnd(n, Hkv, D) for n in ctx], [rnd(1, Hq, D) for _ in ctx]
    kc, vt = _make_cache(kd, vd, 768, dev)
    print("case decode 32/8 heads", ctx, flush=True)
    dec = ops.bi_attention_bf16(torch.cat(qd), kc, vt, i32([0, 1, 2, 3]), i32([1] * 4), i32(ctx), 1, scale)
    for b in range(4):
        check(dec[b:b + 1], qd[b], kd[b], vd[b], list(range(Hq)), f"decode seq {b}")
    kc2, vt2 = _make_cache(kd, vd, 780, dev)
    assert torch.equal(ops.bi_attention_bf16(torch.cat(qd), kc2, vt2, i32([0, 1, 2, 3]), i32([1] * 4), i32(ctx), 1, scale), dec)

    # ---- a long context: 2304 keys; decode (all heads), a chunk of 40 new tokens (all heads), and the whole prefill
    # on four heads (one per position inside a KV group)
    L = 2304
    k1, v1, q1 = rnd(L, Hkv, D), rnd(L, Hkv, D), rnd(L, Hq, D)
    kc, vt = _make_cache([k1], [v1], L, dev)
    print("case long context", L, flush=True)
    full = ops.bi_attention_bf16(q1, kc, vt, i32([0]), i32([L]), i32([L]), L, scale)
    check(full, q1, k1, v1, [1, 6, 19, 28], "prefill 2304")
    one = ops.bi_attention_bf16(q1[-1:], kc, vt, i32([0]), i32([1]), i32([L]), 1, scale)
    check(one, q1[-1:], k1, v1, list(range(Hq)), "decode 2304")
    assert torch.equal(one[0], full[-1])
    chunk = ops.bi_attention_bf16(q1[-40:], kc, vt, i32([0]), i32([40]), i32([L]), 40, scale)
    check(chunk, q1[-40:], k1, v1, list(range(Hq)), "chunk of 40 at 2304")
    assert torch.equal(chunk, full[-40:])
    kc2, vt2 = _make_cache([k1], [v1], L + 4, dev)
    assert torch.equal(ops.bi_attention_bf16(q1[-40:], kc2, vt2, i32([0]), i32([40]), i32([L]), 40, scale), chunk)


SMALL = DecoderConfig(vocab_size=3000, hidden_size=1024, num_layers=2, num_q_heads=16, num_kv_heads=4, head_dim=128,
                      intermediate_size=4096)


def _prompts(n, seed=1):
    g = torch.Generator().manual_seed(seed)
    lens = [37, 64, 5, 48, 21, 33, 16, 50][:n]
    return [torch.randint(0, SMALL.vocab_size, (L,), generator=g).tolist() for L in lens]


def test_greedy_decode_is_identical_across_tp_and_batch(dev):
    prompts = _prompts(8)
    new = 10
    base_model = Qwen3Decoder(SMALL, tp_size=1, seed=0, device=dev)
    base_ids, base_logits = base_model.generate(prompts, new, return_logits=True)
    assert base_ids.shape == (8, new)
    assert torch.isfinite(base_logits.float()).all()
    # batch composition: each prompt alone, and a sub-batch, must reproduce its row bit for bit (logits included)
    for b in (0, 2, 7):
        ids, logits = base_model.generate([prompts[b]], new, return_logits=True)
        assert torch.equal(ids[0], base_ids[b]), b
        assert torch.equal(logits[0], base_logits[b]), b
    ids3 = base_model.generate(prompts[2:5], new)
    assert torch.equal(ids3, base_ids[2:5])
    del base_model
    # simulated tensor parallelism: same seed -> same weights, row-split layers sharded 2/4/8 ways
    for tp in (2, 4, 8):
        m = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev)
        ids, logits = m.generate(prompts, new, return_logits=True)
        assert torch.equal(ids, base_ids), tp
        assert torch.equal(logits, base_logits), tp
        one = m.generate([prompts[5]], new)
        assert torch.equal(one[0], base_ids[5]), tp
        del m


def test_fused_qk_norm_rope_cache_matches_the_unfused_composition(dev):
    from llm_reproducibility_amd.bio.batch_invariant_ops import rms_norm
    from llm_reproducibility_amd.patch.patch_training_inference_align import compute_inv_freq
    torch.manual_seed(2)
    Hq, Hkv, D, B, L, T = 8, 2, 128, 3, 64, 37
    qkv = torch.randn((T, (Hq + 2 * Hkv) * D), device=dev).to(torch.bfloat16)
    qw = (1 + 0.1 * torch.randn(D, device=dev)).to(torch.bfloat16)
    kw = (1 + 0.1 * torch.randn(D, device=dev)).to(torch.bfloat16)
    inv = compute_inv_freq(D, 1e6, dev)
    seq = torch.randint(0, B, (T,), device=dev)
    pos = torch.stack([torch.randperm(L, device=dev)[:T] for _ in range(1)])[0]   # distinct positions: no write races
    kc = torch.zeros((B, Hkv, L, D), dtype=torch.bfloat16, device=dev)
    vt = torch.zeros((B, Hkv, D, L), dtype=torch.bfloat16, device=dev)
    q = ops.bi_qk_norm_rope_cache_bf16(qkv, qw, kw, inv, pos, seq, kc, vt, Hq, Hkv, 1e-6)

    def rope(x):
        ang = pos.float()[:, None] * inv[None, :]
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        xf = x.float()
        a, b = xf[..., :64], xf[..., 64:]
        return torch.cat((a * cos - b * sin, b * cos + a * sin), -1).to(torch.bfloat16)

    q_ref = rope(rms_norm(qkv[:, : Hq * D].reshape(T, Hq, D).contiguous(), qw, 1e-6))
    k_ref = rope(rms_norm(qkv[:, Hq * D: (Hq + Hkv) * D].reshape(T, Hkv, D).contiguous(), kw, 1e-6))
    v_ref = qkv[:, (Hq + Hkv) * D:].reshape(T, Hkv, D)
    tol = lambda got, want: ((got.float() - want.float()).abs() <= 2.0 ** -7 * want.float().abs().clamp_min(2.0 ** -5)).all()  # noqa: E731
    assert tol(q, q_ref)
    assert tol(kc[seq, :, pos], k_ref)
    # the CPU oracle (norm as `rmsnorm`, float64 rotation from the fp32 frequency table): 1 ulp OR 2^-8 of the scale
    qc = qkv.cpu()
    q_want = O.qk_norm_rope(qc[:, : Hq * D].reshape(T, Hq, D), qw.cpu(), 1e-6, pos.cpu(), inv.cpu())
    k_want = O.qk_norm_rope(qc[:, Hq * D: (Hq + Hkv) * D].reshape(T, Hkv, D), kw.cpu(), 1e-6, pos.cpu(), inv.cpu())
    assert torch.equal(inv.cpu(), O.rope_inv_freq(D, 1e6))
    assert not O.outside_tolerance(q, q_want).any(), O.bf16_ulp_distance(q.cpu(), q_want).max()
    assert not O.outside_tolerance(kc[seq, :, pos], k_want).any()
    assert torch.equal(vt[seq, :, :, pos], v_ref)
    # nothing else in the caches was touched
    mask = torch.zeros((B, L), dtype=torch.bool, device=dev)
    mask[seq, pos] = True
    assert (kc.permute(0, 2, 1, 3)[~mask] == 0).all() and (vt.permute(0, 3, 1, 2)[~mask] == 0).all()
    # row i alone == row i in the batch
    kc1, vt1 = torch.zeros_like(kc), torch.zeros_like(vt)
    q1 = ops.bi_qk_norm_rope_cache_bf16(qkv[5:6], qw, kw, inv, pos[5:6], seq[5:6], kc1, vt1, Hq, Hkv, 1e-6)
    assert torch.equal(q1[0], q[5]) and torch.equal(kc1[seq[5], :, pos[5]], kc[seq[5], :, pos[5]])
    # the decoder with and without the fused kernel: same tokens on a short run, logits within tolerance
    prompts = _prompts(3, seed=9)
    a = Qwen3Decoder(SMALL, tp_size=1, seed=0, device=dev, fused_rope=True).generate(prompts, 3, return_logits=True)
    b = Qwen3Decoder(SMALL, tp_size=1, seed=0, device=dev, fused_rope=False).generate(prompts, 3, return_logits=True)
    assert (a[1].float() - b[1].float()).abs().max() < 0.05 * b[1].float().abs().max()


@pytest.mark.parametrize("hq,hkv,ctxs,max_len", [
    (32, 8, [1, 32, 33, 64, 65, 96, 128, 129, 160, 161, 577, 700, 736], 736),   # the new key in tile 0 .. 22, at tile edges
    (8, 2, [5, 31, 100, 128, 0, 200], 224),                                      # a sequence without tokens is skipped
    (16, 2, [40, 129, 7], 160),
    (4, 2, [64, 1, 97], 128),
    (2, 2, [33, 160, 2, 95], 160),
])
def test_decode_step_in_one_launch_equals_norm_rope_cache_write_then_attention(dev, hq, hkv, ctxs, max_len):
    """q/k norm + rotary embedding + cache write + attention of one new token per sequence in ONE launch (the work-group
    of a (sequence, KV head) forms its heads itself and patches the new key and value into the tiles its loaders bring in)
    against the two launches: outputs and both caches bit for bit, wherever the new key falls in its tile and whichever
    tile of the prefetch ring it is."""
    from llm_reproducibility_amd import _lib
    from llm_reproducibility_amd.patch.patch_training_inference_align import compute_inv_freq
    torch.manual_seed(hq + len(ctxs))
    D, B, scale, eps = 128, len(ctxs), 1.0 / math.sqrt(128), 1e-6
    qkv = torch.randn((B, (hq + 2 * hkv) * D), device=dev).to(torch.bfloat16)
    qw = (1 + 0.1 * torch.randn(D, device=dev)).to(torch.bfloat16)
    kw = (1 + 0.1 * torch.randn(D, device=dev)).to(torch.bfloat16)
    inv = compute_inv_freq(D, 1e6, dev)
    kc0 = torch.randn((B, hkv, max_len, D), device=dev).to(torch.bfloat16)      # the history (and junk behind it)
    vt0 = torch.randn((B, hkv, D, max_len), device=dev).to(torch.bfloat16)
    ctx = torch.tensor(ctxs, dtype=torch.int32, device=dev)
    live = [b for b, c in enumerate(ctxs) if c > 0]
    print("case one-launch decode step", hq, hkv, ctxs, max_len, flush=True)
    # the two launches, on the live sequences
    kc_a, vt_a = kc0.clone(), vt0.clone()
    pos = (ctx[live] - 1).to(torch.int64)
    seq = torch.tensor(live, dtype=torch.int64, device=dev)
    q = ops.bi_qk_norm_rope_cache_bf16(qkv[live], qw, kw, inv, pos, seq, kc_a, vt_a, hq, hkv, eps)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    want = ops.bi_attention_bf16(q, kc_a[live].contiguous(), vt_a[live].contiguous(), i32(list(range(len(live)))), i32([1] * len(live)),
                                 ctx[live].contiguous(), 1, scale)
    # one launch (the raw entry point takes the shape: the wrapper below did not fall back)
    kc_b, vt_b = kc0.clone(), vt0.clone()
    out = torch.full((B, hq, D), 7.0, dtype=torch.bfloat16, device=dev)
    rc = _lib.lib().bi_attention_decode_qkv_bf16(qkv.data_ptr(), qkv.stride(0), qw.data_ptr(), kw.data_ptr(), inv.data_ptr(),
                                                 kc_b.data_ptr(), vt_b.data_ptr(), out.data_ptr(), ctx.data_ptr(), B, hq, hkv, D,
                                                 max_len, scale, eps, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.TBIK_OK
    assert torch.equal(out[live], want)
    assert torch.equal(kc_b, kc_a) and torch.equal(vt_b, vt_a)
    for b, c in enumerate(ctxs):
        if c <= 0:
            assert (out[b] == 7.0).all()          # nothing written for a sequence without tokens
    kc_c, vt_c = kc0.clone(), vt0.clone()
    if len(live) == B:
        got = ops.bi_attention_decode_qkv(qkv, qw, kw, inv, kc_c, vt_c, ctx, hq, hkv, scale, eps)
        assert torch.equal(got, want) and torch.equal(kc_c, kc_a) and torch.equal(vt_c, vt_a)
    # a sequence on its own gives the same bits as in the batch
    b = live[-1]
    kc1, vt1 = kc0[b:b + 1].clone(), vt0[b:b + 1].clone()
    alone = ops.bi_attention_decode_qkv(qkv[b:b + 1], qw, kw, inv, kc1, vt1, ctx[b:b + 1].contiguous(), hq, hkv, scale, eps)
    assert torch.equal(alone[0], out[b])
    # a cache length that is not a whole number of tiles: the entry point declines, the wrapper makes the two calls
    if len(live) == B:
        L2 = max_len + 4
        kc2 = torch.zeros((B, hkv, L2, D), dtype=torch.bfloat16, device=dev)
        vt2 = torch.zeros((B, hkv, D, L2), dtype=torch.bfloat16, device=dev)
        kc2[:, :, :max_len], vt2[:, :, :, :max_len] = kc0, vt0
        assert _lib.lib().bi_attention_decode_qkv_bf16(qkv.data_ptr(), qkv.stride(0), qw.data_ptr(), kw.data_ptr(), inv.data_ptr(),
                                                       kc2.data_ptr(), vt2.data_ptr(), out.data_ptr(), ctx.data_ptr(), B, hq, hkv, D,
                                                       L2, scale, eps, torch.cuda.current_stream().cuda_stream) == _lib.TBIK_ERR_UNSUPPORTED
        got2 = ops.bi_attention_decode_qkv(qkv, qw, kw, inv, kc2, vt2, ctx, hq, hkv, scale, eps)
        assert torch.equal(got2, want) and torch.equal(kc2[:, :, :max_len], kc_a) and torch.equal(vt2[:, :, :, :max_len], vt_a)


def test_decoder_with_and_without_the_one_launch_decode_step_gives_the_same_bits(dev):
    prompts = _prompts(6, seed=11)
    for tp in (1, 2):
        a = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_attention_step=True)
        b = Qwen3Decoder(SMALL, tp_size=tp, seed=0, device=dev, fused_attention_step=False)
        for batch in (1, 3, 6):
            print("case decoder one-launch decode step tp", tp, "batch", batch, flush=True)
            ia, la = a.generate(prompts[:batch], 8, return_logits=True)
            ib, lb = b.generate(prompts[:batch], 8, return_logits=True)
            assert torch.equal(ia, ib) and torch.equal(la, lb), (tp, batch)
        del a, b


def test_graph_replayed_decode_steps_equal_eager_steps(dev):
    """Every replay of the captured decode step must give the eager step's bits (token ids and logits)."""
    prompts = _prompts(5, seed=7)
    eager = Qwen3Decoder(SMALL, tp_size=2, seed=0, device=dev)
    graphed = Qwen3Decoder(SMALL, tp_size=2, seed=0, device=dev, use_graphs=True)
    ids_e, log_e = eager.generate(prompts, 9, return_logits=True)
    torch.cuda.synchronize()
    ids_g, log_g = graphed.generate(prompts, 9, return_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(ids_g, ids_e)
    for step in range(log_e.shape[1]):
        assert torch.equal(log_g[:, step], log_e[:, step]), step
    # a second generation on the same object (new capture, new caches) and another batch size
    ids_g2 = graphed.generate(prompts[:2], 6)
    assert torch.equal(ids_g2, eager.generate(prompts[:2], 6))


def test_decoder_logits_agree_with_plain_pytorch_math(dev):
    """Tolerance check of the whole stack against a straightforward fp32 PyTorch forward of the same weights."""
    cfg = DecoderConfig(vocab_size=512, hidden_size=512, num_layers=2, num_q_heads=8, num_kv_heads=2, head_dim=128,
                        intermediate_size=2048)
    m = Qwen3Decoder(cfg, tp_size=2, seed=3, device=dev)
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, cfg.vocab_size, (29,), generator=g).tolist()
    _, logits = m.generate([prompt], 1, return_logits=True)

    def norm(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.rms_eps) * w.float()

    x = m.embed[torch.tensor(prompt, device=dev)].float()
    pos = torch.arange(len(prompt), device=dev)
    ang = pos.float()[:, None] * m.inv_freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rope(t):
        a, b = t[..., :64], t[..., 64:]
        return torch.cat((a * cos - b * sin, b * cos + a * sin), -1)

    Hq, Hkv, D = cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim
    for layer in m.layers:
        h = norm(x, layer.input_norm)
        qkv = h @ layer.qkv_w.float().t()
        q = rope(norm(qkv[:, : Hq * D].reshape(-1, Hq, D), layer.q_norm))
        k = rope(norm(qkv[:, Hq * D: (Hq + Hkv) * D].reshape(-1, Hkv, D), layer.k_norm))
        v = qkv[:, (Hq + Hkv) * D:].reshape(-1, Hkv, D)
        att = _ref_attention(q, k, v, m.scale).reshape(-1, Hq * D)
        x = x + att @ layer.o_proj.weight.float().t()
        h = norm(x, layer.post_norm)
        gu = h @ layer.gate_up_w.float().t()
        x = x + (torch.nn.functional.silu(gu[:, : cfg.intermediate_size]) * gu[:, cfg.intermediate_size:]) @ layer.down_proj.weight.float().t()
    want = norm(x[-1:], m.final_norm) @ m.lm_head.float().t()
    got = logits[0, 0].float()
    assert (got - want[0]).abs().max() <= 0.05 * want.abs().max() + 0.02, ((got - want[0]).abs().max(), want.abs().max())
    # against the CPU oracle composed of the per-op oracles (same rounding points as the kernels, so much tighter):
    # every op is within 1 bf16 ulp of its oracle; through 2 layers x 7 ops those single steps spread to a few 2^-8 of
    # the logit scale -- 2^-6 of the scale is asserted (the fp32 library forward above needs 5 %)
    cpu = lambda t: t.detach().cpu()  # noqa: E731
    weights = {"embed": cpu(m.embed), "lm_head": cpu(m.lm_head), "final_norm": cpu(m.final_norm),
               "layers": [{"input_norm": cpu(l.input_norm), "post_norm": cpu(l.post_norm), "q_norm": cpu(l.q_norm),
                           "k_norm": cpu(l.k_norm), "qkv_w": cpu(l.qkv_w), "gate_up_w": cpu(l.gate_up_w),
                           "o_w": cpu(l.o_proj.weight), "down_w": cpu(l.down_proj.weight)} for l in m.layers]}
    ow = O.decoder_prefill_logits(weights, prompt, Hq, Hkv, D, cfg.rms_eps, cfg.rope_theta).float()
    err = (logits[0, 0].cpu().float() - ow).abs().max().item()
    assert err <= 2.0 ** -6 * ow.abs().max().item(), (err, ow.abs().max().item())
    assert int(ops.bi_argmax(logits[0, :1].contiguous())[0]) == int(O.argmax_lowest_index(logits[0, :1].cpu())[0])


def test_config5_full_size_greedy_decode_is_identical_across_tp_and_batch(dev):
    """The end-to-end configuration at its stated size: random-init Qwen3-8B architecture (36 layers, hidden 4096,
    32/8 heads of 128, MLP 12288, vocab 151936), 128 prompts of 512 uniform-random token ids, 256 greedy tokens;
    generated ids identical across simulated TP 1/2/4/8 and batch sizes 1/32/128 (the reference's simple_inference.py
    check: same prompts, different (TP, batch) settings).  Weights are drawn on the GPU (8.2 G parameters)."""
    cfg = DecoderConfig()
    assert (cfg.num_layers, cfg.hidden_size, cfg.num_q_heads, cfg.num_kv_heads, cfg.intermediate_size, cfg.vocab_size) == \
        (36, 4096, 32, 8, 12288, 151936)
    g = torch.Generator().manual_seed(1)
    prompts = torch.randint(0, cfg.vocab_size, (128, 512), generator=g).tolist()
    new = 256
    model = Qwen3Decoder(cfg, tp_size=1, seed=0, device=dev, init_on_device=True)
    print("case config5 reference run tp=1 batch=128", flush=True)
    ref = model.generate(prompts, new).cpu()
    assert ref.shape == (128, new)
    assert len(set(ref.flatten().tolist())) > 100          # the model does not collapse to one token
    for tp in (1, 2, 4, 8):
        model.set_tp(tp)
        for bs in (1, 32, 128):
            if tp == 1 and bs == 128:
                continue
            print("case config5 tp", tp, "batch", bs, flush=True)
            ids = model.generate(prompts[:bs], new).cpu()
            assert torch.equal(ids, ref[:bs]), (tp, bs, int((ids != ref[:bs]).sum()))
    del model
    torch.cuda.empty_cache()
