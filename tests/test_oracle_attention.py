"""Pins the CPU oracles of the callers around the row-split GEMM -- causal attention, rotary embedding, greedy token
choice -- against library routines in float64, closed forms and brute force (no GPU)."""
import math

import torch

from oracle import tbik_oracle as O


def _sdpa_f64(q, k, v, scale):
    """The library's scaled_dot_product_attention in float64 with an explicit causal mask for the last n positions."""
    n, Hq, _ = q.shape
    L, Hkv, _ = k.shape
    rep = Hq // Hkv
    qd = q.double().permute(1, 0, 2)[None]                                   # [1, Hq, n, D]
    kd = k.double().repeat_interleave(rep, dim=1).permute(1, 0, 2)[None]     # [1, Hq, L, D]
    vd = v.double().repeat_interleave(rep, dim=1).permute(1, 0, 2)[None]
    mask = torch.arange(L)[None, :] <= torch.arange(L - n, L)[:, None]       # True = attend
    out = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, attn_mask=mask, scale=scale)
    return out[0].permute(1, 0, 2)


def test_causal_attention_matches_the_library_in_float64():
    g = torch.Generator().manual_seed(0)
    for (n, L, Hq, Hkv, D) in ((70, 70, 8, 2, 128), (1, 33, 4, 4, 64), (5, 40, 6, 3, 32), (17, 17, 2, 1, 128)):
        q = torch.randn((n, Hq, D), generator=g).to(torch.bfloat16)
        k = torch.randn((L, Hkv, D), generator=g).to(torch.bfloat16)
        v = torch.randn((L, Hkv, D), generator=g).to(torch.bfloat16)
        scale = 1.0 / math.sqrt(D)
        got = O.causal_attention(q, k, v, scale)
        want = _sdpa_f64(q, k, v, scale)
        assert got.dtype == torch.float64
        assert (got - want).abs().max() < 1e-12, (n, L, Hq, Hkv, D)


def test_causal_attention_closed_forms():
    L, Hq, Hkv, D = 9, 4, 2, 16
    g = torch.Generator().manual_seed(1)
    v = torch.randn((L, Hkv, D), generator=g)
    # all scores equal (q = 0): row i is the mean of v[0..i] -- a causal mask off by one, or a mask on the wrong
    # side, changes every row but the last
    out = O.causal_attention(torch.zeros((L, Hq, D)), torch.randn((L, Hkv, D), generator=g), v, 0.25)
    for i in range(L):
        for h in range(Hq):
            assert torch.allclose(out[i, h], v[: i + 1, h // 2].double().mean(0), atol=1e-13), (i, h)
    # one key dominates: the output is that key's value (query head -> KV head map h // rep checked by distinct values)
    k = torch.zeros((L, Hkv, D))
    k[3, 0, 0] = 100.0
    k[5, 1, 0] = 100.0
    q = torch.zeros((1, Hq, D))
    q[..., 0] = 10.0
    out = O.causal_attention(q, k, v, 1.0)      # the single query sits at the last position and sees every key
    assert torch.allclose(out[0, 0], v[3, 0].double(), atol=1e-9) and torch.allclose(out[0, 1], v[3, 0].double(), atol=1e-9)
    assert torch.allclose(out[0, 2], v[5, 1].double(), atol=1e-9) and torch.allclose(out[0, 3], v[5, 1].double(), atol=1e-9)
    # decode row == the last row of the prefill; chunked prefill == the tail of the prefill
    g2 = torch.Generator().manual_seed(2)
    q, k = torch.randn((L, Hq, D), generator=g2), torch.randn((L, Hkv, D), generator=g2)
    full = O.causal_attention(q, k, v, 0.3)
    assert torch.allclose(O.causal_attention(q[-1:], k, v, 0.3)[0], full[-1], atol=1e-14)
    assert torch.allclose(O.causal_attention(q[-4:], k, v, 0.3), full[-4:], atol=1e-14)


def test_rotary_embedding_closed_forms():
    inv = O.rope_inv_freq(128, 1e6)
    assert inv.dtype == torch.float32 and inv.shape == (64,)
    assert inv[0].item() == 1.0 and abs(inv[32].item() - 1e-3) < 1e-9      # base ** -(64/128) = 1e-3
    assert abs(inv[63].item() - 1e6 ** (-126.0 / 128.0)) < 1e-12
    g = torch.Generator().manual_seed(3)
    x = torch.randn((6, 2, 128), generator=g)
    pos = torch.tensor([0, 1, 2, 50, 511, 4095])
    y = O.rotate_half_rope(x, pos, inv)
    assert torch.equal(y[0], x[0])                                         # position 0: identity
    # a rotation: the norm of every (i, i+64) pair is preserved
    n_in = x[..., :64] ** 2 + x[..., 64:] ** 2
    n_out = y[..., :64] ** 2 + y[..., 64:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)
    # channel 0 turns by exactly `position` radians (inv_freq[0] = 1): compare with the complex exponential
    z = torch.complex(x[..., 0].double(), x[..., 64].double()) * torch.exp(1j * pos.double())[:, None]
    assert torch.allclose(y[..., 0].double(), z.real, atol=1e-6) and torch.allclose(y[..., 64].double(), z.imag, atol=1e-6)
    # composition: turning by p1 then p2 equals turning by p1 + p2 (a sign error in the sine term breaks this)
    a = O.rotate_half_rope(O.rotate_half_rope(x.double(), torch.full((6,), 7), inv), torch.full((6,), 5), inv)
    b = O.rotate_half_rope(x.double(), torch.full((6,), 12), inv)
    assert torch.allclose(a, b, atol=1e-9)
    # q/k norm in front of it: unit weight, +-c row -> +-1 * rsqrt(1 + eps/c^2) -> rotation of a +-1 vector
    s = torch.ones((1, 1, 128), dtype=torch.bfloat16) * 3
    got = O.qk_norm_rope(s, torch.ones(128, dtype=torch.bfloat16), 1e-6, torch.tensor([0]), inv)
    assert torch.equal(got, torch.ones((1, 1, 128), dtype=torch.bfloat16))


def test_argmax_lowest_index_matches_brute_force():
    g = torch.Generator().manual_seed(4)
    x = torch.randint(-3, 4, (50, 37), generator=g).to(torch.bfloat16)     # many ties
    got = O.argmax_lowest_index(x)
    for r in range(x.shape[0]):
        row = x[r].tolist()
        want = max(range(len(row)), key=lambda i: (row[i], -i))
        assert got[r].item() == want, r
    y = torch.tensor([[1.0, float("nan"), 5.0, 5.0], [float("nan")] * 4, [-float("inf")] * 4])
    assert O.argmax_lowest_index(y).tolist() == [2, 0, 0]
    assert O.argmax_lowest_index(torch.tensor([[0.0, -0.0, 0.0]])).tolist() == [0]   # -0 == +0: still the lowest index


def test_composed_decoder_oracle_matches_the_hf_qwen3_module():
    """The per-op oracles wired into a decoder agree with Hugging Face's Qwen3ForCausalLM (a library implementation of
    the same architecture, built from a local config object, fp32) on the same bf16-valued weights: the difference is
    the oracle's rounding to bf16 at every op boundary, far below what a wiring mistake (head order, q/k norm on the
    wrong side of the rotation, residual stream, rotate-half pairing, GQA map) would produce."""
    import pytest
    tr = pytest.importorskip("transformers")
    H, L, Hq, Hkv, D, I, V = 256, 2, 4, 2, 64, 512, 320
    cfg = tr.Qwen3Config(vocab_size=V, hidden_size=H, intermediate_size=I, num_hidden_layers=L, num_attention_heads=Hq,
                         num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
                         attention_bias=False, max_position_embeddings=512, use_sliding_window=False)
    if hasattr(cfg, "rope_parameters") and isinstance(getattr(cfg, "rope_parameters", None), dict):
        cfg.rope_parameters["rope_theta"] = 1e6
    torch.manual_seed(0)
    model = tr.Qwen3ForCausalLM(cfg).float().eval()
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name:
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g)).to(torch.bfloat16).float())
            else:
                p.copy_((0.05 * torch.randn(p.shape, generator=g)).to(torch.bfloat16).float())
    bf = lambda t: t.detach().to(torch.bfloat16)  # noqa: E731
    layers = []
    for lyr in model.model.layers:
        a, m = lyr.self_attn, lyr.mlp
        layers.append({"input_norm": bf(lyr.input_layernorm.weight), "post_norm": bf(lyr.post_attention_layernorm.weight),
                       "q_norm": bf(a.q_norm.weight), "k_norm": bf(a.k_norm.weight),
                       "qkv_w": bf(torch.cat((a.q_proj.weight, a.k_proj.weight, a.v_proj.weight), 0)),
                       "gate_up_w": bf(torch.cat((m.gate_proj.weight, m.up_proj.weight), 0)),
                       "o_w": bf(a.o_proj.weight), "down_w": bf(m.down_proj.weight)})
    weights = {"embed": bf(model.model.embed_tokens.weight), "lm_head": bf(model.lm_head.weight),
               "final_norm": bf(model.model.norm.weight), "layers": layers}
    prompt = torch.randint(0, V, (23,), generator=g).tolist()
    with torch.no_grad():
        want = model(torch.tensor([prompt])).logits[0, -1]
    got = O.decoder_prefill_logits(weights, prompt, Hq, Hkv, D, 1e-6, 1e6).float()
    scale = want.abs().max().item()
    assert (got - want).abs().max().item() <= 2.0 ** -5 * scale, ((got - want).abs().max().item(), scale)
    # the comparison has teeth: swapping the rotary pairing or dropping the q/k norm moves the logits by far more
    assert scale > 0.1
