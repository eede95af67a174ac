"""A self-contained Qwen3-architecture decoder that drives the invariant kernels end to end.

It plays the role the vLLM engine plays for the reference (simple_inference.py:62-105: same prompts, different
(TP, batch) settings, compare outputs): RMSNorm -> qkv projection (batch-invariant mm) -> per-head q/k RMSNorm ->
rotary embedding -> fixed-order attention -> o_proj (tree matmul, K sharded over `tp_size` simulated ranks and
combined in the all-reduce tree order) -> gated MLP with down_proj as a tree matmul -> lm_head -> greedy argmax.
Every op either is elementwise or fixes its reduction order per row, so the generated token ids are identical
for every simulated TP degree and every batch composition.

Random-initialised weights only (N(0, 0.02), norm weights 1): this is a correctness and benchmarking vehicle,
not a checkpoint loader.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch

from . import ops
from .bio.batch_invariant_ops import matmul_persistent, rms_norm
from .layers import SimulatedTPRowLinear
from .patch.patch_training_inference_align import compute_inv_freq


@dataclass
class DecoderConfig:
    vocab_size: int = 151936
    hidden_size: int = 4096
    num_layers: int = 36
    num_q_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 12288
    rope_theta: float = 1e6
    rms_eps: float = 1e-6


def _normal_bf16(shape, gen: torch.Generator, device) -> torch.Tensor:
    """N(0, 0.02) in bf16 on `device`, drawn where the generator lives (CPU: the same values on every machine;
    GPU: seconds instead of minutes for the 8B-parameter configuration)."""
    w = torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device)
    return w.mul_(0.02).to(torch.bfloat16).to(device)


class _Layer:
    def __init__(self, cfg: DecoderConfig, tp_size: int, gen: torch.Generator, device):
        def w(*shape):
            return _normal_bf16(shape, gen, device)
        H, D = cfg.hidden_size, cfg.head_dim
        self.input_norm = torch.ones(H, dtype=torch.bfloat16, device=device)
        self.post_norm = torch.ones(H, dtype=torch.bfloat16, device=device)
        self.q_norm = torch.ones(D, dtype=torch.bfloat16, device=device)
        self.k_norm = torch.ones(D, dtype=torch.bfloat16, device=device)
        self.qkv_w = w((cfg.num_q_heads + 2 * cfg.num_kv_heads) * D, H)          # column-parallel in a real TP run
        self.gate_up_w = w(2 * cfg.intermediate_size, H)
        self.o_proj = SimulatedTPRowLinear(w(H, cfg.num_q_heads * D), tp_size)    # row-parallel: K sharded
        self.down_proj = SimulatedTPRowLinear(w(H, cfg.intermediate_size), tp_size)


class Qwen3Decoder:
    def __init__(self, cfg: DecoderConfig, tp_size: int = 1, seed: int = 0, device="cuda:0", use_graphs: bool = False,
                 fused_rope: bool = True, init_on_device: bool = False, fused_producers: bool = True,
                 fused_consumers: bool = True, fused_attention_step: bool = True):
        assert cfg.head_dim == 128, "the attention kernel is built for head_dim 128"
        self.cfg, self.tp_size, self.device = cfg, tp_size, torch.device(device)
        # decode steps replayed from one captured HIP graph (same kernels, same order, same bits as eager; the
        # per-step host work shrinks to one graph launch, which is what bounds small batches)
        self.use_graphs = use_graphs
        self.fused_rope = fused_rope
        # RMSNorm inside the projection that consumes it and SiLU*up inside down_proj (one launch each for a handful of
        # rows, the two launches otherwise; bit-identical either way, so the switch only exists for the tests)
        self.fused_producers = fused_producers
        # beyond a handful of rows: the add-RMSNorm behind o_proj and down_proj inside the launch that combines the layer's
        # K shards (bit-identical to the separate norm; the switch only exists for the tests)
        self.fused_consumers = fused_consumers
        # decode steps (one new token per sequence): q/k norm, rotary embedding, cache write and attention in one launch
        # (bit-identical to the two launches; the switch only exists for the tests)
        self.fused_attention_step = fused_attention_step and fused_rope
        gen = torch.Generator(device=self.device if init_on_device else "cpu").manual_seed(seed)
        emb = lambda *shape: _normal_bf16(shape, gen, self.device)  # noqa: E731
        self.embed = emb(cfg.vocab_size, cfg.hidden_size)
        self.layers = [_Layer(cfg, tp_size, gen, self.device) for _ in range(cfg.num_layers)]
        self.final_norm = torch.ones(cfg.hidden_size, dtype=torch.bfloat16, device=self.device)
        self.lm_head = emb(cfg.vocab_size, cfg.hidden_size)
        self.inv_freq = compute_inv_freq(cfg.head_dim, cfg.rope_theta, self.device)  # fp32 table built on the CPU
        self.scale = 1.0 / math.sqrt(cfg.head_dim)

    def set_tp(self, tp_size: int) -> None:
        """Re-shard the row-split layers (o_proj, down_proj) of THIS model over `tp_size` simulated ranks: the
        weights stay where they are, only the K slices and the shard tree change."""
        for layer in self.layers:
            for lin in (layer.o_proj, layer.down_proj):
                assert lin.weight.shape[1] % tp_size == 0
                lin.tp_size = tp_size
        self.tp_size = tp_size

    # ------------------------------------------------------------------------------------------
    def _rope(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Rotate-half rotary embedding in fp32, rounded once to bf16 (elementwise: batch invariant)."""
        ang = positions.to(torch.float32)[:, None] * self.inv_freq[None, :]            # [tokens, D/2]
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        xf = x.float()
        x1, x2 = xf[..., : x.shape[-1] // 2], xf[..., x.shape[-1] // 2:]
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(torch.bfloat16)

    def _forward(self, token_ids: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                 q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, cache) -> torch.Tensor:
        cfg = self.cfg
        Hq, Hkv, D = cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim
        x = self.embed[token_ids]                                   # [tokens, H]
        residual: Optional[torch.Tensor] = None
        fused = self.fused_producers and (x.shape[0] <= 4 or not self.fused_consumers)   # the one-launch producers take a handful of rows
        h: Optional[torch.Tensor] = None     # the layer's normalised input, when the previous layer's down_proj produced it
        for li, layer in enumerate(self.layers):
            if fused:
                qkv, new_res = ops.rmsnorm_gemm(x, layer.input_norm, cfg.rms_eps, residual, layer.qkv_w.t())
                residual = x if residual is None else new_res
            else:
                if h is None:
                    if residual is None:
                        residual = x
                        h = rms_norm(x, layer.input_norm, cfg.rms_eps)
                    else:
                        h, residual = rms_norm(x, layer.input_norm, cfg.rms_eps, residual=residual)
                qkv = matmul_persistent(h, layer.qkv_w.t())
                h = None
            k_cache, vt_cache = cache[li]
            if self.fused_attention_step and max_q_len == 1 and qkv.shape[0] == ctx_len.numel():
                # a decode step: token b is sequence b's, at position ctx_len[b] - 1
                attn = ops.bi_attention_decode_qkv(qkv, layer.q_norm, layer.k_norm, self.inv_freq, k_cache, vt_cache, ctx_len,
                                                   Hq, Hkv, self.scale, cfg.rms_eps)
            elif self.fused_rope:
                # per-head q/k norm, rotary embedding and the cache write in one kernel
                q = ops.bi_qk_norm_rope_cache_bf16(qkv, layer.q_norm, layer.k_norm, self.inv_freq, positions, seq_of_token,
                                                   k_cache, vt_cache, Hq, Hkv, cfg.rms_eps)
            else:
                q = qkv[:, : Hq * D].reshape(-1, Hq, D)
                k = qkv[:, Hq * D: (Hq + Hkv) * D].reshape(-1, Hkv, D)
                v = qkv[:, (Hq + Hkv) * D:].reshape(-1, Hkv, D)
                q = self._rope(rms_norm(q.contiguous(), layer.q_norm, cfg.rms_eps), positions)
                k = self._rope(rms_norm(k.contiguous(), layer.k_norm, cfg.rms_eps), positions)
                k_cache[seq_of_token, :, positions] = k             # [tokens, Hkv, D] -> [B, Hkv, L, D]
                vt_cache[seq_of_token, :, :, positions] = v         # stored transposed: [B, Hkv, D, L]
            if not (self.fused_attention_step and max_q_len == 1 and qkv.shape[0] == ctx_len.numel()):
                attn = ops.bi_attention_bf16(q, k_cache, vt_cache, q_start, q_len, ctx_len, max_q_len, self.scale)
            if fused:
                x = layer.o_proj(attn.reshape(-1, Hq * D))
                gu, residual = ops.rmsnorm_gemm(x, layer.post_norm, cfg.rms_eps, residual, layer.gate_up_w.t())
                x = layer.down_proj.forward_gated(gu)
            elif self.fused_consumers:
                # the add-RMSNorm behind each row-split layer runs in the launch that combines the layer's K shards
                hp, residual = layer.o_proj.forward_add_norm(attn.reshape(-1, Hq * D), residual, layer.post_norm, cfg.rms_eps)
                act = ops.gemm_silu_mul(hp, layer.gate_up_w)     # the activation inside the projection for 5 .. 64 rows
                if li + 1 < len(self.layers):
                    h, residual = layer.down_proj.forward_add_norm(act, residual, self.layers[li + 1].input_norm, cfg.rms_eps)
                else:
                    x = layer.down_proj(act)    # the final norm runs on the rows the caller selects
            else:
                x = layer.o_proj(attn.reshape(-1, Hq * D))
                hp, residual = rms_norm(x, layer.post_norm, cfg.rms_eps, residual=residual)
                gu = matmul_persistent(hp, layer.gate_up_w.t())
                act = ops.bi_silu_mul(gu)
                x = layer.down_proj(act)
        return x, residual

    def _logits(self, x: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        """Final norm and lm_head for the given rows (the norm is per row, so rows may be selected first)."""
        if self.fused_producers:
            return ops.rmsnorm_gemm(x, self.final_norm, self.cfg.rms_eps, residual, self.lm_head.t())[0]
        h, _ = rms_norm(x, self.final_norm, self.cfg.rms_eps, residual=residual)
        return matmul_persistent(h, self.lm_head.t())

    # ------------------------------------------------------------------------------------------
    @torch.no_grad()
    def generate(self, prompts: List[List[int]], max_new_tokens: int, return_logits: bool = False):
        """Greedy decoding of a batch of prompts (ragged lengths allowed). Returns [batch, max_new_tokens] ids."""
        cfg, dev = self.cfg, self.device
        B = len(prompts)
        lens = [len(p) for p in prompts]
        max_len = ((max(lens) + max_new_tokens + 31) // 32) * 32
        cache = [(torch.zeros((B, cfg.num_kv_heads, max_len, cfg.head_dim), dtype=torch.bfloat16, device=dev),
                  torch.zeros((B, cfg.num_kv_heads, cfg.head_dim, max_len), dtype=torch.bfloat16, device=dev))
                 for _ in range(cfg.num_layers)]
        # ---- prefill: all prompt tokens, token-major
        tok = torch.tensor([t for p in prompts for t in p], dtype=torch.long, device=dev)
        pos = torch.tensor([i for n in lens for i in range(n)], dtype=torch.long, device=dev)
        seq = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.long, device=dev)
        starts = [0]
        for n in lens[:-1]:
            starts.append(starts[-1] + n)
        q_start = torch.tensor(starts, dtype=torch.int32, device=dev)
        q_len = torch.tensor(lens, dtype=torch.int32, device=dev)
        ctx = torch.tensor(lens, dtype=torch.int32, device=dev)
        x, res = self._forward(tok, pos, seq, q_start, q_len, ctx, max(lens), cache)
        last = torch.tensor([s + n - 1 for s, n in zip(starts, lens)], dtype=torch.long, device=dev)
        logits = self._logits(x[last].contiguous(), res[last].contiguous())
        all_logits = [logits] if return_logits else None
        # ---- decode: one token per sequence per step
        q_start = torch.arange(B, dtype=torch.int32, device=dev)
        q_len = torch.ones(B, dtype=torch.int32, device=dev)
        seq = torch.arange(B, dtype=torch.long, device=dev)
        # The step works on static tensors, so that it can be captured once and replayed.  The token choice writes the
        # next token, files it in the output and advances the positions and cache lengths in its own launch: at a
        # small batch a step is a chain of short kernels, and each of those updates would be one more.
        ids = torch.zeros((B, max_new_tokens), dtype=torch.long, device=dev)
        n_out = torch.zeros(B, dtype=torch.long, device=dev)
        tok_s = torch.empty(B, dtype=torch.long, device=dev)
        pos_s = torch.tensor(lens, dtype=torch.long, device=dev)
        ctx_s = (pos_s + 1).to(torch.int32)
        ops.bi_argmax_advance(logits, tok_s, ids, n_out)       # the prompt's last position chooses the first new token

        def step():
            logits = self._logits(*self._forward(tok_s, pos_s, seq, q_start, q_len, ctx_s, 1, cache))
            ops.bi_argmax_advance(logits, tok_s, ids, n_out, pos_s, ctx_s)
            return logits

        def record(logits):
            if return_logits:
                all_logits.append(logits.clone())

        steps = max_new_tokens - 1
        if self.use_graphs and steps >= 3:
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                record(step())           # first step eagerly on the capture stream (also warms every kernel up)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                static_logits = step()
            torch.cuda.current_stream(dev).wait_stream(side)
            for _ in range(steps - 1):
                graph.replay()
                record(static_logits)
        else:
            for _ in range(steps):
                record(step())
        return (ids, torch.stack(all_logits, dim=1)) if return_logits else ids
