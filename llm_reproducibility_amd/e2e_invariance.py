"""End-to-end invariance check on a random-init Qwen3-8B-architecture decoder (36 layers, hidden 4096, 32/8 heads,
MLP 12288, vocab 151936): greedy-decode the same prompts under simulated TP = 1/2/4/8 and batch sizes 1/32/128 and
report whether every generated token id is identical.

    python -m llm_reproducibility_amd.e2e_invariance                      # the full configuration (a few minutes)
    python -m llm_reproducibility_amd.e2e_invariance --layers 4 --prompts 16 --prompt-len 64 --new-tokens 16

This is the analogue of the reference's simple_inference.py (same prompts under different (TP, batch) settings).
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from .decoder import DecoderConfig, Qwen3Decoder


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--prompts", type=int, default=128)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--tp", type=int, nargs="+", default=[1, 2, 4, 8])
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 32, 128])
    args = ap.parse_args(argv)
    cfg = DecoderConfig(num_layers=args.layers)
    g = torch.Generator().manual_seed(1)
    prompts = torch.randint(0, cfg.vocab_size, (args.prompts, args.prompt_len), generator=g).tolist()
    results, ref = [], None
    ok = True
    model = Qwen3Decoder(cfg, tp_size=args.tp[0], seed=0, init_on_device=True)
    for tp in args.tp:
        model.set_tp(tp)
        for bs in args.batches:
            bs = min(bs, args.prompts)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ids = model.generate(prompts[:bs], args.new_tokens).cpu()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            if ref is None:
                ref = model.generate(prompts, args.new_tokens).cpu() if bs < args.prompts else ids
            same = bool(torch.equal(ids, ref[:bs]))
            ok = ok and same
            results.append({"tp": tp, "batch": bs, "identical_to_reference_run": same, "seconds": round(dt, 2),
                            "new_tokens_per_s": round(bs * args.new_tokens / dt, 1)})
            print(json.dumps(results[-1]), flush=True)
    print(json.dumps({"config": vars(args), "all_identical": ok}))
    return 0 if ok else 1


if __name__ == "__main__":
    raise SystemExit(main())
