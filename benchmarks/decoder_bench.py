#!/usr/bin/env python3
"""Prefill and decode throughput of the hybrid decoders (Lebepel; Pemidra with ``--models pemidra,lebepel``;
Fusasun with ``--models fusasun,llama``; Lumedra with ``--models lumedra,fusasun,llama``) beside a Llama decoder of the same width, depth, heads, head size, feed-forward and vocabulary (random
weights, bf16, one GPU), all through the same engine: prefill = S fresh prompts of L tokens in one step, decode = B sequences at
context C, one token each per step (hipGraph replay).  ``bench.py --decoder-bench`` runs this.

    python benchmarks/decoder_bench.py [--sizes 1024,2048,4096] [--models lebepel,llama] [--json-out FILE]

One JSON line per (size, model), then a table.  Per-kernel times come from running it under
``rocprofv3 --kernel-trace --stats`` with ``--sizes`` set to one size.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

# width -> (layers, heads, kv heads, head size, feed-forward, ssm heads, ssm head size P, state N, groups)
SIZES = {
    1024: (8, 8, 2, 128, 2816, 32, 64, 64, 4),
    2048: (8, 16, 4, 128, 5632, 64, 64, 128, 8),
    4096: (4, 32, 8, 128, 14336, 128, 64, 128, 8),
}
VOCAB = 32768


def models(width: int, which: str, device):
    from llm_kubernetes_minikube_sharp4dev_amd.models import build_decoder
    from llm_kubernetes_minikube_sharp4dev_amd.models.configs import (FusasunConfig, LebepelConfig, LumedraConfig, PemidraConfig,
                                                                      decoder_config, fusasun_layers, lebepel_layers, lumedra_layers,
                                                                      pemidra_layers)

    L, H, G, D, FF, sh, sp, sn, sg = SIZES[width]
    if which == "lebepel":
        cfg = LebepelConfig(f"lebepel-w{width}", VOCAB, width, lebepel_layers(L, width, H, G, D, FF, sh, sp, sn, sg, 4, sg),
                            max_position=8192, residual_mult=0.5, logit_softcap=30.0)
    elif which == "pemidra":
        # general_delta / retention / parallel (attention in chunks of 256 beside a gated delta rule, with the
        # feed-forward) in turn; the same heads and head size for every mixer, two-layer projections of rank 128
        cfg = PemidraConfig(f"pemidra-w{width}", VOCAB, width, pemidra_layers(L, H, D, FF, kv_heads=G, chunk=256, lora=128),
                            postln_alpha=2.0)
    elif which == "fusasun":
        # pooled-window attention (window 512, blocks of 64) and latent attention (window 512, latent 512 + 64 rotated)
        # in turn, the same heads and head size; 16 experts of half the dense feed-forward, two per token: the
        # products a token runs are those of the dense model
        cfg = FusasunConfig(f"fusasun-w{width}", VOCAB, width,
                            fusasun_layers(L, H, D, FF // 2, 16, 2, kv_heads=G, window=512, pool=64, rot_dim=64,
                                           q_rank=max(512, width // 2), kv_rank=512), embed_scale=1.0, canon_taps=4)
    elif which == "lumedra":
        # capped-window attention (window 512 + 4 kept positions, values blended), causal latent attention (latent 512 + 64
        # rotated) and lightning attention in turn, the same heads and head size; the first feed-forward dense, the others 16
        # experts of a quarter of it in 4 groups (2 kept), two per token, beside a shared expert of half of it: the products a
        # token runs are those of the dense model
        cfg = LumedraConfig(f"lumedra-w{width}", VOCAB, width,
                            lumedra_layers(L, H, D, FF // 4, 16, 2, kv_heads=G, window=512, keep_first=4, rot_dim=64,
                                           q_rank=max(512, width // 2), kv_rank=512, groups=4, keep=2, shared_ff=FF // 2))
        cfg.layers[0].mlp["ff"] = FF
    else:
        cfg = decoder_config("llama-3-8b", num_layers=L, hidden=width, num_heads=H, num_kv_heads=G, head_dim=D,
                             intermediate=FF, vocab_size=VOCAB, max_position=8192)
        cfg.name = f"llama-w{width}"
    return build_decoder(cfg, device=device, seed=0)


def run(width: int, which: str, a) -> dict:
    import torch

    from llm_kubernetes_minikube_sharp4dev_amd.engine.llm_engine import LLMEngine
    from llm_kubernetes_minikube_sharp4dev_amd.engine.sampling import SamplingParams

    dev = torch.device("cuda", 0)
    m = models(width, which, dev)
    B = a.decode_batch
    eng = LLMEngine(m, None, max_model_len=8192, max_num_seqs=max(B, a.prefill_seqs), kv_cache_gb=8,
                    max_num_batched_tokens=a.prefill_seqs * a.prefill_len, enable_prefix_caching=False, eos_ids=set(),
                    token_align=1, prefill_hold=0)
    g = torch.Generator().manual_seed(1)
    prompt = lambda n: torch.randint(0, VOCAB, (n,), generator=g).tolist()
    # ---- prefill: S prompts of L tokens, one generated token each: one engine step per round
    pre = []
    for r in range(a.rounds + 1):
        seqs = [eng.add_request(prompt(a.prefill_len), SamplingParams.greedy(1)) for _ in range(a.prefill_seqs)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.run_until_done(seqs)
        torch.cuda.synchronize()
        if r:
            pre.append(time.perf_counter() - t0)
    # ---- decode: B sequences at context C, timed single-token steps
    seqs = [eng.add_request(prompt(a.context), SamplingParams.greedy(a.decode_steps + 8)) for _ in range(B)]
    while any(len(s.output_ids) < 4 for s in seqs):   # prompts in, graphs captured, a few decode steps warm
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n0 = sum(len(s.output_ids) for s in seqs)
    for _ in range(a.decode_steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ntok = sum(len(s.output_ids) for s in seqs) - n0
    for s in seqs:
        eng.abort(s.req_id)
    captured = [k for k, st in eng.runner.graphs.items() if st.get("graph") is not None]
    return {"model": m.cfg.name, "width": width, "layers": m.cfg.num_layers,
            "prefill_tokens_per_s": a.prefill_seqs * a.prefill_len / statistics.median(pre),
            "prefill_ms": 1e3 * statistics.median(pre), "prefill_rows": a.prefill_seqs * a.prefill_len,
            "decode_tokens_per_s": ntok / dt, "decode_ms_per_step": 1e3 * dt / a.decode_steps, "decode_batch": B,
            "context": a.context, "decode_graphs": len(captured), "dtype": "bf16", "data": "synthetic"}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="1024,2048,4096")
    ap.add_argument("--models", default="lebepel,llama", help="comma list of lebepel, pemidra, fusasun, lumedra, llama")
    ap.add_argument("--prefill-seqs", type=int, default=4)
    ap.add_argument("--prefill-len", type=int, default=1024)
    ap.add_argument("--decode-batch", type=int, default=64)
    ap.add_argument("--context", type=int, default=1024)
    ap.add_argument("--decode-steps", type=int, default=32)
    ap.add_argument("--rounds", type=int, default=3)
    ap.add_argument("--json-out", default=None)
    a = ap.parse_args(argv)
    rows = []
    for w in (int(x) for x in a.sizes.split(",")):
        for which in a.models.split(","):
            r = run(w, which, a)
            rows.append(r)
            print(json.dumps(r), flush=True)
    print(f"{'model':18s} {'prefill tok/s':>14s} {'ms':>8s} {'decode tok/s':>13s} {'ms/step':>8s}", file=sys.stderr)
    for r in rows:
        print(f"{r['model']:18s} {r['prefill_tokens_per_s']:14.0f} {r['prefill_ms']:8.2f} {r['decode_tokens_per_s']:13.0f} "
              f"{r['decode_ms_per_step']:8.3f}", file=sys.stderr)
    if a.json_out:
        with open(a.json_out, "w") as f:
            json.dump(rows, f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
