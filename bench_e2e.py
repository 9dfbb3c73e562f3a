"""End-to-end sparse generation at Qwen3-4B shape (the end-to-end benchmark configuration): random-init bf16 weights,
36 layers, routing on the upper 18, a synthetic pooled memory bank, top-16 documents, a 4K-token
local context per query, batch 16, greedy decoding.

    python bench_e2e.py [--bank-tokens 10000000] [--batch 16] [--context 4096] [--steps 256]

Prints one JSON line with prefill time and decode tokens/s.  The bank is synthetic at the pooled
level (N(0,1) rows, K_r L2-normalised): encoding 10M tokens through a 4B-parameter model is not part
of what this measures.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import numpy as np
import torch

import os

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from msa_amd.config import GenerateConfig, MemoryConfig, ModelConfig, MSAConfig
from msa_amd.model import MSAForCausalLM, encode_block
from msa_amd.msa_service import MSAService
from msa_amd.prefill import Document, num_chunks, prepare_block_inputs


def build_service(cfg: MSAConfig, bank_tokens: int, seed: int = 0) -> MSAService:
    dev = torch.device("cuda:0")
    P = cfg.msa_config.pooling_kernel_size
    g = np.random.default_rng(seed)
    lens, left = [], bank_tokens
    while left > 0:
        n = min(int(g.integers(256, 2049)), left)
        lens.append(n)
        left -= n
    docs = [Document(doc_id=i, num_chunks=num_chunks(n, P)) for i, n in enumerate(lens)]
    C = sum(d.num_chunks for d in docs)
    Hkv, D = cfg.num_key_value_heads, cfg.head_dim
    svc = MSAService(0, GenerateConfig(devices=[0]),
                     ModelConfig(doc_top_k=cfg.msa_config.top_k_docs, pooling_kernel_size=P,
                                 router_layer_idx=cfg.msa_config.router_layer_idx),
                     MemoryConfig(pooling_kernel_size=P), cfg)
    tg = torch.Generator(device=dev).manual_seed(seed)
    rk, k, v = {}, {}, {}
    for layer in svc.router_layer_ids:
        x = torch.randn((C, Hkv, D), generator=tg, device=dev)
        rk[layer] = (x / x.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
        for store in (k, v):
            h = torch.empty((C, Hkv, D), dtype=torch.bfloat16, pin_memory=True)
            h.copy_(torch.randn((C, Hkv, D), generator=tg, device=dev).to(torch.bfloat16))
            store[layer] = h
    prefix = {l: (torch.randn((1, Hkv, 3, D), generator=tg, device=dev).to(torch.bfloat16),
                  torch.randn((1, Hkv, 3, D), generator=tg, device=dev).to(torch.bfloat16))
              for l in range(cfg.num_hidden_layers)}
    svc.load_pooled(docs, rk, k, v, prefix)
    return svc


def time_stage1(model: MSAForCausalLM, cfg: MSAConfig, tokens: int, seed: int = 1) -> dict:
    """Stage 1 (encode) of one packed block of ragged documents, lengths U[256, 2048]: document-wise causal attention
    and the pooled K / V / K_r of every layer.  Returns the second run's time (the first pays allocator warm-up)."""
    dev = next(model.parameters()).device
    g = np.random.default_rng(seed)
    docs, left = [], tokens
    while left > 0:
        n = min(int(g.integers(256, 2049)), left)
        docs.append(Document(doc_id=len(docs), input_ids=g.integers(0, cfg.vocab_size, size=n).tolist()))
        left -= n
    blk = prepare_block_inputs(docs, [1, 2, 3], cfg.msa_config.pooling_kernel_size)
    dt = 0.0
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cache = encode_block(model, blk, dev)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        del cache
    return {"block_tokens": tokens, "documents": len(docs), "seconds": round(dt, 4), "tokens_per_s": round(tokens / dt)}


def main(argv=None, quiet: bool = False):
    """Runs the workload and prints one JSON line (``quiet`` only returns the dict)."""
    ap = argparse.ArgumentParser()
    ap.add_argument("--bank-tokens", type=int, default=10_000_000)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--encode-tokens", type=int, default=32768,
                    help="also time stage 1 (encode) on one packed block of this many tokens; 0 skips it")
    ap.add_argument("--encode-only", action="store_true", help="time stage 1 (encode) and stop: no bank, no decode")
    ap.add_argument("--eager", action="store_true", help="do not capture the decode step as a HIP graph")
    ap.add_argument("--verify-graph", type=int, default=0, metavar="N",
                    help="also decode N steps eagerly and require identical tokens from the graph replays")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("bench_e2e: no GPU visible; the HIP path has no CPU fallback")
    dev = torch.device("cuda:0")
    cfg = MSAConfig(num_hidden_layers=args.layers)
    if args.layers != 36:
        half = args.layers // 2
        cfg.msa_config.router_layer_idx = ",".join(str(i) for i in range(half, args.layers))
    t0 = time.perf_counter()
    with torch.device(dev):
        model = MSAForCausalLM(cfg).to(torch.bfloat16)
    model.init_random_(0.02, seed=0).eval()
    if args.encode_only:
        out = {"metric": "stage-1 encode tokens/s (one packed block)", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
               "config": {"workload": "Qwen3-4B shape, random init, ragged documents U[256, 2048]", "layers": args.layers},
               **time_stage1(model, cfg, max(args.encode_tokens, 1024))}
        out["value"] = out["tokens_per_s"]
        if not quiet:
            print(json.dumps(out), flush=True)
        return out
    svc = build_service(cfg, args.bank_tokens)
    svc.setup_memory_client(model)
    for layer in model.model.layers:
        layer.self_attn.decode_reserve = args.steps + 8
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    stage1 = time_stage1(model, cfg, args.encode_tokens) if args.encode_tokens > 0 else None
    g = torch.Generator(device=dev).manual_seed(3)
    B, S = args.batch, args.context
    ids = torch.randint(0, cfg.vocab_size, (B, S), generator=g, device=dev)
    mask = torch.ones((B, S), dtype=torch.long, device=dev)
    doc_ids = torch.zeros((B, S), dtype=torch.long, device=dev)
    model.generate_greedy(ids[:, :64].contiguous(), mask[:, :64].contiguous(), doc_ids[:, :64].contiguous(), 4)   # warm-up
    timings = {}
    toks, cache = model.generate_greedy(ids, mask, doc_ids, args.steps, require_recall_topk=True, timings=timings,
                                        use_graph=not args.eager)
    verified = None
    if args.verify_graph:
        ref, _ = model.generate_greedy(ids, mask, doc_ids, args.verify_graph, use_graph=False)
        verified = bool(torch.equal(ref, toks[:, :args.verify_graph]))
        if not verified:
            diff = ref != toks[:, :args.verify_graph]
            first = int(diff.any(dim=0).nonzero()[0])
            sys.exit(f"bench_e2e: graph replays and eager decoding produced different tokens: first at step {first}, "
                     f"{int(diff.any(dim=1).sum())} of {B} samples differ")
    last_router = svc.router_layer_ids[-1]
    kv = cache.cache_kwargs[last_router]["kv_lengths"].cpu().tolist()
    out = {"metric": "sparse decode tok/s (end to end, greedy)", "value": round(B * timings["decode_steps"] / timings["decode_s"], 1),
           "unit": "tokens/s", "ms_per_decode_step": round(timings["decode_s"] / timings["decode_steps"] * 1e3, 3),
           "prefill_s": round(timings["prefill_s"], 3), "setup_s": round(setup_s, 1), "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "configs[4]: Qwen3-4B shape, random init, routing on the upper half of the layers",
                      "layers": args.layers, "bank_tokens": args.bank_tokens, "batch": B, "context_tokens": S,
                      "decode_steps": args.steps, "top_k": cfg.msa_config.top_k_docs,
                      "kv_rows_last_router_layer": kv[:4]},
           "stage1_encode": stage1,
           "decode_mode": "eager" if args.eager else "hip graph replay", "graph_equals_eager": verified,
           "generated_shape": list(toks.shape)}
    del model, svc, cache
    if not quiet:
        print(json.dumps(out), flush=True)
    return out


if __name__ == "__main__":
    main()
