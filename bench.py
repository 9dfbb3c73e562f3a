#!/usr/bin/env python3
"""Benchmark of the MSA routing hot path on one MI355X.

A step is one routed batch at the 100M-token bank: B = 16 queries of S = 128 tokens scored against
the HBM-resident pooled K_r of each of 18 routed layers (cosine, mean over 32 heads, max over
tokens, max over a document's chunks), top-16 documents per query and layer, and the selected
documents' pooled K / V copied from pinned host memory on a side stream while the next layer is
being scored.  Inputs are synthetic (seeded), resident in HBM / pinned memory before timing starts.

Prints ONE JSON line: routed queries/s, plus the roofline of the dominant kernel (the scoring
kernel, timed with HIP event pairs around each of its launches on its own stream) and the CPU
baseline (the reference's torch op sequence on a bounded slice of the same bank, host cores).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
HQ, HKV, D, P, TOPK = 32, 8, 128, 64, 16
PROFILES = os.path.join(ROOT, "profiles")


def measured_traffic(kernel: str, workload: str):
    """Bytes past L2 per launch of `kernel` at `workload`, from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    summaries under profiles/: a line `TRAFFIC kernel=<k> workload=<w> fetch_kib=<n> write_kib=<n> fetch_scale=<f>
    write_scale=<f>` (KiB per dispatch and the factors a plain device copy of known size gives for the same
    counters).  None when no summary covers the workload."""
    try:
        names = sorted(os.listdir(PROFILES))
    except OSError:
        return None
    for name in names:
        if not name.endswith((".txt", ".md")):
            continue
        for line in open(os.path.join(PROFILES, name), errors="replace"):
            if not line.startswith("TRAFFIC "):
                continue
            kv = dict(f.split("=", 1) for f in line.split()[1:] if "=" in f)
            if kv.get("kernel") == kernel and kv.get("workload") == workload:
                return (float(kv["fetch_scale"]) * float(kv["fetch_kib"]) + float(kv["write_scale"]) * float(kv["write_kib"])) * 1024
    return None


def traffic_source(kernel: str, workload: str):
    """Where measured_traffic()'s figure comes from: the committed profile summary (an earlier rocprofv3 --pmc run,
    not this run) that holds the matching TRAFFIC line, or None."""
    try:
        names = sorted(os.listdir(PROFILES))
    except OSError:
        return None
    for name in names:
        if name.endswith((".txt", ".md")):
            for line in open(os.path.join(PROFILES, name), errors="replace"):
                if line.startswith("TRAFFIC ") and f"kernel={kernel} " in line and f"workload={workload} " in line:
                    return f"profiles/{name} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run, scaled by a plain copy)"
    return None


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def make_doc_lens(total_tokens: int, seed: int):
    g = np.random.default_rng(seed)
    lens, left = [], total_tokens
    while left > 0:
        n = int(g.integers(256, 2049))
        n = min(n, left)
        lens.append(n)
        left -= n
    return lens


def build_kr_layer(C_total: int, seed: int, device) -> torch.Tensor:
    """N(0,1) rows L2-normalised per (chunk, head), bf16, generated on the device slice by slice."""
    g = torch.Generator(device=device).manual_seed(seed)
    kr = torch.empty((C_total, HKV, D), dtype=torch.bfloat16, device=device)
    step = 1 << 17
    for s in range(0, C_total, step):
        e = min(C_total, s + step)
        x = torch.randn((e - s, HKV, D), generator=g, device=device)
        kr[s:e] = (x / x.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
    return kr


def plant_needles(kr, q, doc_chunk_off, n_docs, seed):
    """For every query plants TOPK documents whose middle chunk has, per KV head, cosine 0.98, 0.955,
    ... with the pre-summed heads of one query token (the remainder is the chunk's own noise made
    orthogonal to it).  The planted scores are cos * mean_g |sum of the group's unit heads| / 4,
    about 0.49 * cos, so ranks are separated by ~1e-2 (>> the 1e-3 contract gap) and far above the
    ~0.06 of un-planted chunks.  Returns the expected [B, TOPK] document ids in rank order."""
    B, S = q.shape[0], q.shape[1]
    g = np.random.default_rng(seed)
    want = np.zeros((B, TOPK), dtype=np.int64)
    used = set()
    toks, cs = [], []
    for b in range(B):
        toks.append(int(g.integers(0, S)))
        docs = []
        while len(docs) < TOPK:
            d = int(g.integers(0, n_docs))
            if d not in used:
                used.add(d)
                docs.append(d)
        for r, d in enumerate(docs):
            cs.append((int(doc_chunk_off[d]) + int(doc_chunk_off[d + 1])) // 2)
            want[b, r] = d
    # all B * TOPK chunks in one batch of device operations (the planted chunks are distinct)
    dev = kr.device
    qt = q[torch.arange(B, device=dev), torch.tensor(toks, device=dev)].float()                 # [B, HQ, D]
    qn = (qt / qt.norm(dim=-1, keepdim=True)).view(B, HKV, HQ // HKV, D).sum(2)
    direction = (qn / qn.norm(dim=-1, keepdim=True)).repeat_interleave(TOPK, dim=0)           # [B * TOPK, HKV, D]
    cos = (0.98 - 0.025 * torch.arange(TOPK, device=dev, dtype=torch.float32)).repeat(B).view(-1, 1, 1)
    idx = torch.tensor(cs, device=dev)
    noise = kr[idx].float()
    perp = noise - (noise * direction).sum(-1, keepdim=True) * direction
    perp = perp / perp.norm(dim=-1, keepdim=True)
    kr[idx] = (cos * direction + (1 - cos * cos).sqrt() * perp).to(torch.bfloat16)
    return want


def cpu_baseline(kr0, q0, doc_chunks, budget_s=25.0):
    """Reference op sequence (oracle.reference_style) on the first ~200k chunks of the bank (about
    10 s of work per dtype on 16 cores), on the host cores, extrapolated linearly in chunks and
    layers to the whole routed batch."""
    from oracle import reference_style as rs
    C_total = int(sum(doc_chunks))
    target = min(C_total, 200_000)
    n, acc = 0, 0
    while n < len(doc_chunks) and acc < target:
        acc += doc_chunks[n]
        n += 1
    sub_chunks = doc_chunks[:n]
    Cs = int(sum(sub_chunks))
    pool_ids = torch.repeat_interleave(torch.arange(1, n + 1), torch.as_tensor(sub_chunks))
    out = {}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        rk = kr0[:Cs].to("cpu").to(dt).transpose(0, 1).unsqueeze(0).contiguous()       # [1, Hkv, Cs, D]
        qh = torch.nn.functional.normalize(q0.to("cpu").to(dt).permute(0, 2, 1, 3).contiguous(), p=2, dim=-1)
        q5, m5 = rs.group_queries(qh, torch.ones(qh.shape[0], qh.shape[2], dtype=torch.bool), HQ // HKV, -1.0)
        t0 = time.perf_counter()
        rs.stage2_scores_topk(q5, m5, rk, pool_ids, sub_chunks, TOPK)
        dt_s = time.perf_counter() - t0
        out[name] = dt_s
        if dt_s > budget_s:
            break
    return out, Cs


def time_cuda(fn, reps, warm=2):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / reps


def extra_pooling(dev):
    """configs[1]: chunk-mean pooling of K (rotated in the kernel), V and K_r (normalised) over 1M tokens of
    ragged documents, bf16, 8 KV heads x 128, chunk 64; one layer per launch."""
    from msa_amd import ops
    lens = make_doc_lens(1_000_000, 1)
    T = sum(lens)
    g = torch.Generator(device=dev).manual_seed(11)
    k, v, kr = (torch.randn((T, HKV, D), generator=g, device=dev).to(torch.bfloat16) for _ in range(3))
    table = ops.chunk_table(lens, P, device=dev)
    rope = ops.rope_tables(2048, D, 1e6, device=dev)
    ms = time_cuda(lambda: ops.pool_chunks(k, v, kr, table, rope=rope, normalize_kr=True), 10)
    by = 3 * T * HKV * D * 2 + 3 * table.C * HKV * D * 2
    return {"workload": "configs[1]: 1M tokens, docs U[256,2048], K (RoPE fused) + V + K_r (normalised), bf16",
            "tokens": T, "chunks": table.C, "ms_per_layer": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
            "frac_hbm": round(by / ms / 1e6 / HBM_PEAK_GBS, 4), "tokens_per_s": round(T / ms * 1e3)}


def extra_decode(dev):
    """configs[4] attention share: one decode step of one layer, B=16, 32 Q / 8 KV heads, context
    3 + 16 docs x 18 chunks + 4096 local tokens, bf16, cache appended in place."""
    from msa_amd import ops
    B, L = 16, 3 + 288 + 4096
    Lcap = L + 64
    g = torch.Generator(device=dev).manual_seed(12)
    kc = torch.randn((B, Lcap, HKV, D), generator=g, device=dev).to(torch.bfloat16)
    vc = torch.randn((B, Lcap, HKV, D), generator=g, device=dev).to(torch.bfloat16)
    q = torch.randn((B, HQ, D), generator=g, device=dev).to(torch.bfloat16)
    kn, vn = q[:, :HKV].contiguous(), q[:, HKV:2 * HKV].contiguous()
    kv_off = torch.arange(B, dtype=torch.int64, device=dev) * Lcap
    kv_len = torch.full((B,), L, dtype=torch.int32, device=dev)

    def step():                       # the context grows by one row per step, as in a real decode
        ops.cache_append(kn, vn, kc, vc, kv_len)
        ops.sparse_attn(q, kc.view(-1, HKV, D), vc.view(-1, HKV, D), kv_off, kv_len, Lcap)
    ms = time_cuda(step, 20)
    by = 2 * B * (L + 12) * HKV * D * 2        # mean context over the 22 steps run
    # the form the end-to-end decode uses: q/k norm + rotary + append + attention from the fused projection output,
    # replayed from a HIP graph (no Python launch cost between the two kernels)
    kv_len.fill_(L)
    qkv = torch.randn((B, (HQ + 2 * HKV) * D), generator=g, device=dev).to(torch.bfloat16)
    pos = torch.full((B,), L, dtype=torch.int64, device=dev)
    nw = torch.ones((D,), device=dev, dtype=torch.bfloat16)
    rope = ops.rope_tables(8192, D, 1e6, device=dev)

    def fused():
        ops.decode_attn_fused(qkv, HQ, HKV, D, pos, nw, nw, 1e-6, rope, kc, vc, kv_len)
    fused()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fused()
    ms_fused = time_cuda(graph.replay, 20)
    return {"workload": "configs[4] attention share: 1 layer-step, B=16, L=4388, GQA 32/8, bf16",
            "ms_per_layer_step": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
            "frac_hbm": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
            "attention_only_tok_per_s_36_layers": round(B / (36 * ms) * 1e3),
            "fused_norm_rope_append_attention_in_graph": {"ms_per_layer_step": round(ms_fused, 4),
                                                          "GB/s": round(by / ms_fused / 1e6, 1),
                                                          "frac_hbm": round(by / ms_fused / 1e6 / HBM_PEAK_GBS, 4)}}


def extra_mfma_ceiling(dev):
    """What the matrix cores sustain with nothing but MFMAs running (a register-only loop at the scoring kernel's
    occupancy): the rate with operands that toggle is the ceiling the scoring kernel's fraction can be read against."""
    from msa_amd import _lib
    lib = _lib.load()
    wgs, iters = 256 * 4, 20000
    sink = torch.empty(wgs * 512, dtype=torch.float32, device=dev)
    flops = C.c_double(0)
    out = {"workload": f"register-only v_mfma_f32_32x32x16_bf16 loop, {wgs} workgroups x 8 wavefronts x {iters} x 8 MFMAs"}
    # mode + 16 * extra: other VALU work per 8 MFMAs (what the attention kernel's softmax asks of the issue port)
    for mode, name in ((0, "zero_operands"), (2, "toggling_operands"), (16, "zero_operands_plus_24_fma"),
                       (32, "zero_operands_plus_48_fma"), (48, "zero_operands_plus_24_exp"), (64, "zero_operands_plus_48_exp"),
                       (80, "zero_operands_plus_24_cvt_pk_bf16"), (96, "zero_operands_plus_24_dot2c_bf16"),
                       (112, "zero_operands_plus_24_max3")):
        ms = []
        for rep in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _lib.check(lib.msa_diag_mfma_loop(wgs, iters, mode, sink.data_ptr(), C.byref(flops), torch.cuda.current_stream().cuda_stream),
                       "msa_diag_mfma_loop")
            b.record()
            torch.cuda.synchronize()
            ms.append(a.elapsed_time(b))
        best = min(ms[1:])
        out[name] = {"ms": round(best, 3), "TFLOP/s": round(flops.value / best / 1e9, 1),
                     "frac_mfma_peak": round(flops.value / best / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}
    return out


def extra_hbm_read_ceiling(dev):
    """What the memory system gives loops that only read, in the access patterns of the HBM-bound kernels: the rates the
    pooling and decode-attention fractions can be read against (the published 8 TB/s is not reached by any read loop)."""
    from msa_amd import _lib
    lib = _lib.load()
    nbytes = 4 << 30
    src = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
    src.random_(0, 1 << 31)
    dst = torch.empty(nbytes // 64 // 4, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    out = {"workload": "read-only loops over 4 GiB (rows of 2 KB), best of 3 x 5 launches"}
    for mode, name in ((0, "rows_nontemporal (pooling's reads)"), (1, "rows_plus_2KB_store_per_128KB (pooling's reads and writes)"),
                       (2, "one_head_256B_pieces_2KB_apart (decode attention's reads)")):
        def run():
            _lib.check(lib.msa_diag_read_stream(src.data_ptr(), nbytes, dst.data_ptr(), mode, st), "msa_diag_read_stream")
        ms = min(time_cuda(run, 5, warm=2) for _ in range(3))
        out[name] = {"ms": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    # launches of a decode layer-step's size (the K and V rows of 16 samples x 4400 tokens = 288 MB) over 14 distinct
    # pieces of the buffer, back to back: what a launch that short gets, start and end included
    piece = 16 * 4400 * 2 * 2048 // 131072 * 131072
    for mode, name in ((0, "rows_nontemporal, 288 MB per launch"), (2, "one_head_256B_pieces_2KB_apart, 288 MB per launch")):
        def run():
            for i in range(nbytes // piece):
                _lib.check(lib.msa_diag_read_stream(src.data_ptr() + i * piece, piece, dst.data_ptr(), mode, st), "msa_diag_read_stream")
        ms = min(time_cuda(run, 3, warm=1) for _ in range(3)) / (nbytes // piece)
        out[name] = {"us": round(ms * 1e3, 2), "GB/s": round(piece / ms / 1e6, 1), "frac_hbm": round(piece / ms / 1e6 / HBM_PEAK_GBS, 4)}
    return out


def extra_decode_projections(dev):
    """configs[4] projection share: the four weight-streaming linears of a decode layer and the LM head at B=16
    (Qwen3-4B shapes, bf16), each replayed from a HIP graph over distinct weight copies so that neither the Python
    launch cost nor the Infinity Cache flatter the number (a launch inside the graph costs about 4 us whatever its
    work, which is most of the small matrices' distance from the HBM peak)."""
    from msa_amd import ops
    M, H, I, V = 16, 2560, 9728, 151936
    g = torch.Generator(device=dev).manual_seed(14)
    shapes = [("qkv (norm folded)", 6144, H, "norm"), ("o_proj (+residual)", H, 4096, "res"),
              ("gate/up (norm, silu-mul)", 2 * I, H, "silu"), ("down_proj (+residual)", H, I, "res"),
              ("lm_head (norm folded)", V, H, "norm")]
    out = {}
    for name, N, K, kind in shapes:
        copies = 2 if N * K * 2 > (300 << 20) else 10
        ws = [(torch.randn((N, K), generator=g, device=dev) * K ** -0.5).to(torch.bfloat16) for _ in range(copies)]
        x = torch.randn((M, K), generator=g, device=dev).to(torch.bfloat16)
        nw = torch.ones((K,), device=dev, dtype=torch.bfloat16)
        res = torch.zeros((M, N), device=dev, dtype=torch.bfloat16)

        def run():
            for w in ws:
                if kind == "norm":
                    ops.skinny_linear(x, w, norm_weight=nw, eps=1e-6)
                elif kind == "silu":
                    ops.skinny_linear(x, w, silu_mul=True, norm_weight=nw, eps=1e-6)
                else:
                    ops.skinny_linear(x, w, residual=res)
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        us = time_cuda(graph.replay, 5) * 1e3 / copies
        by = N * K * 2
        out[name] = {"N": N, "K": K, "us": round(us, 2), "GB/s": round(by / us / 1e3, 1),
                     "frac_hbm": round(by / us / 1e3 / HBM_PEAK_GBS, 4)}
        del ws
    return {"workload": "configs[4] projection share: weight-streaming linears of one decode layer + LM head, B=16, bf16",
            "kernels": out}


def extra_routing_10m(dev):
    """configs[2]: router scoring + top-k on a 10M-token bank (about 156k chunks), batch 32 x 128 query tokens,
    top-16, one routed layer per call (the 18 layers of a model cost 18 of these)."""
    from msa_amd import ops
    B, S = 32, 128
    doc_chunks = [-(-n // P) for n in make_doc_lens(10_000_000, 2)]
    off = np.concatenate([[0], np.cumsum(doc_chunks)])
    bank = ops.Bank(1, off.tolist(), list(range(len(doc_chunks))), HKV, D, torch.bfloat16)
    kr = build_kr_layer(int(off[-1]), 21, dev)
    bank.set_layer(0, kr)
    g = torch.Generator(device=dev).manual_seed(22)
    q = torch.randn((B, S, HQ, D), generator=g, device=dev).to(torch.bfloat16)
    ms = time_cuda(lambda: ops.route_topk(bank, 0, q, None, "cosine", 1.0, TOPK), 10)
    fl = 2.0 * B * S * HKV * D * int(off[-1])
    return {"workload": "configs[2]: 10M-token bank, B=32 x S=128, top-16, bf16, one layer",
            "chunks": int(off[-1]), "docs": len(doc_chunks), "ms_per_layer": round(ms, 4),
            "queries_per_s_18_layers": round(B / (18 * ms) * 1e3, 1), "TFLOP/s": round(fl / ms / 1e9, 1),
            "frac_mfma_peak": round(fl / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}


def extra_prefill_attention(dev):
    """Stage-2 prefill attention of the end-to-end shape: B=16 queries of 4096 tokens over
    [3 + 288 memory rows | the 4096 query tokens], causal, GQA 32/8, bf16 (MFMA flash kernel)."""
    from msa_amd import ops
    B, S, M = 16, 4096, 3 + 288
    L = M + S
    g = torch.Generator(device=dev).manual_seed(13)
    q = torch.randn((B * S, HQ, D), generator=g, device=dev).to(torch.bfloat16)
    kc = torch.randn((B * L, HKV, D), generator=g, device=dev).to(torch.bfloat16)
    vc = torch.randn((B * L, HKV, D), generator=g, device=dev).to(torch.bfloat16)
    kv_off = torch.arange(B, dtype=torch.int64, device=dev) * L
    kv_len = torch.full((B,), L, dtype=torch.int32, device=dev)
    cu_q = (torch.arange(B + 1, dtype=torch.int32, device=dev) * S)
    from msa_amd import _lib
    lib = _lib.load()
    run = lambda: ops.sparse_attn(q, kc, vc, kv_off, kv_len, L, cu_q=cu_q, max_sq=S, causal=True)
    # (ten warm-up launches each: the chip's power management takes about that long to settle on a kernel's load)
    ms = time_cuda(run, 10, warm=10)
    # the 32-column form of the kernel in the same process, for comparison (the call above picks the wide form)
    _lib.check(lib.msa_flash_set_form(1), "msa_flash_set_form")
    try:
        ms32 = time_cuda(run, 10, warm=10)
    finally:
        _lib.check(lib.msa_flash_set_form(0), "msa_flash_set_form")
    pairs = B * (S * M + S * (S + 1) // 2)
    fl = 4.0 * pairs * HQ * D
    return {"workload": "stage-2 prefill attention: B=16 x 4096 query tokens over 4387 keys, causal, GQA 32/8, bf16",
            "kernel": "flash_wide_kernel", "ms_per_layer": round(ms, 3), "TFLOP/s": round(fl / ms / 1e9, 1),
            "frac_mfma_peak": round(fl / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "columns32_form_ms": round(ms32, 3), "columns32_form_frac": round(fl / ms32 / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--tokens", type=int, default=100_000_000, help="bank size in tokens")
    ap.add_argument("--layers", type=int, default=18, help="routed layers resident in HBM")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--seq", type=int, default=128)
    ap.add_argument("--host-kv-layers", type=int, default=0,
                    help="distinct pinned host K/V layer buffers (routed layers share them round-robin); 0: as many as "
                         "the box pins, up to 8 (the boxes of this pool refuse pinned memory past about 56 GB, i.e. the "
                         "17th 3.3 GB buffer at the 100M-token bank)")
    ap.add_argument("--gather", choices=["device", "fused", "memcpy"], default="fused",
                    help="device: plan + copy kernels read the pinned bank directly, no ids on the host; "
                         "fused: the same plan + copy inside the next layer's scan launch (one workgroup of it); "
                         "memcpy: ids to the host, one hipMemcpyAsync per document run")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--sweep-only", action="store_true",
                    help="run the bandwidth-regime sweep (one query per scan) and stop; with --layers 1 this is the "
                         "short run the rocprofv3 summaries of that regime come from")
    ap.add_argument("--no-extras", action="store_true", help="skip the pooling and decode-attention side measurements")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end sparse decode run among the extras")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (reference point for rocprof FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--ceiling-only", action="store_true",
                    help="run only the register-only MFMA loop (other_kernels.mfma_ceiling) and print its figures")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no sharding, no collectives); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")

    from msa_amd import _lib, ops
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.ceiling_only:
        print(json.dumps({"mfma_ceiling": extra_mfma_ceiling(dev)}), flush=True)
        return
    B, S, L = args.batch, args.seq, args.layers

    t_setup = time.perf_counter()
    doc_lens = make_doc_lens(args.tokens, 0)
    doc_chunks = [(n + P - 1) // P for n in doc_lens]
    doc_chunk_off = np.concatenate([[0], np.cumsum(doc_chunks)]).astype(np.int64)
    n_docs, C_total = len(doc_lens), int(doc_chunk_off[-1])
    log(f"bank: {args.tokens} tokens, {n_docs} docs, {C_total} chunks, {L} layers, "
        f"{C_total * HKV * D * 2 * L / 1e9:.1f} GB of K_r")
    bank = ops.Bank(L, doc_chunk_off.tolist(), list(range(n_docs)), HKV, D, torch.bfloat16)

    # Pinned host K / V: distinct layer buffers, filled from the device.  The configuration names pinned K / V for
    # every routed layer; this pool's boxes refuse pinned allocations past about 56 GB, so the bench takes as many
    # layer buffers as the box pins (each K + V pair is allocated before it counts; one buffer of head room is kept
    # below the point of refusal), up to 8 by default, and the routed layers share them round-robin.
    auto = args.host_kv_layers <= 0
    n_want = max(1, min(8 if auto else args.host_kv_layers, L))
    buf_gb = C_total * HKV * D * 2 / 1e9
    host_k, host_v, refused_at_gb = [], [], None
    for i in range(n_want):
        try:
            pair = [torch.empty((C_total, HKV, D), dtype=torch.bfloat16, pin_memory=True) for _ in range(2)]
        except RuntimeError as e:
            refused_at_gb = round((2 * len(host_k) + 1) * buf_gb, 1)
            log(f"host K/V: pinned allocation refused at about {refused_at_gb} GB ({str(e).splitlines()[0][:80]})")
            pair = None
            if len(host_k) > 1:           # head room: give the last pair back
                host_k.pop(); host_v.pop()
            break
        host_k.append(pair[0]); host_v.append(pair[1])
    pair = None
    if not host_k:
        sys.exit("bench.py: could not pin one layer of host K / V")
    n_host = len(host_k)
    for i in range(n_host):
        for h, seed in ((host_k[i], 1000 + i), (host_v[i], 2000 + i)):
            g = torch.Generator(device=dev).manual_seed(seed)
            step = 1 << 18
            for s0 in range(0, C_total, step):
                e0 = min(C_total, s0 + step)
                h[s0:e0].copy_(torch.randn((e0 - s0, HKV, D), generator=g, device=dev).to(torch.bfloat16))
        if n_host > 2:
            log(f"host K/V: layer buffer {i + 1} of {n_host} filled")
    pinned_gb = round(2 * n_host * buf_gb, 1)
    log(f"host K/V: {n_host} layer buffer(s), {pinned_gb} GB pinned")

    qs, wants, krs = [], [], []
    gq = torch.Generator(device=dev).manual_seed(7)
    for li in range(L):
        kr = build_kr_layer(C_total, 100 + li, dev)
        q = torch.randn((B, S, HQ, D), generator=gq, device=dev).to(torch.bfloat16)
        wants.append(plant_needles(kr, q, doc_chunk_off, n_docs, 500 + li))
        bank.set_layer(li, kr, host_k[li % n_host], host_v[li % n_host])
        krs.append(kr)
        qs.append(q)
    torch.cuda.synchronize()
    log(f"setup {time.perf_counter() - t_setup:.1f} s")

    ws = bank.workspace(B, S, HQ, TOPK, dev)
    scores = [torch.empty((B, TOPK), dtype=torch.float32, device=dev) for _ in range(L)]
    docs = [torch.empty((B, TOPK), dtype=torch.int32, device=dev) for _ in range(L)]
    gids = [torch.empty((B, TOPK), dtype=torch.int64, device=dev) for _ in range(L)]
    docs_host = [torch.empty((B, TOPK), dtype=torch.int32, pin_memory=True) for _ in range(L)]
    ready = [torch.cuda.Event() for _ in range(L)]
    scored = [torch.cuda.Event() for _ in range(L)]
    ids_stream = torch.cuda.Stream()
    cap_chunks = B * TOPK * 32
    gk = [torch.empty((cap_chunks, HKV, D), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    gv = [torch.empty((cap_chunks, HKV, D), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    side = torch.cuda.Stream()
    main_stream = torch.cuda.current_stream()
    sel_chunks = [0] * L

    host_s = {"wait": 0.0, "copy_calls": 0.0, "route_calls": 0.0}   # host time: waiting for a layer's ids, issuing its copies, its kernels

    def route(li):
        t_r = time.perf_counter()
        _lib.check(lib.msa_route_topk(bank.handle, li, qs[li].data_ptr(), None, B, S, HQ, _lib.MODE_COSINE, 1.0, TOPK,
                                      scores[li].data_ptr(), docs[li].data_ptr(), gids[li].data_ptr(), ws.data_ptr(),
                                      ws.numel(), main_stream.cuda_stream), "msa_route_topk")
        # The ids leave on a stream of their own: a copy queued on the scan's stream would hold the next layer's
        # kernels back whenever the copy engine is still busy with the previous layer's K / V.
        scored[li].record(main_stream)
        ids_stream.wait_event(scored[li])
        with torch.cuda.stream(ids_stream):
            docs_host[li].copy_(docs[li], non_blocking=True)
        ready[li].record(ids_stream)
        host_s["route_calls"] += time.perf_counter() - t_r


    def gather(li):
        t_a = time.perf_counter()
        ready[li].synchronize()
        t_b = time.perf_counter()
        cu = torch.empty(B + 1, dtype=torch.int64)
        _lib.check(lib.msa_gather_plan(bank.handle, docs_host[li].data_ptr(), B, TOPK, cu.data_ptr()), "msa_gather_plan")
        sel_chunks[li] = int(cu[-1])
        _lib.check(lib.msa_gather_kv(bank.handle, li, docs_host[li].data_ptr(), B, TOPK, gk[li & 1].data_ptr(),
                                     gv[li & 1].data_ptr(), cap_chunks, side.cuda_stream), "msa_gather_kv")
        host_s["wait"] += t_b - t_a
        host_s["copy_calls"] += time.perf_counter() - t_b

    cu_dev = [torch.empty(B + 1, dtype=torch.int32, device=dev) for _ in range(L)]
    gws = torch.empty(lib.msa_gather_device_workspace_bytes(B, TOPK), dtype=torch.uint8, device=dev)

    def gather_device(li):
        side.wait_event(scored[li])        # no host wait: the side stream picks the ids up on the device
        _lib.check(lib.msa_gather_kv_device(bank.handle, li, docs[li].data_ptr(), B, TOPK, gk[li & 1].data_ptr(),
                                            gv[li & 1].data_ptr(), cap_chunks, cu_dev[li].data_ptr(), gws.data_ptr(),
                                            gws.numel(), side.cuda_stream), "msa_gather_kv_device")

    def route_fused(li, prev):             # layer li's scan; one of its workgroups fetches layer prev's selection
        t_r = time.perf_counter()
        _lib.check(lib.msa_route_topk_gather(bank.handle, li, qs[li].data_ptr(), None, B, S, HQ, _lib.MODE_COSINE, 1.0,
                                             TOPK, scores[li].data_ptr(), docs[li].data_ptr(), gids[li].data_ptr(),
                                             ws.data_ptr(), ws.numel(), prev, docs[prev].data_ptr(), B, TOPK,
                                             gk[prev & 1].data_ptr(), gv[prev & 1].data_ptr(), cap_chunks,
                                             cu_dev[prev].data_ptr(), gws.data_ptr(), gws.numel(),
                                             main_stream.cuda_stream), "msa_route_topk_gather")
        scored[li].record(main_stream)
        host_s["route_calls"] += time.perf_counter() - t_r

    pending = [None]                  # layer whose selected K / V have not been fetched yet

    def step():
        if args.gather == "device":
            for li in range(L):
                route(li)
                gather_device(li)          # runs on the side stream under the next layer's scan
            return
        if args.gather == "fused":
            for li in range(L):
                if pending[0] is None:
                    route(li)
                else:
                    route_fused(li, pending[0])
                pending[0] = li
            return
        for li in range(L):
            route(li)                      # layer li is being scored ...
            if pending[0] is not None:
                gather(pending[0])         # ... while the previous layer's K / V come over from the host (the last
            pending[0] = li                # layer's under the first scan of the next batch)

    def drain():                           # the last batch's last layer has no scan left to hide under
        if pending[0] is not None:
            gather_device(pending[0]) if args.gather == "fused" else gather(pending[0])
            pending[0] = None

    for _ in range(args.warmup):
        step()
    drain()
    torch.cuda.synchronize()
    _lib.check(lib.msa_profile_enable(args.steps * L), "msa_profile_enable")
    torch.cuda.synchronize()
    host_s["wait"] = host_s["copy_calls"] = host_s["route_calls"] = 0.0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    drain()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_buf = (C.c_float * (args.steps * L))()
    n_rec = C.c_int32(0)
    _lib.check(lib.msa_profile_collect(ms_buf, args.steps * L, C.byref(n_rec)), "msa_profile_collect")
    kern_ms = float(np.mean(list(ms_buf)[: n_rec.value]))
    _lib.check(lib.msa_profile_enable(0), "msa_profile_enable")

    # ---- parity at full size: planted needles must come back exactly, in rank order; gathered rows
    # ---- of the last layer must equal the host rows
    for li in range(L):
        got = docs[li].cpu().numpy().astype(np.int64)
        if not np.array_equal(got, wants[li]):
            bad = np.nonzero((got != wants[li]).any(axis=1))[0]
            log(f"layer {li}: rows {bad.tolist()} differ; got {got[bad[0]].tolist()} want {wants[li][bad[0]].tolist()} "
                f"scores {scores[li][bad[0]].cpu().tolist()}")
            sys.exit(f"bench.py: PARITY FAILURE at layer {li}: top-k ids differ from the planted documents")
    last = L - 1
    from oracle import closed_form as cf
    wk, wv, wcu, _ = cf.gather_selected(host_k[last % n_host], host_v[last % n_host], doc_chunk_off,
                                        torch.as_tensor(wants[last]))
    n_sel = int(wcu[-1])
    if args.gather in ("device", "fused"):
        sel_chunks = [int(c[-1]) for c in cu_dev]
    if n_sel != sel_chunks[last] or not torch.equal(gk[last & 1][:n_sel].cpu(), wk) or \
            not torch.equal(gv[last & 1][:n_sel].cpu(), wv):
        sys.exit("bench.py: PARITY FAILURE: gathered K / V rows differ from the host bank")

    ms_per_step = elapsed / args.steps * 1e3
    qps = B * args.steps / elapsed
    flops = 2.0 * B * S * HKV * D * C_total                       # pre-summed GQA form, per launch
    bytes_layer = C_total * HKV * D * 2 + B * S * HQ * D * 2 + C_total * 4 + B * TOPK * 16
    tflops = flops / (kern_ms * 1e-3) / 1e12
    intensity = flops / bytes_layer
    bound = "mfma" if intensity > MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9) else "hbm"
    if bound == "mfma":
        roof = {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}
    else:
        gbs = bytes_layer / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}
    scan_kernel = "score_scan4_kernel" if B * ((S + 31) // 32 * 32) > 128 else "score_gemm_kernel"
    roof["traffic"] = measured_traffic(scan_kernel, f"tokens={args.tokens},B={B},S={S}")
    roof["traffic_source"] = traffic_source(scan_kernel, f"tokens={args.tokens},B={B},S={S}")
    roof.update({"kernel": scan_kernel, "kernel_ms": round(kern_ms, 4), "launches_timed": n_rec.value,
                 "flops_per_launch": flops, "algorithmic_bytes_per_launch": bytes_layer,
                 "hbm_gbs_at_this_batch": round(bytes_layer / (kern_ms * 1e-3) / 1e9, 1)})

    if args.calibrate_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).fill_(1.0)     # 1 GiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- bandwidth-bound regime: one query (and fewer tokens) per scan of layer 0.  `call_ms` is the whole
    # msa_route_topk call (prologue, scan with the per-document max in its epilogue, top-k select and merge) timed
    # with events on its stream over back-to-back calls; `frac_hbm` is the algorithmic bytes over that time.
    sweep = []
    if not args.no_sweep:
        for b1, s1 in ((1, 1), (1, 16), (1, 64), (1, 128), (2, 128), (4, 128)):
            q1 = qs[0][:b1, :s1].contiguous()
            sc = torch.empty((b1, TOPK), dtype=torch.float32, device=dev)
            dc = torch.empty((b1, TOPK), dtype=torch.int32, device=dev)
            reps = 10

            def call():
                _lib.check(lib.msa_route_topk(bank.handle, 0, q1.data_ptr(), None, b1, s1, HQ, _lib.MODE_COSINE, 1.0,
                                              TOPK, sc.data_ptr(), dc.data_ptr(), None, ws.data_ptr(), ws.numel(),
                                              main_stream.cuda_stream), "msa_route_topk")
            call_ms = time_cuda(call, reps)
            torch.cuda.synchronize()
            _lib.check(lib.msa_profile_enable(reps), "msa_profile_enable")
            for _ in range(reps):
                call()
            torch.cuda.synchronize()
            buf = (C.c_float * reps)()
            _lib.check(lib.msa_profile_collect(buf, reps, C.byref(n_rec)), "msa_profile_collect")
            ms1 = float(np.mean(list(buf)[: n_rec.value]))
            by = C_total * HKV * D * 2 + b1 * s1 * HQ * D * 2 + C_total * 4 + b1 * TOPK * 16
            sweep.append({"B": b1, "S": s1, "call_ms": round(call_ms, 4), "GB/s": round(by / call_ms / 1e6, 1),
                          "frac_hbm": round(by / call_ms / 1e6 / HBM_PEAK_GBS, 4), "scan_kernel_ms": round(ms1, 4),
                          "scan_kernel_frac_hbm": round(by / ms1 / 1e6 / HBM_PEAK_GBS, 4), "algorithmic_bytes": by,
                          "scan_TFLOP/s": round(2.0 * b1 * ((s1 + 31) // 32 * 32) * HKV * D * C_total / ms1 / 1e9, 1),
                          "scan_kernel": "score_scan4_kernel" if b1 * ((s1 + 31) // 32 * 32) > 128 else "score_gemm_kernel",
                          "traffic": measured_traffic("score_scan4_kernel" if b1 * ((s1 + 31) // 32 * 32) > 128 else "score_gemm_kernel",
                                                      f"tokens={args.tokens},B={b1},S={s1}")})
        _lib.check(lib.msa_profile_enable(0), "msa_profile_enable")
    if args.sweep_only:
        print(json.dumps({"hbm_regime_sweep": sweep}), flush=True)
        return

    extras = None
    if not args.no_extras:
        extras = {"pooling": extra_pooling(dev), "routing_10M_bank": extra_routing_10m(dev), "decode_attention": extra_decode(dev),
                  "prefill_attention": extra_prefill_attention(dev), "decode_projections": extra_decode_projections(dev),
                  "mfma_ceiling": extra_mfma_ceiling(dev),
                  "hbm_read_ceiling": extra_hbm_read_ceiling(dev)}

    cpu = None
    if not args.no_cpu_baseline:
        times, Cs = cpu_baseline(krs[0], qs[0], doc_chunks)
        best = min(times.values())
        full = best * (C_total / Cs) * L
        cpu = {"value": round(B / full, 5), "unit": "queries/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"reference op sequence (matmul, masked_fill, mean, max, scatter_reduce amax, topk) on the "
                         f"first {Cs} of {C_total} chunks of layer 0 for the same {B}x{S} queries; "
                         f"{', '.join(f'{k} {v:.2f} s' for k, v in times.items())}; best extrapolated linearly "
                         f"x{C_total / Cs:.1f} chunks x{L} layers",
               "host_cpus": os.cpu_count(), "cpu_model": cpu_model()}

    if extras is not None and not args.no_e2e:
        # configs[4] end to end (the "sparse decode tok/s" half of the metric); ~25 GB next to the 100M bank's 60 GB
        import gc
        import bench_e2e
        # the 100M-token bank's pinned host K / V go back to the system first: the boxes refuse pinned memory past
        # about 56 GB and the end-to-end run pins a bank of its own
        torch.cuda.synchronize()
        bank._keep.clear()
        del bank, wk, wv
        host_k.clear(); host_v.clear()
        gc.collect()
        torch._C._host_emptyCache()
        r = bench_e2e.main(["--steps", "256"], quiet=True)
        extras["e2e_sparse_decode"] = {"workload": r["config"]["workload"] + ", 10M-token bank, B=16, 4K context, greedy",
                                       "tokens_per_s": r["value"], "ms_per_decode_step": r["ms_per_decode_step"],
                                       "prefill_s": r["prefill_s"], "decode_steps": r["config"]["decode_steps"],
                                       "decode_mode": r["decode_mode"], "stage1_encode": r["stage1_encode"]}

    out = {
        "metric": "routed queries/s at the 100M-token bank (router scoring + top-k + host gather, 18 layers)",
        "value": round(qps, 2), "unit": "queries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[3]: 100M-token bank, K_r HBM-resident, K/V pinned host, B=16 x S=128, top-16",
                   "bank_tokens": args.tokens, "chunks": C_total, "docs": n_docs, "routed_layers": L, "batch": B,
                   "query_tokens": S, "top_k": TOPK, "kr_hbm_gb": round(C_total * HKV * D * 2 * L / 1e9, 1),
                   "host_kv_layer_buffers": n_host, "host_kv_pinned_gb": pinned_gb, "pinned_refused_at_gb": refused_at_gb,
                   "host_kv_note": "fewer layer buffers than routed layers: the box refuses pinned host memory past "
                                   "about 56 GB; the routed layers share the buffers round-robin" if n_host < L else None,
                   "gather": args.gather,
                   "gather_host_ms_per_layer": {k: round(v / (args.steps * L) * 1e3, 3) for k, v in host_s.items()}, "selected_chunks_per_layer": int(np.mean(sel_chunks)),
                   "mode": "cosine/mean-heads/max-tokens/max-chunks"},
        "roofline": roof, "cpu_baseline": cpu, "hbm_regime_sweep": sweep, "other_kernels": extras, "parity": "needles exact on all layers",
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
