"""GPU tests of the two largest benchmark configurations at their real shapes.

* 100M-token bank: one routed layer resident in HBM (3.3 GB of K_r), its pooled K / V in pinned host memory filled
  with a pattern that is a function of (chunk, head, dim), so a gathered row proves where it came from without the
  host bank being read back; batch of 16 queries x 128 tokens, top-16; the gather of one scan's winners runs on a
  side stream under the next scan.
* End-to-end generation at Qwen3-4B shape (36 layers, routing on the upper 18, 10M-token bank, batch 16, 4K-token
  context): a few greedy steps, HIP-graph replay against eager decoding, and the routed layer's results (selected
  documents, assembled context, stage-2 and decode attention) against the fp64 oracle on sampled rows.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

HQ, HKV, D, P, TOPK = 32, 8, 128, 64, 16


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible")
    from msa_amd import ops as _ops
    return _ops


def _doc_tokens(total, seed):
    rng = np.random.default_rng(seed)
    lens, left = [], total
    while left > 0:
        n = min(int(rng.integers(256, 2049)), left)
        lens.append(n)
        left -= n
    return lens


def _pattern_k(c, h, d):
    return ((c * 7 + h * 13 + d) % 255 - 127).to(torch.bfloat16)      # integers up to 127: exact in bf16


def _pattern_v(c, h, d):
    return ((c * 3 + h * 5 + 2 * d) % 251 - 125).to(torch.bfloat16)


def _pattern_rows(fn, chunks, device="cpu"):
    c = torch.as_tensor(chunks, dtype=torch.int64, device=device).view(-1, 1, 1)
    h = torch.arange(HKV, device=device).view(1, -1, 1)
    d = torch.arange(D, device=device).view(1, 1, -1)
    return fn(c, h, d)


def test_config3_hundred_million_token_bank(ops):
    say("configs[3]: 100M-token bank, one routed layer, pinned host K/V, gather under the next scan")
    from msa_amd import _lib
    lib = _lib.load()
    B, S = 16, 128
    doc_tokens = _doc_tokens(100_000_000, 0)
    doc_chunks = [(n + P - 1) // P for n in doc_tokens]
    dco = np.concatenate([[0], np.cumsum(doc_chunks)]).astype(np.int64)
    n_docs, C = len(doc_chunks), int(dco[-1])
    assert C > 1_560_000 and n_docs > 80_000
    dev = torch.device("cuda:0")

    # K_r: N(0,1) rows normalised per (chunk, head), generated on the device slice by slice
    g = torch.Generator(device=dev).manual_seed(100)
    kr = torch.empty((C, HKV, D), dtype=torch.bfloat16, device=dev)
    for s0 in range(0, C, 1 << 17):
        e0 = min(C, s0 + (1 << 17))
        x = torch.randn((e0 - s0, HKV, D), generator=g, device=dev)
        kr[s0:e0] = (x / x.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
    q = torch.randn((B, S, HQ, D), generator=g, device=dev).to(torch.bfloat16)

    # planted winners: rank r of query b has cosine 0.98 - 0.025 r with one token's head-summed direction
    rng = np.random.default_rng(500)
    all_docs = rng.choice(n_docs, size=B * TOPK, replace=False).reshape(B, TOPK)
    planted_chunks = []
    for b in range(B):
        tok = int(rng.integers(0, S))
        qn = cf.l2_normalize(q[b, tok].cpu().double()).view(HKV, HQ // HKV, D).sum(1)
        direction = cf.l2_normalize(qn)
        for r, d in enumerate(all_docs[b]):
            c = (int(dco[d]) + int(dco[d + 1])) // 2
            noise = kr[c].cpu().double()
            perp = cf.l2_normalize(noise - (noise * direction).sum(-1, keepdim=True) * direction)
            cos = 0.98 - 0.025 * r
            kr[c] = (cos * direction + (1 - cos * cos) ** 0.5 * perp).to(torch.bfloat16).to(dev)
            planted_chunks.append(c)
    want_docs = all_docs.astype(np.int64)

    # pinned host K / V of the layer, filled with the pattern from the device in slices
    kh = torch.empty((C, HKV, D), dtype=torch.bfloat16, pin_memory=True)
    vh = torch.empty((C, HKV, D), dtype=torch.bfloat16, pin_memory=True)
    for s0 in range(0, C, 1 << 18):
        e0 = min(C, s0 + (1 << 18))
        idx = torch.arange(s0, e0, device=dev)
        kh[s0:e0].copy_(_pattern_rows(_pattern_k, idx, dev))
        vh[s0:e0].copy_(_pattern_rows(_pattern_v, idx, dev))
    torch.cuda.synchronize()

    bank = ops.Bank(1, dco.tolist(), (np.arange(n_docs, dtype=np.int64) * 5 + 3).tolist(), HKV, D, torch.bfloat16)
    bank.set_layer(0, kr, kh, vh)
    scores, doc, gid = ops.route_topk(bank, 0, q, None, "cosine", 1.0, TOPK)
    torch.cuda.synchronize()
    assert np.array_equal(doc.cpu().numpy().astype(np.int64), want_docs)            # exact, in rank order
    assert (scores[:, :-1] > scores[:, 1:]).all()
    assert torch.equal(gid.cpu(), doc.cpu().long() * 5 + 3)

    # second scan on the main stream, the first scan's winners fetched on a side stream underneath it
    main, side = torch.cuda.current_stream(), torch.cuda.Stream()
    ids_host = torch.empty((B, TOPK), dtype=torch.int32, pin_memory=True)
    ids_host.copy_(doc, non_blocking=True)
    ready = torch.cuda.Event()
    ready.record(main)
    scores2, doc2, _ = ops.route_topk(bank, 0, q, None, "cosine", 1.0, TOPK)          # enqueued, about 6 ms of work
    ready.synchronize()
    K, V, cu = ops.gather_kv(bank, 0, ids_host, dev, stream=side)                     # DMA copies under the scan
    side.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(doc2, doc) and torch.equal(scores2, scores)                    # the scan is deterministic
    _, _, wcu, _ = cf.gather_selected(torch.zeros((C, 1, 1)), torch.zeros((C, 1, 1)), dco, torch.as_tensor(want_docs))
    assert cu.tolist() == wcu.tolist()
    exp_chunks = np.concatenate([np.arange(dco[d], dco[d + 1]) for b in range(B) for d in sorted(want_docs[b])])
    assert K.shape[0] == len(exp_chunks) == int(wcu[-1])
    assert torch.equal(K.cpu(), _pattern_rows(_pattern_k, exp_chunks)) and torch.equal(V.cpu(), _pattern_rows(_pattern_v, exp_chunks))
    # the device-planned gather reads the same pinned rows without the ids leaving the device
    cap = B * TOPK * bank.max_doc_chunks
    Kd, Vd, cud = ops.gather_kv_device(bank, 0, doc, cap)
    torch.cuda.synchronize()
    n = len(exp_chunks)
    assert cud.cpu().tolist() == wcu.tolist()
    assert torch.equal(Kd[:n].cpu(), _pattern_rows(_pattern_k, exp_chunks)) and torch.equal(Vd[:n].cpu(), _pattern_rows(_pattern_v, exp_chunks))

    # the same gather carried by a scan's launch (one workgroup of it copies, the others score; at this size the
    # scan's last N tiles are a pool the workgroups draw from): both calls' results, bit for bit
    (s3, d3, g3), (Kf, Vf, cuf) = ops.route_topk_gather(bank, 0, q, None, "cosine", 1.0, TOPK, 0, doc, cap)
    torch.cuda.synchronize()
    assert torch.equal(d3, doc) and torch.equal(s3, scores) and torch.equal(g3, gid)
    assert cuf.cpu().tolist() == wcu.tolist()
    assert torch.equal(Kf[:n].cpu(), _pattern_rows(_pattern_k, exp_chunks)) and torch.equal(Vf[:n].cpu(), _pattern_rows(_pattern_v, exp_chunks))
    del Kf, Vf, Kd, Vd

    # oracle parity of the chunk scores on a sample (random chunks plus every planted one)
    cs_all = ops.chunk_scores(bank, 0, q, None, "cosine", 1.0)
    torch.cuda.synchronize()
    sample = np.unique(np.concatenate([rng.integers(0, C, size=400), planted_chunks, [0, C - 1]]))
    want = cf.chunk_scores(q.cpu(), torch.ones(B, S, dtype=torch.bool), kr[sample].cpu(), "cosine")
    assert cf.rel_err(cs_all[:, sample].cpu(), want) < 1e-2
    # a document's score is the max of its chunks' scores; fused (routing) and per-chunk epilogues agree exactly
    for b in (0, 7, B - 1):
        for r in (0, TOPK - 1):
            d = int(doc[b, r])
            assert float(scores[b, r]) == float(cs_all[b, int(dco[d]):int(dco[d + 1])].max())
    # the whole-bank invariant behind the top-k: no document outside the returned ones scores above the k-th
    ds_max = torch.empty((B, n_docs), dtype=torch.float32, device=dev)
    seg = torch.repeat_interleave(torch.arange(n_docs, device=dev), torch.as_tensor(doc_chunks, device=dev))
    ds_max.fill_(float("-inf")).scatter_reduce_(1, seg.expand(B, -1), cs_all, reduce="amax")
    kth = scores[:, -1:]
    above = (ds_max > kth).sum(dim=1)
    assert above.cpu().tolist() == [TOPK - 1] * B
    del cs_all, ds_max, kr, kh, vh


def test_config4_end_to_end_qwen3_4b_shape(ops):
    say("configs[4]: Qwen3-4B shape, 36 layers, 10M-token bank, B=16, 4K context")
    import bench_e2e
    from msa_amd.config import MSAConfig
    from msa_amd.model import MSAForCausalLM
    dev = torch.device("cuda:0")
    cfg = MSAConfig()
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (36, 2560, 32, 8)
    with torch.device(dev):
        model = MSAForCausalLM(cfg).to(torch.bfloat16)
    model.init_random_(0.02, seed=0).eval()
    svc = bench_e2e.build_service(cfg, 10_000_000)
    svc.setup_memory_client(model)
    bank = svc.bank
    dco = bank.off_host.numpy().astype(np.int64)
    n_docs = bank.n_docs
    B, S, steps = 16, 4096, 8
    g = torch.Generator(device=dev).manual_seed(3)
    ids = torch.randint(0, cfg.vocab_size, (B, S), generator=g, device=dev)
    mask = torch.ones((B, S), dtype=torch.long, device=dev)
    doc_ids = torch.zeros((B, S), dtype=torch.long, device=dev)

    layer_idx = svc.router_layer_ids[0]                     # 18: the first routed layer
    attn = model.model.layers[layer_idx].self_attn
    grabbed = {}
    # the layer's input at stage 2 (its router projection runs inside the fused projection kernel; the oracle side
    # projects the same hidden states with the router weights below)
    def grab(module, args):                                  # a pre-hook that returns something replaces the inputs
        grabbed.setdefault("h", args[0].detach().clone())
    hook = attn.register_forward_pre_hook(grab)
    tok_eager, cache = model.generate_greedy(ids, mask, doc_ids, steps, require_recall_topk=True, use_graph=False)
    hook.remove()
    tok_graph, cache_g = model.generate_greedy(ids, mask, doc_ids, steps, use_graph=True)
    torch.cuda.synchronize()
    assert tok_eager.shape == (B, steps)
    assert torch.equal(tok_eager, tok_graph)                # graph replays == eager decoding, token for token
    ck = cache.cache_kwargs[layer_idx]
    kv_len = ck["kv_lengths"].cpu().tolist()
    assert kv_len == cache_g.cache_kwargs[layer_idx]["kv_lengths"].cpu().tolist()

    # ---- routing of the first routed layer against the oracle on sampled documents
    assert grabbed["h"].shape == (B, S, cfg.hidden_size)
    rq = torch.nn.functional.linear(grabbed["h"], attn.router_q_proj[0].weight).view(B, S, HQ, D)
    rec = ck["recall_topk"]
    rng = np.random.default_rng(9)
    slot = svc._layer_slot[layer_idx]
    kr = bank._keep[slot][0]
    kh, vh = bank._keep[slot][1], bank._keep[slot][2]
    for b in (0, B - 1):
        sel = [int(x) for x in rec[b]["topk_doc_ids"]]
        got_scores = torch.tensor(rec[b]["score"], dtype=torch.float64)
        assert len(set(sel)) == TOPK and (got_scores[:-1] >= got_scores[1:]).all()
        others = [int(x) for x in rng.choice(n_docs, size=100, replace=False) if int(x) not in sel]
        docs = sel + others
        chunks = np.concatenate([np.arange(dco[d], dco[d + 1]) for d in docs])
        off = np.concatenate([[0], np.cumsum([dco[d + 1] - dco[d] for d in docs])])
        cs = cf.chunk_scores(rq[b:b + 1].cpu(), torch.ones(1, S, dtype=torch.bool), kr[chunks].cpu(), "cosine")
        ds = cf.doc_scores(cs, off)[0]
        assert cf.rel_err(got_scores, ds[:TOPK]) < 1e-2
        assert float(ds[TOPK:].max()) <= float(got_scores[-1]) + 1e-3       # no sampled outsider beats the k-th

        # ---- the assembled context of this sample: [prefix | selected chunks, ascending documents | query tokens]
        kc, vc = ck["compacked_key_cache"][b], ck["compacked_value_cache"][b]
        sel_sorted = sorted(sel)
        mem_chunks = np.concatenate([np.arange(dco[d], dco[d + 1]) for d in sel_sorted])
        n_mem = len(mem_chunks)
        assert kv_len[b] == 3 + n_mem + S + (steps - 1)
        pk, pv = svc.get_template_prefix_kvcaches(layer_idx)
        assert torch.equal(kc[:3].cpu(), pk[0].transpose(0, 1).cpu()) and torch.equal(vc[:3].cpu(), pv[0].transpose(0, 1).cpu())
        assert torch.equal(kc[3:3 + n_mem].cpu(), kh[mem_chunks]) and torch.equal(vc[3:3 + n_mem].cpu(), vh[mem_chunks])

        # ---- stage-2 attention at this shape: the sample's 4096 query rows over its context, causal, sampled rows
        L2 = 3 + n_mem + S
        gq = torch.Generator().manual_seed(40 + b)
        qrows = torch.randn((S, HQ, D), generator=gq).to(torch.bfloat16)
        out = ops.sparse_attn(qrows.to(dev), kc, vc, torch.zeros(1, dtype=torch.int64, device=dev),
                              torch.tensor([L2], dtype=torch.int32, device=dev), L2,
                              cu_q=torch.tensor([0, S], dtype=torch.int32, device=dev), max_sq=S, causal=True).cpu()
        kcpu, vcpu = kc[:L2].cpu(), vc[:L2].cpu()
        for i in (0, 1, 63, 64, 2047, S - 1):
            vis = L2 - S + i + 1
            want = cf.attention(qrows[i:i + 1], kcpu[:vis], vcpu[:vis], causal=False)
            assert cf.rel_err(out[i:i + 1], want) < 1e-2, (b, i)

        # ---- decode attention over the whole compact cache (L about 4390): one row for this sample
        L = kv_len[b]
        qd = torch.randn((1, HQ, D), generator=gq).to(torch.bfloat16)
        got = ops.sparse_attn(qd.to(dev), kc, vc, torch.zeros(1, dtype=torch.int64, device=dev),
                              torch.tensor([L], dtype=torch.int32, device=dev), L).cpu()
        assert cf.rel_err(got, cf.attention(qd, kc[:L].cpu(), vc[:L].cpu())) < 1e-2
    # a lower (non-routed) layer holds [prefix | query tokens | decoded tokens] only
    assert cache.cache_kwargs[0]["kv_lengths"].cpu().tolist() == [3 + S + steps - 1] * B
    del model, svc, cache, cache_g
