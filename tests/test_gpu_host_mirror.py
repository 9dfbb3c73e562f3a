"""GPU tests of the reference-shaped host interface: ``MemorySparseAttention`` (stage 1, stage 2,
decode), ``Memory.prefill_stage2`` / ``MSAService.doc_query`` and the greedy loop.  Dense
projections are re-done in fp64 torch on the CPU with the layer's own weights; everything the HIP
library computes is checked against the closed-form oracle."""
import copy
import sys

import numpy as np
import pytest
import torch

from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

P, HID, HQ, HKV, D, TOPK = 8, 256, 4, 2, 128, 3
HEAD_IDS = [7, 8, 9]
TOL = 3e-5


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def env():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible")
    from msa_amd import config, memory_sparse_attention as msa, model, msa_service, prefill
    cfg = config.MSAConfig(hidden_size=HID, num_hidden_layers=2, num_attention_heads=HQ, num_key_value_heads=HKV,
                           head_dim=D, intermediate_size=512, vocab_size=500,
                           msa_config=dict(config.default_msa_config(), top_k_docs=TOPK, pooling_kernel_size=P,
                                           router_layer_idx="1"))
    return dict(cfg=cfg, config=config, msa=msa, model=model, svc=msa_service, prefill=prefill)


def _layer(env, seed=0):
    torch.manual_seed(seed)
    layer = env["msa"].MemorySparseAttention(env["cfg"], 1).float()
    with torch.no_grad():
        for p in layer.parameters():
            if p.dim() > 1:
                p.copy_(torch.randn(p.shape) * 0.08)
            else:
                p.copy_(1.0 + 0.1 * torch.randn(p.shape))
    return layer.eval()


def _tables(env, position_ids):
    cos, sin = env["msa"].rotary_embedding(position_ids, D, env["cfg"].rope_theta, torch.float32)
    return cos, sin


def _docs(env, lens, first_id=100):
    pf = env["prefill"]
    g = np.random.default_rng(5)
    return [pf.Document(doc=f"d{i}", doc_id=first_id + i, num_chunks=pf.num_chunks(n, P),
                        input_ids=[int(x) for x in g.integers(10, 400, size=n)]) for i, n in enumerate(lens)]


def test_layer_stage1_stage2_decode_against_oracle(env):
    say("layer: stage 1 -> bank -> stage 2 -> decode")
    pf, svc_mod = env["prefill"], env["svc"]
    layer = _layer(env)
    layer64 = copy.deepcopy(layer).double()
    layer = layer.cuda()
    lens = [5, 8, 17, 1, 30, 9, 16, 23, 12]
    docs = _docs(env, lens)
    blocks = pf.split_docs(docs, 8)
    assert len(blocks) >= 2
    service = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                 env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                 env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    service.begin(docs)
    g = torch.Generator().manual_seed(3)
    bank_k, bank_v, bank_rk, prefix = [], [], [], None
    for blk in blocks:
        inp = pf.prepare_block_inputs(blk, HEAD_IDS, P)
        T = inp.doc_ids.shape[1]
        hs = torch.randn((1, T, HID), generator=g)
        cos, sin = _tables(env, inp.position_ids)
        cache = env["model"].create_cache()
        cache.record_kwargs(1, {"stage": "prefill_stage1"})
        with torch.no_grad():
            out, _ = layer(hs.cuda(), inp.doc_ids.cuda(), inp.doc_attention_mask.cuda(), (cos.cuda(), sin.cuda()), cache)
            q64, k64, v64 = layer64._project(hs.double(), (cos.double(), sin.double()))
            rk64 = layer64.router_k_proj(hs.double()).view(T, HKV, D)
        _, _, cs, cl, cd = cf.chunk_table(inp.doc_lens, P, 3)
        want_k, want_v = cf.pool_chunks(k64[0], cs, cl), cf.pool_chunks(v64[0], cs, cl)
        want_rk = cf.l2_normalize(cf.pool_chunks(rk64, cs, cl))
        pk, pv = cache.get_kvcache(1)
        assert pk.shape == (1, HKV, len(cs), D)                              # the reference's [1, Hkv, C, D] view
        assert cf.rel_err(pk[0].transpose(0, 1).cpu(), want_k) < TOL
        assert cf.rel_err(pv[0].transpose(0, 1).cpu(), want_v) < TOL
        assert cf.rel_err(cache.get_router_kcache(1)[0].transpose(0, 1).cpu(), want_rk) < TOL
        kw = cache.cache_kwargs[1]
        assert kw["pooled_doc_ids"].cpu().tolist() == (cd + 1).tolist()      # 1-based within the block
        assert kw["template_prefix_kcache"].shape == (1, HKV, 3, D)
        assert cf.rel_err(kw["template_prefix_kcache"][0].transpose(0, 1).cpu(), k64[0, :3]) < TOL
        # document-wise causal attention, template head as its own segment
        seg = [3] + inp.doc_lens
        edges = np.concatenate([[0], np.cumsum(seg)])
        want_attn = cf.attention_ragged(q64[0], edges, k64[0], v64[0], edges, causal=True)
        with torch.no_grad():
            want_out = layer64.o_proj(want_attn.reshape(1, T, HQ * D))
        assert cf.rel_err(out.cpu(), want_out) < TOL
        bank_k.append(want_k); bank_v.append(want_v); bank_rk.append(want_rk)
        if prefix is None:
            prefix = (k64[0, :3], v64[0, :3])
        service.add_block(cache)
    service.finish()
    bank_k, bank_v, bank_rk = torch.cat(bank_k), torch.cat(bank_v), torch.cat(bank_rk)
    _, dco, _, _, _ = cf.chunk_table(lens, P)
    assert service.block_desc.pool_ids_cpu.tolist() == (np.repeat(np.arange(len(lens)), np.diff(dco)) + 1).tolist()
    layer.set_memory_client(service)

    # ---- stage 2: two left-padded queries
    n_q = [7, 4]
    B, S = 2, max(n_q)
    hs2 = torch.randn((B, S, HID), generator=g)
    mask = torch.tensor([[1] * 7, [0] * 3 + [1] * 4])
    pos = torch.tensor([pf.query_position_ids(n, TOPK, 3, S - n) for n in n_q])
    cos, sin = _tables(env, pos)
    cache2 = env["model"].create_cache()
    cache2.meta["require_recall_topk"] = True
    cache2.record_kwargs(1, {"stage": "prefill_stage2"})
    dz = torch.zeros((B, S), dtype=torch.long)
    with torch.no_grad():
        out2, _ = layer(hs2.cuda(), dz.cuda(), mask.cuda(), (cos.cuda(), sin.cuda()), cache2)
        q64, k64, v64 = layer64._project(hs2.double(), (cos.double(), sin.double()))
        rq64 = layer64.router_q_proj(hs2.double()).view(B, S, HQ, D)
    ds = cf.doc_scores(cf.chunk_scores(rq64, mask.bool(), bank_rk, "cosine"), dco)
    want_s, want_i = cf.topk_docs(ds, TOPK)
    recall = cache2.cache_kwargs[1]["recall_topk"]
    got_i = torch.tensor([[d - 100 for d in r["topk_doc_ids"]] for r in recall])
    assert not cf.topk_acceptable(ds, got_i, TOPK, gap=1e-4)
    if float((want_s[:, :-1] - want_s[:, 1:]).min()) > 1e-4:
        assert torch.equal(got_i, want_i)
    assert cf.rel_err(torch.tensor([r["score"] for r in recall]), torch.gather(ds, 1, got_i)) < TOL
    mk, mv, cu_sel, _ = cf.gather_selected(bank_k, bank_v, dco, got_i)
    want_rows = []
    for b in range(B):
        lo = S - n_q[b]
        kk = torch.cat([prefix[0], mk[cu_sel[b]:cu_sel[b + 1]], k64[b, lo:]])
        vv = torch.cat([prefix[1], mv[cu_sel[b]:cu_sel[b + 1]], v64[b, lo:]])
        want_rows.append((cf.attention(q64[b, lo:], kk, vv, causal=True), kk, vv))
    with torch.no_grad():
        for b in range(B):
            lo = S - n_q[b]
            want_out = layer64.o_proj(want_rows[b][0].reshape(1, n_q[b], HQ * D))
            assert cf.rel_err(out2[b:b + 1, lo:].cpu(), want_out) < TOL
            assert float(out2[b, :lo].abs().max()) == 0.0 if lo else True
    kw2 = cache2.cache_kwargs[1]
    assert kw2["kv_lengths"].cpu().tolist() == [3 + int(cu_sel[b + 1] - cu_sel[b]) + n_q[b] for b in range(B)]

    # ---- two decode steps
    for i in range(cache2.get_layer_length()):
        cache2.cache_kwargs[1]["stage"] = "generate"
    ctx = [(r[1], r[2]) for r in want_rows]
    for step in range(2):
        hs3 = torch.randn((B, 1, HID), generator=g)
        pos3 = pos[:, -1:] + 1 + step
        cos, sin = _tables(env, pos3)
        with torch.no_grad():
            out3, _ = layer(hs3.cuda(), torch.full((B, 1), -1).cuda(), torch.ones(B, 1, dtype=torch.long).cuda(),
                            (cos.cuda(), sin.cuda()), cache2)
            q64, k64, v64 = layer64._project(hs3.double(), (cos.double(), sin.double()))
            for b in range(B):
                ctx[b] = (torch.cat([ctx[b][0], k64[b]]), torch.cat([ctx[b][1], v64[b]]))
                want = layer64.o_proj(cf.attention(q64[b], ctx[b][0], ctx[b][1]).reshape(1, 1, HQ * D))
                assert cf.rel_err(out3[b:b + 1].cpu(), want) < TOL

    # ---- the scorer / client surface with the reference's argument conventions
    with torch.no_grad():
        rq = torch.nn.functional.normalize(layer.router_q_proj(hs2.cuda()).view(B, S, HQ, D).transpose(1, 2), p=2, dim=-1)
    q5 = rq.reshape(B, HKV, HQ // HKV, S, D)                                 # [B, Hkv, G, S, D], cosine: not scaled
    m5 = mask.bool().cuda().view(B, 1, 1, S, 1)
    s, local, gids = service.prefill_stage2(1, q5, m5)
    assert s.shape == (B, TOPK) and local.dtype == torch.int64
    assert not cf.topk_acceptable(ds, local.cpu() - 1, TOPK, gap=1e-4)       # local ids are 1-based
    assert torch.equal(gids.cpu(), local.cpu() + 99)
    K, V, s2, n_sel, g2 = service.doc_query(rq, mask.bool().cuda(), 1)
    assert K.shape == (HKV, int(cu_sel[-1]), D) and V.shape == K.shape        # the reference's [Hkv, n, D]
    assert n_sel.cpu().tolist() == np.diff(cu_sel).tolist() and n_sel.dtype == torch.int64
    assert cf.rel_err(K.permute(1, 0, 2).cpu(), mk) < TOL and cf.rel_err(V.permute(1, 0, 2).cpu(), mv) < TOL
    assert torch.equal(g2.cpu(), got_i + 100)

    # fewer documents than top-k: the dummy slot 0 pads the tail with the dtype's lowest value
    small = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                               env["config"].ModelConfig(doc_top_k=16, pooling_kernel_size=P, router_layer_idx="1"),
                               env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    small.block_desc = service.block_desc
    small.bank, small._layer_slot = service.bank, service._layer_slot
    s, local, gids = small.prefill_stage2(1, q5, m5)
    assert s.shape == (B, len(lens) + 1) and (local[:, -1] == 0).all() and (gids[:, -1] == 0).all()
    assert float(s[0, -1]) == torch.finfo(torch.float32).min
    assert sorted(local[0, :-1].cpu().tolist()) == list(range(1, len(lens) + 1))

    # ---- stored bank: serialize, stream back into a fresh service, same answers bit for bit
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        service.serialize(tmp)
        fresh = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                   env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                   env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
        fresh.deserialize(tmp)
    assert [d.doc for d in fresh.block_desc.docs] == [d.doc for d in docs]
    assert torch.equal(fresh.block_desc.pool_ids_cpu, service.block_desc.pool_ids_cpu)
    K2, V2, s3, n2, g3 = fresh.doc_query(rq, mask.bool().cuda(), 1)
    assert torch.equal(K2, K) and torch.equal(V2, V) and torch.equal(s3, s2) and torch.equal(g3, g2) and torch.equal(n2, n_sel)
    pk_a, pv_a = service.get_template_prefix_kvcaches(1)
    pk_b, pv_b = fresh.get_template_prefix_kvcaches(1)
    assert torch.equal(pk_a, pk_b) and torch.equal(pv_a, pv_b)

    # ---- the same bank in the reference's own file layout ([1, Hkv, C, D] tensors, one file each) converts
    with tempfile.TemporaryDirectory() as tmp:
        for tag, src in (("rk", service._rk), ("k", service._k), ("v", service._v)):
            torch.save(src[1].cpu().transpose(0, 1).unsqueeze(0).contiguous(), f"{tmp}/layer_1_{tag}.pt")
        torch.save({l: (a.cpu(), b.cpu()) for l, (a, b) in service.template_prefix_kvcache.items()},
                   f"{tmp}/prefix_cache.pt")
        conv = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                  env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                  env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
        conv.load_reference_bank(tmp, docs)
    K4, V4, s4, n4, g4 = conv.doc_query(rq, mask.bool().cuda(), 1)
    assert torch.equal(K4, K) and torch.equal(V4, V) and torch.equal(s4, s2) and torch.equal(g4, g2) and torch.equal(n4, n_sel)
    assert conv._k[1].is_pinned() and conv._rk[1].is_cuda


def test_unsupported_reductions_raise(env):
    say("unsupported reduce methods")
    cfgm = env["config"]
    bad = cfgm.MSAConfig(msa_config=dict(cfgm.default_msa_config(), head_reduce_method="max"))
    with pytest.raises(NotImplementedError, match="Unsupported head reduce method"):
        env["svc"].Memory(0, cfgm.GenerateConfig(devices=[0]), cfgm.ModelConfig(), cfgm.MemoryConfig(), bad)
    bad = cfgm.MSAConfig(msa_config=dict(cfgm.default_msa_config(), chunk_reduce_method="median"))
    with pytest.raises(ValueError, match="Invalid chunk reduction method"):
        env["svc"].Memory(0, cfgm.GenerateConfig(devices=[0]), cfgm.ModelConfig(), cfgm.MemoryConfig(), bad)
    bad = cfgm.MSAConfig(msa_config=dict(cfgm.default_msa_config(), query_reduce_method="first"))
    with pytest.raises(NotImplementedError, match="Unsupported query reduce method"):
        env["svc"].Memory(0, cfgm.GenerateConfig(devices=[0]), cfgm.ModelConfig(), cfgm.MemoryConfig(), bad)
    # the reference's other token / chunk reductions are accepted (src/msa_service.py:751-811)
    ok = cfgm.MSAConfig(msa_config=dict(cfgm.default_msa_config(), query_reduce_method="mean", chunk_reduce_method="mean"))
    mem = env["svc"].Memory(0, cfgm.GenerateConfig(devices=[0]), cfgm.ModelConfig(), cfgm.MemoryConfig(), ok)
    assert (mem.query_reduce_method, mem.chunk_reduce_method) == ("mean", "mean")
    layer = _layer(env).cuda()
    with pytest.raises(Exception, match="error!"):
        layer(torch.zeros(1, 1, HID).cuda(), torch.zeros(1, 1).long().cuda())


def test_model_greedy_generation_runs_and_is_deterministic(env):
    say("model: encode -> bank -> greedy generation (bf16)")
    pf, svc_mod, M = env["prefill"], env["svc"], env["model"]
    model = M.MSAForCausalLM(env["cfg"]).init_random(0.05, seed=1).to(torch.bfloat16).cuda().eval()
    lens = [20, 33, 9, 41, 16, 27]
    docs = _docs(env, lens, first_id=0)
    service = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                 env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                 env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    service.begin(docs)
    for blk in pf.split_docs(docs, 12):
        service.add_block(M.encode_block(model, pf.prepare_block_inputs(blk, HEAD_IDS, P), "cuda"))
    service.finish()
    assert set(service.template_prefix_kvcache) == {0, 1}                    # every layer keeps its template prefix
    service.setup_memory_client(model)
    ids = torch.tensor([[5, 6, 7, 8, 9, 10], [0, 0, 11, 12, 13, 14]]).cuda()
    mask = torch.tensor([[1] * 6, [0, 0, 1, 1, 1, 1]]).cuda()
    dz = torch.zeros_like(ids)
    t1, c1 = model.generate_greedy(ids, mask, dz, 5, require_recall_topk=True)
    t2, _ = model.generate_greedy(ids, mask, dz, 5)
    assert t1.shape == (2, 5) and torch.equal(t1, t2)
    # a captured decode step replayed as a HIP graph must give the eager tokens, replay after replay
    t3, _ = model.generate_greedy(ids, mask, dz, 12, use_graph=False)
    t4, c4 = model.generate_greedy(ids, mask, dz, 12, use_graph=True)
    assert torch.equal(t3[:, :5], t1) and torch.equal(t3, t4)
    # 5 tokens = stage 2 + 4 decode steps, 12 tokens = stage 2 + 11: the graph run appended 7 rows more per sample
    assert c4.cache_kwargs[1]["kv_lengths"].cpu().tolist() == [x + 7 for x in c1.cache_kwargs[1]["kv_lengths"].cpu().tolist()]
    rec = c1.cache_kwargs[1]["recall_topk"]
    assert len(rec) == 2 and all(len(set(r["topk_doc_ids"])) == TOPK for r in rec)
    assert "recall_topk" not in c1.cache_kwargs[0]                           # layer 0 is not a router layer
    assert c1.cache_kwargs[1]["kv_lengths"].cpu().tolist()[0] > c1.cache_kwargs[0]["kv_lengths"].cpu().tolist()[0]


def test_decode_rows_path_matches_generic_layer_path(env):
    """The weight-streaming decode step (norms, silu-mul and residual adds folded into the projections) against
    the same decoder layers run through the separate norm / projection / activation kernels."""
    say("model: weight-streaming decode step vs generic layer path")
    pf, svc_mod, M = env["prefill"], env["svc"], env["model"]
    model = M.MSAForCausalLM(env["cfg"]).init_random(0.05, seed=4).to(torch.bfloat16).cuda().eval()
    docs = _docs(env, [20, 33, 9, 41], first_id=0)
    service = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                 env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                 env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    service.begin(docs)
    for blk in pf.split_docs(docs, 12):
        service.add_block(M.encode_block(model, pf.prepare_block_inputs(blk, HEAD_IDS, P), "cuda"))
    service.finish()
    service.setup_memory_client(model)
    ids = torch.tensor([[5, 6, 7, 8, 9, 10], [0, 0, 11, 12, 13, 14]]).cuda()
    mask = torch.tensor([[1] * 6, [0, 0, 1, 1, 1, 1]]).cuda()
    _, cache = model.generate_greedy(ids, mask, torch.zeros_like(ids), 1)
    for i in range(env["cfg"].num_hidden_layers):
        cache.cache_kwargs[i]["stage"] = "generate"
    layer = model.model.layers[1]
    h = (torch.randn((2, 1, HID), generator=torch.Generator().manual_seed(9)) * 2).bfloat16().cuda()
    pos = torch.tensor([[30], [28]]).cuda()
    gen_ids = torch.full((2, 1), -1).cuda()
    ones = torch.ones((2, 1), dtype=torch.long).cuda()
    lens0 = cache.cache_kwargs[1]["kv_lengths"].clone()
    assert layer._decode_rows_ok(h, cache, pos)
    with torch.no_grad():
        fast = layer(h.clone(), gen_ids, ones, None, cache, position_ids=pos)
        cache.cache_kwargs[1]["kv_lengths"].copy_(lens0)                     # same cache row for the second run
        layer._decode_rows_ok = lambda *a: False
        slow = layer(h.clone(), gen_ids, ones, None, cache, position_ids=pos)
        del layer._decode_rows_ok
    assert fast.shape == slow.shape == (2, 1, HID)
    assert cf.rel_err(fast.cpu(), slow.double().cpu()) < 1e-2


def test_injected_block_equals_token_by_token_decode(env):
    """Memory-Interleave source-context injection: a ragged left-padded block of new tokens fed in one forward of
    the decode stage must leave the caches and the last hidden state where feeding the same tokens one decode
    step at a time leaves them."""
    say("model: multi-token block in the decode stage vs token-by-token")
    pf, svc_mod, M = env["prefill"], env["svc"], env["model"]
    model = M.MSAForCausalLM(env["cfg"]).init_random(0.05, seed=6).to(torch.bfloat16).cuda().eval()
    docs = _docs(env, [20, 33, 9, 41], first_id=0)
    service = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                 env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                 env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    service.begin(docs)
    for blk in pf.split_docs(docs, 12):
        service.add_block(M.encode_block(model, pf.prepare_block_inputs(blk, HEAD_IDS, P), "cuda"))
    service.finish()
    service.setup_memory_client(model)
    ids = torch.tensor([[5, 6, 7, 8, 9, 10], [0, 0, 11, 12, 13, 14]]).cuda()
    mask = torch.tensor([[1] * 6, [0, 0, 1, 1, 1, 1]]).cuda()
    blocks = [[21, 22, 23, 24, 25], [31, 32]]

    def run(block_mode):
        _, cache = model.generate_greedy(ids, mask, torch.zeros_like(ids), 1)
        for i in range(env["cfg"].num_hidden_layers):
            cache.cache_kwargs[i]["stage"] = "generate"
        lens0 = [cache.cache_kwargs[i]["kv_lengths"].clone() for i in range(2)]
        pos0 = torch.tensor([3 + TOPK + 6 - 1, 3 + TOPK + 4 - 1]).cuda()
        with torch.no_grad():
            if block_mode:
                x = torch.tensor([blocks[0], [0, 0, 0] + blocks[1]]).cuda()
                m = torch.tensor([[1] * 5, [0, 0, 0, 1, 1]]).cuda()
                p = torch.stack([pos0[0] + 1 + torch.arange(5).cuda(), torch.tensor([0, 0, 0, 1, 2]).cuda() + pos0[1] + (torch.tensor([1, 1, 1, 0, 0]).cuda())])
                h = model.model(x, m, p, cache, torch.zeros_like(x))
                last = h[:, -1]
            else:
                last = [None, None]
                for t in range(5):
                    tok = torch.tensor([[blocks[0][t]], [blocks[1][min(t, 1)]]]).cuda()
                    h = model.model(tok, torch.ones_like(tok), (pos0 + 1 + t).unsqueeze(1), cache, torch.full_like(tok, -1))
                    last[0] = h[0, 0]
                    if t == 1:
                        last[1] = h[1, 0]
                last = torch.stack(last)
        return last, cache, lens0

    a, ca, lens0 = run(True)
    b, cb, _ = run(False)
    assert cf.rel_err(a.cpu(), b.double().cpu()) < 2e-2
    for layer in range(2):
        la = ca.cache_kwargs[layer]["kv_lengths"].cpu()
        assert la.tolist() == (lens0[layer].cpu() + torch.tensor([5, 2])).tolist()
        ka, kb = ca.cache_kwargs[layer]["compacked_key_cache"], cb.cache_kwargs[layer]["compacked_key_cache"]
        for s_, n in enumerate([5, 2]):
            lo = int(lens0[layer][s_])
            assert cf.rel_err(ka[s_, lo:lo + n].cpu(), kb[s_, lo:lo + n].double().cpu()) < 2e-2

    # the round loop itself: a hook that injects once, every sample keeps generating afterwards
    calls = []

    def inject(step, toks):
        calls.append((step, tuple(toks.shape)))
        return [[21, 22, 23], []] if step == 2 else None

    toks, cache = M.generate_interleaved(model, ids, mask, torch.zeros_like(ids), 5, inject)
    assert toks.shape == (2, 5) and calls[0] == (1, (2, 1)) and calls[-1] == (4, (2, 4))
    plain, c0 = model.generate_greedy(ids, mask, torch.zeros_like(ids), 5)
    assert torch.equal(toks[:, :2], plain[:, :2])                           # identical until the injection
    grown = cache.cache_kwargs[1]["kv_lengths"].cpu() - c0.cache_kwargs[1]["kv_lengths"].cpu()
    assert grown.tolist() == [2, 0]                                         # 3 injected tokens replaced 1 generated one


class _StubAttention(torch.nn.Module):
    """Stands in for the attention block: a fixed linear map, so the decoder layer's own norm / residual / MLP
    wiring can be compared between its fused-kernel path on the GPU and the plain torch path on the CPU."""

    def __init__(self, hid, seed):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.a = torch.nn.Parameter(torch.randn((hid, hid), generator=g) * hid ** -0.5)
        self.layer_idx = 0

    def forward(self, hidden_states, *args, **kwargs):
        return hidden_states @ self.a.to(hidden_states.dtype), None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decoder_layer_glue_matches_plain_torch(env, dtype):
    say(f"decoder layer: fused norm / residual / MLP kernels vs plain torch, dtype={dtype}")
    M = env["model"]
    torch.manual_seed(3)
    layer = M.MSADecoderLayer(env["cfg"], 0)
    layer.self_attn = _StubAttention(HID, 5)
    with torch.no_grad():
        for p in layer.parameters():
            if p.dim() == 1:
                p.copy_(1.0 + 0.1 * torch.randn(p.shape))
    layer = layer.eval()
    x = torch.randn((3, 7, HID), generator=torch.Generator().manual_seed(8))
    with torch.no_grad():
        want = layer.double()(x.double(), None, None, None, object())                 # CPU: the plain torch branch
        got = layer.to(dtype).cuda()(x.to(dtype).cuda(), None, None, None, object(), position_ids=None)
    assert cf.rel_err(got.cpu(), want) < (2e-2 if dtype == torch.bfloat16 else 1e-5)
    # the weight-streaming MLP of the decode step against the same module's torch arithmetic
    if dtype == torch.bfloat16:
        h = torch.randn((5, HID), generator=torch.Generator().manual_seed(9)).bfloat16().cuda()
        n2 = layer.post_attention_layernorm
        with torch.no_grad():
            got = layer.mlp.decode_rows(h, n2.weight, n2.variance_epsilon)
            hd = h.double().cpu()
            w = {k: v.double().cpu() for k, v in layer.state_dict().items()}
            normed = hd * torch.rsqrt((hd * hd).mean(-1, keepdim=True) + n2.variance_epsilon) * w["post_attention_layernorm.weight"]
            act = torch.nn.functional.silu(normed @ w["mlp.gate_proj.weight"].T) * (normed @ w["mlp.up_proj.weight"].T)
            want = hd + act @ w["mlp.down_proj.weight"].T
        assert cf.rel_err(got.cpu(), want) < 2e-2


def _layer_bank(env, layer, layer64, lens, g):
    """Stage 1 of a single router layer over `lens` documents, fed to a service block by block; returns the service
    and the fp64 oracle's pooled bank, template prefix and document table."""
    pf, svc_mod = env["prefill"], env["svc"]
    docs = _docs(env, lens)
    service = svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                 env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                 env["config"].MemoryConfig(pooling_kernel_size=P), env["cfg"])
    service.begin(docs)
    bank_k, bank_v, bank_rk, prefix = [], [], [], None
    for blk in pf.split_docs(docs, 8):
        inp = pf.prepare_block_inputs(blk, HEAD_IDS, P)
        T = inp.doc_ids.shape[1]
        hs = torch.randn((1, T, HID), generator=g)
        cos, sin = _tables(env, inp.position_ids)
        cache = env["model"].create_cache()
        cache.record_kwargs(1, {"stage": "prefill_stage1"})
        with torch.no_grad():
            layer(hs.cuda(), inp.doc_ids.cuda(), inp.doc_attention_mask.cuda(), (cos.cuda(), sin.cuda()), cache)
            _, k64, v64 = layer64._project(hs.double(), (cos.double(), sin.double()))
            rk64 = layer64.router_k_proj(hs.double()).view(T, HKV, D)
        _, _, cs, cl, _ = cf.chunk_table(inp.doc_lens, P, 3)
        bank_k.append(cf.pool_chunks(k64[0], cs, cl))
        bank_v.append(cf.pool_chunks(v64[0], cs, cl))
        bank_rk.append(cf.l2_normalize(cf.pool_chunks(rk64, cs, cl)))
        if prefix is None:
            prefix = (k64[0, :3], v64[0, :3])
        service.add_block(cache)
    service.finish()
    _, dco, _, _, _ = cf.chunk_table(lens, P)
    return service, torch.cat(bank_k), torch.cat(bank_v), torch.cat(bank_rk), prefix, dco


def _stage2_with_oracle(env, layer, layer64, bank, hs2, mask, doc_ids, n_q):
    """Stage 2 of the layer on a left-padded batch; returns the cache and, per sample, the oracle's context rows
    ``(K, V)`` = [prefix | selected chunks | the sample's own tokens] built from the documents the layer recalled
    (which are checked against the oracle's scores of the tokens marked 0 in ``doc_ids``)."""
    pf = env["prefill"]
    bank_k, bank_v, bank_rk, prefix, dco = bank
    B, S = mask.shape
    pos = torch.tensor([pf.query_position_ids(n, TOPK, 3, S - n) for n in n_q])
    cos, sin = _tables(env, pos)
    cache = env["model"].create_cache()
    cache.meta["require_recall_topk"] = True
    cache.record_kwargs(1, {"stage": "prefill_stage2"})
    with torch.no_grad():
        out, _ = layer(hs2.cuda(), doc_ids.cuda(), mask.cuda(), (cos.cuda(), sin.cuda()), cache)
        q64, k64, v64 = layer64._project(hs2.double(), (cos.double(), sin.double()))
        rq64 = layer64.router_q_proj(hs2.double()).view(B, S, HQ, D)
    scored = (doc_ids == 0) & mask.bool()                       # only the marked tokens query the memory
    ds = cf.doc_scores(cf.chunk_scores(rq64, scored, bank_rk, "cosine"), dco)
    got_i = torch.tensor([[d - 100 for d in r["topk_doc_ids"]] for r in cache.cache_kwargs[1]["recall_topk"]])
    assert not cf.topk_acceptable(ds, got_i, TOPK, gap=1e-4)
    mk, mv, cu_sel, _ = cf.gather_selected(bank_k, bank_v, dco, got_i)
    ctx = []
    for b in range(B):
        lo = S - n_q[b]
        kk = torch.cat([prefix[0], mk[cu_sel[b]:cu_sel[b + 1]], k64[b, lo:]])
        vv = torch.cat([prefix[1], mv[cu_sel[b]:cu_sel[b + 1]], v64[b, lo:]])
        want = cf.attention(q64[b, lo:], kk, vv, causal=True)
        with torch.no_grad():
            assert cf.rel_err(out[b:b + 1, lo:].cpu(), layer64.o_proj(want.reshape(1, n_q[b], HQ * D))) < TOL
        ctx.append((kk, vv))
    return cache, ctx, pos, ds, got_i


def test_injected_block_rerouted_hop_and_masked_step_against_oracle(env):
    """The Memory-Interleave pieces against the fp64 oracle on one router layer (fp32): a ragged left-padded block of
    source tokens injected in the decode stage at the reference's positions (src/msa/generate.py:235-236) attends
    over the explicit [stage-2 context | block so far] keys and lands in the compact cache; the decode step after it
    sees all of it; a step whose attention mask is 0 for a sample (qa_mode, src/msa/memory_sparse_attention.py:
    375-380) gives that sample no new key; and a second hop routes again with only the tokens its regenerated prompt
    marks with 0 (src/msa_service.py:1734-1770)."""
    say("layer: injected block, masked step and re-routed hop against the oracle")
    pf = env["prefill"]
    layer = _layer(env, seed=2)
    layer64 = copy.deepcopy(layer).double()
    layer = layer.cuda()
    g = torch.Generator().manual_seed(13)
    lens = [5, 8, 17, 1, 30, 9, 16, 23, 12, 7, 40]
    service, bank_k, bank_v, bank_rk, prefix, dco = _layer_bank(env, layer, layer64, lens, g)
    bank = (bank_k, bank_v, bank_rk, prefix, dco)
    layer.set_memory_client(service)
    n_q = [7, 4]
    B, S = 2, 7
    mask = torch.tensor([[1] * 7, [0] * 3 + [1] * 4])
    hs2 = torch.randn((B, S, HID), generator=g)
    cache, ctx, pos, ds1, sel1 = _stage2_with_oracle(env, layer, layer64, bank, hs2, mask, torch.zeros((B, S), dtype=torch.long), n_q)
    cache.cache_kwargs[1]["stage"] = "generate"
    len0 = cache.cache_kwargs[1]["kv_lengths"].cpu().tolist()

    # ---- the injected block: 5 and 2 source tokens, left-padded to 5 columns
    n_new, W = [5, 2], 5
    last_pos = pos[:, -1].tolist()
    p_blk = torch.tensor(pf.source_block_position_ids(last_pos, n_new, W))
    m_blk = torch.tensor([[1] * 5, [0, 0, 0, 1, 1]])
    # the reference's arithmetic, on the columns that hold tokens
    ref_pos = torch.arange(W).unsqueeze(0).expand(B, -1) + pos[:, -1:] + m_blk.sum(dim=1, keepdim=True) - W + 1
    assert torch.equal(p_blk[m_blk.bool()], ref_pos[m_blk.bool()])
    assert p_blk[0].tolist() == [last_pos[0] + 1 + i for i in range(5)] and p_blk[1, 3:].tolist() == [last_pos[1] + 1, last_pos[1] + 2]
    hs_blk = torch.randn((B, W, HID), generator=g)
    cos, sin = _tables(env, p_blk)
    with torch.no_grad():
        out_blk, _ = layer(hs_blk.cuda(), torch.zeros((B, W), dtype=torch.long).cuda(), m_blk.cuda(),
                           (cos.cuda(), sin.cuda()), cache)
        q64, k64, v64 = layer64._project(hs_blk.double(), (cos.double(), sin.double()))
    kw = cache.cache_kwargs[1]
    assert kw["kv_lengths"].cpu().tolist() == [len0[b] + n_new[b] for b in range(B)]
    for b in range(B):
        lo = W - n_new[b]
        ctx[b] = (torch.cat([ctx[b][0], k64[b, lo:]]), torch.cat([ctx[b][1], v64[b, lo:]]))
        want = cf.attention(q64[b, lo:], ctx[b][0], ctx[b][1], causal=True)        # row i sees the block up to i
        with torch.no_grad():
            assert cf.rel_err(out_blk[b:b + 1, lo:].cpu(), layer64.o_proj(want.reshape(1, n_new[b], HQ * D))) < TOL
        assert float(out_blk[b, :lo].abs().max()) == 0.0 if lo else True
        L = len0[b] + n_new[b]
        assert cf.rel_err(kw["compacked_key_cache"][b, :L].cpu(), ctx[b][0]) < TOL       # the whole context, row for row
        assert cf.rel_err(kw["compacked_value_cache"][b, :L].cpu(), ctx[b][1]) < TOL

    # ---- the decode step behind the block sees [context | block | itself]
    last_pos = [last_pos[b] + n_new[b] for b in range(B)]
    hs3 = torch.randn((B, 1, HID), generator=g)
    pos3 = torch.tensor([[x + 1] for x in last_pos])
    cos, sin = _tables(env, pos3)
    with torch.no_grad():
        out3, _ = layer(hs3.cuda(), torch.full((B, 1), -1).cuda(), torch.ones(B, 1, dtype=torch.long).cuda(),
                        (cos.cuda(), sin.cuda()), cache)
        q64, k64, v64 = layer64._project(hs3.double(), (cos.double(), sin.double()))
        for b in range(B):
            ctx[b] = (torch.cat([ctx[b][0], k64[b]]), torch.cat([ctx[b][1], v64[b]]))
            want = layer64.o_proj(cf.attention(q64[b], ctx[b][0], ctx[b][1]).reshape(1, 1, HQ * D))
            assert cf.rel_err(out3[b:b + 1].cpu(), want) < TOL

    # ---- qa_mode: a step whose mask is 0 for sample 1 appends nothing for it
    cache.meta["qa_mode"] = True
    before = kw["kv_lengths"].cpu().tolist()
    hs4 = torch.randn((B, 1, HID), generator=g)
    pos4 = pos3 + 1
    cos, sin = _tables(env, pos4)
    with torch.no_grad():
        out4, _ = layer(hs4.cuda(), torch.full((B, 1), -1).cuda(), torch.tensor([[1], [0]]).cuda(),
                        (cos.cuda(), sin.cuda()), cache)
        q64, k64, v64 = layer64._project(hs4.double(), (cos.double(), sin.double()))
        want = layer64.o_proj(cf.attention(q64[0], torch.cat([ctx[0][0], k64[0]]), torch.cat([ctx[0][1], v64[0]])).reshape(1, 1, HQ * D))
    assert kw["kv_lengths"].cpu().tolist() == [before[0] + 1, before[1]]
    assert cf.rel_err(out4[0:1].cpu(), want) < TOL and float(out4[1].abs().max()) == 0.0

    # ---- second hop: a regenerated prompt routes again, with the tokens it marks 0 only
    n_q2 = [6, 9]
    S2 = 9
    mask2 = torch.tensor([[0] * 3 + [1] * 6, [1] * 9])
    doc2 = torch.tensor([[-1, -1, -1, 0, 0, -1, -1, 0, -1], [0, 0, 0, -1, -1, -1, -1, -1, 0]])
    hs5 = torch.randn((B, S2, HID), generator=g)
    cache2, _, _, ds2, sel2 = _stage2_with_oracle(env, layer, layer64, bank, hs5, mask2, doc2, n_q2)
    # had every token been scored the documents' scores would differ: the mask reached the router
    with torch.no_grad():
        rq_all = layer64.router_q_proj(hs5.double()).view(B, S2, HQ, D)
    ds_all = cf.doc_scores(cf.chunk_scores(rq_all, mask2.bool(), bank_rk, "cosine"), dco)
    assert float((ds_all - ds2).abs().max()) > 1e-3
    assert cache2 is not cache and "compacked_key_cache" in cache2.cache_kwargs[1]    # a new, independent compact cache


def test_generate_blocks_worker_surface_and_hop_loop(env, tmp_path, monkeypatch):
    """``Memory.generate_blocks(docs)`` with a stage-1 worker (src/msa_service.py:497-582, src/prefill.py:142-157,
    300-303) builds the same bank, bit for bit, as feeding the blocks by hand; with MEMORY_DATA_PATH it dumps the
    bank and a second service loads the dump instead of encoding.  Then the hop loop: every hop is a fresh stage-2
    pass over the regenerated prompt."""
    say("model: generate_blocks through the worker, stored bank, hop loop")
    pf, svc_mod, M = env["prefill"], env["svc"], env["model"]
    model = M.MSAForCausalLM(env["cfg"]).init_random(0.05, seed=7).to(torch.bfloat16).cuda().eval()
    docs = _docs(env, [20, 33, 9, 41, 16, 27, 11], first_id=0)

    def new_service():
        return svc_mod.MSAService(0, env["config"].GenerateConfig(devices=[0]),
                                  env["config"].ModelConfig(doc_top_k=TOPK, pooling_kernel_size=P, router_layer_idx="1"),
                                  env["config"].MemoryConfig(block_size=12, pooling_kernel_size=P), env["cfg"])
    by_hand = new_service()
    by_hand.begin(docs)
    for blk in pf.split_docs(docs, 12):
        by_hand.add_block(M.encode_block(model, pf.prepare_block_inputs(blk, HEAD_IDS, P), "cuda"))
    by_hand.finish()

    worker = pf.PrefillStage1Worker(0, model, HEAD_IDS, P)
    meta = worker.inference(pf.split_docs(docs, 12)[0])
    assert set(meta) == {"chunk_sizes", "past_key_values", "nr_docs", "doc_ids", "nr_chunks"}
    first = pf.split_docs(docs, 12)[0]
    assert meta["nr_docs"] == len(first) and meta["doc_ids"] == [d.doc_id for d in first]
    assert meta["nr_chunks"] == [d.num_chunks for d in first] == meta["chunk_sizes"]
    pkv = meta["past_key_values"]
    assert pkv.get_kvcache(1)[0].shape == (1, HKV, sum(meta["chunk_sizes"]), D) and pkv.get_router_kcache(1) is not None
    assert {"pooled_doc_ids", "template_prefix_kcache", "template_prefix_vcache"} <= set(pkv.cache_kwargs[1])

    monkeypatch.setenv("MEMORY_DATA_PATH", str(tmp_path))
    built = new_service()
    built.generate_blocks(docs, worker)
    for a, b in ((by_hand._rk[1], built._rk[1]), (by_hand._k[1], built._k[1]), (by_hand._v[1], built._v[1])):
        assert torch.equal(a.cpu(), b.cpu())
    assert torch.equal(by_hand.block_desc.pool_ids_cpu, built.block_desc.pool_ids_cpu)
    assert torch.equal(by_hand.block_desc.doc_offsets_cpu, built.block_desc.doc_offsets_cpu)
    assert (tmp_path / "gpu1" / "0").exists()
    loaded = new_service()
    loaded.generate_blocks(docs)                               # no worker: the dump is there
    assert torch.equal(loaded._rk[1].cpu(), built._rk[1].cpu()) and torch.equal(loaded._k[1], built._k[1])
    monkeypatch.delenv("MEMORY_DATA_PATH")
    with pytest.raises(ValueError, match="stage-1 worker"):
        new_service().generate_blocks(docs)

    # ---- hop loop on the loaded bank
    loaded.setup_memory_client(model)
    ids = torch.tensor([[5, 6, 7, 8, 9, 10], [0, 0, 11, 12, 13, 14]]).cuda()
    mask = torch.tensor([[1] * 6, [0, 0, 1, 1, 1, 1]]).cuda()
    ids2 = torch.tensor([[41, 42, 43, 44, 45, 46, 47, 48], [0, 0, 0, 51, 52, 53, 54, 55]]).cuda()
    mask2 = torch.tensor([[1] * 8, [0, 0, 0, 1, 1, 1, 1, 1]]).cuda()
    doc2 = torch.tensor([[0, 0, -1, -1, -1, 0, -1, -1], [0, 0, 0, -1, 0, 0, -1, -1]]).cuda()
    seen = []

    def regenerate(hop, toks):
        seen.append((hop, tuple(toks.shape)))
        return (ids2, mask2, doc2) if hop == 0 else None

    passes = M.generate_with_hops(model, ids, mask, torch.zeros_like(ids), 4, regenerate)
    assert len(passes) == 2 and seen == [(0, (2, 4)), (1, (2, 4))]
    (t1, c1), (t2, c2) = passes
    direct, cd = M.generate_interleaved(model, ids2, mask2, doc2, 4, None, require_recall_topk=True)
    assert torch.equal(t2, direct)                             # hop 2 is a complete pass of its own over the new prompt
    r2, rd = c2.cache_kwargs[1]["recall_topk"], cd.cache_kwargs[1]["recall_topk"]
    assert [r["topk_doc_ids"] for r in r2] == [r["topk_doc_ids"] for r in rd]
    assert c2 is not c1 and t1.shape == t2.shape == (2, 4)
