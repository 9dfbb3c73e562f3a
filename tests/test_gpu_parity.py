"""GPU parity: the HIP path (called through the C ABI) against the fp64 closed-form oracle on the
same seeded inputs.  Tolerances are the contract's: 1e-2 (bf16) / 1e-5 (fp32) relative to the
reference's max magnitude; integer and index work is bit-exact; top-k is exact wherever the
boundary gap exceeds 1e-3."""
import math
import sys

import numpy as np
import pytest
import torch

from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 1e-2, torch.float32: 1e-5}


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests need an MI355X")
    from msa_amd import ops as _ops
    return _ops


def _ragged(seed, n_docs, lo, hi):
    g = np.random.default_rng(seed)
    return [int(x) for x in g.integers(lo, hi + 1, size=n_docs)]


def _randn(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


# ------------------------------------------------------------------ chunk table
@pytest.mark.parametrize("P,first", [(64, 3), (4, 0)])
def test_chunk_table(ops, P, first):
    say(f"chunk_table P={P} first={first}")
    lens = _ragged(2, 1500, 1, 40 * P // 8 + 5) + [1, P, P + 1, 2 * P]
    t = ops.chunk_table(lens, P, first)
    torch.cuda.synchronize()
    ds, dco, cs, cl, cd = cf.chunk_table(lens, P, first)
    assert int(t.n_chunks.item()) == len(cs) == t.C
    assert t.doc_chunk_off.cpu().tolist() == dco.tolist()
    assert t.chunk_start.cpu().tolist() == cs.tolist()
    assert t.chunk_len.cpu().tolist() == cl.tolist()
    assert t.chunk_doc.cpu().tolist() == cd.tolist()


# ------------------------------------------------------------------ pooling
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rope", [False, True])
def test_pool_chunks(ops, dtype, rope):
    say(f"pool dtype={dtype} rope={rope}")
    P, H, D, first, theta = 64, 8, 128, 3, 1e6
    lens = _ragged(3, 40, 1, 700) + [1, 64, 65, 128, 2048]
    T = first + sum(lens)
    k, v, kr = (_randn((T, H, D), s, dtype) for s in (10, 11, 12))
    t = ops.chunk_table(lens, P, first)
    tables = ops.rope_tables(2048, D, theta) if rope else None
    pk, pv, pkr = ops.pool_chunks(k.cuda(), v.cuda(), kr.cuda(), t, rope=tables, normalize_kr=True)
    torch.cuda.synchronize()
    _, _, cs, cl, _ = cf.chunk_table(lens, P, first)
    k_ref = k.double()
    if rope:
        k_ref = cf.apply_rope(k_ref, torch.as_tensor(cf.doc_positions(lens, first)), theta)
    want_k = cf.pool_chunks(k_ref, cs, cl)
    want_v = cf.pool_chunks(v, cs, cl)
    want_kr = cf.l2_normalize(cf.pool_chunks(kr, cs, cl))
    tol = TOL[dtype]
    assert cf.rel_err(pk.cpu(), want_k) < tol
    assert cf.rel_err(pv.cpu(), want_v) < tol
    assert cf.rel_err(pkr.cpu(), want_kr) < tol
    # identity on a length-1 document: its only chunk is the token itself (bit-exact without rope)
    if not rope:
        c1 = int(np.nonzero(cl == 1)[0][0])
        assert torch.equal(pv[c1].cpu(), v[int(cs[c1])])


def test_pool_subset_of_tensors_and_linearity(ops):
    say("pool subset / linearity")
    P, H, D = 64, 8, 128
    lens = _ragged(4, 30, 10, 300)
    T = sum(lens)
    x, y = _randn((T, H, D), 1, torch.float32), _randn((T, H, D), 2, torch.float32)
    t = ops.chunk_table(lens, P)
    (_, px, _) = ops.pool_chunks(None, x.cuda(), None, t)
    (_, _, py) = ops.pool_chunks(None, None, y.cuda(), t)
    (pz, _, _) = ops.pool_chunks((2 * x - 0.5 * y).cuda(), None, None, t)
    torch.cuda.synchronize()
    assert cf.rel_err(pz.cpu(), 2 * px.cpu().double() - 0.5 * py.cpu().double()) < 1e-5
    const = torch.full((T, H, D), 0.375)
    (pc, _, _) = ops.pool_chunks(const.cuda(), None, None, t)
    assert torch.allclose(pc.cpu(), torch.full_like(pc.cpu(), 0.375), rtol=1e-6)


# ------------------------------------------------------------------ scoring + top-k
def _make_bank(ops, doc_chunks, Hkv, D, dtype, seed, normalize=True, with_kv=False):
    _, dco, _, _, _ = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    Ctot = int(dco[-1])
    kr = _randn((Ctot, Hkv, D), seed, torch.float32)
    if normalize:
        kr = cf.l2_normalize(kr).float()
    kr = kr.to(dtype)
    gids = [1000 + 7 * d for d in range(len(doc_chunks))]
    bank = ops.Bank(2, dco.tolist(), gids, Hkv, D, dtype)
    kr_dev = kr.cuda()
    kh = vh = None
    if with_kv:
        kh = _randn((Ctot, Hkv, D), seed + 1, dtype).pin_memory()
        vh = _randn((Ctot, Hkv, D), seed + 2, dtype).pin_memory()
    bank.set_layer(1, kr_dev, kh, vh)
    return bank, kr, dco, gids, kh, vh


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["cosine", "scaled_dot"])
@pytest.mark.parametrize("B,S", [(1, 64), (3, 50), (5, 128)])
def test_chunk_scores(ops, dtype, mode, B, S):
    say(f"chunk_scores dtype={dtype} mode={mode} B={B} S={S}")
    Hq, Hkv, D = 32, 8, 128
    doc_chunks = _ragged(5, 150, 1, 9)                       # C not a multiple of the tile
    bank, kr, dco, _, _, _ = _make_bank(ops, doc_chunks, Hkv, D, dtype, 21, normalize=(mode == "cosine"))
    q = _randn((B, S, Hq, D), 22, dtype)
    mask = torch.ones(B, S, dtype=torch.bool)
    if B > 1:
        mask[1, : S // 2] = False                            # left padding
        mask[2, 5] = False
    got = ops.chunk_scores(bank, 1, q.cuda(), mask.cuda(), mode, D ** -0.5)
    torch.cuda.synchronize()
    want = cf.chunk_scores(q, mask, kr, mode)
    assert cf.rel_err(got.cpu(), want) < TOL[dtype]
    # no mask == all-ones mask
    got2 = ops.chunk_scores(bank, 1, q.cuda(), None, mode, D ** -0.5)
    want2 = cf.chunk_scores(q, torch.ones(B, S, dtype=torch.bool), kr, mode)
    assert cf.rel_err(got2.cpu(), want2) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["cosine", "scaled_dot"])
@pytest.mark.parametrize("query_reduce,chunk_reduce", [("mean", "max"), ("last", "max"), ("max", "mean"), ("mean", "mean"),
                                                        ("last", "mean")])
def test_route_topk_other_reductions(ops, dtype, mode, query_reduce, chunk_reduce):
    """query_reduce_method mean / last and chunk_reduce_method mean (src/msa_service.py:751-811) against the oracle:
    scores of the returned documents within tolerance, the selection by the acceptance rule, a query without scored
    tokens all -inf."""
    say(f"route_topk_reduce dtype={dtype} mode={mode} query={query_reduce} chunk={chunk_reduce}")
    B, S, Hq, Hkv, D, k = 6, 50, 32, 8, 128, 8
    doc_chunks = _ragged(8, 700, 1, 7)
    bank, kr, dco, gids, _, _ = _make_bank(ops, doc_chunks, Hkv, D, dtype, 61, normalize=(mode == "cosine"))
    q = _randn((B, S, Hq, D), 62, dtype)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[1, S // 2:] = False                                  # a prefix of scored tokens
    mask[2, 3] = False; mask[2, 10] = False                   # holes (position count - 1 is scored)
    mask[3] = False                                           # nothing scored
    mask[4, 1:] = False                                       # one token
    scores, doc, gid = ops.route_topk(bank, 1, q.cuda(), mask.cuda(), mode, D ** -0.5, k, query_reduce=query_reduce,
                                      chunk_reduce=chunk_reduce)
    torch.cuda.synchronize()
    scores, doc = scores.cpu(), doc.cpu().long()
    ds = cf.doc_scores(cf.chunk_scores(q, mask, kr, mode, query_reduce=query_reduce), dco, chunk_reduce)
    live = [b for b in range(B) if b != 3]
    assert torch.isinf(scores[3]).all() and (scores[3] < 0).all()
    # mean scores sit close together: the acceptance gap is widened by the dtype's score error
    scale = float(ds[live].abs().max())
    gap = max(1e-3, 2 * TOL[dtype] * scale)
    assert not cf.topk_acceptable(ds[live], doc[live], k, gap=gap)
    picked = torch.gather(ds[live], 1, doc[live])
    assert cf.rel_err(scores[live], picked) < TOL[dtype]
    assert (scores[live][:, :-1] >= scores[live][:, 1:]).all()


def test_chunk_scores_fully_masked_query(ops):
    say("chunk_scores fully masked")
    bank, kr, *_ = _make_bank(ops, [3, 4, 5], 8, 128, torch.bfloat16, 31)
    q = _randn((2, 40, 32, 128), 32, torch.bfloat16)
    mask = torch.ones(2, 40, dtype=torch.bool); mask[0] = False
    got = ops.chunk_scores(bank, 1, q.cuda(), mask.cuda()).cpu()
    assert torch.isinf(got[0]).all() and (got[0] < 0).all() and torch.isfinite(got[1]).all()


def _plant(q, kr, dco, b, t, doc, strength, dtype):
    """Makes one chunk of `doc` point along query token (b, t): its cosine score becomes ~strength."""
    Hq, D = q.shape[2], q.shape[3]
    Hkv = kr.shape[1]
    G = Hq // Hkv
    qn = cf.l2_normalize(q[b, t].double()).view(Hkv, G, D).sum(1)              # [Hkv, D]
    direction = cf.l2_normalize(qn)
    c = int(dco[doc]) + (int(dco[doc + 1]) - int(dco[doc])) // 2
    noise = cf.l2_normalize(kr[c].double())
    mix = cf.l2_normalize(strength * direction + (1 - strength) * noise)
    kr[c] = mix.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_route_topk_needles_and_acceptance(ops, dtype):
    say(f"route_topk dtype={dtype}")
    B, S, Hq, Hkv, D, k = 4, 70, 32, 8, 128, 16
    doc_chunks = _ragged(6, 9000, 1, 6)                      # > 4096 documents: several candidate blocks
    _, dco, _, _, _ = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    kr = cf.l2_normalize(_randn((int(dco[-1]), Hkv, D), 41, torch.float32)).float().to(dtype)
    q = _randn((B, S, Hq, D), 42, dtype)
    g = np.random.default_rng(7)
    planted = {}
    for b in range(B):
        docs = g.choice(len(doc_chunks), size=k, replace=False)
        planted[b] = [int(d) for d in docs]
        tok = int(g.integers(0, S))                          # one token per query: score is monotone in strength
        for r, d in enumerate(docs):
            _plant(q, kr, dco, b, tok, int(d), 0.9 - 0.04 * r, dtype)                     # separated by >> 1e-3
    gids = [5 * d + 3 for d in range(len(doc_chunks))]
    bank = ops.Bank(1, dco.tolist(), gids, Hkv, D, dtype)
    kr_dev = kr.cuda()
    bank.set_layer(0, kr_dev)
    mask = torch.ones(B, S, dtype=torch.bool)
    scores, doc, gid = ops.route_topk(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0, k)
    torch.cuda.synchronize()
    scores, doc, gid = scores.cpu(), doc.cpu().long(), gid.cpu()
    ds = cf.doc_scores(cf.chunk_scores(q, mask, kr, "cosine"), dco)
    want_s, want_i = cf.topk_docs(ds, k)
    gaps = (want_s[:, :-1] - want_s[:, 1:]).min()
    assert float(gaps) > 1e-3, "fixture must separate every rank by more than the contract's gap"
    assert torch.equal(doc, want_i)                          # bit-exact ids, in order
    for b in range(B):
        assert sorted(doc[b].tolist()) == sorted(planted[b])
    assert torch.equal(gid, torch.as_tensor(gids)[doc])
    assert cf.rel_err(scores, want_s) < TOL[dtype]
    assert (scores[:, :-1] >= scores[:, 1:]).all()


def test_route_topk_random_bank_acceptance_and_small_bank(ops):
    say("route_topk acceptance on an un-planted bank; fewer docs than k")
    B, S, Hq, Hkv, D, k = 3, 33, 32, 8, 128, 16
    doc_chunks = _ragged(8, 5000, 1, 5)
    bank, kr, dco, gids, _, _ = _make_bank(ops, doc_chunks, Hkv, D, torch.bfloat16, 51)
    q = _randn((B, S, Hq, D), 52, torch.bfloat16)
    scores, doc, gid = ops.route_topk(bank, 1, q.cuda(), None, "cosine", 1.0, k)
    ds = cf.doc_scores(cf.chunk_scores(q, torch.ones(B, S, dtype=torch.bool), kr, "cosine"), dco)
    # bf16 scores carry ~1e-2 relative error, so the index contract is the gap rule
    errs = cf.topk_acceptable(ds, doc.cpu().long(), k, gap=1e-3)
    assert not errs, errs
    # returned scores are the kernel's own doc scores, sorted, and match the oracle's for those docs
    picked = torch.gather(ds, 1, doc.cpu().long())
    assert cf.rel_err(scores.cpu(), picked) < 1e-2
    # 5 documents, k = 16: tail is (-inf, -1)
    bank2, kr2, dco2, gids2, _, _ = _make_bank(ops, [2, 1, 3, 1, 2], Hkv, D, torch.bfloat16, 53)
    s2, d2, g2 = ops.route_topk(bank2, 1, q.cuda(), None, "cosine", 1.0, k)
    d2 = d2.cpu()
    assert (d2[:, 5:] == -1).all() and (g2.cpu()[:, 5:] == -1).all() and torch.isinf(s2.cpu()[:, 5:]).all()
    for b in range(B):
        assert sorted(d2[b, :5].tolist()) == [0, 1, 2, 3, 4]


def test_route_topk_ties_are_broken_by_lower_doc(ops):
    say("route_topk ties")
    Hkv, D = 8, 128
    doc_chunks = [1] * 40
    _, dco, _, _, _ = cf.chunk_table([4] * 40, 4)
    row = cf.l2_normalize(_randn((1, Hkv, D), 61, torch.float32)).float()
    kr = row.expand(40, Hkv, D).contiguous().to(torch.bfloat16)          # every document scores the same
    bank = ops.Bank(1, dco.tolist(), list(range(40)), Hkv, D, torch.bfloat16)
    kr_dev = kr.cuda()
    bank.set_layer(0, kr_dev)
    q = _randn((2, 8, 32, D), 62, torch.bfloat16)
    s, d, _ = ops.route_topk(bank, 0, q.cuda(), None, "cosine", 1.0, 16)
    assert d.cpu().tolist() == [list(range(16))] * 2
    assert float((s.cpu().max(1).values - s.cpu().min(1).values).max()) == 0.0


# ------------------------------------------------------------------ gather
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gather_kv_exact(ops, dtype):
    say(f"gather dtype={dtype}")
    doc_chunks = _ragged(9, 300, 1, 8)
    bank, _, dco, _, kh, vh = _make_bank(ops, doc_chunks, 8, 128, dtype, 71, with_kv=True)
    sel = torch.tensor([[5, 6, 7, 290, 0, 12, -1, 12], [299, 298, 1, 0, 2, 150, 151, 3], [-1] * 8, [42] * 8],
                       dtype=torch.int32)
    side = torch.cuda.Stream()
    K, V, cu = ops.gather_kv(bank, 1, sel, "cuda", stream=side)
    side.synchronize()
    wk, wv, wcu, _ = cf.gather_selected(kh, vh, dco, sel)
    assert cu.tolist() == wcu.tolist()
    assert torch.equal(K.cpu(), wk) and torch.equal(V.cpu(), wv)
    # device-side gather: same rows, same order, ids never leave the device; out-of-range ids are skipped
    sel_dev = torch.cat([sel, torch.tensor([[300, -5, 7, 7, 7, 7, 7, 6]], dtype=torch.int32)]).cuda()
    cap = sel_dev.shape[0] * sel_dev.shape[1] * bank.max_doc_chunks
    Kd, Vd, cud = ops.gather_kv_device(bank, 1, sel_dev, cap)
    torch.cuda.synchronize()
    sel_ref = torch.cat([sel, torch.tensor([[-1, -1, 7, 7, 7, 7, 7, 6]], dtype=torch.int32)])
    wk2, wv2, wcu2, _ = cf.gather_selected(kh, vh, dco, sel_ref)
    assert cud.cpu().tolist() == wcu2.tolist()
    n = int(wcu2[-1])
    assert torch.equal(Kd[:n].cpu(), wk2) and torch.equal(Vd[:n].cpu(), wv2)
    # a short output drops the overflowing rows instead of writing past the end
    Ks, Vs, cus = ops.gather_kv_device(bank, 1, sel_dev, 10)
    torch.cuda.synchronize()
    # ... and the prefix sums stop at the capacity, so no consumer addresses a row that was never filled
    assert torch.equal(Ks.cpu(), wk2[:10]) and cus.cpu().tolist() == [min(int(x), 10) for x in wcu2.tolist()]
    # documents shared by several samples (fetched from the host once, copied on the device for the others;
    # src/msa_service.py:1214): every sample still gets its own complete rows, on both gather paths
    shared = torch.tensor([[9, 3, 200, 7], [3, 9, 7, 200], [200, 200, 3, 5], [5, 3, 9, 7], [1, 2, 3, 4]], dtype=torch.int32)
    wk3, wv3, wcu3, _ = cf.gather_selected(kh, vh, dco, shared)
    K3, V3, cu3 = ops.gather_kv(bank, 1, shared, "cuda", stream=side)
    side.synchronize()
    assert cu3.tolist() == wcu3.tolist() and torch.equal(K3.cpu(), wk3) and torch.equal(V3.cpu(), wv3)
    Kd3, Vd3, cud3 = ops.gather_kv_device(bank, 1, shared.cuda(), shared.numel() * bank.max_doc_chunks)
    torch.cuda.synchronize()
    n3 = int(wcu3[-1])
    assert cud3.cpu().tolist() == wcu3.tolist() and torch.equal(Kd3[:n3].cpu(), wk3) and torch.equal(Vd3[:n3].cpu(), wv3)
    with pytest.raises(Exception, match="outside"):
        ops.gather_kv(bank, 1, torch.tensor([[300]], dtype=torch.int32), "cuda")
    with pytest.raises(Exception, match="no host K"):
        ops.gather_kv(bank, 0, sel, "cuda")


# ------------------------------------------------------------------ assembly, append, attention
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_assemble_append_attention(ops, dtype):
    say(f"assemble/append/attention dtype={dtype}")
    B, Hq, Hkv, D = 3, 32, 8, 128
    n_sel = [37, 0, 300]
    n_loc = [64, 5, 200]
    prefix_k, prefix_v = _randn((3, Hkv, D), 80, dtype), _randn((3, Hkv, D), 81, dtype)
    mem_k, mem_v = _randn((sum(n_sel), Hkv, D), 82, dtype), _randn((sum(n_sel), Hkv, D), 83, dtype)
    loc_k, loc_v = _randn((sum(n_loc), Hkv, D), 84, dtype), _randn((sum(n_loc), Hkv, D), 85, dtype)
    cu_sel = np.concatenate([[0], np.cumsum(n_sel)])
    cu_loc = np.concatenate([[0], np.cumsum(n_loc)])
    Lcap = 3 + max(a + b for a, b in zip(n_sel, n_loc)) + 4
    dev = lambda t: t.cuda()
    i32 = lambda a: torch.as_tensor(a, dtype=torch.int32).cuda()
    kc, vc, kv_len = ops.assemble_context(dev(prefix_k), dev(prefix_v), dev(mem_k), dev(mem_v), i32(cu_sel),
                                          dev(loc_k), dev(loc_v), i32(cu_loc), B, Lcap)
    torch.cuda.synchronize()
    wk, wcu = cf.assemble_context(prefix_k, mem_k, cu_sel, loc_k, cu_loc)
    wv, _ = cf.assemble_context(prefix_v, mem_v, cu_sel, loc_v, cu_loc)
    lens = np.diff(wcu)
    assert kv_len.cpu().tolist() == lens.tolist()
    for b in range(B):
        assert torch.equal(kc[b, : lens[b]].cpu(), wk[wcu[b]: wcu[b + 1]])
        assert torch.equal(vc[b, : lens[b]].cpu(), wv[wcu[b]: wcu[b + 1]])

    # stage-2 style: the query's own S_b rows are the last S_b keys; causal, bottom-right aligned
    q_rows = n_loc
    q = _randn((sum(q_rows), Hq, D), 86, dtype)
    kv_off = (torch.arange(B, dtype=torch.int64) * Lcap).cuda()
    out = ops.sparse_attn(dev(q), kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), kv_off, kv_len, int(lens.max()),
                          cu_q=i32(cu_loc), max_sq=max(q_rows), causal=True)
    torch.cuda.synchronize()
    want = cf.attention_ragged(q, cu_loc, wk, wv, wcu, causal=True)
    assert cf.rel_err(out.cpu(), want) < TOL[dtype]

    # decode: append one row per sample, one query row per sample over everything
    k_new, v_new = _randn((B, Hkv, D), 87, dtype), _randn((B, Hkv, D), 88, dtype)
    ops.cache_append(dev(k_new), dev(v_new), kc, vc, kv_len)
    assert kv_len.cpu().tolist() == (lens + 1).tolist()
    qd = _randn((B, Hq, D), 89, dtype)
    outd = ops.sparse_attn(dev(qd), kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), kv_off, kv_len, int(lens.max()) + 1)
    torch.cuda.synchronize()
    for b in range(B):
        kk = torch.cat([wk[wcu[b]: wcu[b + 1]], k_new[b: b + 1]])
        vv = torch.cat([wv[wcu[b]: wcu[b + 1]], v_new[b: b + 1]])
        assert cf.rel_err(outd[b: b + 1].cpu(), cf.attention(qd[b: b + 1], kk, vv)) < TOL[dtype]


def test_attention_long_context_splits_and_special_cases(ops):
    say("attention long / special cases")
    Hq, Hkv, D = 32, 8, 128
    L = [4500, 1, 777]
    B = len(L)
    Lcap = max(L)
    k = _randn((B, Lcap, Hkv, D), 90, torch.bfloat16)
    v = _randn((B, Lcap, Hkv, D), 91, torch.bfloat16)
    q = _randn((B, Hq, D), 92, torch.bfloat16)
    kv_off = (torch.arange(B, dtype=torch.int64) * Lcap).cuda()
    kv_len = torch.tensor(L, dtype=torch.int32).cuda()
    out = ops.sparse_attn(q.cuda(), k.cuda().view(-1, Hkv, D), v.cuda().view(-1, Hkv, D), kv_off, kv_len, Lcap).cpu()
    for b in range(B):
        want = cf.attention(q[b: b + 1], k[b, : L[b]], v[b, : L[b]])
        assert cf.rel_err(out[b: b + 1], want) < 1e-2
    # a single key returns its value exactly (bf16 in, bf16 out)
    assert torch.equal(out[1].view(Hkv, 4, D), v[1, 0][:, None, :].expand(Hkv, 4, D))


# ------------------------------------------------------------------ the CPU-runnable routing layer
def test_config1_routing_layer_fp32(ops):
    """1,000 documents of 512 tokens, 8 KV heads, head_dim 128, pooled at 64; 64 query tokens,
    32 Q heads; cosine / mean heads / max tokens / max chunks; top-16; gather; one decode step over
    [memory | 64 local tokens].  Pooling runs in blocks of 100 documents as stage 1 does."""
    say("config 1 (fp32, seed 0)")
    n_docs, doc_len, P, Hq, Hkv, D, k, S = 1000, 512, 64, 32, 8, 128, 16, 64
    per_block = 100
    g = torch.Generator().manual_seed(0)
    pooled = {"k": [], "v": [], "kr": []}
    oracle_pooled = {"k": [], "v": [], "kr": []}
    for blk in range(n_docs // per_block):
        lens = [doc_len] * per_block
        T = sum(lens)
        kk, vv, rr = (torch.randn((T, Hkv, D), generator=g) for _ in range(3))
        t = ops.chunk_table(lens, P)
        pk, pv, pkr = ops.pool_chunks(kk.cuda(), vv.cuda(), rr.cuda(), t, normalize_kr=True)
        pooled["k"].append(pk.cpu()); pooled["v"].append(pv.cpu()); pooled["kr"].append(pkr)
        if blk in (0, 9):                                   # whole chunks: the library routine pins the mean
            for name, x in (("k", kk), ("v", vv)):
                want = x.double().view(-1, P, Hkv, D).mean(1)
                assert cf.rel_err(pooled[name][-1], want) < 1e-5
            assert cf.rel_err(pkr.cpu(), cf.l2_normalize(rr.double().view(-1, P, Hkv, D).mean(1))) < 1e-5
    k_bank = torch.cat(pooled["k"]).pin_memory()
    v_bank = torch.cat(pooled["v"]).pin_memory()
    kr_bank = torch.cat(pooled["kr"])
    C = kr_bank.shape[0]
    assert C == 8000
    dco = (np.arange(n_docs + 1) * (doc_len // P)).astype(np.int64)
    bank = ops.Bank(1, dco.tolist(), list(range(n_docs)), Hkv, D, torch.float32)
    bank.set_layer(0, kr_bank, k_bank, v_bank)
    q = torch.randn((1, S, Hq, D), generator=g)
    mask = torch.ones(1, S, dtype=torch.bool)
    scores, doc, gid = ops.route_topk(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0, k)
    cs = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0)
    torch.cuda.synchronize()
    kr_cpu = kr_bank.cpu()
    want_cs = cf.chunk_scores(q, mask, kr_cpu, "cosine")
    assert cf.rel_err(cs.cpu(), want_cs) < 1e-5
    ds = cf.doc_scores(want_cs, dco)
    assert not cf.topk_acceptable(ds, doc.cpu().long(), k, gap=1e-3)
    want_s, want_i = cf.topk_docs(ds, k)
    assert cf.rel_err(scores.cpu(), want_s) < 1e-5
    # fp32 error is ~1e-7, far below typical rank gaps: ids agree wherever ranks are separated by > 1e-5
    sep = (want_s[0, :-1] - want_s[0, 1:]) > 1e-5
    if bool(sep.all()):
        assert torch.equal(doc.cpu().long(), want_i)
    # gather + decode over [memory | 64 local tokens]
    K, V, cu = ops.gather_kv(bank, 0, doc.cpu(), "cuda")
    torch.cuda.synchronize()
    wk, wv, wcu, _ = cf.gather_selected(k_bank, v_bank, dco, doc.cpu().long())
    assert torch.equal(K.cpu(), wk) and torch.equal(V.cpu(), wv) and int(cu[-1]) == 16 * 8
    loc_k, loc_v = torch.randn((64, Hkv, D), generator=g), torch.randn((64, Hkv, D), generator=g)
    qd = torch.randn((1, Hq, D), generator=g)
    i32 = lambda a: torch.as_tensor(a, dtype=torch.int32).cuda()
    kc, vc, kv_len = ops.assemble_context(None, None, K, V, i32(cu.tolist()), loc_k.cuda(), loc_v.cuda(),
                                          i32([0, 64]), 1, 256)
    out = ops.sparse_attn(qd.cuda(), kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), torch.zeros(1, dtype=torch.int64).cuda(),
                          kv_len, 192)
    torch.cuda.synchronize()
    want = cf.attention(qd, torch.cat([wk, loc_k]), torch.cat([wv, loc_v]))
    assert cf.rel_err(out.cpu(), want) < 1e-5


# ------------------------------------------------------------------ fused projection GEMM
def test_qkv_proj_refuses_operands_the_kernel_would_misread(ops):
    """fp32 norm weights, a rotary table of the wrong width or type, and a misaligned weight view are refused on the
    host instead of being read as something else."""
    say("qkv_proj argument checks")
    D, T, K = 128, 64, 128
    x = torch.zeros((T, K), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((4 * D, K), dtype=torch.bfloat16, device="cuda")
    pos = torch.zeros(T, dtype=torch.int64, device="cuda")
    nw = torch.ones(D, dtype=torch.bfloat16, device="cuda")
    rope = ops.rope_tables(16, D, 1e6)
    ops.qkv_proj(x, w, 2, 1, pos, nw, nw, 1e-6, rope)
    with pytest.raises(ValueError, match="q_norm_w"):
        ops.qkv_proj(x, w, 2, 1, pos, nw.float(), nw, 1e-6, rope)
    with pytest.raises(ValueError, match="k_norm_w"):
        ops.qkv_proj(x, w, 2, 1, pos, nw, nw[:64], 1e-6, rope)
    with pytest.raises(ValueError, match="table"):
        ops.qkv_proj(x, w, 2, 1, pos, nw, nw, 1e-6, (rope[0].double(), rope[1].double()))
    with pytest.raises(ValueError, match="table"):
        ops.qkv_proj(x, w, 2, 1, pos, nw, nw, 1e-6, (rope[0][:, :32].contiguous(), rope[1][:, :32].contiguous()))
    wide = torch.zeros((4 * D * K + 4,), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="aligned"):
        ops.qkv_proj(x, wide[4:].view(4 * D, K), 2, 1, pos, nw, nw, 1e-6, rope)


@pytest.mark.parametrize("T,K,Hq,Hkv,front,back", [(300, 320, 4, 2, 2, 0), (70, 64, 8, 1, 0, 8), (513, 2560, 32, 8, 8, 0),
                                                    (1000, 2560, 32, 8, 0, 32), (257, 192, 3, 1, 0, 0)])
def test_qkv_proj_gemm_with_norm_rope_epilogue(ops, T, K, Hq, Hkv, front, back):
    """x . [router | q | k | v | router]^T with the q / k RMSNorm + rotary in the GEMM's epilogue against fp64
    F.linear + Qwen3RMSNorm + the rotary by the table entries the kernel reads (and the fp64 rotary at small
    positions); v and the router heads are the plain projection.  Ragged token counts (partial M tiles), head
    counts that leave half an N tile empty, router heads in front (stage 1) or behind (stage 2)."""
    say(f"qkv_proj T={T} K={K} Hq={Hq} Hkv={Hkv} router front={front} back={back}")
    D, eps, theta = 128, 1e-6, 1e6
    heads = front + Hq + 2 * Hkv + back
    x = _randn((T, K), 300 + T, torch.bfloat16)
    w = (_randn((heads * D, K), 301 + K, torch.float32) * K ** -0.5).to(torch.bfloat16)
    qw = (1 + 0.1 * _randn((D,), 302, torch.float32)).to(torch.bfloat16)
    kw = (1 + 0.1 * _randn((D,), 303, torch.float32)).to(torch.bfloat16)
    g = torch.Generator().manual_seed(304)
    pos = torch.randint(0, 4000, (T,), generator=g, dtype=torch.int64)
    pos[: min(T, 40)] = torch.arange(min(T, 40))
    rope = ops.rope_tables(4096, D, theta)
    q, k, v, r = ops.qkv_proj(x.cuda(), w.cuda(), Hq, Hkv, pos.cuda(), qw.cuda(), kw.cuda(), eps, rope,
                              router_front=front, router_back=back)
    torch.cuda.synchronize()
    y = (x.double() @ w.double().T).view(T, heads, D)

    def norm(t, wt):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * wt.double()
    c, s_ = rope[0].cpu().double()[pos][:, None, :], rope[1].cpu().double()[pos][:, None, :]

    def rot(t):
        a, b = t[..., :64], t[..., 64:]
        return torch.cat([a * c - b * s_, b * c + a * s_], dim=-1)
    nq, nk = norm(y[:, front:front + Hq], qw), norm(y[:, front + Hq:front + Hq + Hkv], kw)
    tol = 1e-2
    assert q.shape == (T, Hq, D) and k.shape == (T, Hkv, D) and v.shape == (T, Hkv, D)
    assert cf.rel_err(q.cpu(), rot(nq)) < tol and cf.rel_err(k.cpu(), rot(nk)) < tol
    small = pos < 64
    assert cf.rel_err(q.cpu()[small], cf.apply_rope(nq[small], pos[small], theta)) < tol
    assert cf.rel_err(v.cpu(), y[:, front + Hq + Hkv:front + Hq + 2 * Hkv]) < tol
    if front + back:
        want_r = torch.cat([y[:, :front], y[:, front + Hq + 2 * Hkv:]], dim=1)
        assert r.shape == (T, front + back, D) and cf.rel_err(r.cpu(), want_r) < tol
    else:
        assert r is None
    # the two-step path (vendor GEMM, then the norm + rotary kernel) lands on the same values up to bf16 rounding
    qkv = torch.nn.functional.linear(x.cuda(), w.cuda()[front * D:(front + Hq + 2 * Hkv) * D])
    q2, k2, v2 = ops.qk_norm_rope(qkv, Hq, Hkv, D, pos.cuda(), qw.cuda(), kw.cuda(), eps, rope)
    assert cf.rel_err(q.cpu(), q2.double().cpu()) < 2e-2 and cf.rel_err(k.cpu(), k2.double().cpu()) < 2e-2


# ------------------------------------------------------------------ fused layer helpers
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_qk_norm_rope_rmsnorm_silu(ops, dtype):
    say(f"qk_norm_rope / rmsnorm / silu_mul dtype={dtype}")
    N, Hq, Hkv, D, theta, eps = 37, 32, 8, 128, 1e6, 1e-6
    qkv = _randn((N, (Hq + 2 * Hkv) * D), 100, dtype)
    qw, kw = (1 + 0.1 * _randn((D,), 101, torch.float32)).to(dtype), (1 + 0.1 * _randn((D,), 102, torch.float32)).to(dtype)
    pos = torch.tensor([0, 1, 5, 19, 4387, 2047] + list(range(100, 131)), dtype=torch.int64)
    rope = ops.rope_tables(8192, D, theta)
    q, k, v = ops.qk_norm_rope(qkv.cuda(), Hq, Hkv, D, pos.cuda(), qw.cuda(), kw.cuda(), eps, rope)
    x = qkv.double().view(N, Hq + 2 * Hkv, D)

    def norm(t, w):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    nq, nk = norm(x[:, :Hq], qw), norm(x[:, Hq:Hq + Hkv], kw)
    # (a) small positions against the fp64 rotary (pins pairing and signs; fp32 angle error is negligible there)
    small = pos < 64
    assert cf.rel_err(q.cpu()[small], cf.apply_rope(nq[small], pos[small], theta)) < TOL[dtype]
    assert cf.rel_err(k.cpu()[small], cf.apply_rope(nk[small], pos[small], theta)) < TOL[dtype]
    # (b) every position against a rotation by the SAME fp32 table entries the kernel reads: the tables carry the
    # fp32 angle rounding of Qwen3's rotary embedding (about 4387 * 2^-24 rad at the largest position here)
    c, s_ = rope[0].cpu().double()[pos][:, None, :], rope[1].cpu().double()[pos][:, None, :]

    def rot(t):
        a, b = t[..., :64], t[..., 64:]
        return torch.cat([a * c - b * s_, b * c + a * s_], dim=-1)
    assert cf.rel_err(q.cpu(), rot(nq)) < TOL[dtype] and cf.rel_err(k.cpu(), rot(nk)) < TOL[dtype]
    assert torch.equal(v.cpu(), qkv.view(N, Hq + 2 * Hkv, D)[:, Hq + Hkv:])

    H = 2560
    xs, res, w = _randn((N, H), 103, dtype), _randn((N, H), 104, dtype), (1 + 0.1 * _randn((H,), 105, torch.float32)).to(dtype)
    out = ops.rmsnorm(xs.cuda(), w.cuda(), eps)
    assert cf.rel_err(out.cpu(), norm(xs.double(), w)) < TOL[dtype]
    res_dev = res.cuda()
    out2 = ops.rmsnorm(xs.cuda(), w.cuda(), eps, residual=res_dev)
    summed = (xs.double() + res.double()).to(dtype)                       # the sum is stored in the model dtype
    assert torch.equal(res_dev.cpu(), summed)
    assert cf.rel_err(out2.cpu(), norm(summed.double(), w)) < TOL[dtype]

    gu = _randn((N, 2 * 1024), 106, dtype)
    got = ops.silu_mul(gu.cuda())
    g64, u64 = gu.double()[:, :1024], gu.double()[:, 1024:]
    assert cf.rel_err(got.cpu(), g64 * torch.sigmoid(g64) * u64) < TOL[dtype]


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (8, 8), (16, 8), (16, 2), (6, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_attention_blocks(ops, Hq, Hkv, causal):
    say(f"flash attention Hq={Hkv} Hkv={Hkv} causal={causal}")
    D = 128
    sq = [130, 1, 33, 64, 17]                 # ragged query blocks, including a single row and non-multiples of the tile
    L = [400, 70, 33, 1000, 90]               # keys per sample (>= sq for the causal alignment)
    B = len(sq)
    cu_q = np.concatenate([[0], np.cumsum(sq)])
    cu_kv = np.concatenate([[0], np.cumsum(L)])
    q = _randn((int(cu_q[-1]), Hq, D), 200, torch.bfloat16)
    k = _randn((int(cu_kv[-1]), Hkv, D), 201, torch.bfloat16)
    v = _randn((int(cu_kv[-1]), Hkv, D), 202, torch.bfloat16)
    kv_off = torch.as_tensor(cu_kv[:-1], dtype=torch.int64).cuda()
    kv_len = torch.as_tensor(L, dtype=torch.int32).cuda()
    out = ops.sparse_attn(q.cuda(), k.cuda(), v.cuda(), kv_off, kv_len, max(L),
                          cu_q=torch.as_tensor(cu_q, dtype=torch.int32).cuda(), max_sq=max(sq), causal=causal)
    torch.cuda.synchronize()
    want = cf.attention_ragged(q, cu_q, k, v, cu_kv, causal=causal)
    assert cf.rel_err(out.cpu(), want) < 1e-2
    # the split-KV kernel (forced by a high threshold) must agree with the flash kernel
    old = ops.FLASH_MIN_ROWS
    try:
        ops.FLASH_MIN_ROWS = 1 << 30
        out2 = ops.sparse_attn(q.cuda(), k.cuda(), v.cuda(), kv_off, kv_len, max(L),
                               cu_q=torch.as_tensor(cu_q, dtype=torch.int32).cuda(), max_sq=max(sq), causal=causal)
    finally:
        ops.FLASH_MIN_ROWS = old
    assert cf.rel_err(out2.cpu(), want) < 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_by_hand_fixture_through_the_c_abi(ops, dtype):
    """tests/golden/by_hand.json (numbers derived by hand on one-hot vectors) through the HIP path: exact in both
    dtypes, since every operand and every result is a small dyadic number."""
    say(f"by-hand fixture dtype={dtype}")
    from tests.golden import by_hand
    fx = by_hand.load()
    q, mask, kr, dco = by_hand.tensors(fx, dtype)
    bank = ops.Bank(1, dco.tolist(), [10, 20, 30], fx["Hkv"], fx["D"], dtype)
    kr_dev = kr.cuda()
    kh = torch.arange(6, dtype=torch.float32).view(6, 1, 1).expand(6, 2, 128).to(dtype).contiguous().pin_memory()
    bank.set_layer(0, kr_dev, kh, kh)
    cs = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0).cpu()
    assert torch.equal(cs, torch.tensor(fx["chunk_scores_cosine"]))
    sd = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda(), "scaled_dot", fx["D"] ** -0.5).cpu()
    assert torch.allclose(sd, torch.tensor(fx["chunk_scores_cosine"]) * fx["scaled_dot_factor"], rtol=1e-6)
    for k, key in ((2, "top2"), (3, "top3")):
        s, doc, gid = ops.route_topk(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0, k)
        assert doc.cpu().tolist() == fx[key]                                  # the tie goes to the lower document id
        assert gid.cpu().tolist() == [[10 * (d + 1) for d in row] for row in fx[key]]
        want = torch.tensor(fx["doc_scores_cosine"]).gather(1, torch.tensor(fx[key]))
        assert torch.equal(s.cpu(), want)
    p = fx["pool"]
    t = ops.chunk_table(p["doc_lens"], p["P"])
    assert (t.chunk_start.cpu().tolist(), t.chunk_len.cpu().tolist(), t.chunk_doc.cpu().tolist()) == \
        (p["chunk_start"], p["chunk_len"], p["chunk_doc"])
    x = (torch.arange(sum(p["doc_lens"]), dtype=torch.float32) + 1).view(-1, 1, 1).expand(-1, 8, 128).to(dtype).contiguous().cuda()
    pk, pv, pkr = ops.pool_chunks(x, x, x, t, normalize_kr=True)
    assert torch.equal(pv[:, 0, 0].float().cpu(), torch.tensor(p["chunk_mean"]))
    assert torch.allclose(pkr.float().cpu(), torch.full((3, 8, 128), p["normalized_element"]), rtol=TOL[dtype])
    gth = fx["gather"]
    sel = torch.tensor(gth["selected"], dtype=torch.int32)
    mk, mv, cu = ops.gather_kv(bank, 0, sel, "cuda")
    torch.cuda.synchronize()
    assert cu.tolist() == gth["cu_sel"] and mk[:, 0, 0].float().cpu().tolist() == [float(c) for row in gth["chunks"] for c in row]
    mk2, mv2, cu2 = ops.gather_kv_device(bank, 0, sel.cuda(), 8)
    torch.cuda.synchronize()
    assert cu2.cpu().tolist() == gth["cu_sel"] and torch.equal(mk2[:6].cpu(), mk.cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("B,S,dtype", [(6, 128, torch.bfloat16), (3, 200, torch.bfloat16), (2, 40, torch.bfloat16),
                                      (4, 96, torch.float32)])
def test_route_topk_gather_equals_the_two_calls(B, S, dtype):
    """msa_route_topk_gather (routing of one layer with the gather of another layer's selection inside the scan's
    launch) returns exactly what msa_route_topk and msa_gather_kv_device return by themselves: for the large-tile
    form of the scan, which carries the copy in one of its workgroups, and for the forms that cannot (few query rows,
    fp32), where the gather's own kernels run first.  The gathered selection shares documents between samples and
    holds a duplicate and an out-of-range id."""
    from msa_amd import ops
    rng = np.random.default_rng(77 + B)
    doc_chunks = rng.integers(1, 9, size=300).tolist()
    dco = np.concatenate([[0], np.cumsum(doc_chunks)])
    C, Hkv, D = int(dco[-1]), 8, 128
    g = torch.Generator().manual_seed(5 + S)
    bank = ops.Bank(2, dco.tolist(), list(range(len(doc_chunks))), Hkv, D, dtype)
    keep = []
    for layer in range(2):
        kr = torch.nn.functional.normalize(torch.randn((C, Hkv, D), generator=g), dim=-1).to(dtype).cuda()
        kh = torch.randn((C, Hkv, D), generator=g).to(dtype).pin_memory()
        vh = torch.randn((C, Hkv, D), generator=g).to(dtype).pin_memory()
        bank.set_layer(layer, kr, kh, vh)
        keep.append((kr, kh, vh))
    q = torch.randn((B, S, 32, D), generator=g).to(dtype).cuda()
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[0, S // 2:] = False
    sel = torch.from_numpy(rng.integers(0, len(doc_chunks), size=(5, 7)).astype(np.int32))
    sel[1, :3] = sel[0, :3]          # documents shared between samples
    sel[2, 4] = sel[2, 3]            # a duplicate inside a sample
    sel[3, 0] = -1                   # skipped
    sel = sel.cuda()
    cap = 5 * 7 * 8
    want_r = ops.route_topk(bank, 1, q, mask.cuda(), "cosine", 1.0, 8)
    want_g = ops.gather_kv_device(bank, 0, sel, cap)
    (s_, d_, gid_), (k_, v_, cu_) = ops.route_topk_gather(bank, 1, q, mask.cuda(), "cosine", 1.0, 8, 0, sel, cap)
    torch.cuda.synchronize()
    assert torch.equal(d_, want_r[1]) and torch.equal(gid_, want_r[2]) and torch.equal(s_, want_r[0])
    assert torch.equal(cu_, want_g[2])
    n = int(cu_[-1])
    assert n > 0 and torch.equal(k_[:n], want_g[0][:n]) and torch.equal(v_[:n], want_g[1][:n])
    # outputs too small for the selection: both forms stop at the capacity (cu_sel clamps there, later rows are
    # dropped, nothing past the capacity is written), also where a shared document's second use lies past it
    sel[4, 1] = sel[0, 1]
    full = ops.gather_kv_device(bank, 0, sel, cap)
    short = int(full[2][-1]) // 2
    bufs = [tuple(torch.full((cap, Hkv, D), 7.0, dtype=dtype, device="cuda") for _ in range(2)) for _ in range(2)]
    want_g = ops.gather_kv_device(bank, 0, sel, short, out=bufs[0])
    _, (k_, v_, cu_) = ops.route_topk_gather(bank, 1, q, mask.cuda(), "cosine", 1.0, 8, 0, sel, short, out=bufs[1])
    torch.cuda.synchronize()
    assert int(cu_[-1]) == short and torch.equal(cu_, want_g[2]) and torch.equal(cu_, full[2].clamp(max=short))
    for got, alone, whole in ((k_, want_g[0], full[0]), (v_, want_g[1], full[1])):
        assert torch.equal(got[:short], whole[:short]) and torch.equal(alone[:short], whole[:short])
        assert (got[short:] == 7.0).all() and (alone[short:] == 7.0).all()
