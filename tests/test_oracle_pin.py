"""Pins the CPU oracle by mathematics: library special cases, closed forms,
invariants, brute force, and agreement of its two independent restatements.
The reference ships no golden vectors for this path, so these checks are what
stands between the oracle and a dropped term / wrong index / transposed operand.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import closed_form as cf
from oracle import reference_style as rs

torch.manual_seed(0)


def _ragged(seed, n_docs, lo, hi):
    g = np.random.default_rng(seed)
    return [int(x) for x in g.integers(lo, hi + 1, size=n_docs)]


# ------------------------------------------------------------------ chunk table
@pytest.mark.parametrize("P", [4, 64])
def test_chunk_table_invariants(P):
    lens = _ragged(1, 37, 1, 5 * P + 3) + [P, 2 * P, 1, P + 1]
    ds, dco, cs, cl, cd = cf.chunk_table(lens, P, first_token=3)
    assert ds[0] == 3 and ds[-1] == 3 + sum(lens)
    assert dco[-1] == len(cs) == sum(math.ceil(n / P) for n in lens)
    assert np.all(np.diff(cd) >= 0)
    for d, n in enumerate(lens):
        idx = np.nonzero(cd == d)[0]
        assert len(idx) == math.ceil(n / P)
        assert cl[idx].sum() == n
        assert np.all(cl[idx[:-1]] == P)
        assert cl[idx[-1]] == n - P * ((n - 1) // P)
        assert np.all(cs[idx] == ds[d] + P * np.arange(len(idx)))
    # chunks tile the document tokens exactly, in order, without overlap
    assert np.all(cs[1:] == cs[:-1] + cl[:-1])


def test_chunk_table_matches_reference_style_ids():
    P = 4
    lens = [5, 4, 1, 9, 8]
    head = 3
    ds, dco, cs, cl, cd = cf.chunk_table(lens, P, first_token=head)
    doc_ids = torch.tensor([[-2] * head + sum(([i + 1] * n for i, n in enumerate(lens)), [])])
    am = torch.ones_like(doc_ids)
    where, gchunk, pooled = rs.stage1_chunk_ids(doc_ids, am, P)
    assert pooled.tolist() == (cd + 1).tolist()
    _, lengths = torch.unique_consecutive(gchunk, return_counts=True)
    assert lengths.tolist() == cl.tolist()
    assert where[:, 1].tolist() == list(range(head, head + sum(lens)))
    pos = cf.doc_positions(lens, head)
    assert pos[:head].tolist() == [0, 1, 2]
    for d in range(len(lens)):
        assert pos[ds[d]:ds[d + 1]].tolist() == list(range(lens[d]))


# ------------------------------------------------------------------ pooling
def test_pool_whole_chunks_is_view_mean():
    P, H, D = 8, 2, 16
    lens = [P * 3, P, P * 2]
    x = torch.randn(sum(lens), H, D, dtype=torch.float64)
    _, _, cs, cl, _ = cf.chunk_table(lens, P)
    got = cf.pool_chunks(x, cs, cl)
    assert torch.allclose(got, x.view(-1, P, H, D).mean(1), atol=1e-14)


def test_pool_special_cases_and_linearity():
    P, H, D = 8, 2, 16
    lens = [1, 7, 8, 9, 17, 1]
    T = sum(lens) + 2
    _, _, cs, cl, cd = cf.chunk_table(lens, P, first_token=2)
    const = torch.full((T, H, D), 3.25, dtype=torch.float64)
    assert torch.allclose(cf.pool_chunks(const, cs, cl), torch.full((len(cs), H, D), 3.25, dtype=torch.float64))
    x, y = torch.randn(T, H, D, dtype=torch.float64), torch.randn(T, H, D, dtype=torch.float64)
    px, py = cf.pool_chunks(x, cs, cl), cf.pool_chunks(y, cs, cl)
    assert torch.allclose(px[0], x[2]) and torch.allclose(px[-1], x[T - 1])      # length-1 docs: identity
    assert torch.allclose(cf.pool_chunks(2.0 * x - 0.5 * y, cs, cl), 2.0 * px - 0.5 * py, atol=1e-13)
    # the partial chunk divides by its true length: doc of 9 -> chunks of 8 and 1
    c9 = int(np.nonzero(cd == 3)[0][1])
    assert cl[c9] == 1 and torch.allclose(px[c9], x[cs[c9]])
    # template tokens in front are not pooled
    x2 = x.clone(); x2[:2] += 100.0
    assert torch.allclose(cf.pool_chunks(x2, cs, cl), px)


def test_pool_reference_style_agrees():
    P, H, D = 16, 4, 32
    lens = _ragged(3, 25, 1, 100)
    head = 3
    T = head + sum(lens)
    x = torch.randn(1, H, T, D)
    doc_ids = torch.tensor([[-2] * head + sum(([i + 1] * n for i, n in enumerate(lens)), [])])
    where, gchunk, _ = rs.stage1_chunk_ids(doc_ids, torch.ones_like(doc_ids), P)
    ref = rs.stage1_pool(x, where, gchunk)                                       # [1, H, C, D]
    _, _, cs, cl, _ = cf.chunk_table(lens, P, first_token=head)
    mine = cf.pool_chunks(x[0].transpose(0, 1), cs, cl)                          # [C, H, D]
    assert cf.rel_err(ref[0].transpose(0, 1), mine) < 2e-5                       # fp32 cumsum difference
    refn = rs.stage1_pool(x, where, gchunk, normalize=True)[0].transpose(0, 1)
    assert cf.rel_err(refn, cf.l2_normalize(mine)) < 2e-5
    assert torch.allclose(cf.l2_normalize(mine).norm(dim=-1), torch.ones(len(cs), H, dtype=torch.float64))


# ------------------------------------------------------------------ rope
def test_rope_invariants():
    T, H, D, theta = 9, 2, 16, 1e6
    x, y = torch.randn(T, H, D, dtype=torch.float64), torch.randn(T, H, D, dtype=torch.float64)
    zero = torch.zeros(T, dtype=torch.int64)
    assert torch.allclose(cf.apply_rope(x, zero, theta), x)
    pos = torch.arange(T) * 7 + 1
    rx = cf.apply_rope(x, pos, theta)
    half = D // 2
    assert torch.allclose(rx[..., :half] ** 2 + rx[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)
    # relative-position property
    a = (cf.apply_rope(x, pos, theta) * cf.apply_rope(y, pos + 5, theta)).sum(-1)
    b = (cf.apply_rope(x, pos + 100, theta) * cf.apply_rope(y, pos + 105, theta)).sum(-1)
    assert torch.allclose(a, b, atol=1e-10)
    # first pair rotates by exactly pos radians (inv_freq_0 = 1); sign convention pinned
    e = torch.zeros(1, 1, D, dtype=torch.float64); e[0, 0, 0] = 1.0
    r = cf.apply_rope(e, torch.tensor([1]), theta)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-12 and abs(float(r[0, 0, half]) - math.sin(1.0)) < 1e-12
    # last pair has inv_freq theta^-(D-2)/D
    e2 = torch.zeros(1, 1, D, dtype=torch.float64); e2[0, 0, half - 1] = 1.0
    r2 = cf.apply_rope(e2, torch.tensor([1000]), theta)
    assert abs(float(r2[0, 0, half - 1]) - math.cos(1000 * theta ** (-(D - 2) / D))) < 1e-12
    cos, sin = cf.rope_tables(64, D, theta)
    assert torch.allclose(cos[5], torch.cos(5 * theta ** (-torch.arange(0, D, 2, dtype=torch.float64) / D)))


def test_rope_reference_style_agrees():
    T, H, D, theta = 50, 3, 32, 1e6
    x = torch.randn(1, H, T, D)
    pos = torch.tensor(cf.doc_positions([20, 27], 3))[None]
    ref = rs.rotary(x, pos, theta)[0].transpose(0, 1)
    mine = cf.apply_rope(x[0].transpose(0, 1), pos[0], theta)
    assert cf.rel_err(ref, mine) < 1e-5


# ------------------------------------------------------------------ scoring
def _bank(seed, lens_chunks, Hkv, D, normalize=True):
    g = torch.Generator().manual_seed(seed)
    C = sum(lens_chunks)
    kr = torch.randn(C, Hkv, D, generator=g)
    return cf.l2_normalize(kr).float() if normalize else kr


def test_scores_gqa_presum_and_needle_and_permutation():
    B, S, Hq, Hkv, D = 2, 5, 8, 2, 16
    G = Hq // Hkv
    C = 23
    kr = _bank(0, [C], Hkv, D).double()
    q = torch.randn(B, S, Hq, D, dtype=torch.float64)
    mask = torch.ones(B, S, dtype=torch.bool); mask[1, :2] = False
    cs = cf.chunk_scores(q, mask, kr, "cosine")
    # brute force over explicit loops
    qn = q / q.norm(dim=-1, keepdim=True)
    brute = torch.full((B, C), float("-inf"), dtype=torch.float64)
    for b in range(B):
        for c in range(C):
            for t in range(S):
                if not mask[b, t]:
                    continue
                s = sum(float(qn[b, t, h] @ kr[c, h // G]) for h in range(Hq)) / Hq
                brute[b, c] = max(brute[b, c], s)
    assert torch.allclose(cs, brute, atol=1e-12)
    # GQA pre-sum identity: summing the G normalised query heads per kv head first
    pres = qn.view(B, S, Hkv, G, D).sum(3).reshape(B, S, Hkv * D)
    s2 = (pres @ kr.reshape(C, Hkv * D).T / Hq).masked_fill(~mask[:, :, None], float("-inf")).max(1).values
    assert torch.allclose(cs, s2, atol=1e-12)
    # permutation equivariance in chunk order
    perm = torch.randperm(C)
    assert torch.allclose(cf.chunk_scores(q, mask, kr[perm], "cosine"), cs[:, perm], atol=1e-12)
    # planted needle: every kv head of a chunk equals the direction of one token's (identical) heads -> score 1
    qq = q.clone()
    v = torch.randn(D, dtype=torch.float64)
    qq[0, 3] = v * 2.5
    kr2 = kr.clone(); kr2[7] = v / v.norm()
    cs2 = cf.chunk_scores(qq, mask, kr2, "cosine")
    assert abs(float(cs2[0, 7]) - 1.0) < 1e-12 and float(cs2[0].max()) == float(cs2[0, 7])
    # scaled-dot mode: no normalisation, D^-0.5
    sd = cf.chunk_scores(q, mask, kr, "scaled_dot")
    s3 = (q.view(B, S, Hkv, G, D).sum(3).reshape(B, S, -1) @ kr.reshape(C, -1).T / Hq * D ** -0.5)
    assert torch.allclose(sd, s3.masked_fill(~mask[:, :, None], float("-inf")).max(1).values, atol=1e-12)
    # fully masked query
    none = torch.zeros(B, S, dtype=torch.bool)
    assert torch.isinf(cf.chunk_scores(q, none, kr, "cosine")).all()


@pytest.mark.parametrize("mode", ["cosine", "scaled_dot"])
def test_scores_topk_reference_style_agrees(mode):
    B, S, Hq, Hkv, D, k = 3, 6, 8, 2, 32, 4
    G = Hq // Hkv
    doc_chunks = _ragged(5, 300, 1, 9)
    _, dco, _, _, cd = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    kr = _bank(1, doc_chunks, Hkv, D, normalize=(mode == "cosine"))
    q = torch.randn(B, S, Hq, D)
    mask = torch.ones(B, S, dtype=torch.bool); mask[2, :3] = False
    cs = cf.chunk_scores(q, mask, kr, mode)
    ds = cf.doc_scores(cs, dco)
    want_s, want_i = cf.topk_docs(ds, k)
    # the reference sequence: q normalised by the layer, scaling -1 in cosine mode
    qh = q.permute(0, 2, 1, 3).contiguous()                                     # [B, Hq, S, D]
    if mode == "cosine":
        qh = F.normalize(qh, p=2, dim=-1)
    q5, m5 = rs.group_queries(qh, mask, G, -1.0 if mode == "cosine" else D ** -0.5)
    rk = kr.transpose(0, 1).unsqueeze(0)                                        # [1, Hkv, C, D]
    got_s, got_i = rs.stage2_scores_topk(q5, m5, rk, torch.as_tensor(cd + 1), doc_chunks, k,
                                         slice_chunk_size=256)                   # several slices + tail merge
    assert cf.rel_err(got_s, want_s) < 1e-5
    assert not cf.topk_acceptable(ds, got_i - 1, k, gap=1e-5)
    assert (got_i >= 1).all()                                                   # dummy slot 0 never wins


@pytest.mark.parametrize("query_reduce,chunk_reduce", [("mean", "max"), ("last", "max"), ("max", "mean"), ("mean", "mean"),
                                                        ("last", "mean")])
def test_other_reductions_brute_force_and_reference_style_agree(query_reduce, chunk_reduce):
    """The reference's other reductions over tokens and chunks (src/msa_service.py:751-811), pinned by plain loops over
    every (query, token, head, chunk) and by the reference-style op sequence (several slices)."""
    B, S, Hq, Hkv, D, k = 3, 7, 8, 2, 16, 4
    G = Hq // Hkv
    doc_chunks = _ragged(11, 40, 1, 6)
    _, dco, _, _, cd = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    kr = _bank(2, doc_chunks, Hkv, D, normalize=False).double()
    q = torch.randn(B, S, Hq, D).double()
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[1, 4:] = False                       # a prefix of 4 scored tokens
    mask[2, 0] = False; mask[2, 3] = False    # holes: 5 scored tokens, position 4 is scored
    sc = D ** -0.5
    C = kr.shape[0]
    # brute force
    want_c = torch.empty(B, C, dtype=torch.float64)
    for b in range(B):
        seen = [t for t in range(S) if mask[b, t]]
        for c in range(C):
            per_tok = []
            for t in range(S):
                tot = 0.0
                for h in range(Hq):
                    tot += float(q[b, t, h] @ kr[c, h // G]) * sc
                per_tok.append(tot / Hq)
            if query_reduce == "mean":
                want_c[b, c] = sum(per_tok[t] for t in seen) / max(len(seen), 1)
            else:
                want_c[b, c] = per_tok[len(seen) - 1] if mask[b, len(seen) - 1] else -math.inf
                if query_reduce == "max":
                    want_c[b, c] = max(per_tok[t] for t in seen)
    got_c = cf.chunk_scores(q, mask, kr, "scaled_dot", query_reduce=query_reduce)
    assert torch.allclose(got_c, want_c, atol=1e-12)
    want_d = torch.empty(B, len(doc_chunks), dtype=torch.float64)
    for d in range(len(doc_chunks)):
        cols = [float("nan")] * 0
        for b in range(B):
            vals = [float(want_c[b, c]) for c in range(int(dco[d]), int(dco[d + 1]))]
            want_d[b, d] = max(vals) if chunk_reduce == "max" else sum(vals) / len(vals)
    got_d = cf.doc_scores(got_c, dco, chunk_reduce)
    assert torch.allclose(got_d, want_d, atol=1e-12)
    # the reference-style sequence (fp64 here), slices of 32 chunks
    qh = q.permute(0, 2, 1, 3).contiguous()
    q5, m5 = rs.group_queries(qh, mask, G, sc)
    rk = kr.transpose(0, 1).unsqueeze(0)
    got_s, got_i = rs.stage2_scores_topk(q5, m5, rk, torch.as_tensor(cd + 1), doc_chunks, k, slice_chunk_size=32,
                                         query_reduce=query_reduce, chunk_reduce=chunk_reduce)
    want_s, want_i = cf.topk_docs(want_d, k)
    assert torch.allclose(got_s, want_s, atol=1e-9)
    assert torch.equal(got_i - 1, want_i)


def test_make_slices_doc_aligned_and_tail_merge():
    chunks = [600] * 5 + [100]
    sl = rs.make_slices(chunks, 1024)
    assert sl == [(0, 1200), (1200, 3100)]          # tail of 700 (<1024) joins the previous slice
    sl2 = rs.make_slices([600] * 5 + [1100], 1024)
    assert sl2 == [(0, 1200), (1200, 2400), (2400, 4100)]
    assert rs.make_slices([5, 5], 1024) == [(0, 10)]


def test_topk_against_sort_and_ties():
    g = torch.Generator().manual_seed(4)
    ds = torch.randn(5, 200, generator=g, dtype=torch.float64)
    s, i = cf.topk_docs(ds, 16)
    srt = torch.sort(ds, dim=1, descending=True)
    assert torch.equal(s, srt.values[:, :16]) and torch.equal(i, srt.indices[:, :16])
    tie = torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0]], dtype=torch.float64)
    s, i = cf.topk_docs(tie, 3)
    assert i.tolist() == [[1, 2, 4]]
    s, i = cf.topk_docs(tie, 8)
    assert i.tolist() == [[1, 2, 4, 3, 0, -1, -1, -1]] and torch.isinf(s[0, 5:]).all()
    assert not cf.topk_acceptable(tie, torch.tensor([[2, 4, 1]]), 3)
    assert cf.topk_acceptable(tie, torch.tensor([[2, 4, 3]]), 2 + 1)             # 3 is below the boundary
    assert cf.topk_acceptable(tie, torch.tensor([[1, 1, 2]]), 3)                 # duplicates


# ------------------------------------------------------------------ gather
def test_gather_exact_and_reference_style_agrees():
    Hkv, D = 2, 8
    doc_chunks = [3, 1, 4, 2, 5, 1]
    _, dco, _, _, _ = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    C = int(dco[-1])
    kb = torch.arange(C * Hkv * D, dtype=torch.float32).view(C, Hkv, D)
    vb = -kb
    sel = torch.tensor([[4, 0, 2], [2, 5, -1], [1, 1, 3]])
    K, V, cu, rows = cf.gather_selected(kb, vb, dco, sel)
    assert cu.tolist() == [0, 3 + 4 + 5, 12 + 4 + 1, 17 + 1 + 2]
    assert rows[:12].tolist() == [0, 1, 2] + [4, 5, 6, 7] + [10, 11, 12, 13, 14]
    assert torch.equal(K, kb[rows]) and torch.equal(V, vb[rows])
    # reference-style regroup with dummy slot 0 tables and 1-based ids
    lens = torch.tensor([0] + doc_chunks)
    offs = torch.cumsum(torch.tensor([0] + [0] + doc_chunks[:-1]), 0)
    gids = torch.tensor([0] + [100 + d for d in range(len(doc_chunks))])
    scores = torch.ones(3, 3); scores[1, 2] = -3e38
    local = (sel + 1).clamp_min(0)
    k_r, v_r, n_sel = rs.gather_regroup(kb.transpose(0, 1)[None], vb.transpose(0, 1)[None], offs, lens, gids,
                                        scores, local)
    assert n_sel.tolist() == np.diff(cu).tolist()
    assert torch.equal(k_r.permute(1, 0, 2), K) and torch.equal(v_r.permute(1, 0, 2), V)


def test_assemble_and_positions():
    H, D = 2, 4
    prefix = torch.full((3, H, D), -1.0)
    mem = torch.arange(5.0)[:, None, None].expand(5, H, D)
    local = 10 + torch.arange(4.0)[:, None, None].expand(4, H, D)
    ctx, cu = cf.assemble_context(prefix, mem, np.array([0, 2, 5]), local, np.array([0, 3, 4]))
    assert cu.tolist() == [0, 3 + 2 + 3, 8 + 3 + 3 + 1]
    assert ctx[:, 0, 0].tolist() == [-1, -1, -1, 0, 1, 10, 11, 12, -1, -1, -1, 2, 3, 4, 13]
    assert cf.query_positions(4, 16).tolist() == [19, 20, 21, 22]
    assert cf.query_positions(2, 16, left_pad=2).tolist() == [19, 19, 19, 20]


# ------------------------------------------------------------------ attention
def test_attention_against_sdpa_and_special_cases():
    Sq, L, Hq, Hkv, D = 5, 12, 8, 2, 16
    q = torch.randn(Sq, Hq, D, dtype=torch.float64)
    k = torch.randn(L, Hkv, D, dtype=torch.float64)
    v = torch.randn(L, Hkv, D, dtype=torch.float64)
    out = cf.attention(q, k, v)
    i = torch.arange(Sq)[:, None]; j = torch.arange(L)[None, :]
    allowed = j <= (L - Sq + i)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], rs.repeat_kv(k.transpose(0, 1)[None], 4),
                                         rs.repeat_kv(v.transpose(0, 1)[None], 4), attn_mask=allowed)
    assert torch.allclose(out, ref[0].transpose(0, 1), atol=1e-12)
    # first query row of a bottom-right causal block sees exactly L-Sq+1 keys
    only = cf.attention(q[:1], k[: L - Sq + 1], v[: L - Sq + 1], causal=False)
    assert torch.allclose(out[:1], only, atol=1e-12)
    # one key -> its value; identical keys -> mean of values
    assert torch.allclose(cf.attention(q[:1], k[:1], v[:1]), rs.repeat_kv(v[:1].transpose(0, 1)[None], 4)[0].transpose(0, 1))
    same = k[:1].expand(L, -1, -1)
    mv = v.mean(0, keepdim=True)
    assert torch.allclose(cf.attention(q[:1], same, v), rs.repeat_kv(mv.transpose(0, 1)[None], 4)[0].transpose(0, 1), atol=1e-12)


def test_decode_step_reference_style_agrees():
    B, Hq, Hkv, D = 3, 8, 2, 16
    lens = [7, 4, 9]
    Lmax = max(lens)
    ck = torch.zeros(B, Hkv, Lmax, D); cv = torch.zeros(B, Hkv, Lmax, D)
    ks, vs = [], []
    for b, n in enumerate(lens):
        kk, vv = torch.randn(n, Hkv, D), torch.randn(n, Hkv, D)
        ks.append(kk); vs.append(vv)
        ck[b, :, Lmax - n:] = kk.transpose(0, 1); cv[b, :, Lmax - n:] = vv.transpose(0, 1)
    ck[1, :, : Lmax - 4] = 55.0                      # garbage in the padding must be ignored
    q = torch.randn(B, Hq, 1, D); kn = torch.randn(B, Hkv, 1, D); vn = torch.randn(B, Hkv, 1, D)
    out, fk, fv = rs.decode_step(q, ck, cv, kn, vn, torch.tensor(lens))
    assert fk.shape[2] == Lmax + 1
    for b in range(B):
        kk = torch.cat([ks[b], kn[b].transpose(0, 1)]); vv = torch.cat([vs[b], vn[b].transpose(0, 1)])
        want = cf.attention(q[b].transpose(0, 1), kk, vv)
        assert cf.rel_err(out[b].transpose(0, 1), want) < 1e-5


def test_by_hand_fixture_pins_the_oracle():
    """tests/golden/by_hand.json: numbers worked out by hand on one-hot vectors (masking, head mean, token max,
    chunk max, tie order, pooling means, gather order, positions).  A wrong axis, sign, offset or tie rule fails."""
    from tests.golden import by_hand
    fx = by_hand.load()
    q, mask, kr, dco = by_hand.tensors(fx)
    cs = cf.chunk_scores(q, mask, kr, "cosine")
    assert torch.allclose(cs, torch.tensor(fx["chunk_scores_cosine"], dtype=cs.dtype), atol=1e-12)
    sd = cf.chunk_scores(q, mask, kr, "scaled_dot", scale=fx["D"] ** -0.5)
    assert torch.allclose(sd, torch.tensor(fx["chunk_scores_cosine"], dtype=sd.dtype) * fx["scaled_dot_factor"], atol=1e-12)
    ds = cf.doc_scores(cs, dco)
    assert torch.allclose(ds, torch.tensor(fx["doc_scores_cosine"], dtype=ds.dtype), atol=1e-12)
    assert cf.topk_docs(ds, 2)[1].tolist() == fx["top2"] and cf.topk_docs(ds, 3)[1].tolist() == fx["top3"]
    # the reference's own op order gives the same numbers
    qh = torch.nn.functional.normalize(q.permute(0, 2, 1, 3), p=2, dim=-1)
    q5, m5 = rs.group_queries(qh, mask, fx["Hq"] // fx["Hkv"], -1.0)
    chunks = np.diff(dco).tolist()
    pool_ids = torch.repeat_interleave(torch.arange(1, len(chunks) + 1), torch.as_tensor(chunks))
    s_ref, i_ref = rs.stage2_scores_topk(q5, m5, kr.transpose(0, 1).unsqueeze(0), pool_ids, chunks, 2)
    assert torch.allclose(s_ref.double(), torch.tensor([[1.0, 0.5], [1.0, 0.5]], dtype=torch.float64), atol=1e-6)
    assert (i_ref[:, 0] - 1).tolist() == [r[0] for r in fx["top2"]]          # 1-based pool ids; rank 0 has no tie
    # pooling
    p = fx["pool"]
    _, off, cstart, clen, cdoc = cf.chunk_table(p["doc_lens"], p["P"])
    assert (cstart.tolist(), clen.tolist(), cdoc.tolist(), off.tolist()) == (p["chunk_start"], p["chunk_len"], p["chunk_doc"],
                                                                            p["doc_chunk_off"])
    x = (torch.arange(sum(p["doc_lens"]), dtype=torch.float64) + 1).view(-1, 1, 1).expand(-1, 2, 128)
    pooled = cf.pool_chunks(x, cstart, clen)
    assert torch.allclose(pooled[:, 0, 0], torch.tensor(p["chunk_mean"], dtype=torch.float64), atol=1e-12)
    assert torch.allclose(cf.l2_normalize(pooled), torch.full_like(pooled, p["normalized_element"]), atol=1e-12)
    # gather order and positions
    gth = fx["gather"]
    bank = torch.arange(6, dtype=torch.float64).view(6, 1, 1).expand(6, 2, 128)
    mk, _, cu, _ = cf.gather_selected(bank, bank, dco, torch.tensor(gth["selected"]))
    assert cu.tolist() == gth["cu_sel"] and mk[:, 0, 0].tolist() == [float(c) for row in gth["chunks"] for c in row]
    ps = fx["positions"]
    assert cf.query_positions(ps["n_query"], ps["top_k"], ps["n_prefix"], ps["left_pad"]).tolist() == ps["position_ids"]
