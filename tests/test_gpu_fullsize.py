"""GPU tests at the full sizes of the benchmark configurations, where the fp64 oracle cannot run
over everything: size-independent properties over the whole output (checksums, permutation
equivariance, sortedness, planted answers) plus oracle parity on random samples of it."""
import sys

import numpy as np
import pytest
import torch

from oracle import closed_form as cf

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible")
    from msa_amd import ops as _ops
    return _ops


def test_pooling_one_million_tokens(ops):
    """Encode-side pooling at 1M tokens, ragged documents of 256..2048 tokens, bf16, K with fused RoPE."""
    say("full size: pooling 1M tokens")
    P, H, D, theta = 64, 8, 128, 1e6
    rng = np.random.default_rng(0)
    lens = []
    while sum(lens) < 1_000_000:
        lens.append(int(rng.integers(256, 2049)))
    T = sum(lens)
    g = torch.Generator(device="cuda").manual_seed(1)
    k, v, kr = (torch.randn((T, H, D), generator=g, device="cuda").bfloat16() for _ in range(3))
    t = ops.chunk_table(lens, P)
    tables = ops.rope_tables(2048, D, theta)
    pk, pv, pkr = ops.pool_chunks(k, v, kr, t, rope=tables, normalize_kr=True)
    torch.cuda.synchronize()
    _, _, cs, cl, cd = cf.chunk_table(lens, P)
    C = len(cs)
    assert pk.shape == pv.shape == pkr.shape == (C, H, D)
    assert torch.equal(t.chunk_start.cpu(), torch.as_tensor(cs, dtype=torch.int32))
    assert torch.equal(t.chunk_len.cpu(), torch.as_tensor(cl, dtype=torch.int32))
    # checksum of checksums: sum over chunks of len * mean == sum over tokens (per head and dim), in fp64
    w = torch.as_tensor(cl, dtype=torch.float64, device="cuda").view(C, 1, 1)
    got = (pv.double() * w).sum(0)
    want = v.double().sum(0)
    assert float((got - want).abs().max()) < 1e-2 * float(want.abs().max()) + 0.05 * np.sqrt(C) * 2 ** -8
    # every normalised routing key has unit norm per head
    norms = pkr.float().norm(dim=-1)
    assert float((norms - 1).abs().max()) < 1e-2
    # oracle parity on a sample of chunks: full first / last chunks, the partial tails, random ones
    tails = np.nonzero(cl < P)[0]
    sample = np.unique(np.concatenate([[0, C - 1], tails[:40], rng.integers(0, C, size=120)]))
    pos = cf.doc_positions(lens)
    for tensor, out, rope, norm in ((k, pk, True, False), (v, pv, False, False), (kr, pkr, False, True)):
        worst = 0.0
        for c in sample:
            rows = slice(int(cs[c]), int(cs[c]) + int(cl[c]))
            x = tensor[rows].cpu().double()
            if rope:
                x = cf.apply_rope(x, torch.as_tensor(pos[rows]), theta)
            ref = x.mean(0)
            if norm:
                ref = cf.l2_normalize(ref)
            worst = max(worst, float((out[c].cpu().double() - ref).abs().max() / ref.abs().max()))
        assert worst < 1e-2, worst


def test_routing_ten_million_token_bank(ops):
    """Router scoring + top-k on a 10M-token bank (about 156k chunks), batch 32 x 128 query tokens, top-16."""
    say("full size: routing over a 10M-token bank")
    B, S, Hq, Hkv, D, k, P = 32, 128, 32, 8, 128, 16, 64
    rng = np.random.default_rng(2)
    doc_tokens = []
    while sum(doc_tokens) < 10_000_000:
        doc_tokens.append(int(rng.integers(256, 2049)))
    _, dco, _, _, _ = cf.chunk_table(doc_tokens, P)
    C, n_docs = int(dco[-1]), len(doc_tokens)
    g = torch.Generator(device="cuda").manual_seed(3)
    kr = torch.randn((C, Hkv, D), generator=g, device="cuda")
    kr = (kr / kr.norm(dim=-1, keepdim=True)).bfloat16()
    q = torch.randn((B, S, Hq, D), generator=g, device="cuda").bfloat16()
    mask = torch.ones((B, S), dtype=torch.bool, device="cuda")
    mask[1, :37] = False                                      # a left-padded query
    # plant k needles per query on one of its tokens: per KV head the chunk has cosine 0.98 - 0.025 r with the
    # (head-summed) query direction, so the ranks are separated by 0.025 * mean|q_sum| / G >> 1e-3
    planted = []
    all_docs = rng.choice(n_docs, size=B * k, replace=False).reshape(B, k)     # no document is planted twice
    for b in range(B):
        docs = all_docs[b]
        tok = int(rng.integers(40, S))
        qn = cf.l2_normalize(q[b, tok].cpu().double()).view(Hkv, Hq // Hkv, D).sum(1)
        direction = cf.l2_normalize(qn)
        for r, d in enumerate(docs):
            c = int(dco[d]) + (int(dco[d + 1]) - int(dco[d])) // 2
            noise = kr[c].cpu().double()
            perp = cf.l2_normalize(noise - (noise * direction).sum(-1, keepdim=True) * direction)
            cos = 0.98 - 0.025 * r
            kr[c] = (cos * direction + (1 - cos * cos) ** 0.5 * perp).bfloat16().cuda()
        planted.append([int(d) for d in docs])
    gids = (np.arange(n_docs, dtype=np.int64) * 3 + 11).tolist()
    bank = ops.Bank(1, dco.tolist(), gids, Hkv, D, torch.bfloat16)
    bank.set_layer(0, kr)
    scores, doc, gid = ops.route_topk(bank, 0, q, mask, "cosine", 1.0, k)
    cs_all = ops.chunk_scores(bank, 0, q, mask, "cosine", 1.0)
    torch.cuda.synchronize()
    # planted answers, exactly and in rank order; ids unique; scores sorted; global ids follow the table
    assert doc.cpu().tolist() == planted
    assert (scores[:, :-1] >= scores[:, 1:]).all()
    assert torch.equal(gid.cpu(), torch.as_tensor(gids)[doc.cpu().long()])
    # the returned score of a document is the max of its chunk scores (same kernel output, exact)
    for b in (0, 1, B - 1):
        for r in (0, k - 1):
            d = int(doc[b, r])
            assert float(scores[b, r]) == float(cs_all[b, int(dco[d]):int(dco[d + 1])].max())
    # oracle parity on a random sample of chunks (plus the planted ones of query 0)
    sample = np.unique(np.concatenate([rng.integers(0, C, size=1500),
                                       [int(dco[d]) + (int(dco[d + 1]) - int(dco[d])) // 2 for d in planted[0]]]))
    want = cf.chunk_scores(q.cpu(), mask.cpu(), kr[sample].cpu(), "cosine")
    assert cf.rel_err(cs_all[:, sample].cpu(), want) < 1e-2
    # the same with the needles left out: their scores (about 3x an ordinary chunk's largest) set the scale of the
    # relative error above, so ordinary chunks are also held to 1e-2 of the largest ordinary score
    needles = np.array([int(dco[d]) + (int(dco[d + 1]) - int(dco[d])) // 2 for row in planted for d in row])
    plain = np.setdiff1d(sample, needles)
    want_plain = cf.chunk_scores(q.cpu(), mask.cpu(), kr[plain].cpu(), "cosine")
    assert float(want_plain.max()) < 0.5 * float(want.max())
    assert cf.rel_err(cs_all[:, plain].cpu(), want_plain) < 1e-2
    # permutation equivariance, bit for bit: a chunk's score does not depend on where it sits in the bank
    perm = torch.randperm(C, generator=torch.Generator().manual_seed(4)).cuda()
    bank2 = ops.Bank(1, dco.tolist(), gids, Hkv, D, torch.bfloat16)
    kr2 = kr[perm].contiguous()
    bank2.set_layer(0, kr2)
    cs_perm = ops.chunk_scores(bank2, 0, q, mask, "cosine", 1.0)
    assert torch.equal(cs_perm, cs_all[:, perm])


def test_prefill_attention_full_size_properties(ops):
    """The stage-2 prefill attention of the end-to-end workload at its real shape (16 samples of 4096 query tokens over
    291 memory rows + the 4096 tokens, bottom-right causal mask, 32 query / 8 KV heads), where the fp64 oracle cannot
    run over everything.  Size-independent properties that pin the mask boundary and the normalisation of every row:
    (1) values of ones: every row must come out as ones whatever the scores (the probabilities the kernel multiplies
        sum to the denominator it divides by);
    (2) queries of zeros: every visible key has the same weight, so row i of a sample is the mean of the first
        M + i + 1 value rows, which a prefix sum gives exactly: one key too many or too few in any row shows;
    (3) random rows of the random case against the fp64 oracle."""
    say("full size: prefill attention B=16 S=4096 L=4387")
    B, S, M, Hq, Hkv, D = 16, 4096, 291, 32, 8, 128
    L = M + S
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(77)
    q = torch.randn((B * S, Hq, D), generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn((B * L, Hkv, D), generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn((B * L, Hkv, D), generator=g, device=dev).to(torch.bfloat16)
    kv_off = torch.arange(B, dtype=torch.int64, device=dev) * L
    kv_len = torch.full((B,), L, dtype=torch.int32, device=dev)
    cu_q = torch.arange(B + 1, dtype=torch.int32, device=dev) * S
    run = lambda qq, vv: ops.sparse_attn(qq, k, vv, kv_off, kv_len, L, cu_q=cu_q, max_sq=S, causal=True)
    # (1)
    out = run(q, torch.ones_like(v))
    torch.cuda.synchronize()
    assert (out.float() - 1.0).abs().max().item() < 1e-2
    # (2)
    out = run(torch.zeros_like(q), v).float().view(B, S, Hq, D)
    prefix = torch.cumsum(v.float().view(B, L, Hkv, D), dim=1)                      # fp32 sums of bf16 values
    counts = (M + 1 + torch.arange(S, device=dev)).float().view(1, S, 1, 1)
    want = (prefix[:, M:M + S] / counts).repeat_interleave(Hq // Hkv, dim=2)        # [B, S, Hq, D]
    # the means are at most ~0.3 in size, so bf16 rounding of the output is at most 1e-3; a key too many or too few
    # moves the first rows (292 keys) by up to |v| / 292 ~ 0.014
    err = (out - want).abs().max().item()
    assert err < 3e-3, err
    first = (out[:, :64] - want[:, :64]).abs().max().item()                        # the rows with the fewest keys
    assert first < 2e-3, first
    # (3)
    out = run(q, v).view(B, S, Hq, D)
    rng = np.random.default_rng(5)
    qh, kh, vh = q.view(B, S, Hq, D), k.view(B, L, Hkv, D), v.view(B, L, Hkv, D)
    for _ in range(6):
        b, i = int(rng.integers(B)), int(rng.integers(S))
        want_row = cf.attention(qh[b, i:i + 1].cpu(), kh[b, :M + i + 1].cpu(), vh[b, :M + i + 1].cpu(), causal=True)
        assert cf.rel_err(out[b, i:i + 1].cpu(), want_row) < 1e-2, (b, i)
