"""GPU edge cases of the C ABI: odd head counts, tiny and ragged shapes, extreme top-k, error codes.
Everything is compared with the fp64 oracle on the same seeded inputs."""
import ctypes as C
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


def _randn(shape, seed, dtype):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


def _bank(ops, doc_chunks, Hkv, dtype, seed):
    _, dco, _, _, _ = cf.chunk_table([n * 4 for n in doc_chunks], 4)
    kr = cf.l2_normalize(_randn((int(dco[-1]), Hkv, 128), seed, torch.float32)).float().to(dtype)
    bank = ops.Bank(1, dco.tolist(), list(range(len(doc_chunks))), Hkv, 128, dtype)
    dev = kr.cuda()
    bank.set_layer(0, dev)
    return bank, kr, dco, dev


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (16, 16), (4, 1), (64, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_scores_head_layouts(ops, Hq, Hkv, dtype):
    say(f"scores Hq={Hq} Hkv={Hkv} {dtype}")
    bank, kr, dco, _ = _bank(ops, [3, 1, 7, 2, 9, 4] * 30, Hkv, dtype, 300 + Hq)
    q = _randn((3, 37, Hq, 128), 301, dtype)
    mask = torch.ones(3, 37, dtype=torch.bool); mask[0, 30:] = False
    got = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda())
    assert cf.rel_err(got.cpu(), cf.chunk_scores(q, mask, kr, "cosine")) < (1e-2 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("B,S,topk", [(1, 1, 1), (33, 3, 64), (2, 200, 16), (300, 2, 5)])
def test_route_extreme_shapes(ops, B, S, topk):
    say(f"route B={B} S={S} topk={topk}")
    bank, kr, dco, _ = _bank(ops, list(np.random.default_rng(3).integers(1, 5, size=700)), 8, torch.float32, 310)
    q = _randn((B, S, 32, 128), 311, torch.float32)
    s, d, g = ops.route_topk(bank, 0, q.cuda(), None, "cosine", 1.0, topk)
    ds = cf.doc_scores(cf.chunk_scores(q, torch.ones(B, S, dtype=torch.bool), kr, "cosine"), dco)
    assert not cf.topk_acceptable(ds, d.cpu().long(), topk, gap=1e-5)
    ws, wi = cf.topk_docs(ds, topk)
    assert cf.rel_err(s.cpu(), ws) < 1e-5
    assert torch.equal(g.cpu(), d.cpu().long())


def test_tiny_bank_and_single_chunk(ops):
    say("bank smaller than one tile; one document of one chunk")
    for doc_chunks in ([1], [2, 1, 1], [5]):
        bank, kr, dco, _ = _bank(ops, doc_chunks, 8, torch.bfloat16, 320)
        q = _randn((2, 9, 32, 128), 321, torch.bfloat16)
        got = ops.chunk_scores(bank, 0, q.cuda())
        assert cf.rel_err(got.cpu(), cf.chunk_scores(q, torch.ones(2, 9, dtype=torch.bool), kr, "cosine")) < 1e-2
        s, d, _ = ops.route_topk(bank, 0, q.cuda(), None, "cosine", 1.0, 16)
        n = len(doc_chunks)
        assert (d.cpu()[:, n:] == -1).all() and sorted(d.cpu()[0, :n].tolist()) == list(range(n))


@pytest.mark.parametrize("H", [1, 2, 4, 16, 32])
@pytest.mark.parametrize("P", [1, 7, 64])
def test_pool_head_counts_and_chunk_sizes(ops, H, P):
    say(f"pool H={H} P={P}")
    lens = [1, 2, P, P + 1, 3 * P + 2, 5]
    T = sum(lens) + 1
    x = _randn((T, H, 128), 330 + H, torch.float32)
    t = ops.chunk_table(lens, P, first_token=1)
    rope = ops.rope_tables(256, 128, 1e4)
    pk, pv, pr = ops.pool_chunks(x.cuda(), x.cuda(), x.cuda(), t, rope=rope, normalize_kr=True)
    _, _, cs, cl, _ = cf.chunk_table(lens, P, 1)
    pos = torch.as_tensor(cf.doc_positions(lens, 1))
    assert cf.rel_err(pv.cpu(), cf.pool_chunks(x, cs, cl)) < 1e-5
    assert cf.rel_err(pr.cpu(), cf.l2_normalize(cf.pool_chunks(x, cs, cl))) < 1e-5
    assert cf.rel_err(pk.cpu(), cf.pool_chunks(cf.apply_rope(x, pos, 1e4), cs, cl)) < 2e-5


@pytest.mark.parametrize("Hq,Hkv", [(8, 1), (8, 8), (16, 2)])
def test_decode_attention_group_sizes(ops, Hq, Hkv):
    say(f"decode attention Hq={Hq} Hkv={Hkv}")
    L = [1, 63, 64, 65, 700]
    B, cap = len(L), max(L)
    for dtype, tol in ((torch.bfloat16, 1e-2), (torch.float32, 1e-5)):
        k, v = _randn((B, cap, Hkv, 128), 340, dtype), _randn((B, cap, Hkv, 128), 341, dtype)
        q = _randn((B, Hq, 128), 342, dtype)
        out = ops.sparse_attn(q.cuda(), k.cuda().view(-1, Hkv, 128), v.cuda().view(-1, Hkv, 128),
                              (torch.arange(B, dtype=torch.int64) * cap).cuda(), torch.tensor(L, dtype=torch.int32).cuda(), cap)
        for b in range(B):
            assert cf.rel_err(out[b:b + 1].cpu(), cf.attention(q[b:b + 1], k[b, :L[b]], v[b, :L[b]])) < tol


def test_error_codes(ops):
    say("error codes")
    from msa_amd import _lib
    lib = _lib.load()
    bank, kr, dco, kr_dev = _bank(ops, [2, 3], 8, torch.bfloat16, 350)
    q = _randn((1, 4, 32, 128), 351, torch.bfloat16).cuda()
    out = torch.empty(1, bank.C, device="cuda")
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")
    rc = lib.msa_chunk_scores(bank.handle, 0, q.data_ptr(), None, 1, 4, 32, 0, 1.0, out.data_ptr(), ws.data_ptr(), 1024, None)
    assert rc == -3 and b"workspace" in lib.msa_last_error()                      # MSA_ESIZE
    two = ops.Bank(2, dco.tolist(), [0, 1], 8, 128, torch.bfloat16)
    two.set_layer(0, kr_dev)
    with pytest.raises(_lib.MsaError, match="no K_r") as ei:
        ops.chunk_scores(two, 1, q)
    assert ei.value.code == -4                                                    # MSA_ESTATE
    with pytest.raises(_lib.MsaError, match="out of range"):
        ops.chunk_scores(two, 2, q)
    with pytest.raises(_lib.MsaError, match="multiple of Hkv"):
        ops.chunk_scores(two, 0, _randn((1, 4, 12, 128), 352, torch.bfloat16).cuda())
    with pytest.raises(NotImplementedError):
        ops.chunk_scores(two, 0, q, mode="l2")
    with pytest.raises(ValueError, match="pinned"):
        two.set_layer(1, kr_dev, kr.clone(), kr.clone())
    # attention: rows move in 16-byte pieces, so a misaligned tensor is refused, not read
    aq = _randn((64 * 32 * 128 + 8,), 354, torch.bfloat16).cuda()
    ak = _randn((64 * 8 * 128 + 8,), 355, torch.bfloat16).cuda()
    off = torch.zeros(1, dtype=torch.int64, device="cuda"); ln = torch.full((1,), 64, dtype=torch.int32, device="cuda")
    cu = torch.tensor([0, 64], dtype=torch.int32, device="cuda")
    rc = lib.msa_flash_attn(aq.data_ptr() + 2, cu.data_ptr(), ak.data_ptr(), ak.data_ptr(), off.data_ptr(), ln.data_ptr(),
                            1, 64, 32, 8, 128, 128 ** -0.5, 1, aq.data_ptr(), None)
    assert rc == -1 and b"16-byte aligned" in lib.msa_last_error()                # MSA_EINVAL
    rc = lib.msa_sparse_attn(aq.data_ptr(), cu.data_ptr(), ak.data_ptr() + 2, ak.data_ptr(), off.data_ptr(), ln.data_ptr(),
                             1, 64, 64, 64, 32, 8, 128, 0, 128 ** -0.5, 1, aq.data_ptr(), ws.data_ptr(), 1024, None)
    assert rc == -1 and b"16-byte aligned" in lib.msa_last_error()
    with pytest.raises(_lib.MsaError, match="rotary table"):
        t = ops.chunk_table([300], 64)
        x = _randn((300, 8, 128), 353, torch.bfloat16).cuda()
        ops.pool_chunks(x, None, None, t, rope=ops.rope_tables(128, 128, 1e4))


# ---------------------------------------------------------------------------------------------
# weight-streaming linear layer of the decode step
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 48, 128), (5, 500, 256), (16, 2560, 4096), (16, 6144, 2560), (7, 2560, 9728),
                                   (16, 16400, 2560), (3, 8210, 2560), (16, 20000, 2560),
                                   (16, 20, 384)])
def test_skinny_linear_plain_and_residual(ops, M, N, K):
    say(f"skinny_linear M={M} N={N} K={K}")
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn((M, K), generator=g).bfloat16()
    w = (torch.randn((N, K), generator=g) * K ** -0.5).bfloat16()
    res = torch.randn((M, N), generator=g).bfloat16()
    want = x.double() @ w.double().T
    got = ops.skinny_linear(x.cuda(), w.cuda()).cpu()
    assert got.shape == (M, N) and cf.rel_err(got, want) < 1e-2
    got_r = ops.skinny_linear(x.cuda(), w.cuda(), residual=res.cuda()).cpu()
    assert cf.rel_err(got_r, want.bfloat16().double() + res.double()) < 1e-2
    # a fixed summation order: the same call twice gives the same bits
    assert torch.equal(ops.skinny_linear(x.cuda(), w.cuda()).cpu(), got)


@pytest.mark.parametrize("M,I,K", [(16, 9728, 2560), (3, 64, 256), (16, 528, 1024), (7, 8208, 2560), (16, 4112, 2560),
                                   (16, 4104, 2560), (5, 8, 128), (16, 2056, 2560)])
def test_skinny_linear_norm_and_silu_mul(ops, M, I, K):
    say(f"skinny_linear norm + silu-mul M={M} I={I} K={K}")
    g = torch.Generator().manual_seed(I + K)
    x = (torch.randn((M, K), generator=g) * 3).bfloat16()
    gate = (torch.randn((I, K), generator=g) * K ** -0.5).bfloat16()
    up = (torch.randn((I, K), generator=g) * K ** -0.5).bfloat16()
    nw = (1 + 0.1 * torch.randn((K,), generator=g)).bfloat16()
    eps = 1e-6
    xd = x.double()
    normed = (xd * torch.rsqrt((xd * xd).mean(-1, keepdim=True) + eps) * nw.double()).bfloat16().double()
    # RMSNorm folded in, plain epilogue
    want = normed @ gate.double().T
    got = ops.skinny_linear(x.cuda(), gate.cuda(), norm_weight=nw.cuda(), eps=eps).cpu()
    assert cf.rel_err(got, want) < 1e-2
    # and with the silu-mul epilogue over interleaved gate / up row groups
    wi = ops.interleave_gate_up(gate.cuda(), up.cuda())
    assert wi.shape == (2 * I, K) and torch.equal(wi[:8].cpu(), gate[:8]) and torch.equal(wi[8:16].cpu(), up[:8])
    a, b = (normed @ gate.double().T).bfloat16().double(), (normed @ up.double().T).bfloat16().double()
    got = ops.skinny_linear(x.cuda(), wi, silu_mul=True, norm_weight=nw.cuda(), eps=eps).cpu()
    assert got.shape == (M, I) and cf.rel_err(got, torch.nn.functional.silu(a) * b) < 1.5e-2


def test_skinny_linear_errors(ops):
    say("skinny_linear argument checks")
    from msa_amd import _lib
    x, w = torch.zeros((17, 128), dtype=torch.bfloat16).cuda(), torch.zeros((16, 128), dtype=torch.bfloat16).cuda()
    with pytest.raises(_lib.MsaError, match="rows"):
        ops.skinny_linear(x, w)
    with pytest.raises(_lib.MsaError, match="multiple of 128"):
        ops.skinny_linear(torch.zeros((2, 96), dtype=torch.bfloat16).cuda(), torch.zeros((16, 96), dtype=torch.bfloat16).cuda())
    with pytest.raises(_lib.MsaError, match="bf16 only"):
        ops.skinny_linear(torch.zeros((2, 128)).cuda(), torch.zeros((16, 128)).cuda())


def test_qk_norm_rope_append_equals_separate_kernels(ops):
    say("qk_norm_rope_append vs qk_norm_rope + cache_append")
    B, Hq, Hkv, D, Lcap = 5, 8, 2, 128, 12
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn((B, (Hq + 2 * Hkv) * D), generator=g).bfloat16().cuda()
    pos = torch.tensor([3, 700, 0, 41, 9], dtype=torch.int64).cuda()
    qw, kw = (1 + 0.1 * torch.randn(D, generator=g)).bfloat16().cuda(), (1 + 0.1 * torch.randn(D, generator=g)).bfloat16().cuda()
    rope = ops.rope_tables(1024, D, 1e6, device="cuda")
    lens = torch.tensor([0, 11, 12, 5, 7], dtype=torch.int32)                 # sample 2 is full: its row is dropped
    kc0 = torch.randn((B, Lcap, Hkv, D), generator=g).bfloat16().cuda()
    vc0 = torch.randn((B, Lcap, Hkv, D), generator=g).bfloat16().cuda()
    q, k, v = ops.qk_norm_rope(qkv, Hq, Hkv, D, pos, qw, kw, 1e-6, rope)
    kc1, vc1, l1 = kc0.clone(), vc0.clone(), lens.clone().cuda()
    ops.cache_append(k, v, kc1, vc1, l1)
    kc2, vc2, l2 = kc0.clone(), vc0.clone(), lens.clone().cuda()
    q2 = ops.qk_norm_rope_append(qkv, Hq, Hkv, D, pos, qw, kw, 1e-6, rope, kc2, vc2, l2)
    assert torch.equal(q2, q) and torch.equal(kc2, kc1) and torch.equal(vc2, vc1)
    assert l2.cpu().tolist() == l1.cpu().tolist() == [1, 12, 12, 6, 8]
    assert torch.equal(kc2[2], kc0[2]) and not torch.equal(kc2[0, 0], kc0[0, 0])


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (32, 8), (16, 2)])
def test_decode_attn_fused_equals_the_separate_launches(ops, Hq, Hkv):
    """q / k norm + rotary + cache append + attention in one call against msa_qk_norm_rope_append followed by
    msa_sparse_attn: identical cache rows and lengths, outputs equal up to the order of the fp32 sums, including an
    empty cache (the token sees only itself), a full cache (the row is dropped) and lengths around the batch of 4
    keys and the split of the key range."""
    say(f"decode_attn_fused Hq={Hq} Hkv={Hkv}")
    D, Lcap = 128, 700
    lens = [0, 1, 3, 4, 5, 699, 700, 257, 512, 31]
    B = len(lens)
    g = torch.Generator().manual_seed(Hq * 100 + Hkv)
    qkv = torch.randn((B, (Hq + 2 * Hkv) * D), generator=g).bfloat16().cuda()
    pos = torch.tensor([3, 700, 0, 41, 9, 1023, 5000, 77, 512, 30], dtype=torch.int64).cuda()   # 5000 clamps to the table
    qw, kw = (1 + 0.1 * torch.randn(D, generator=g)).bfloat16().cuda(), (1 + 0.1 * torch.randn(D, generator=g)).bfloat16().cuda()
    rope = ops.rope_tables(1024, D, 1e6, device="cuda")
    kc0 = torch.randn((B, Lcap, Hkv, D), generator=g).bfloat16().cuda()
    vc0 = torch.randn((B, Lcap, Hkv, D), generator=g).bfloat16().cuda()
    kc1, vc1, l1 = kc0.clone(), vc0.clone(), torch.tensor(lens, dtype=torch.int32).cuda()
    q = ops.qk_norm_rope_append(qkv, Hq, Hkv, D, pos, qw, kw, 1e-6, rope, kc1, vc1, l1)
    kv_off = torch.arange(B, dtype=torch.int64, device="cuda") * Lcap
    want = ops.sparse_attn(q, kc1.view(-1, Hkv, D), vc1.view(-1, Hkv, D), kv_off, l1, Lcap, causal=True)
    kc2, vc2, l2 = kc0.clone(), vc0.clone(), torch.tensor(lens, dtype=torch.int32).cuda()
    got = ops.decode_attn_fused(qkv, Hq, Hkv, D, pos, qw, kw, 1e-6, rope, kc2, vc2, l2)
    torch.cuda.synchronize()
    assert l2.cpu().tolist() == l1.cpu().tolist() == [min(n + 1, Lcap) for n in lens]
    assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1)
    assert cf.rel_err(got.cpu(), want.cpu()) < 2e-3
    # and against the oracle from the raw projection output (sample 5: a long row; sample 0: the token alone)
    for b in (0, 5, 9):
        n = int(l2[b])
        ref = cf.attention(q[b:b + 1].cpu(), kc2[b, :n].cpu(), vc2[b, :n].cpu(), causal=True)
        assert cf.rel_err(got[b:b + 1].cpu(), ref) < 1e-2


def test_cache_append_rows_ragged_and_clamped(ops):
    say("cache_append_rows: ragged blocks, empty block, capacity clamp")
    B, Lcap, Hkv, D = 4, 10, 2, 128
    g = torch.Generator().manual_seed(3)
    kc0, vc0 = torch.randn((B, Lcap, Hkv, D), generator=g), torch.randn((B, Lcap, Hkv, D), generator=g)
    n_new = [3, 0, 5, 1]
    lens = [2, 4, 7, 10]                                       # sample 2 has room for 3 of its 5 rows, sample 3 for none
    kn, vn = torch.randn((sum(n_new), Hkv, D), generator=g), torch.randn((sum(n_new), Hkv, D), generator=g)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(n_new)]), dtype=torch.int32)
    for dtype in (torch.float32, torch.bfloat16):
        kc, vc = kc0.to(dtype).cuda(), vc0.to(dtype).cuda()
        kv_len = torch.tensor(lens, dtype=torch.int32).cuda()
        ops.cache_append_rows(kn.to(dtype).cuda(), vn.to(dtype).cuda(), cu.cuda(), max(n_new), kc, vc, kv_len)
        want_k, want_v = kc0.to(dtype).clone(), vc0.to(dtype).clone()
        for b in range(B):
            fit = min(n_new[b], Lcap - lens[b])
            want_k[b, lens[b]:lens[b] + fit] = kn.to(dtype)[cu[b]:cu[b] + fit]
            want_v[b, lens[b]:lens[b] + fit] = vn.to(dtype)[cu[b]:cu[b] + fit]
        assert torch.equal(kc.cpu(), want_k) and torch.equal(vc.cpu(), want_v)
        assert kv_len.cpu().tolist() == [5, 4, 10, 10]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H", [8, 100, 2560, 5120, 9000])
def test_rmsnorm_and_silu_mul_widths(ops, dtype, H):
    """Row widths on and off the 8-element vector path, and rows longer than what the kernel keeps in registers."""
    say(f"rmsnorm / silu_mul H={H} dtype={dtype}")
    g = torch.Generator().manual_seed(H)
    N, eps = 5, 1e-6
    x, res = torch.randn((N, H), generator=g).to(dtype), torch.randn((N, H), generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5

    def ref(v):
        v = v.double()
        return v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * w.double()

    assert cf.rel_err(ops.rmsnorm(x.cuda(), w.cuda(), eps).cpu(), ref(x)) < tol
    res_dev = res.clone().cuda()
    out = ops.rmsnorm(x.cuda(), w.cuda(), eps, residual=res_dev).cpu()
    summed = (x.double() + res.double()).to(dtype)
    assert torch.equal(res_dev.cpu(), summed) and cf.rel_err(out, ref(summed)) < tol
    gu = torch.randn((N, 2 * H), generator=g).to(dtype)
    want = torch.nn.functional.silu(gu[:, :H].double()) * gu[:, H:].double()
    assert cf.rel_err(ops.silu_mul(gu.cuda()).cpu(), want) < tol


@pytest.fixture(params=[1, 2], ids=["columns32", "wide"])
def flash_form(request):
    """Runs a test once per form of the flash kernel (see msa_flash_set_form), and puts the choice by size back."""
    from msa_amd import _lib
    lib = _lib.load()
    _lib.check(lib.msa_flash_set_form(request.param), "msa_flash_set_form")
    yield request.param
    _lib.check(lib.msa_flash_set_form(0), "msa_flash_set_form")


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (8, 8), (16, 8), (16, 2), (6, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_kernel_through_the_c_abi(ops, Hq, Hkv, causal, flash_form):
    """msa_flash_attn called directly (the host wrapper only picks it for large batches), both forms of its kernel:
    every position of the tile pipelines (1, 2, 3, 4, 7, 16 tiles of 64 keys; the wide form's statements repeat every
    six tiles), a sample without keys, a causal sample with more query rows than keys (the leading rows see nothing
    and come out as zeros), single-row and ragged query blocks."""
    say(f"flash kernel direct Hq={Hq} Hkv={Hkv} causal={causal} form={flash_form}")
    from msa_amd import _lib
    D = 128
    sq = [130, 1, 33, 64, 200, 5, 7, 40, 300]
    L = [400, 70, 33, 1000, 200, 192, 0, 10, 777]
    cu_q = np.concatenate([[0], np.cumsum(sq)])
    cu_kv = np.concatenate([[0], np.cumsum(L)])
    q = _randn((int(cu_q[-1]), Hq, D), 300, torch.bfloat16)
    k = _randn((int(cu_kv[-1]), Hkv, D), 301, torch.bfloat16)
    v = _randn((int(cu_kv[-1]), Hkv, D), 302, torch.bfloat16)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    kv_off = torch.as_tensor(cu_kv[:-1], dtype=torch.int64).cuda()
    kv_len = torch.as_tensor(L, dtype=torch.int32).cuda()
    cu_q_dev = torch.as_tensor(cu_q, dtype=torch.int32).cuda()
    out = torch.full_like(qd, float("nan"))
    lib = _lib.load()
    _lib.check(lib.msa_flash_attn(_lib.ptr(qd), _lib.ptr(cu_q_dev), _lib.ptr(kd), _lib.ptr(vd), _lib.ptr(kv_off),
                                  _lib.ptr(kv_len), len(sq), int(cu_q[-1]), Hq, Hkv, D, D ** -0.5, int(causal),
                                  _lib.ptr(out), torch.cuda.current_stream().cuda_stream), "msa_flash_attn")
    torch.cuda.synchronize()
    out = out.cpu()
    assert not torch.isnan(out).any()
    for b in range(len(sq)):
        rows = slice(int(cu_q[b]), int(cu_q[b + 1]))
        keys = slice(int(cu_kv[b]), int(cu_kv[b + 1]))
        blind = sq[b] if L[b] == 0 else (max(0, sq[b] - L[b]) if causal else 0)     # leading rows that see no key
        assert (out[rows][:blind] == 0).all()
        if blind < sq[b]:
            want = cf.attention(q[rows][blind:], k[keys], v[keys], causal=causal)
            assert cf.rel_err(out[rows][blind:], want) < 1e-2, (b, sq[b], L[b])


def test_flash_kernel_one_row_per_sample_without_cu_q(ops, flash_form):
    """cu_q = NULL means one query row per sample (total_q == B): both forms, causal (the row sees all its keys)."""
    say(f"flash kernel, one row per sample, no cu_q, form={flash_form}")
    from msa_amd import _lib
    lib = _lib.load()
    Hq, Hkv, D = 32, 8, 128
    L = [70, 1, 129, 300, 64, 5]
    cu_kv = np.concatenate([[0], np.cumsum(L)])
    q = _randn((len(L), Hq, D), 330, torch.bfloat16)
    k = _randn((int(cu_kv[-1]), Hkv, D), 331, torch.bfloat16)
    v = _randn((int(cu_kv[-1]), Hkv, D), 332, torch.bfloat16)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    kv_off = torch.as_tensor(cu_kv[:-1], dtype=torch.int64).cuda()
    kv_len = torch.as_tensor(L, dtype=torch.int32).cuda()
    out = torch.full_like(qd, float("nan"))
    _lib.check(lib.msa_flash_attn(_lib.ptr(qd), None, _lib.ptr(kd), _lib.ptr(vd), _lib.ptr(kv_off), _lib.ptr(kv_len),
                                  len(L), len(L), Hq, Hkv, D, D ** -0.5, 1, _lib.ptr(out),
                                  torch.cuda.current_stream().cuda_stream), "msa_flash_attn")
    torch.cuda.synchronize()
    for b in range(len(L)):
        want = cf.attention(q[b:b + 1], k[int(cu_kv[b]):int(cu_kv[b + 1])], v[int(cu_kv[b]):int(cu_kv[b + 1])], causal=True)
        assert cf.rel_err(out[b:b + 1].cpu(), want) < 1e-2, b


def test_flash_hint_keeps_ragged_batches_on_the_32_column_form(ops):
    """msa_flash_attn_hint with the longest query block named: a ragged batch takes the 32-column form, an even one of
    at least 4096 columns the wide form (bit-identical outputs with the forms forced tell which one ran)."""
    say("flash hint: ragged batch -> 32-column form")
    from msa_amd import _lib
    lib = _lib.load()
    Hq, Hkv, D = 32, 8, 128
    st = torch.cuda.current_stream().cuda_stream

    def run(entry, sq, extra=()):
        L = [s + 100 for s in sq]
        cu_q = np.concatenate([[0], np.cumsum(sq)])
        cu_kv = np.concatenate([[0], np.cumsum(L)])
        q = _randn((int(cu_q[-1]), Hq, D), 320, torch.bfloat16).cuda()
        k = _randn((int(cu_kv[-1]), Hkv, D), 321, torch.bfloat16).cuda()
        v = _randn((int(cu_kv[-1]), Hkv, D), 322, torch.bfloat16).cuda()
        kv_off = torch.as_tensor(cu_kv[:-1], dtype=torch.int64).cuda()
        kv_len = torch.as_tensor(L, dtype=torch.int32).cuda()
        cu = torch.as_tensor(cu_q, dtype=torch.int32).cuda()
        out = torch.full_like(q, float("nan"))
        _lib.check(getattr(lib, entry)(_lib.ptr(q), _lib.ptr(cu), _lib.ptr(k), _lib.ptr(v), _lib.ptr(kv_off), _lib.ptr(kv_len),
                                       len(sq), int(cu_q[-1]), Hq, Hkv, D, D ** -0.5, 1, _lib.ptr(out), *extra, st), entry)
        torch.cuda.synchronize()
        return out

    for sq, want_form in (([700, 90, 130, 60, 50, 40], 1), ([200] * 6, 2)):
        got = run("msa_flash_attn_hint", sq, (max(sq),))
        forced = {}
        for form in (1, 2):
            _lib.check(lib.msa_flash_set_form(form), "msa_flash_set_form")
            try:
                forced[form] = run("msa_flash_attn", sq)
            finally:
                _lib.check(lib.msa_flash_set_form(0), "msa_flash_set_form")
        assert not torch.equal(forced[1], forced[2])            # the forms round differently somewhere
        assert torch.equal(got, forced[want_form]), (sq, want_form)
    assert lib.msa_flash_attn_hint(None, None, None, None, None, None, 1, 1, Hq, Hkv, D, C.c_float(1.0), 1, None, 0, st) != 0


@pytest.mark.parametrize("causal", [True, False])
def test_flash_kernel_ignores_stale_lds(ops, causal, flash_form):
    """The flash kernel's K / V tiles arrive in LDS by direct loads; rows past a sample's last key are not loaded.
    With every compute unit's LDS filled with NaN patterns beforehand (LDS is not cleared between kernels), ragged
    samples whose last tile is partly or almost wholly empty must still give the oracle's result: scores of rows that
    were not loaded are masked by a select, and V rows that were not loaded are never multiplied (0 x NaN)."""
    say(f"flash kernel after an LDS fill of NaNs causal={causal} form={flash_form}")
    import ctypes as C
    from msa_amd import _lib
    lib = _lib.load()
    Hq, Hkv, D = 32, 8, 128
    sq = [1, 40, 64, 3, 100, 130]
    L = [1, 65, 64, 127, 129, 200]
    cu_q = np.concatenate([[0], np.cumsum(sq)])
    cu_kv = np.concatenate([[0], np.cumsum(L)])
    q = _randn((int(cu_q[-1]), Hq, D), 310, torch.bfloat16)
    k = _randn((int(cu_kv[-1]), Hkv, D), 311, torch.bfloat16)
    v = _randn((int(cu_kv[-1]), Hkv, D), 312, torch.bfloat16)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    kv_off = torch.as_tensor(cu_kv[:-1], dtype=torch.int64).cuda()
    kv_len = torch.as_tensor(L, dtype=torch.int32).cuda()
    cu_q_dev = torch.as_tensor(cu_q, dtype=torch.int32).cuda()
    st = torch.cuda.current_stream().cuda_stream
    check = torch.zeros(2048, dtype=torch.int32, device="cuda")
    for word in (0x7fc07fc0, 0xffffffff):                    # bf16 NaN pairs; all ones (NaN as bf16 and as fp32)
        _lib.check(lib.msa_diag_fill_lds(word, _lib.ptr(check), 2048, st), "msa_diag_fill_lds")
        out = torch.full_like(qd, float("nan"))
        _lib.check(lib.msa_flash_attn(_lib.ptr(qd), _lib.ptr(cu_q_dev), _lib.ptr(kd), _lib.ptr(vd), _lib.ptr(kv_off),
                                      _lib.ptr(kv_len), len(sq), int(cu_q[-1]), Hq, Hkv, D, D ** -0.5, int(causal),
                                      _lib.ptr(out), st), "msa_flash_attn")
        torch.cuda.synchronize()
        assert (check.cpu().view(torch.uint8).view(-1, 4) == torch.tensor(list(word.to_bytes(4, "little")), dtype=torch.uint8)).all()
        out = out.cpu()
        assert not torch.isnan(out).any()
        for b in range(len(sq)):
            rows = slice(int(cu_q[b]), int(cu_q[b + 1]))
            keys = slice(int(cu_kv[b]), int(cu_kv[b + 1]))
            blind = max(0, sq[b] - L[b]) if causal else 0
            assert (out[rows][:blind] == 0).all()
            want = cf.attention(q[rows][blind:], k[keys], v[keys], causal=causal)
            assert cf.rel_err(out[rows][blind:], want) < 1e-2, (b, sq[b], L[b])
    assert lib.msa_diag_fill_lds(0, None, 0, st) != 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,V", [(16, 151936), (3, 1000), (1, 31), (5, 65)])
def test_greedy_sample_against_argmax(ops, dtype, B, V):
    """Row-wise argmax + the token bookkeeping of a decode step; ties go to the smallest index (bf16 logits of this
    width tie often), -inf rows and the write window of `out` are covered."""
    say(f"greedy_sample B={B} V={V} dtype={dtype}")
    g = torch.Generator().manual_seed(B * 7 + V)
    logits = torch.randn((B, V), generator=g).to(dtype)
    if V > 40:
        logits[0, 7] = logits[0, 33] = 100.0                   # a planted tie: the first index wins
        logits[B - 1] = float("-inf")
        logits[B - 1, V - 1] = -5.0                            # a single finite value at the very end
    want = torch.stack([torch.nonzero(r == r.max())[0, 0] for r in logits.float()])     # first index of the maximum
    dev = logits.cuda()
    tok = torch.full((B, 1), -1, dtype=torch.int64, device="cuda")
    pos = torch.arange(B, dtype=torch.int64, device="cuda").view(B, 1) * 10
    out = torch.full((B, 3), -7, dtype=torch.int64, device="cuda")
    col = torch.ones((B, 1), dtype=torch.int64, device="cuda")
    for step in range(3):                                      # the third call finds col == 3 == max_new: no write
        ops.greedy_sample(dev, tok, pos, out, col)
    torch.cuda.synchronize()
    assert tok.view(-1).cpu().tolist() == want.tolist()
    assert pos.view(-1).cpu().tolist() == [10 * b + 3 for b in range(B)]
    assert col.view(-1).cpu().tolist() == [4] * B
    assert out.cpu()[:, 0].tolist() == [-7] * B and out.cpu()[:, 1].tolist() == want.tolist() == out.cpu()[:, 2].tolist()
    tok2 = torch.empty(B, dtype=torch.int64, device="cuda")
    ops.greedy_sample(dev, tok2)                               # argmax only
    assert tok2.cpu().tolist() == want.tolist()


@pytest.mark.parametrize("B,S", [(16, 128), (4, 64), (3, 96), (2, 200), (1, 128), (5, 32), (9, 1), (20, 128)])
def test_score_epilogue_forms_on_a_dirty_workspace(ops, B, S):
    """The scoring epilogue merges keys with atomicMax into a plane that the prologue kernel clears (per chunk for
    chunk_scores, per document for route_topk) and reads row masks that the prologue writes word by word.  Both must
    give the oracle's scores whatever the workspace held before, for queries that fit one wavefront's tile and for
    queries that span several, and a query without a scored token must come back as -inf everywhere."""
    say(f"epilogue forms B={B} S={S}")
    bank, kr, dco, _ = _bank(ops, [3, 1, 7, 2, 9, 4, 1, 1, 12] * 41, 8, torch.bfloat16, 900 + B)
    q = _randn((B, S, 32, 128), 901 + S, torch.bfloat16)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[0, S // 2 + 1:] = False
    if B > 1:
        mask[B - 1] = False
    bank.workspace(B, S, 32, 16, "cuda", chunk_plane=True).fill_(0xFF)
    got = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda()).cpu()
    want = cf.chunk_scores(q, mask, kr, "cosine")
    live = mask.any(dim=1)
    assert cf.rel_err(got[live], want[live]) < 1e-2
    assert torch.isinf(got[~live]).all() and (got[~live] < 0).all()
    bank.workspace(B, S, 32, 16, "cuda").fill_(0xFF)
    s, d, _ = ops.route_topk(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0, 16)
    ds = cf.doc_scores(want, dco)
    assert not cf.topk_acceptable(ds[live], d.cpu().long()[live], 16)
    assert torch.isinf(s.cpu()[~live]).all()


@pytest.mark.parametrize("B,S,Hkv", [(24, 100, 4), (9, 250, 8), (40, 33, 2)])
def test_scores_many_query_tiles(ops, B, S, Hkv):
    """More than eight 256-row query tiles (they are then walked in groups of eight per K_r tile, the last group
    ragged), a ragged last K_r tile, and depths of 4 to 16 K steps per tile through the large-tile form; a masked
    tail of one query and a query whose padded rows end inside a tile."""
    say(f"many query tiles B={B} S={S} Hkv={Hkv}")
    bank, kr, dco, _ = _bank(ops, [5, 1, 8, 2, 11, 3] * 37, Hkv, torch.bfloat16, 950 + B)
    q = _randn((B, S, 4 * Hkv, 128), 951 + S, torch.bfloat16)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[1, S // 3:] = False
    got = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda()).cpu()
    want = cf.chunk_scores(q, mask, kr, "cosine")
    assert cf.rel_err(got, want) < 1e-2
    s_, d, _ = ops.route_topk(bank, 0, q.cuda(), mask.cuda(), "cosine", 1.0, 8)
    assert not cf.topk_acceptable(cf.doc_scores(want, dco), d.cpu().long(), 8)


@pytest.mark.parametrize("topk", [1, 16, 64])
def test_topk_windows_long_documents_and_filtering(ops, topk):
    """Documents longer than the top-k kernel's LDS window (2044 keys) among one-chunk documents, more documents
    than one workgroup's block, and planted winners at both ends of the bank: ids and order must be exact."""
    say(f"top-k windows topk={topk}")
    rng = np.random.default_rng(11)
    doc_chunks = [1] * 3000 + [5000] + list(rng.integers(1, 40, size=2500)) + [2045, 2044, 4089] + [1] * 700
    bank, kr, dco, dev = _bank(ops, doc_chunks, 8, torch.bfloat16, 930)
    n_docs = len(doc_chunks)
    B, S = 3, 8
    q = _randn((B, S, 32, 128), 931, torch.bfloat16)
    # plant winners: the last chunk of a chosen document becomes the direction one query token has after the
    # pre-sum over each group's heads, scaled down by rank (6 % steps, far above bf16 noise); every query gets its
    # own documents, spread over both ends of the bank and the long documents
    edge = [0, 2999, 3000, 3001, n_docs - 1, n_docs - 702, n_docs - 703, 4000, 1, 2998, 3100, n_docs - 2,
            n_docs - 701, n_docs - 704, 4001, 2, 2997, 3500, n_docs - 3, n_docs - 700, 3200, 4002, 3, 2996]
    assert len(set(edge)) == len(edge) and doc_chunks[n_docs - 702] == 2044 and doc_chunks[3000] == 5000
    n_win = max(1, min(8, topk))
    qf = cf.l2_normalize(q.double())
    for b in range(B):
        for r, dsel in enumerate(edge[b::B][:n_win]):
            c = int(dco[dsel + 1]) - 1
            v = qf[b, r % S].view(8, 4, 128).mean(dim=1)                   # [Hkv, D]
            kr[c] = (cf.l2_normalize(v) * (1.0 - 0.06 * r)).to(torch.bfloat16)
    dev.copy_(kr.cuda())
    s, d, _ = ops.route_topk(bank, 0, q.cuda(), None, "cosine", 1.0, topk)
    ds = cf.doc_scores(cf.chunk_scores(q, torch.ones(B, S, dtype=torch.bool), kr, "cosine"), dco)
    assert not cf.topk_acceptable(ds, d.cpu().long(), topk)
    ws, wi = cf.topk_docs(ds, topk)
    assert cf.rel_err(s.cpu(), ws) < 1e-2
    sc = s.cpu()
    assert (sc[:, :-1] >= sc[:, 1:]).all()
    # clear winners (gap above the rest far larger than bf16 noise) must match the oracle id for id, in order
    got = d.cpu().long()[:, :n_win]
    assert torch.equal(got, wi[:, :n_win]), (got, wi[:, :n_win])
    for b in range(B):
        assert sorted(got[b].tolist()) == sorted(edge[b::B][:n_win])


@pytest.mark.parametrize("Hq,Hkv", [(4, 1), (8, 2), (32, 8), (24, 3)])
@pytest.mark.parametrize("B,S", [(1, 40), (2, 20), (1, 5)])
def test_scores_at_most_64_query_rows(ops, Hq, Hkv, B, S):
    """The narrow tile with two K tiles of loads in flight: even and odd K-tile counts (Hkv * 128 / 64), a bank that
    is not a multiple of the tile, masked tokens."""
    say(f"narrow tile Hq={Hq} Hkv={Hkv} B={B} S={S}")
    bank, kr, dco, _ = _bank(ops, [3, 1, 7, 2, 9, 4, 5] * 53, Hkv, torch.bfloat16, 950 + Hkv)
    q = _randn((B, S, Hq, 128), 951 + S, torch.bfloat16)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[0, ::3] = False
    got = ops.chunk_scores(bank, 0, q.cuda(), mask.cuda())
    assert cf.rel_err(got.cpu(), cf.chunk_scores(q, mask, kr, "cosine")) < 1e-2


@pytest.mark.gpu
def test_mfma_loop_diagnostic_counts_exactly():
    """msa_diag_mfma_loop with operands of ones: every MFMA adds 16 to each accumulator element, eight accumulators per
    thread are summed, so every thread reports 128 * iters; the reported operation count is workgroups x 8 wavefronts x
    iters x 8 MFMAs x 2 * 32 * 32 * 16.  The other two modes (zero and toggling operands) run and stay finite."""
    import ctypes as C
    from msa_amd import _lib
    lib = _lib.load()
    wgs, iters = 8, 1000
    sink = torch.full((wgs * 512,), -1.0, device="cuda")
    flops = C.c_double(0)
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.msa_diag_mfma_loop(wgs, iters, 1, sink.data_ptr(), C.byref(flops), st), "msa_diag_mfma_loop")
    torch.cuda.synchronize()
    assert torch.equal(sink.cpu(), torch.full((wgs * 512,), 128.0 * iters))
    assert flops.value == wgs * 8 * iters * 8 * 2 * 32 * 32 * 16
    _lib.check(lib.msa_diag_mfma_loop(wgs, iters, 0, sink.data_ptr(), None, st), "msa_diag_mfma_loop")
    torch.cuda.synchronize()
    assert torch.equal(sink.cpu(), torch.zeros(wgs * 512))
    _lib.check(lib.msa_diag_mfma_loop(wgs, iters, 2, sink.data_ptr(), None, st), "msa_diag_mfma_loop")
    torch.cuda.synchronize()
    assert torch.isfinite(sink).all() and (sink != 0).any()
    assert lib.msa_diag_mfma_loop(0, iters, 1, sink.data_ptr(), None, st) != 0
    # the variants with other VALU work between the products (mode + 16 * extra) run; their sink is not defined
    for extra in range(1, 8):
        _lib.check(lib.msa_diag_mfma_loop(wgs, 50, 16 * extra, sink.data_ptr(), C.byref(flops), st), "msa_diag_mfma_loop")
        assert flops.value == wgs * 8 * 50 * 8 * 2 * 32 * 32 * 16
    torch.cuda.synchronize()
    assert lib.msa_diag_mfma_loop(wgs, 50, 16 * 8, sink.data_ptr(), None, st) != 0
    assert lib.msa_diag_mfma_loop(wgs, 50, 3, sink.data_ptr(), None, st) != 0


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_route_topk_mid_size_banks_with_the_tile_pool(seed):
    """Random mid-size banks (130k - 300k chunks, 9 - 24 queries of 64 - 200 tokens, 4 or 8 KV heads, ragged masks, both
    modes): large enough for the scan's tile pool (the last eighth of the N tiles, drawn dynamically) to be active with
    ragged last tiles.  Checked against the whole-bank property the top-k must have, computed by plain fp32 torch
    matmuls on the device from the same bf16 inputs: the returned scores are the documents' true scores, they come in
    descending order, and no returned document scores below the true k-th score (beyond the tie tolerance)."""
    from msa_amd import ops
    rng = np.random.default_rng(seed)
    g = torch.Generator(device="cuda").manual_seed(seed)
    D = 128
    Hkv = int(rng.choice([4, 8])); Hq = Hkv * 4
    B = int(rng.integers(9, 25)); S = int(rng.integers(64, 200))
    n_docs = int(rng.integers(9000, 16000))
    doc_chunks = rng.integers(4, 33, size=n_docs)
    dco = np.concatenate([[0], np.cumsum(doc_chunks)]); C = int(dco[-1])
    mode = ["cosine", "scaled_dot"][seed % 2]
    k = [4, 16, 32][seed % 3]
    say(f"mid-size bank seed={seed} B={B} S={S} Hkv={Hkv} C={C} docs={n_docs} mode={mode} k={k}")
    bank = ops.Bank(1, dco.tolist(), list(range(n_docs)), Hkv, D, torch.bfloat16)
    kr = torch.randn((C, Hkv, D), generator=g, device="cuda")
    if mode == "cosine":
        kr = kr / kr.norm(dim=-1, keepdim=True)
    kr = kr.to(torch.bfloat16)
    bank.set_layer(0, kr)
    q = torch.randn((B, S, Hq, D), generator=g, device="cuda").to(torch.bfloat16)
    mask = torch.rand((B, S), generator=g, device="cuda") > 0.2
    mask[:, 0] = True
    scale = D ** -0.5
    sc, doc, gid = ops.route_topk(bank, 0, q, mask, mode, scale, k)
    torch.cuda.synchronize()
    qf = q.float()
    if mode == "cosine":
        qf = qf / qf.norm(dim=-1, keepdim=True)
    qs = qf.view(B, S, Hkv, 4, D).sum(3).to(torch.bfloat16).float()        # rounded as the kernel's pre-sum rounds them
    krf = kr.float().view(C, Hkv * D)
    seg = torch.repeat_interleave(torch.arange(n_docs, device="cuda"), torch.as_tensor(doc_chunks, device="cuda"))
    mul = (1.0 if mode == "cosine" else scale) / Hq
    for b in range(B):
        s_bc = (qs[b].reshape(S, Hkv * D) @ krf.T) * mul
        s_bc[~mask[b]] = float("-inf")
        ds = torch.full((n_docs,), float("-inf"), device="cuda").scatter_reduce_(0, seg, s_bc.max(0).values, reduce="amax")
        true_of_returned = ds[doc[b].long()]
        kth = torch.topk(ds, k).values[-1]
        assert torch.allclose(sc[b], true_of_returned, rtol=1e-2, atol=2e-3)
        assert bool((true_of_returned >= kth - 1e-3).all())                  # the 1e-3 gap rule at the k boundary
        assert bool((sc[b][:-1] >= sc[b][1:]).all())
        assert torch.equal(gid[b], doc[b].long())


def test_asm_scheduled_kernels_were_loaded_without_scratch(ops):
    """The loaded code object's routing scan and wide flash kernel use no scratch memory (their asm statements keep
    state in physical registers across statements; the library would refuse to launch them otherwise) and the whole
    register file of a SIMD lane (one wavefront per SIMD)."""
    say("resources of the asm-scheduled kernels")
    from msa_amd import _lib
    lib = _lib.load()
    for which in (0, 1):
        regs, scratch = C.c_int32(-1), C.c_int32(-1)
        _lib.check(lib.msa_diag_asm_kernel_resources(which, C.byref(regs), C.byref(scratch)), "msa_diag_asm_kernel_resources")
        print(f"[resources] kernel {which}: {regs.value} registers, {scratch.value} bytes of scratch", flush=True)
        assert scratch.value == 0
        assert regs.value == 512
    assert lib.msa_diag_asm_kernel_resources(2, C.byref(regs), C.byref(scratch)) != 0


def test_read_stream_diagnostic_reads_what_it_says(ops):
    """The measurement aid behind the HBM ceilings: its storing form writes, per 128 KB read, the xor of the 32
    4 KB slices of that block (so every byte was loaded once); the two non-storing forms leave dst alone; sizes that
    are no multiple of 128 KB and unknown modes are refused."""
    say("read-stream diagnostic, 3 x 128 KB")
    from msa_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    groups = 3
    src = torch.randint(0, 1 << 31, (groups, 32, 1024), dtype=torch.int32, generator=torch.Generator().manual_seed(5))
    want = src[:, 0].clone()
    for i in range(1, 32):
        want ^= src[:, i]
    want = want[:, :512]                                     # lanes 0 - 127: 2 KB
    d_src = src.cuda()
    dst = torch.full((groups, 512), -7, dtype=torch.int32, device="cuda")
    _lib.check(lib.msa_diag_read_stream(d_src.data_ptr(), groups * 131072, dst.data_ptr(), 1, st), "msa_diag_read_stream")
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), want)
    for mode in (0, 2):
        dst.fill_(-7)
        _lib.check(lib.msa_diag_read_stream(d_src.data_ptr(), groups * 131072, dst.data_ptr(), mode, st), "msa_diag_read_stream")
        torch.cuda.synchronize()
        assert bool((dst == -7).all())
    assert lib.msa_diag_read_stream(d_src.data_ptr(), 131072 + 2048, dst.data_ptr(), 0, st) != 0
    assert lib.msa_diag_read_stream(d_src.data_ptr(), 131072, dst.data_ptr(), 3, st) != 0
    assert lib.msa_diag_read_stream(None, 131072, dst.data_ptr(), 0, st) != 0
