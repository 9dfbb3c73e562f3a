"""The allocation-free routing entry point against the workspace one, through the C ABI: same kernels, scratch in a
device array of the library.  Two calls in a row, the second smaller, so anything a call leaves behind in the shared
scratch would show."""
import sys

import numpy as np
import pytest
import torch

from oracle import closed_form as cf

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _route_both(lib, _lib, bank, q, mask, topk):
    B, S, Hq, _ = q.shape
    dev = q.device
    outs = []
    for static in (False, True):
        sc = torch.full((B, topk), 7.0, dtype=torch.float32, device=dev)
        dc = torch.full((B, topk), -7, dtype=torch.int32, device=dev)
        gd = torch.full((B, topk), -7, dtype=torch.int64, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        m = None if mask is None else mask.to(torch.uint8).contiguous()
        if static:
            _lib.check(lib.msa_route_topk_static(bank.handle, 0, q.data_ptr(), _lib.ptr(m), B, S, Hq, _lib.MODE_COSINE, 1.0,
                                                 topk, sc.data_ptr(), dc.data_ptr(), gd.data_ptr(), st), "msa_route_topk_static")
        else:
            ws = bank.workspace(B, S, Hq, topk, dev)
            _lib.check(lib.msa_route_topk(bank.handle, 0, q.data_ptr(), _lib.ptr(m), B, S, Hq, _lib.MODE_COSINE, 1.0, topk,
                                          sc.data_ptr(), dc.data_ptr(), gd.data_ptr(), ws.data_ptr(), ws.numel(), st),
                       "msa_route_topk")
        torch.cuda.synchronize()
        outs.append((sc.cpu(), dc.cpu(), gd.cpu()))
    return outs


def test_route_topk_static_matches_workspace_form():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible")
    from msa_amd import _lib, ops
    lib = _lib.load()
    say("allocation-free routing entry point: two calls in a row, the second smaller")
    rng = np.random.default_rng(3)
    doc_chunks = [int(x) for x in rng.integers(1, 30, size=5000)]
    dco = np.concatenate([[0], np.cumsum(doc_chunks)])
    C = int(dco[-1])
    g = torch.Generator().manual_seed(5)
    kr = torch.nn.functional.normalize(torch.randn((C, 8, 128), generator=g), dim=-1).to(torch.bfloat16)
    bank = ops.Bank(1, dco.tolist(), [1000 + 3 * i for i in range(len(doc_chunks))], 8, 128, torch.bfloat16)
    kr_dev = kr.cuda()
    bank.set_layer(0, kr_dev)
    for B, S, topk in ((6, 100, 16), (1, 17, 5)):
        q = torch.randn((B, S, 32, 128), generator=g).to(torch.bfloat16)
        mask = torch.ones(B, S, dtype=torch.bool)
        mask[0, : S // 3] = False
        (s0, d0, g0), (s1, d1, g1) = _route_both(lib, _lib, bank, q.cuda(), mask.cuda(), topk)
        assert torch.equal(d0, d1) and torch.equal(g0, g1) and torch.equal(s0, s1)      # same kernels: bit for bit
        # and both are right: the oracle accepts the selection
        ds = cf.doc_scores(cf.chunk_scores(q, mask, kr, "cosine"), dco)
        assert not cf.topk_acceptable(ds, d1.long(), topk)
        assert (g1 == 1000 + 3 * d1.long()).all()
    # a request whose scratch does not fit the built-in buffer is refused, not truncated
    big = torch.zeros((64, 512, 32, 128), dtype=torch.bfloat16, device="cuda")
    out = torch.empty((64, 16), dtype=torch.float32, device="cuda")
    doc = torch.empty((64, 16), dtype=torch.int32, device="cuda")
    rc = lib.msa_route_topk_static(bank.handle, 0, big.data_ptr(), None, 64, 512, 32, _lib.MODE_COSINE, 1.0, 16,
                                   out.data_ptr(), doc.data_ptr(), None, torch.cuda.current_stream().cuda_stream)
    assert rc == -3 and b"scratch" in lib.msa_last_error()
