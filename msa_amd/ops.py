"""Torch-tensor front end of the C ABI (``include/msa_amd.h``).

PyTorch is used here only to own device / pinned memory and to name streams; every computation
below happens in the HIP library.  All functions enqueue on the current torch stream unless a
stream is given, and raise :class:`msa_amd._lib.MsaError` on any failure.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import MODE_COSINE, MODE_SCALED_DOT, check, dtype_code, ptr

MODES = {"cosine": MODE_COSINE, "scaled_dot": MODE_SCALED_DOT}


def _stream(stream: Optional[torch.cuda.Stream] = None) -> int:
    return (stream or torch.cuda.current_stream()).cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("expected a device tensor (the HIP path has no CPU fallback)")
        if t is not None and not t.is_contiguous():
            raise ValueError("expected a contiguous tensor")


# ------------------------------------------------------------------------------ chunk table
@dataclass
class ChunkTable:
    """Device-side chunking of one packed block (all int32 tensors)."""
    doc_start: torch.Tensor       # [n_docs + 1] token offsets
    doc_chunk_off: torch.Tensor   # [n_docs + 1]
    chunk_start: torch.Tensor     # [C]
    chunk_len: torch.Tensor       # [C]
    chunk_doc: torch.Tensor       # [C] 0-based
    n_chunks: torch.Tensor        # [1] int64, written by the kernel
    P: int
    max_doc_len: int

    @property
    def C(self) -> int:
        return self.chunk_start.numel()


def chunk_table(doc_lens: Sequence[int], P: int, first_token: int = 0, device="cuda") -> ChunkTable:
    """Builds the chunk table on the device from host-side document lengths (the host only sizes
    the outputs: ``C = sum(ceil(len / P))``, as src/prefill.py:225 does)."""
    lib = _lib.load()
    lens = [int(x) for x in doc_lens]
    if not lens or min(lens) <= 0:
        raise ValueError("every document needs at least one token")
    n_chunks = sum((n + P - 1) // P for n in lens)
    starts = torch.tensor([first_token] + lens, dtype=torch.int64).cumsum(0).to(torch.int32)
    doc_start = starts.to(device)
    n_docs = len(lens)
    i32 = dict(dtype=torch.int32, device=device)
    t = ChunkTable(doc_start, torch.empty(n_docs + 1, **i32), torch.empty(n_chunks, **i32),
                   torch.empty(n_chunks, **i32), torch.empty(n_chunks, **i32),
                   torch.zeros(1, dtype=torch.int64, device=device), P, max(lens))
    check(lib.msa_chunk_table(ptr(t.doc_start), n_docs, P, n_chunks, ptr(t.doc_chunk_off), ptr(t.chunk_start),
                              ptr(t.chunk_len), ptr(t.chunk_doc), ptr(t.n_chunks), _stream()), "msa_chunk_table")
    return t


# ------------------------------------------------------------------------------ pooling
def rope_tables(n_rows: int, D: int, theta: float, device="cuda") -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 ``[n_rows, D/2]`` cos / sin tables, computed the way Qwen3RotaryEmbedding does (fp32
    inv_freq, fp32 angles)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.int64).float() / D))
    ang = torch.arange(n_rows, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return ang.cos().contiguous().to(device), ang.sin().contiguous().to(device)


def pool_chunks(k: Optional[torch.Tensor], v: Optional[torch.Tensor], kr: Optional[torch.Tensor], table: ChunkTable,
                rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, normalize_kr: bool = False):
    """Chunk means of token-major ``[T, H, D]`` tensors -> chunk-major ``[C, H, D]`` (same dtype).
    ``rope=(cos, sin)`` rotates K at per-document positions while reading it."""
    lib = _lib.load()
    ref = next(t for t in (k, v, kr) if t is not None)
    _need_cuda(k, v, kr)
    T, H, D = ref.shape
    for t in (k, v, kr):
        if t is not None and (t.shape != ref.shape or t.dtype != ref.dtype):
            raise ValueError("K, V and K_r must share shape and dtype")
    outs = [None if t is None else torch.empty((table.C, H, D), dtype=ref.dtype, device=ref.device) for t in (k, v, kr)]
    cos, sin = rope if rope is not None else (None, None)
    if rope is not None:
        _need_cuda(cos, sin)
        if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != D // 2:
            raise ValueError("rotary tables must be fp32 [rows, D/2]")
    check(lib.msa_pool_chunks(ptr(k), ptr(v), ptr(kr), dtype_code(ref.dtype), T, H, D, ptr(table.chunk_start),
                              ptr(table.chunk_len), ptr(table.chunk_doc), table.C, ptr(table.doc_start), ptr(cos),
                              ptr(sin), 0 if cos is None else cos.shape[0], table.max_doc_len, int(normalize_kr),
                              ptr(outs[0]), ptr(outs[1]), ptr(outs[2]), _stream()), "msa_pool_chunks")
    return tuple(outs)


# ------------------------------------------------------------------------------ bank + routing
class Bank:
    """Owner of an ``msa_bank`` handle plus the tensors it borrows."""

    def __init__(self, n_layers: int, doc_chunk_off: Sequence[int], doc_global_id: Sequence[int], Hkv: int, D: int,
                 dtype: torch.dtype):
        lib = _lib.load()
        self.off_host = torch.as_tensor(doc_chunk_off, dtype=torch.int32).contiguous()
        self.gid_host = torch.as_tensor(doc_global_id, dtype=torch.int64).contiguous()
        self.n_docs = self.gid_host.numel()
        if self.off_host.numel() != self.n_docs + 1:
            raise ValueError("doc_chunk_off must have n_docs + 1 entries")
        self.C = int(self.off_host[-1])
        self.max_doc_chunks = int((self.off_host[1:] - self.off_host[:-1]).max())
        self.n_layers, self.Hkv, self.D, self.dtype = n_layers, Hkv, D, dtype
        self._keep = {}
        self._ws: Optional[torch.Tensor] = None
        h = C.c_void_p()
        check(lib.msa_bank_create(C.byref(h), n_layers, self.C, Hkv, D, dtype_code(dtype), ptr(self.off_host),
                                  ptr(self.gid_host), self.n_docs), "msa_bank_create")
        self.handle = h

    def set_layer(self, layer: int, kr: torch.Tensor, k_host: Optional[torch.Tensor] = None,
                  v_host: Optional[torch.Tensor] = None):
        want = (self.C, self.Hkv, self.D)
        _need_cuda(kr)
        for t in (kr, k_host, v_host):
            if t is not None and (tuple(t.shape) != want or t.dtype != self.dtype or not t.is_contiguous()):
                raise ValueError(f"bank tensors must be contiguous {want} {self.dtype}")
        for t in (k_host, v_host):
            if t is not None and (t.is_cuda or not t.is_pinned()):
                raise ValueError("pooled K / V must live in pinned host memory")
        check(_lib.load().msa_bank_set_layer(self.handle, layer, ptr(kr), ptr(k_host), ptr(v_host)),
              "msa_bank_set_layer")
        self._keep[layer] = (kr, k_host, v_host)

    def workspace(self, B: int, S: int, Hq: int, topk: int, device, chunk_plane: bool = False) -> torch.Tensor:
        """Scratch for ``route_topk`` (pre-summed queries, row masks, one key per document, candidate lists);
        with ``chunk_plane`` also room for the ``[B, C]`` key plane ``chunk_scores`` needs."""
        lib = _lib.load()
        need = (lib.msa_route_workspace_bytes(B, S, Hq, self.Hkv, self.D, self.C, self.n_docs, topk) if chunk_plane
                else lib.msa_route_topk_workspace_bytes(B, S, Hq, self.Hkv, self.D, self.n_docs, topk))
        if self._ws is None or self._ws.numel() < need or self._ws.device != torch.device(device):
            self._ws = torch.empty(need, dtype=torch.uint8, device=device)
        return self._ws

    def close(self):
        if getattr(self, "handle", None):
            _lib.load().msa_bank_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _route_args(bank: Bank, q: torch.Tensor, qmask: Optional[torch.Tensor], mode: str):
    _need_cuda(q, qmask)
    if q.dim() != 4 or q.shape[3] != bank.D or q.dtype != bank.dtype:
        raise ValueError(f"q must be [B, S, Hq, {bank.D}] {bank.dtype}")
    B, S, Hq, _ = q.shape
    if qmask is not None:
        if tuple(qmask.shape) != (B, S):
            raise ValueError("qmask must be [B, S]")
        qmask = qmask.to(torch.uint8).contiguous()
    if mode not in MODES:
        raise NotImplementedError(f"unsupported scoring mode {mode!r}")
    return B, S, Hq, qmask


def chunk_scores(bank: Bank, layer: int, q: torch.Tensor, qmask: Optional[torch.Tensor] = None, mode: str = "cosine",
                 scale: float = 1.0) -> torch.Tensor:
    """fp32 ``[B, C]`` chunk scores (mean over heads, max over scored tokens)."""
    B, S, Hq, qm = _route_args(bank, q, qmask, mode)
    ws = bank.workspace(B, S, Hq, 16, q.device, chunk_plane=True)
    out = torch.empty((B, bank.C), dtype=torch.float32, device=q.device)
    check(_lib.load().msa_chunk_scores(bank.handle, layer, ptr(q), ptr(qm), B, S, Hq, MODES[mode], scale, ptr(out),
                                       ptr(ws), ws.numel(), _stream()), "msa_chunk_scores")
    return out


QUERY_REDUCE = {"max": 0, "mean": 1, "last": 2}     # the reference's query_reduce_method (src/msa_service.py:749-780)
CHUNK_REDUCE = {"max": 0, "mean": 1}                # chunk_reduce_method (:787-811)


def route_topk(bank: Bank, layer: int, q: torch.Tensor, qmask: Optional[torch.Tensor] = None, mode: str = "cosine",
               scale: float = 1.0, topk: int = 16, query_reduce: str = "max", chunk_reduce: str = "max"):
    """``(scores [B, k] fp32, doc [B, k] int32 0-based, doc_global [B, k] int64)``.  ``query_reduce`` / ``chunk_reduce``
    other than "max" take the reference's other reductions (``msa_route_topk_reduce``)."""
    B, S, Hq, qm = _route_args(bank, q, qmask, mode)
    if query_reduce not in QUERY_REDUCE:
        raise NotImplementedError(f"Unsupported query reduce method: {query_reduce}")
    if chunk_reduce not in CHUNK_REDUCE:
        raise ValueError(f"Invalid chunk reduction method: {chunk_reduce}")
    scores = torch.empty((B, topk), dtype=torch.float32, device=q.device)
    doc = torch.empty((B, topk), dtype=torch.int32, device=q.device)
    gid = torch.empty((B, topk), dtype=torch.int64, device=q.device)
    if query_reduce == "max" and chunk_reduce == "max":
        ws = bank.workspace(B, S, Hq, topk, q.device)
        check(_lib.load().msa_route_topk(bank.handle, layer, ptr(q), ptr(qm), B, S, Hq, MODES[mode], scale, topk,
                                         ptr(scores), ptr(doc), ptr(gid), ptr(ws), ws.numel(), _stream()),
              "msa_route_topk")
    else:
        ws = bank.workspace(B, S, Hq, topk, q.device, chunk_plane=chunk_reduce != "max")
        check(_lib.load().msa_route_topk_reduce(bank.handle, layer, ptr(q), ptr(qm), B, S, Hq, MODES[mode], scale,
                                                QUERY_REDUCE[query_reduce], CHUNK_REDUCE[chunk_reduce], topk, ptr(scores),
                                                ptr(doc), ptr(gid), ptr(ws), ws.numel(), _stream()),
              "msa_route_topk_reduce")
    return scores, doc, gid


# ------------------------------------------------------------------------------ gather
def gather_kv(bank: Bank, layer: int, doc_sel_host: torch.Tensor, device, stream: Optional[torch.cuda.Stream] = None):
    """Copies the selected documents' pooled K / V rows from pinned host memory on ``stream``.
    Returns ``(K [sum, Hkv, D], V, cu_sel int64 [B + 1] (host))``; the copies are merely enqueued."""
    lib = _lib.load()
    sel = doc_sel_host.to(torch.int32).contiguous()
    if sel.is_cuda or sel.dim() != 2:
        raise ValueError("doc_sel_host must be a host tensor [B, k]")
    B, k = sel.shape
    cu = torch.empty(B + 1, dtype=torch.int64)
    check(lib.msa_gather_plan(bank.handle, ptr(sel), B, k, ptr(cu)), "msa_gather_plan")
    total = int(cu[-1])
    with torch.cuda.stream(stream) if stream is not None else _null_ctx():
        k_out = torch.empty((total, bank.Hkv, bank.D), dtype=bank.dtype, device=device)
        v_out = torch.empty_like(k_out)
    check(lib.msa_gather_kv(bank.handle, layer, ptr(sel), B, k, ptr(k_out), ptr(v_out), total, _stream(stream)),
          "msa_gather_kv")
    return k_out, v_out, cu


def gather_kv_device(bank: Bank, layer: int, doc_sel: torch.Tensor, capacity_chunks: int,
                     out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
    """Device-side gather: ``doc_sel [B, k]`` int32 on the device (e.g. ``route_topk``'s documents).  Returns
    ``(K [capacity, Hkv, D], V, cu_sel int32 [B + 1] on the device)``; rows ``cu_sel[b] .. cu_sel[b + 1]`` belong to
    sample ``b``.  No host synchronisation."""
    _need_cuda(doc_sel)
    if doc_sel.dtype != torch.int32 or doc_sel.dim() != 2:
        raise ValueError("doc_sel must be int32 [B, k]")
    B, k = doc_sel.shape
    lib = _lib.load()
    dev = doc_sel.device
    if out is None:
        k_out = torch.empty((capacity_chunks, bank.Hkv, bank.D), dtype=bank.dtype, device=dev)
        v_out = torch.empty_like(k_out)
    else:
        k_out, v_out = out
    cu = torch.empty(B + 1, dtype=torch.int32, device=dev)
    ws = torch.empty(lib.msa_gather_device_workspace_bytes(B, k), dtype=torch.uint8, device=dev)
    check(lib.msa_gather_kv_device(bank.handle, layer, ptr(doc_sel), B, k, ptr(k_out), ptr(v_out), capacity_chunks, ptr(cu),
                                   ptr(ws), ws.numel(), _stream()), "msa_gather_kv_device")
    return k_out, v_out, cu


def route_topk_gather(bank: Bank, layer: int, q: torch.Tensor, qmask: Optional[torch.Tensor], mode: str, scale: float,
                      topk: int, gather_layer: int, gather_doc_sel: torch.Tensor, capacity_chunks: int,
                      out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
    """``route_topk`` of ``layer`` with ``gather_kv_device`` of (``gather_layer``, ``gather_doc_sel``) in the same
    launch (one workgroup of the scan copies while the others score).  Returns the two calls' results:
    ``(scores, doc, doc_global), (K, V, cu_sel)``."""
    B, S, Hq, qm = _route_args(bank, q, qmask, mode)
    _need_cuda(gather_doc_sel)
    if gather_doc_sel.dtype != torch.int32 or gather_doc_sel.dim() != 2:
        raise ValueError("gather_doc_sel must be int32 [B, k]")
    gB, gk = gather_doc_sel.shape
    lib = _lib.load()
    dev = q.device
    ws = bank.workspace(B, S, Hq, topk, dev)
    scores = torch.empty((B, topk), dtype=torch.float32, device=dev)
    doc = torch.empty((B, topk), dtype=torch.int32, device=dev)
    gid = torch.empty((B, topk), dtype=torch.int64, device=dev)
    if out is None:
        k_out = torch.empty((capacity_chunks, bank.Hkv, bank.D), dtype=bank.dtype, device=dev)
        v_out = torch.empty_like(k_out)
    else:
        k_out, v_out = out
    cu = torch.empty(gB + 1, dtype=torch.int32, device=dev)
    gws = torch.empty(lib.msa_gather_device_workspace_bytes(gB, gk), dtype=torch.uint8, device=dev)
    check(lib.msa_route_topk_gather(bank.handle, layer, ptr(q), ptr(qm), B, S, Hq, MODES[mode], scale, topk, ptr(scores),
                                    ptr(doc), ptr(gid), ptr(ws), ws.numel(), gather_layer, ptr(gather_doc_sel), gB, gk,
                                    ptr(k_out), ptr(v_out), capacity_chunks, ptr(cu), ptr(gws), gws.numel(), _stream()),
          "msa_route_topk_gather")
    return (scores, doc, gid), (k_out, v_out, cu)


class _null_ctx:
    def __enter__(self):
        return None

    def __exit__(self, *a):
        return False


# ------------------------------------------------------------------------------ cache + attention
def assemble_context(prefix_k, prefix_v, mem_k, mem_v, cu_sel, local_k, local_v, cu_local, B: int, Lcap: int):
    """Builds ``kcache / vcache [B, Lcap, Hkv, D]`` and ``kv_len [B]`` from
    ``[prefix | memory rows of b | local rows of b]``."""
    ref = next(t for t in (prefix_k, mem_k, local_k) if t is not None)
    Hkv, D = ref.shape[-2], ref.shape[-1]
    _need_cuda(prefix_k, prefix_v, mem_k, mem_v, cu_sel, local_k, local_v, cu_local)
    kc = torch.empty((B, Lcap, Hkv, D), dtype=ref.dtype, device=ref.device)
    vc = torch.empty_like(kc)
    kv_len = torch.empty(B, dtype=torch.int32, device=ref.device)
    n_prefix = 0 if prefix_k is None else prefix_k.shape[0]
    check(_lib.load().msa_assemble_context(ptr(prefix_k), ptr(prefix_v), n_prefix, ptr(mem_k), ptr(mem_v),
                                           ptr(cu_sel), ptr(local_k), ptr(local_v), ptr(cu_local), B, Hkv, D,
                                           dtype_code(ref.dtype), ptr(kc), ptr(vc), Lcap, ptr(kv_len), _stream()),
          "msa_assemble_context")
    return kc, vc, kv_len


def cache_append(k_new, v_new, kcache, vcache, kv_len):
    """Writes one ``[B, Hkv, D]`` row per sample at ``kv_len[b]`` and increments it, in place."""
    _need_cuda(k_new, v_new, kcache, vcache, kv_len)
    B, Lcap, Hkv, D = kcache.shape
    check(_lib.load().msa_cache_append(ptr(k_new), ptr(v_new), B, Hkv, D, dtype_code(kcache.dtype), ptr(kcache),
                                       ptr(vcache), Lcap, ptr(kv_len), _stream()), "msa_cache_append")


def cache_append_rows(k_new, v_new, cu_new, max_new: int, kcache, vcache, kv_len):
    """Ragged append: sample ``b`` gets rows ``cu_new[b]:cu_new[b+1]`` of ``k_new / v_new [total, Hkv, D]`` at
    ``kv_len[b]``, which grows by that count (clamped to the capacity), in place."""
    _need_cuda(k_new, v_new, cu_new, kcache, vcache, kv_len)
    B, Lcap, Hkv, D = kcache.shape
    if cu_new.dtype != torch.int32 or cu_new.numel() != B + 1 or k_new.shape[1:] != (Hkv, D) or k_new.shape != v_new.shape:
        raise ValueError("cu_new int32 [B + 1]; k_new / v_new [total, Hkv, D]")
    check(_lib.load().msa_cache_append_rows(ptr(k_new), ptr(v_new), ptr(cu_new), max_new, B, Hkv, D,
                                            dtype_code(kcache.dtype), ptr(kcache), ptr(vcache), Lcap, ptr(kv_len),
                                            _stream()), "msa_cache_append_rows")


_attn_ws = {}
FLASH_MIN_ROWS = 16     # bf16 query blocks at least this long go to the MFMA flash kernel


def sparse_attn(q, k, v, kv_off, kv_len, max_kv: int, cu_q=None, max_sq: int = 1, scale: Optional[float] = None,
                causal: bool = True):
    """GQA attention of ``q [total_q, Hq, D]`` over per-sample key ranges of ``k / v [rows, Hkv, D]``."""
    _need_cuda(q, k, v, kv_off, kv_len, cu_q)
    total_q, Hq, D = q.shape
    Hkv = k.shape[-2]
    B = kv_len.numel()
    if kv_off.dtype != torch.int64 or kv_len.dtype != torch.int32 or (cu_q is not None and cu_q.dtype != torch.int32):
        raise ValueError("kv_off int64, kv_len / cu_q int32")
    lib = _lib.load()
    sc = D ** -0.5 if scale is None else scale
    # long bf16 query blocks: one-pass MFMA flash kernel when there are enough blocks to fill the chip, otherwise the
    # split-KV entry point below (which runs the same MFMA kernel per key range for bf16 blocks of >= 8 rows)
    if q.dtype == torch.bfloat16 and max_sq >= FLASH_MIN_ROWS and total_q * Hkv >= 32 * 512:
        out = torch.empty_like(q)
        check(lib.msa_flash_attn_hint(ptr(q), ptr(cu_q), ptr(k), ptr(v), ptr(kv_off), ptr(kv_len), B, total_q, Hq, Hkv, D,
                                      sc, int(causal), ptr(out), int(max_sq), _stream()), "msa_flash_attn")
        return out
    need = lib.msa_attn_workspace_bytes(total_q, Hq, Hkv, D, max_kv)
    ws = _attn_ws.get(q.device)
    if ws is None or ws.numel() < need:
        ws = _attn_ws[q.device] = torch.empty(need, dtype=torch.uint8, device=q.device)
    out = torch.empty_like(q)
    check(lib.msa_sparse_attn(ptr(q), ptr(cu_q), ptr(k), ptr(v), ptr(kv_off), ptr(kv_len), B, total_q, max_sq, max_kv,
                              Hq, Hkv, D, dtype_code(q.dtype), D ** -0.5 if scale is None else scale, int(causal),
                              ptr(out), ptr(ws), ws.numel(), _stream()), "msa_sparse_attn")
    return out


# ------------------------------------------------------------------------------ fused layer helpers
def qk_norm_rope(qkv: torch.Tensor, Hq: int, Hkv: int, D: int, positions: torch.Tensor, q_norm_w, k_norm_w, eps: float,
                 rope: Tuple[torch.Tensor, torch.Tensor]):
    """``qkv [N, (Hq + 2 Hkv) * D]`` (fused projection output) -> ``q [N, Hq, D]`` and ``k [N, Hkv, D]``
    normalised per head and rotated at ``positions [N]``, plus ``v [N, Hkv, D]`` copied dense."""
    _need_cuda(qkv, positions, q_norm_w, k_norm_w, rope[0], rope[1])
    N, W = qkv.shape
    if W != (Hq + 2 * Hkv) * D or positions.dtype != torch.int64 or positions.numel() != N:
        raise ValueError("qkv must be [N, (Hq + 2 Hkv) D] and positions int64 [N]")
    q = torch.empty((N, Hq, D), dtype=qkv.dtype, device=qkv.device)
    k = torch.empty((N, Hkv, D), dtype=qkv.dtype, device=qkv.device)
    v = torch.empty((N, Hkv, D), dtype=qkv.dtype, device=qkv.device)
    es = qkv.element_size()
    base = qkv.data_ptr()
    check(_lib.load().msa_qk_norm_rope(base, base + Hq * D * es, base + (Hq + Hkv) * D * es, W, W, W, ptr(positions),
                                       ptr(q_norm_w), ptr(k_norm_w), eps, ptr(rope[0]), ptr(rope[1]), rope[0].shape[0],
                                       dtype_code(qkv.dtype), N, Hq, Hkv, D, ptr(q), ptr(k), ptr(v), _stream()),
          "msa_qk_norm_rope")
    return q, k, v


def qkv_proj(x: torch.Tensor, w: torch.Tensor, Hq: int, Hkv: int, positions: torch.Tensor, q_norm_w, k_norm_w, eps: float,
             rope: Tuple[torch.Tensor, torch.Tensor], router_front: int = 0, router_back: int = 0):
    """Fused projection of ``x [T, K]`` (bf16) through ``w [(router_front + Hq + 2 Hkv + router_back) * 128, K]``:
    returns ``q [T, Hq, 128]`` and ``k [T, Hkv, 128]`` (per-head RMSNorm + rotary at ``positions [T]`` done in the
    GEMM's epilogue), ``v [T, Hkv, 128]`` and the router heads ``r [T, router_front + router_back, 128]`` (``None``
    without router heads), all dense."""
    _need_cuda(x, w, positions, q_norm_w, k_norm_w, rope[0], rope[1])
    T, K = x.shape
    D = 128
    heads = router_front + Hq + 2 * Hkv + router_back
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or tuple(w.shape) != (heads * D, K):
        raise ValueError(f"qkv_proj: x [T, K] and w [{heads * D}, K] in bf16")
    if positions.dtype != torch.int64 or positions.numel() != T:
        raise ValueError("qkv_proj: positions int64 [T]")
    for name, nw in (("q_norm_w", q_norm_w), ("k_norm_w", k_norm_w)):
        if nw.dtype != torch.bfloat16 or nw.numel() != D or not nw.is_contiguous():
            raise ValueError(f"qkv_proj: {name} must be {D} contiguous bf16 weights, got {nw.dtype} x {nw.numel()}")
    for name, tab in (("cos", rope[0]), ("sin", rope[1])):
        if tab.dtype != torch.float32 or tab.dim() != 2 or tab.shape[1] != D // 2 or not tab.is_contiguous():
            raise ValueError(f"qkv_proj: the {name} table must be contiguous fp32 [rows, {D // 2}], got {tab.dtype} "
                             f"{tuple(tab.shape)}")
    if rope[0].shape != rope[1].shape:
        raise ValueError("qkv_proj: cos / sin tables differ in shape")
    if not (x.is_contiguous() and w.is_contiguous()) or x.data_ptr() % 16 or w.data_ptr() % 16:
        raise ValueError("qkv_proj: x and w must be contiguous and 16-byte aligned")
    dev = x.device
    q = torch.empty((T, Hq, D), dtype=x.dtype, device=dev)
    k = torch.empty((T, Hkv, D), dtype=x.dtype, device=dev)
    v = torch.empty((T, Hkv, D), dtype=x.dtype, device=dev)
    r = torch.empty((T, router_front + router_back, D), dtype=x.dtype, device=dev) if router_front + router_back else None
    check(_lib.load().msa_qkv_proj(ptr(x), T, K, ptr(w), Hq, Hkv, router_front, router_back, ptr(positions), ptr(q_norm_w),
                                   ptr(k_norm_w), eps, ptr(rope[0]), ptr(rope[1]), rope[0].shape[0], ptr(q), ptr(k), ptr(v),
                                   ptr(r), _stream()), "msa_qkv_proj")
    return q, k, v, r


def qk_norm_rope_append(qkv: torch.Tensor, Hq: int, Hkv: int, D: int, positions: torch.Tensor, q_norm_w, k_norm_w,
                        eps: float, rope: Tuple[torch.Tensor, torch.Tensor], kcache: torch.Tensor, vcache: torch.Tensor,
                        kv_len: torch.Tensor) -> torch.Tensor:
    """Decode-step form of :func:`qk_norm_rope` (one new token per sample): returns ``q [B, Hq, D]`` and writes
    the k / v rows into ``kcache / vcache [B, Lcap, Hkv, D]`` at ``kv_len[b]``, which is incremented in place."""
    _need_cuda(qkv, positions, q_norm_w, k_norm_w, rope[0], rope[1], kcache, vcache, kv_len)
    B, W = qkv.shape
    if W != (Hq + 2 * Hkv) * D or positions.dtype != torch.int64 or positions.numel() != B:
        raise ValueError("qkv must be [B, (Hq + 2 Hkv) D] and positions int64 [B]")
    if (kcache.shape != vcache.shape or kcache.dim() != 4 or kcache.shape[0] != B or tuple(kcache.shape[2:]) != (Hkv, D)
            or kcache.dtype != qkv.dtype or not (kcache.is_contiguous() and vcache.is_contiguous())):
        raise ValueError("kcache / vcache must be contiguous [B, Lcap, Hkv, D] of qkv's dtype")
    if kv_len.dtype != torch.int32 or kv_len.numel() != B:
        raise ValueError("kv_len must be int32 [B]")
    q = torch.empty((B, Hq, D), dtype=qkv.dtype, device=qkv.device)
    es, base = qkv.element_size(), qkv.data_ptr()
    check(_lib.load().msa_qk_norm_rope_append(base, base + Hq * D * es, base + (Hq + Hkv) * D * es, W, W, W,
                                              ptr(positions), ptr(q_norm_w), ptr(k_norm_w), eps, ptr(rope[0]),
                                              ptr(rope[1]), rope[0].shape[0], dtype_code(qkv.dtype), B, Hq, Hkv, D,
                                              ptr(q), ptr(kcache), ptr(vcache), kcache.shape[1], ptr(kv_len), _stream()),
          "msa_qk_norm_rope_append")
    return q


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row RMSNorm of ``x [..., H]``; with ``residual`` (same shape) does ``residual += x`` in place first
    and normalises the sum."""
    _need_cuda(x, weight, residual)
    H = x.shape[-1]
    out = torch.empty_like(x)
    check(_lib.load().msa_rmsnorm(ptr(x), ptr(residual), ptr(weight), dtype_code(x.dtype), x.numel() // H, H, eps,
                                  ptr(out), _stream()), "msa_rmsnorm")
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` for a fused ``[..., 2 I]`` projection output (gate first)."""
    _need_cuda(gate_up)
    I = gate_up.shape[-1] // 2
    out = torch.empty(gate_up.shape[:-1] + (I,), dtype=gate_up.dtype, device=gate_up.device)
    check(_lib.load().msa_silu_mul(ptr(gate_up), dtype_code(gate_up.dtype), gate_up.numel() // (2 * I), I, ptr(out),
                                   _stream()), "msa_silu_mul")
    return out


def decode_attn_fused(qkv: torch.Tensor, Hq: int, Hkv: int, D: int, positions: torch.Tensor, q_norm_w, k_norm_w,
                      eps: float, rope: Tuple[torch.Tensor, torch.Tensor], kcache: torch.Tensor, vcache: torch.Tensor,
                      kv_len: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """One decode step from the fused projection output ``qkv [B, (Hq + 2 Hkv) D]`` (bf16) to the attention output
    ``[B, Hq, D]``: q / k norm + rotary, in-place append of the new K / V row to ``kcache / vcache [B, Lcap, Hkv, D]``
    at ``kv_len`` (advanced by one) and attention over ``[cache | new token]``, in two launches."""
    _need_cuda(qkv, positions, q_norm_w, k_norm_w, rope[0], rope[1], kcache, vcache, kv_len)
    B, W = qkv.shape
    if qkv.dtype != torch.bfloat16 or W != (Hq + 2 * Hkv) * D or positions.dtype != torch.int64 or positions.numel() != B:
        raise ValueError("qkv must be bf16 [B, (Hq + 2 Hkv) D] and positions int64 [B]")
    if kcache.shape != vcache.shape or kcache.dim() != 4 or kcache.shape[0] != B or tuple(kcache.shape[2:]) != (Hkv, D) \
            or kcache.dtype != torch.bfloat16 or kv_len.dtype != torch.int32 or kv_len.numel() != B:
        raise ValueError("caches must be bf16 [B, Lcap, Hkv, D] and kv_len int32 [B]")
    Lcap = kcache.shape[1]
    lib = _lib.load()
    need = lib.msa_attn_workspace_bytes(B, Hq, Hkv, D, Lcap)
    ws = _attn_ws.get(qkv.device)
    if ws is None or ws.numel() < need:
        ws = _attn_ws[qkv.device] = torch.empty(need, dtype=torch.uint8, device=qkv.device)
    out = torch.empty((B, Hq, D), dtype=qkv.dtype, device=qkv.device)
    check(lib.msa_decode_attn_fused(ptr(qkv), W, ptr(positions), ptr(q_norm_w), ptr(k_norm_w), eps, ptr(rope[0]),
                                    ptr(rope[1]), rope[0].shape[0], B, Hq, Hkv, D, ptr(kcache), ptr(vcache), Lcap,
                                    ptr(kv_len), D ** -0.5 if scale is None else scale, ptr(out), ptr(ws), ws.numel(),
                                    _stream()), "msa_decode_attn_fused")
    return out


def greedy_sample(logits: torch.Tensor, tok: torch.Tensor, pos: Optional[torch.Tensor] = None,
                  out: Optional[torch.Tensor] = None, col: Optional[torch.Tensor] = None,
                  scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-wise argmax of ``logits [B, V]`` written to ``tok`` (int64, ``B`` elements) with the bookkeeping of a
    greedy decode step done in place: ``pos += 1``; ``out[b, col[b]] = tok[b]``; ``col += 1``.  Returns ``tok``."""
    _need_cuda(logits, tok, pos, out, col)
    B, V = logits.shape
    if not logits.is_contiguous() or tok.dtype != torch.int64 or tok.numel() != B:
        raise ValueError("logits must be contiguous [B, V] and tok int64 with B elements")
    for t in (pos, col):
        if t is not None and (t.dtype != torch.int64 or t.numel() != B or not t.is_contiguous()):
            raise ValueError("pos / col must be contiguous int64 with B elements")
    if (out is None) != (col is None) or (out is not None and (out.dtype != torch.int64 or out.stride(-1) != 1)):
        raise ValueError("out [B, max_new] int64 and col go together")
    if scratch is None:
        scratch = torch.empty(B * 32, dtype=torch.int64, device=logits.device)
    check(_lib.load().msa_greedy_sample(ptr(logits), dtype_code(logits.dtype), B, V, ptr(scratch), ptr(tok), ptr(pos),
                                        ptr(out), out.stride(0) if out is not None else 0, ptr(col),
                                        out.shape[1] if out is not None else 0, _stream()), "msa_greedy_sample")
    return tok


SKINNY_MAX_ROWS = 16
_linear_ws = {}


def interleave_gate_up(gate_w: torch.Tensor, up_w: torch.Tensor) -> torch.Tensor:
    """``[2 I, K]`` weight with alternating 8-row groups of gate and up rows (rows ``16 i .. 16 i + 7`` are gate
    rows ``8 i .. 8 i + 7``, the next 8 the same up rows): the layout the silu-mul epilogue of ``skinny_linear``
    expects (``I`` a multiple of 8)."""
    I, K = gate_w.shape
    if I % 8 or up_w.shape != gate_w.shape:
        raise ValueError("gate / up weights must be [I, K] with I a multiple of 8")
    return torch.stack([gate_w.view(I // 8, 8, K), up_w.view(I // 8, 8, K)], dim=1).reshape(2 * I, K).contiguous()


def skinny_linear(x: torch.Tensor, w: torch.Tensor, residual: Optional[torch.Tensor] = None,
                  silu_mul: bool = False, norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> torch.Tensor:
    """``x @ w.T`` for up to 16 rows of bf16 ``x [M, K]`` against ``w [N, K]``, streaming ``w`` once.
    ``residual [M, N]`` is added to the bf16-rounded product; ``silu_mul`` takes ``w`` from ``interleave_gate_up``
    and returns ``silu(gate) * up`` of width ``N / 2``; ``norm_weight [K]`` applies RMSNorm to ``x`` first."""
    _need_cuda(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or not x.is_contiguous() or not w.is_contiguous():
        raise ValueError("skinny_linear: x [M, K] and w [N, K], both contiguous")
    if residual is not None and silu_mul:
        raise ValueError("skinny_linear: residual and silu_mul are exclusive")
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty((M, N // 2 if silu_mul else N), dtype=x.dtype, device=x.device)
    if residual is not None and (residual.shape != out.shape or not residual.is_contiguous() or residual.dtype != x.dtype):
        raise ValueError("skinny_linear: residual must be a contiguous [M, N] tensor of x's dtype")
    epi = 2 if silu_mul else (1 if residual is not None else 0)
    if norm_weight is not None and (norm_weight.shape != (K,) or norm_weight.dtype != x.dtype or not norm_weight.is_contiguous()):
        raise ValueError("skinny_linear: norm_weight must be a contiguous [K] tensor of x's dtype")
    lib = _lib.load()
    need = lib.msa_skinny_linear_workspace_bytes(M, N, K)
    ws = _linear_ws.get(x.device)
    if need and (ws is None or ws.numel() < need):
        ws = _linear_ws[x.device] = torch.empty(need, dtype=torch.uint8, device=x.device)
    check(lib.msa_skinny_linear_ws(ptr(x), ptr(w), ptr(residual) if residual is not None else None,
                                   ptr(norm_weight) if norm_weight is not None else None, float(eps), epi,
                                   dtype_code(x.dtype), M, N, K, ptr(out), ptr(ws) if need else None,
                                   ws.numel() if need else 0, _stream()), "msa_skinny_linear_ws")
    return out
