"""fp64 closed-form oracle of the MSA hot path (test infrastructure only).

Layouts are the build's native ones: token-major ``[T, H, D]`` activations,
chunk-major ``[C, H, D]`` pooled tensors, 0-based document indices in bank
order.  Each function cites the reference lines it restates
(paths relative to the reference checkout).
"""
from __future__ import annotations

import math
from typing import List, Sequence, Tuple

import numpy as np
import torch

F64 = torch.float64
NEG_INF = float("-inf")


# --------------------------------------------------------------------------
# chunk table  (src/prefill.py:219-226, src/msa/memory_sparse_attention.py:146-163)
# --------------------------------------------------------------------------
def chunk_table(doc_lens: Sequence[int], P: int, first_token: int = 0):
    """Per-document chunking of a packed block.

    Tokens of document d occupy ``[doc_start[d], doc_start[d]+len_d)``; its
    rank-in-document r maps to chunk ``r // P`` (memory_sparse_attention.py:157)
    so the document has ``ceil(len_d / P)`` chunks (prefill.py:225) and the
    last one may be partial.  ``first_token`` is the number of template tokens
    in front of the first document (prefill.py:204-207); they belong to no
    chunk.

    Returns ``doc_start[n+1]``, ``doc_chunk_off[n+1]``, ``chunk_start[C]``,
    ``chunk_len[C]``, ``chunk_doc[C]`` as int64 numpy arrays.
    """
    doc_start = [first_token]
    doc_chunk_off = [0]
    chunk_start: List[int] = []
    chunk_len: List[int] = []
    chunk_doc: List[int] = []
    for d, n in enumerate(doc_lens):
        n = int(n)
        if n <= 0:
            raise ValueError("documents must have at least one token")
        base = doc_start[-1]
        nch = (n + P - 1) // P
        for j in range(nch):
            chunk_start.append(base + j * P)
            chunk_len.append(min(P, n - j * P))
            chunk_doc.append(d)
        doc_start.append(base + n)
        doc_chunk_off.append(doc_chunk_off[-1] + nch)
    as64 = lambda a: np.asarray(a, dtype=np.int64)
    return as64(doc_start), as64(doc_chunk_off), as64(chunk_start), as64(chunk_len), as64(chunk_doc)


def doc_positions(doc_lens: Sequence[int], first_token: int = 0) -> np.ndarray:
    """Position ids of a packed block: 0..first_token-1 for the template head,
    then restarting at 0 for every document (src/prefill.py:207,223)."""
    pos = list(range(first_token))
    for n in doc_lens:
        pos.extend(range(int(n)))
    return np.asarray(pos, dtype=np.int64)


# --------------------------------------------------------------------------
# RoPE (transformers modeling_qwen3 rotate_half / apply_rotary_pos_emb,
# called at src/msa/memory_sparse_attention.py:132-133)
# --------------------------------------------------------------------------
def rope_tables(max_pos: int, D: int, theta: float, dtype=F64) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin ``[max_pos, D/2]`` with ``inv_freq_i = theta^(-2i/D)``."""
    i = torch.arange(0, D, 2, dtype=F64)
    inv_freq = theta ** (-i / D)
    ang = torch.arange(max_pos, dtype=F64)[:, None] * inv_freq[None, :]
    return ang.cos().to(dtype), ang.sin().to(dtype)


def apply_rope(x: torch.Tensor, pos: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotary on ``x[T, H, D]`` at integer positions ``pos[T]``:
    ``out[:half] = x1*cos - x2*sin``, ``out[half:] = x2*cos + x1*sin``."""
    T, H, D = x.shape
    half = D // 2
    x = x.to(F64)
    i = torch.arange(0, D, 2, dtype=F64)
    inv_freq = theta ** (-i / D)
    ang = pos.to(F64)[:, None] * inv_freq[None, :]  # [T, half]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


# --------------------------------------------------------------------------
# pooling (src/msa/memory_sparse_attention.py:467-486 and :178-190)
# --------------------------------------------------------------------------
def pool_chunks(x: torch.Tensor, chunk_start: np.ndarray, chunk_len: np.ndarray) -> torch.Tensor:
    """Mean of ``x[T, H, D]`` over each chunk's tokens; the partial last chunk
    of a document is divided by its true length (:470-473, :482)."""
    x = x.to(F64)
    C = len(chunk_start)
    out = torch.empty((C,) + tuple(x.shape[1:]), dtype=F64)
    for c in range(C):
        s, n = int(chunk_start[c]), int(chunk_len[c])
        out[c] = x[s : s + n].sum(dim=0) / n
    return out


def l2_normalize(x: torch.Tensor, eps: float = 1e-12) -> torch.Tensor:
    """``x / max(||x||_2, eps)`` over the last dim (F.normalize default,
    src/msa/memory_sparse_attention.py:194, :265)."""
    x = x.to(F64)
    n = x.norm(dim=-1, keepdim=True).clamp_min(eps)
    return x / n


# --------------------------------------------------------------------------
# routing (src/msa_service.py:1095-1100, 703-828)
# --------------------------------------------------------------------------
def chunk_scores(
    q: torch.Tensor,        # [B, S, Hq, D]
    qmask: torch.Tensor,    # [B, S] bool, True = scored token
    kr: torch.Tensor,       # [C, Hkv, D]
    mode: str = "cosine",   # "cosine": q normalised here, kr assumed normalised, scale 1
    scale: float | None = None,
    chunk_block: int = 4096,
    query_reduce: str = "max",
) -> torch.Tensor:
    """``s[b,c] = max_{t valid} (1/Hq) sum_h q'[b,t,h] . kr[c, h // G] * scale``.

    Restates matmul (:730) -> mask (:733) -> mean over the Hq heads (:745) ->
    max over tokens (:750).  A query with no valid token scores -inf.
    ``query_reduce`` "mean": sum over the valid tokens / max(their number, 1)
    (:751-767); "last": the token at position (number of valid tokens - 1), -inf
    if that position is not a valid token (:768-780, where a masked position
    carries the dtype's lowest value).
    """
    B, S, Hq, D = q.shape
    C, Hkv, _ = kr.shape
    G = Hq // Hkv
    q = q.to(F64)
    if mode == "cosine":
        q = l2_normalize(q)
        sc = 1.0
    elif mode == "scaled_dot":
        sc = D ** -0.5 if scale is None else scale
    else:
        raise ValueError(mode)
    kr = kr.to(F64)
    qg = q.view(B, S, Hkv, G, D)
    out = torch.full((B, C), NEG_INF, dtype=F64)
    for c0 in range(0, C, chunk_block):
        kb = kr[c0 : c0 + chunk_block]                      # [c, Hkv, D]
        # per-head dots then mean over all Hq heads
        s = torch.einsum("bsgjd,cgd->bsc", qg, kb) * (sc / Hq)
        if query_reduce == "max":
            s = s.masked_fill(~qmask[:, :, None], NEG_INF)
            red = s.max(dim=1).values
        elif query_reduce == "mean":
            n = qmask.sum(dim=1).clamp(min=1).to(F64)
            red = torch.where(qmask[:, :, None], s, torch.zeros_like(s)).sum(dim=1) / n[:, None]
            red = torch.where((qmask.sum(dim=1) > 0)[:, None], red, torch.full_like(red, NEG_INF))
        elif query_reduce == "last":
            n = qmask.sum(dim=1)
            last = (n - 1).clamp(min=0)
            red = s[torch.arange(B), last]
            ok = qmask[torch.arange(B), last] & (n > 0)
            red = torch.where(ok[:, None], red, torch.full_like(red, NEG_INF))
        else:
            raise NotImplementedError(f"Unsupported query reduce method: {query_reduce}")
        out[:, c0 : c0 + chunk_block] = red
    return out


def doc_scores(cs: torch.Tensor, doc_chunk_off: np.ndarray, chunk_reduce: str = "max") -> torch.Tensor:
    """Max over each document's chunks (scatter_reduce amax, :789-792, :817-820); ``chunk_reduce``
    "mean": their mean (sum / count, :794-811)."""
    B = cs.shape[0]
    n = len(doc_chunk_off) - 1
    out = torch.empty((B, n), dtype=cs.dtype)
    for d in range(n):
        part = cs[:, int(doc_chunk_off[d]) : int(doc_chunk_off[d + 1])]
        if chunk_reduce == "max":
            out[:, d] = part.max(dim=1).values
        elif chunk_reduce == "mean":
            out[:, d] = part.sum(dim=1) / part.shape[1]
        else:
            raise ValueError(f"Invalid chunk reduction method: {chunk_reduce}")
    return out


def topk_docs(ds: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Full-sort top-k (torch.topk at :826).  Ties broken by lower document
    index, which torch.topk leaves unspecified.  If fewer than k documents
    exist the tail is (-inf, -1)."""
    B, n = ds.shape
    scores = torch.full((B, k), NEG_INF, dtype=ds.dtype)
    idx = torch.full((B, k), -1, dtype=torch.int64)
    for b in range(B):
        row = ds[b].tolist()
        order = sorted(range(n), key=lambda d: (-row[d], d))[:k]
        for j, d in enumerate(order):
            scores[b, j] = row[d]
            idx[b, j] = d
    return scores, idx


def topk_acceptable(ds_ref: torch.Tensor, got_idx: torch.Tensor, k: int, gap: float = 1e-3) -> List[str]:
    """The acceptance rule for top-k parity: every document whose reference
    score exceeds the k-th best by more than ``gap`` must be returned, and every
    returned document must score at least (k-th best - gap).  Returns a list of
    violations (empty = pass)."""
    errs = []
    B, n = ds_ref.shape
    kk = min(k, n)
    for b in range(B):
        row = ds_ref[b]
        srt = torch.sort(row, descending=True).values
        s_k = float(srt[kk - 1])
        got = [int(x) for x in got_idx[b].tolist() if int(x) >= 0]
        if len(set(got)) != len(got):
            errs.append(f"b={b}: duplicate docs {got}")
        if len(got) != kk:
            errs.append(f"b={b}: returned {len(got)} docs, want {kk}")
        must = set(torch.nonzero(row > s_k + gap).flatten().tolist())
        missing = must - set(got)
        if missing:
            errs.append(f"b={b}: missing clear winners {sorted(missing)}")
        for d in got:
            if float(row[d]) < s_k - gap:
                errs.append(f"b={b}: doc {d} score {float(row[d]):.6f} below boundary {s_k:.6f}")
    return errs


# --------------------------------------------------------------------------
# gather / regroup (src/msa_service.py:1203-1314)
# --------------------------------------------------------------------------
def gather_selected(
    k_bank: torch.Tensor,      # [C, Hkv, D]
    v_bank: torch.Tensor,
    doc_chunk_off: np.ndarray,  # [n_docs+1]
    sel_docs: torch.Tensor,     # [B, k] 0-based, -1 = none
):
    """Rows of the selected documents' chunks, per sample, documents in
    ascending bank order (the reference fetches ``unique()``-sorted local ids,
    :1214, and regroups in fetched order, :1289-1303), each document once per
    sample.  Returns ``K[sum, Hkv, D]``, ``V``, ``cu_sel[B+1]`` and the chunk
    row indices used."""
    rows: List[int] = []
    cu = [0]
    for b in range(sel_docs.shape[0]):
        docs = sorted({int(d) for d in sel_docs[b].tolist() if int(d) >= 0})
        for d in docs:
            rows.extend(range(int(doc_chunk_off[d]), int(doc_chunk_off[d + 1])))
        cu.append(len(rows))
    ridx = torch.as_tensor(rows, dtype=torch.int64)
    return k_bank[ridx], v_bank[ridx], np.asarray(cu, dtype=np.int64), ridx


# --------------------------------------------------------------------------
# context assembly + positions
# (src/msa/memory_sparse_attention.py:282-329, src/msa_service.py:1823-1836)
# --------------------------------------------------------------------------
def assemble_context(prefix, mem, cu_sel, local, cu_local):
    """Ragged ``[prefix | selected chunks of sample b | local tokens of b]``
    for every sample.  All inputs are ``[n, H, D]``; returns the concatenation
    and ``cu_kv[B+1]``."""
    B = len(cu_sel) - 1
    parts = []
    cu = [0]
    for b in range(B):
        parts.append(prefix)
        parts.append(mem[int(cu_sel[b]) : int(cu_sel[b + 1])])
        parts.append(local[int(cu_local[b]) : int(cu_local[b + 1])])
        cu.append(cu[-1] + prefix.shape[0] + int(cu_sel[b + 1] - cu_sel[b]) + int(cu_local[b + 1] - cu_local[b]))
    return torch.cat(parts, dim=0), np.asarray(cu, dtype=np.int64)


def query_positions(n_tokens: int, top_k: int, template_len: int = 3, left_pad: int = 0) -> np.ndarray:
    """Global RoPE positions of a query: ``template_len + top_k + i``; left
    padding repeats the first position (src/msa_service.py:1823-1864)."""
    first = template_len + top_k
    return np.asarray([first] * left_pad + [first + i for i in range(n_tokens)], dtype=np.int64)


# --------------------------------------------------------------------------
# attention (src/msa/memory_sparse_attention.py:334-339 and :389-399)
# --------------------------------------------------------------------------
def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None = None,
              causal: bool = True) -> torch.Tensor:
    """Naive softmax attention with GQA.  ``q[Sq, Hq, D]``, ``k, v[L, Hkv, D]``.
    With ``causal`` the mask is bottom-right aligned: query row i sees keys
    ``0 .. L - Sq + i`` (flash-attn >= 2.1 semantics for Sq != L; for Sq == 1
    this is plain decode over all L keys)."""
    Sq, Hq, D = q.shape
    L, Hkv, _ = k.shape
    G = Hq // Hkv
    sc = D ** -0.5 if scale is None else scale
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    out = torch.empty((Sq, Hq, D), dtype=F64)
    for h in range(Hq):
        g = h // G
        s = (q[:, h] @ k[:, g].T) * sc                    # [Sq, L]
        if causal:
            i = torch.arange(Sq)[:, None]
            j = torch.arange(L)[None, :]
            s = s.masked_fill(j > (L - Sq + i), NEG_INF)
        p = torch.softmax(s, dim=-1)
        out[:, h] = p @ v[:, g]
    return out


def attention_ragged(q, cu_q, k, v, cu_kv, scale=None, causal=True):
    """Per-sample :func:`attention` over ragged batches."""
    outs = []
    for b in range(len(cu_q) - 1):
        outs.append(attention(q[int(cu_q[b]) : int(cu_q[b + 1])],
                              k[int(cu_kv[b]) : int(cu_kv[b + 1])],
                              v[int(cu_kv[b]) : int(cu_kv[b + 1])], scale, causal))
    return torch.cat(outs, dim=0)


def rel_err(x: torch.Tensor, ref: torch.Tensor, eps: float = 1e-30) -> float:
    """``||x - ref||_inf / max(||ref||_inf, eps)`` — the tolerance metric used
    by every floating-point parity gate."""
    x, ref = x.to(F64), ref.to(F64)
    return float((x - ref).abs().max() / max(float(ref.abs().max()), eps))
