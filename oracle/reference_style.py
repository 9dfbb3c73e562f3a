"""Reference-style CPU path of the MSA hot path (test infrastructure only).

Where ``closed_form`` states *what* is computed, this module executes the same
*sequence of torch ops* the reference runs, in the reference's tensor layouts
and dtype (bf16 rounding after every op when given bf16), on whatever device
the inputs live on (CPU in this build).  It is (a) the CPU baseline that
``bench.py`` times next to the HIP path and (b) an independent second reading
of the semantics that the tests compare with ``closed_form``.

Reference layouts used here: activations ``[1, H, T, D]``, pooled bank
``[1, Hkv, C, D]``, 1-based pool ids per chunk, document slot 0 is a dummy.
"""
from __future__ import annotations

from typing import List, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# stage 1: chunk ids + cumsum-difference pooling
# (src/msa/memory_sparse_attention.py:138-190, 467-486)
# --------------------------------------------------------------------------
def stage1_chunk_ids(doc_ids: torch.Tensor, attention_mask: torch.Tensor, P: int):
    """doc_ids/attention_mask ``[1, T]`` -> (token index pairs, global chunk id
    per document token, pooled_doc_ids per chunk), as :138-163."""
    q_len = doc_ids.shape[1]
    top = int(doc_ids.max().item())
    is_doc = (doc_ids > 0) & (attention_mask == 1)
    where = torch.nonzero(is_doc, as_tuple=False)
    gdoc = where[:, 0] * (top + 1) + doc_ids[is_doc]
    _, per_doc = torch.unique_consecutive(gdoc, return_counts=True)
    starts = F.pad(per_doc.cumsum(0), (1, 0))[:-1]
    rank = torch.arange(gdoc.shape[0]) - torch.repeat_interleave(starts, per_doc)
    width = q_len // P + 1
    gchunk = gdoc * width + rank // P
    uniq, _ = torch.unique_consecutive(gchunk, return_counts=True)
    pooled_doc_ids = uniq // width % (top + 1)
    return where, gchunk, pooled_doc_ids


def _cumsum_pool(states: torch.Tensor, lengths: torch.Tensor) -> torch.Tensor:
    """fp32 running sum over tokens, differenced at chunk boundaries, divided
    by the true chunk length, cast back (:475-482)."""
    n, h, d = states.shape
    flat = states.reshape(n, -1).to(torch.float32)
    run = F.pad(torch.cumsum(flat, dim=0), (0, 0, 1, 0))
    edges = F.pad(torch.cumsum(lengths, 0), (1, 0))
    sums = run[edges[1:]] - run[edges[:-1]]
    return (sums.view(-1, h, d) / lengths.view(-1, 1, 1).to(torch.float32)).to(states.dtype)


def stage1_pool(states: torch.Tensor, where: torch.Tensor, gchunk: torch.Tensor,
                normalize: bool = False) -> torch.Tensor:
    """``states [1, H, T, D]`` -> pooled ``[1, H, C, D]`` (:468, :484, :173;
    optional L2 normalise as :192-194)."""
    picked = states[where[:, 0], :, where[:, 1]]            # [n_doc_tokens, H, D]
    _, lengths = torch.unique_consecutive(gchunk, return_counts=True)
    pooled = _cumsum_pool(picked, lengths).transpose(0, 1).unsqueeze(0)
    if normalize:
        pooled = F.normalize(pooled, p=2, dim=-1)
    return pooled


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def rotary(x: torch.Tensor, position_ids: torch.Tensor, theta: float) -> torch.Tensor:
    """Qwen3 rotary in the model dtype: cos/sin computed in fp32 and cast to
    ``x.dtype`` first; ``x [1, H, T, D]``, ``position_ids [1, T]``."""
    D = x.shape[-1]
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.int64).float() / D))
    freqs = position_ids[0].float()[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos().to(x.dtype)[None, None], emb.sin().to(x.dtype)[None, None]
    return x * cos + rotate_half(x) * sin


# --------------------------------------------------------------------------
# stage 2: slices, scoring, reductions, top-k  (src/msa_service.py:644-828, 1095-1100)
# --------------------------------------------------------------------------
def make_slices(doc_num_chunks: List[int], slice_chunk_size: int) -> List[Tuple[int, int]]:
    """Document-aligned chunk ranges of at least ``slice_chunk_size`` chunks; a
    tail under 1024 chunks joins the previous slice (:650-677)."""
    ends, acc, off = [], 0, 0
    for n in doc_num_chunks:
        acc += n
        off += n
        if acc >= slice_chunk_size:
            ends.append(off)
            acc = 0
    if acc > 0:
        if acc < 1024 and ends:
            ends[-1] = off
        else:
            ends.append(off)
    starts = [0] + ends[:-1]
    return list(zip(starts, ends))


def group_queries(query_states: torch.Tensor, query_mask: torch.Tensor, num_kv_groups: int,
                  scaling: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``[B, Hq, S, D]`` -> ``[B, Hkv, G, S, D]`` (pre-scaled unless
    ``scaling <= 0``) and mask ``[B, 1, 1, S, 1]`` (:1095-1100)."""
    B, Hq, S, D = query_states.shape
    if scaling > 0:
        query_states = query_states * scaling
    return (query_states.view(B, Hq // num_kv_groups, num_kv_groups, S, D),
            query_mask.view(B, 1, 1, S, 1))


def stage2_scores_topk(q5: torch.Tensor, m5: torch.Tensor, rk: torch.Tensor, pool_ids: torch.Tensor,
                       doc_num_chunks: List[int], top_k: int, slice_chunk_size: int = 16 * 1024,
                       query_reduce: str = "max", chunk_reduce: str = "max"):
    """The scorer loop: per slice matmul (:730) -> masked_fill (:733) ->
    mean over heads (:745) -> max over tokens (:750) -> amax chunk->slice doc
    (:787-792) -> amax slice doc->bank doc (:816-820); then topk (:826).

    ``rk [1, Hkv, C, D]``; ``pool_ids [C]`` 1-based.  Returns scores ``[B, k]``
    and 1-based local ids ``[B, k]`` with ``k = min(top_k, n_docs + 1)``.
    """
    B = q5.shape[0]
    dtype = q5.dtype
    lowest = torch.finfo(dtype).min
    blocked = ~m5
    n_docs = len(doc_num_chunks)
    table = torch.full((B, n_docs + 1), lowest, dtype=dtype)
    for start, end in make_slices(doc_num_chunks, slice_chunk_size):
        ids = pool_ids[start:end]
        change = torch.diff(ids) != 0
        local0 = F.pad(torch.cumsum(change.int(), 0), (1, 0)).long()          # 0-based doc in slice
        first = torch.cat([torch.tensor([0]), torch.where(change)[0] + 1])
        bank_ids = ids[first]
        kt = rk[:, :, start:end].transpose(-1, -2).unsqueeze(2)              # [1, Hkv, 1, D, Cs]
        s = torch.matmul(q5, kt)                                             # [B, Hkv, G, S, Cs]
        s.masked_fill_(blocked, lowest)
        s = s.flatten(1, 2).mean(dim=1)                                      # [B, S, Cs]
        if query_reduce == "max":
            s = s.max(dim=1).values                                          # [B, Cs]
        elif query_reduce == "mean":                                         # :751-767
            seen = m5.squeeze(2).squeeze(1)                                  # [B, S, 1]
            s = torch.where(seen, s, torch.zeros_like(s)).sum(dim=1) / seen.sum(dim=1).clamp(min=1.0)
        elif query_reduce == "last":                                         # :768-780
            n_seen = m5.reshape(B, -1).sum(dim=1).long()
            at = (n_seen - 1).clamp(min=0).view(B, 1, 1).expand(-1, 1, s.shape[2])
            s = s.gather(1, at).squeeze(1)
        else:
            raise NotImplementedError(f"Unsupported query reduce method: {query_reduce}")
        index = local0.view(1, -1).expand(B, -1)
        per_doc = torch.full((B, bank_ids.numel()), -float("inf"), dtype=dtype)
        if chunk_reduce == "max":
            per_doc.scatter_reduce_(1, index, s, reduce="amax", include_self=True)
        elif chunk_reduce == "mean":                                         # :794-811
            sums = torch.zeros_like(per_doc).scatter_reduce(1, index, s, reduce="sum", include_self=False)
            counts = torch.zeros_like(per_doc).scatter_reduce(1, index, torch.ones_like(s), reduce="sum", include_self=False)
            per_doc = torch.where(counts > 0, sums / counts.clamp(min=1.0), per_doc)
        else:
            raise ValueError(f"Invalid chunk reduction method: {chunk_reduce}")
        table.scatter_reduce_(1, bank_ids.view(1, -1).expand(B, -1), per_doc, reduce="amax", include_self=True)
    return torch.topk(table, k=min(top_k, table.shape[1]), dim=1)


# --------------------------------------------------------------------------
# host gather + per-sample regroup (src/msa_service.py:1203-1314, world size 1)
# --------------------------------------------------------------------------
def gather_regroup(k_bank: torch.Tensor, v_bank: torch.Tensor, doc_offsets: torch.Tensor,
                   doc_lens: torch.Tensor, doc_ids: torch.Tensor, scores: torch.Tensor,
                   local_ids: torch.Tensor):
    """``k_bank/v_bank [1, Hkv, C, D]``; ``doc_offsets/doc_lens/doc_ids`` are the
    ``[n_docs + 1]`` tables with the dummy slot 0 (:209-216).  Invalid picks
    (score <= -1e9) are dropped (:1190-1191); unique sorted ids fetched once
    (:1214), rows located by ``offset + arange`` (:1236-1244), pulled with
    ``index_select`` (:1253) and regrouped per sample by matching global ids
    (:1289-1306).  Returns ``K [Hkv, sum, D]``, ``V``, ``n_sel [B]``."""
    global_ids = doc_ids[local_ids]
    want = local_ids.masked_fill(~(scores > -1e9), -1)
    uniq = want[want != -1].unique()
    lens = doc_lens[uniq]
    total = int(lens.sum())
    base = torch.repeat_interleave(doc_offsets[uniq], lens)
    inner = torch.arange(total) - torch.repeat_interleave(torch.cumsum(lens, 0) - lens, lens)
    rows = base + inner
    k_sel = k_bank.index_select(2, rows).squeeze(0).transpose(0, 1)          # [sum_u, Hkv, D]
    v_sel = v_bank.index_select(2, rows).squeeze(0).transpose(0, 1)
    row_gid = doc_ids[uniq].repeat_interleave(lens)
    hit = (global_ids.unsqueeze(-1) == row_gid.view(1, 1, -1)).any(dim=1)     # [B, sum_u]
    B = hit.shape[0]
    k_out = k_sel.unsqueeze(0).expand(B, -1, -1, -1)[hit].permute(1, 0, 2).contiguous()
    v_out = v_sel.unsqueeze(0).expand(B, -1, -1, -1)[hit].permute(1, 0, 2).contiguous()
    return k_out, v_out, hit.sum(dim=1)


# --------------------------------------------------------------------------
# decode step (src/msa/memory_sparse_attention.py:372-399)
# --------------------------------------------------------------------------
def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    b, h, l, d = x.shape
    return x[:, :, None].expand(b, h, n_rep, l, d).reshape(b, h * n_rep, l, d)


def decode_step(q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, k_new: torch.Tensor,
                v_new: torch.Tensor, kv_lengths: torch.Tensor):
    """``q [B, Hq, 1, D]``; left-padded caches ``[B, Hkv, Lmax, D]`` with
    ``kv_lengths [B]`` valid entries at the right; appends the new token (cat,
    :372-373), builds the left-pad mask (:382-386), expands KV 4x (:389-390) and
    runs SDPA with the bool mask (:392-399).  Returns ``[B, Hq, 1, D]`` and the
    grown caches."""
    B, Hq = q.shape[0], q.shape[1]
    full_k = torch.cat([cache_k, k_new], dim=2)
    full_v = torch.cat([cache_v, v_new], dim=2)
    L = full_k.shape[2]
    visible = torch.arange(L).unsqueeze(0) >= (L - (kv_lengths + 1).unsqueeze(1))
    mask4 = visible[:, None, None, :].expand(-1, Hq, 1, -1)
    n_rep = Hq // full_k.shape[1]
    out = F.scaled_dot_product_attention(q, repeat_kv(full_k, n_rep), repeat_kv(full_v, n_rep),
                                         attn_mask=mask4, dropout_p=0.0, is_causal=False)
    return out, full_k, full_v
