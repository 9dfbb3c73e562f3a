"""``MemorySparseAttention`` with the reference layer's interface
(src/msa/memory_sparse_attention.py:20-405): same constructor arguments, parameter names,
``set_memory_client``, ``forward`` signature and stage dispatch through
``past_key_value.cache_kwargs[layer_idx]["stage"]``.

The dense projections, RMSNorm and rotary are PyTorch-ROCm (the backbone is not part of the hot
path); chunk pooling, routing, gather, context assembly and attention run in the HIP library.
Inference only: the training branch of the reference (:407-465, 488-852) is not provided.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .config import MSAConfig


class RMSNorm(nn.Module):
    """Qwen3RMSNorm: fp32 statistics, weight applied in the input dtype."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.variance_epsilon = eps

    def forward(self, x):
        dt = x.dtype
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * xf.to(dt)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary_bshd(x, cos, sin):
    """Half-split rotary on ``x [B, S, H, D]`` with ``cos / sin [B, S, D]`` (transformers
    ``apply_rotary_pos_emb`` with the head axis at 2)."""
    return x * cos[:, :, None, :] + rotate_half(x) * sin[:, :, None, :]


def rotary_embedding(position_ids: torch.Tensor, head_dim: int, theta: float, dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(cos, sin) [B, S, D]`` as Qwen3RotaryEmbedding computes them (fp32, then cast)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64, device=position_ids.device).float() / head_dim))
    freqs = position_ids[..., None].float() * inv_freq
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


_ROPE_TABLES = {}


class MemorySparseAttention(nn.Module):
    def __init__(self, config: MSAConfig, layer_idx: int):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = config.head_dim
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads
        self.scaling = self.head_dim ** -0.5
        self.attention_dropout = config.attention_dropout
        hs, Hq, Hkv, D = config.hidden_size, config.num_attention_heads, config.num_key_value_heads, self.head_dim
        self.q_proj = nn.Linear(hs, Hq * D, bias=config.attention_bias)
        self.k_proj = nn.Linear(hs, Hkv * D, bias=config.attention_bias)
        self.v_proj = nn.Linear(hs, Hkv * D, bias=config.attention_bias)
        self.o_proj = nn.Linear(Hq * D, hs, bias=config.attention_bias)
        self.q_norm = RMSNorm(D, eps=config.rms_norm_eps)
        self.k_norm = RMSNorm(D, eps=config.rms_norm_eps)

        mc = config.msa_config
        self.top_k_docs = mc.top_k_docs
        self.pooling_kernel_size = mc.pooling_kernel_size
        ridx = mc.router_layer_idx
        self.router_layer_idx = list(range(config.num_hidden_layers)) if ridx == "all" else [int(i) for i in ridx.split(",")]
        self.is_router_layer = layer_idx in self.router_layer_idx
        self.head_reduce_method, self.query_reduce_method = mc.head_reduce_method, mc.query_reduce_method
        self.chunk_reduce_method, self.decouple_pooling_mode = mc.chunk_reduce_method, mc.decouple_pooling_mode
        self.aux_loss_method, self.decouple_router = mc.aux_loss_method, mc.decouple_router
        if self.is_router_layer and self.decouple_router:
            self.router_k_proj = nn.Sequential(nn.Linear(hs, Hkv * D, bias=False))
            self.router_q_proj = nn.Sequential(nn.Linear(hs, Hq * D, bias=False))
        self.num_kv_heads = Hkv
        self.template_prefix_kcache = None
        self.template_prefix_vcache = None
        self.memory_client = None
        self.decode_reserve = 512      # rows kept free behind the stage-2 context for in-place decode appends
        self._qkv_weight = None        # q / k / v weights concatenated on first use of the fused projection

    def set_memory_client(self, memory_client):
        self.memory_client = memory_client

    def forward(self, hidden_states: torch.Tensor, doc_ids: torch.LongTensor, attention_mask: Optional[torch.Tensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, past_key_value=None, **kwargs):
        if self.training:
            raise NotImplementedError("the training path of the reference layer is not part of this build")
        if past_key_value is None:
            raise Exception("error!")          # same failure as the reference without a cache (:97)
        return self.forward_with_kvcache_for_batch_parrallel(hidden_states, doc_ids, attention_mask,
                                                             position_embeddings, past_key_value, **kwargs)

    # ------------------------------------------------------------------------------------------
    def _project(self, hidden_states, position_embeddings):
        B, S, _ = hidden_states.shape
        D = self.head_dim
        q = self.q_norm(self.q_proj(hidden_states).view(B, S, -1, D))
        k = self.k_norm(self.k_proj(hidden_states).view(B, S, -1, D))
        v = self.v_proj(hidden_states).view(B, S, -1, D)
        cos, sin = position_embeddings
        return apply_rotary_bshd(q, cos, sin).contiguous(), apply_rotary_bshd(k, cos, sin).contiguous(), v.contiguous()

    def _project_fused(self, hidden_states, position_ids, router: Optional[str] = None):
        """Same result as :meth:`_project` from integer positions, plus the router projection the stage needs
        (``router`` = "k": router_k_proj, "q": router_q_proj): ``(q, k, v, r)`` with ``r`` ``None`` when not asked for.
        bf16: one native GEMM over the concatenated weights with the per-head RMSNorm + rotary in its epilogue
        (``ops.qkv_proj``); fp32: one GEMM over q / k / v, the norm + rotary kernel, and the router module."""
        B, S, _ = hidden_states.shape
        Hq, Hkv, D = self.config.num_attention_heads, self.num_kv_heads, self.head_dim
        tables = self._rope_tables(hidden_states.device)
        x = hidden_states.reshape(B * S, -1)
        pos = position_ids.reshape(-1).contiguous()
        has_router = self.is_router_layer and self.decouple_router
        if (hidden_states.dtype == torch.bfloat16 and D == 128 and x.shape[1] % 64 == 0
                and self.q_norm.weight.dtype == torch.bfloat16 and self.k_norm.weight.dtype == torch.bfloat16
                and self.q_proj.weight.dtype == torch.bfloat16):
            w_all = self._all_weight(hidden_states.device)
            lo = Hkv * D if has_router else 0                   # rows of router_k_proj in front of q | k | v
            if has_router and router == "k":
                q, k, v, r = ops.qkv_proj(x.contiguous(), w_all[:lo + (Hq + 2 * Hkv) * D], Hq, Hkv, pos, self.q_norm.weight,
                                          self.k_norm.weight, self.q_norm.variance_epsilon, tables, router_front=Hkv)
            elif has_router and router == "q":
                q, k, v, r = ops.qkv_proj(x.contiguous(), w_all[lo:], Hq, Hkv, pos, self.q_norm.weight, self.k_norm.weight,
                                          self.q_norm.variance_epsilon, tables, router_back=Hq)
            else:
                q, k, v, r = ops.qkv_proj(x.contiguous(), w_all[lo:lo + (Hq + 2 * Hkv) * D], Hq, Hkv, pos, self.q_norm.weight,
                                          self.k_norm.weight, self.q_norm.variance_epsilon, tables)
            r = None if r is None else r.view(B, S, -1, D)
            return q.view(B, S, Hq, D), k.view(B, S, Hkv, D), v.view(B, S, Hkv, D), r
        qkv = F.linear(x, self._fused_weight(hidden_states.device))
        q, k, v = ops.qk_norm_rope(qkv, Hq, Hkv, D, pos, self.q_norm.weight, self.k_norm.weight,
                                   self.q_norm.variance_epsilon, tables)
        r = None
        if has_router and router == "k":
            r = self.router_k_proj(hidden_states).view(B, S, Hkv, D)
        elif has_router and router == "q":
            r = self.router_q_proj(hidden_states).view(B, S, Hq, D)
        return q.view(B, S, Hq, D), k.view(B, S, Hkv, D), v.view(B, S, Hkv, D), r

    def _all_weight(self, device):
        """[router_k_proj | q_proj | k_proj | v_proj | router_q_proj] rows in one matrix (q | k | v alone on layers
        without a decoupled router): stage 1 multiplies by the first four, stage 2 by the last four, a decode step by
        the middle three, all as contiguous row ranges of this one copy."""
        parts = [self.q_proj.weight, self.k_proj.weight, self.v_proj.weight]
        if self.is_router_layer and self.decouple_router:
            parts = [self.router_k_proj[0].weight] + parts + [self.router_q_proj[0].weight]
        # the copy follows its sources: loading a state dict, .to(dtype / device) or an in-place update of any of
        # them changes the storage pointer, the dtype or the version counter, and the copy is rebuilt
        key = tuple((w.data_ptr(), w._version, w.dtype, w.device) for w in parts) + (device,)
        if self._qkv_weight is None or self._qkv_weight_key != key:
            self._qkv_weight = torch.cat([w.detach().to(device) for w in parts], dim=0).contiguous()
            self._qkv_weight_key = key
        return self._qkv_weight

    def _fused_weight(self, device):
        w = self._all_weight(device)
        Hq, Hkv, D = self.config.num_attention_heads, self.num_kv_heads, self.head_dim
        lo = Hkv * D if (self.is_router_layer and self.decouple_router) else 0
        return w[lo:lo + (Hq + 2 * Hkv) * D]

    def _rope_tables(self, device):
        # one row per position the configuration allows; positions beyond it are refused where they are made
        # (check_positions), not clamped in the kernels
        rows = int(self.config.max_position_embeddings)
        key = (device, rows, float(self.config.rope_theta))
        if key not in _ROPE_TABLES:
            _ROPE_TABLES[key] = ops.rope_tables(rows, self.head_dim, self.config.rope_theta, device=device)
        return _ROPE_TABLES[key]

    def check_positions(self, last_position: int) -> None:
        """Raises when a position would fall outside the rotary tables (the reference computes cos / sin for any
        position; here they are tabulated up to ``max_position_embeddings``)."""
        rows = int(self.config.max_position_embeddings)
        if last_position >= rows:
            raise ValueError(f"position {last_position} is beyond max_position_embeddings = {rows}")

    @staticmethod
    def _claim_rows(ck: dict, n_new: int) -> None:
        """Books ``n_new`` more rows per sample against the free rows behind the stage-2 context; raises instead
        of letting the append kernels drop rows (the reference grows its cache without limit, :372-373)."""
        left = ck.get("rows_free")
        if left is None:
            return
        if n_new > left:
            raise RuntimeError(f"compact KV cache is full: {n_new} new rows per sample, {left} free "
                               f"(raise decode_reserve before stage 2)")
        ck["rows_free"] = left - n_new

    def decode_rows(self, residual, norm_weight, eps, position_ids, cache):
        """The decode step of :meth:`_generate` on the residual stream ``[B, hidden]`` (B <= 16, bf16) with the
        layer's dense parts on the weight-streaming kernel: RMSNorm folded into the fused q/k/v projection, and
        the residual add folded into the output projection.  Returns the new residual stream."""
        B = residual.shape[0]
        Hq, Hkv, D = self.config.num_attention_heads, self.num_kv_heads, self.head_dim
        ck = cache.cache_kwargs[self.layer_idx]
        if "compacked_key_cache" not in ck:
            raise ValueError("compact KV cache not found: did prefill stage 2 run?")
        self._claim_rows(ck, 1)
        qkv = ops.skinny_linear(residual, self._fused_weight(residual.device), norm_weight=norm_weight, eps=eps)
        kc, vc, kv_len = ck["compacked_key_cache"], ck["compacked_value_cache"], ck["kv_lengths"]
        if Hq // Hkv in (4, 8) and kc.dim() == 4 and kc.is_contiguous() and vc.is_contiguous():
            # q / k norm + rotary + cache append folded into the attention launch
            out = ops.decode_attn_fused(qkv, Hq, Hkv, D, position_ids.reshape(-1), self.q_norm.weight, self.k_norm.weight,
                                        self.q_norm.variance_epsilon, self._rope_tables(residual.device), kc, vc, kv_len,
                                        scale=self.scaling)
        else:
            q = ops.qk_norm_rope_append(qkv, Hq, Hkv, D, position_ids.reshape(-1), self.q_norm.weight, self.k_norm.weight,
                                        self.q_norm.variance_epsilon, self._rope_tables(residual.device), kc, vc, kv_len)
            out = ops.sparse_attn(q.view(B, Hq, D), kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), ck["kv_offsets"], kv_len,
                                  ck["kv_capacity"], scale=self.scaling, causal=True)
        return ops.skinny_linear(out.view(B, Hq * D), self.o_proj.weight, residual=residual)

    def forward_with_kvcache_for_batch_parrallel(self, hidden_states, doc_ids, attention_mask=None,
                                                 position_embeddings=None, past_key_value=None, position_ids=None,
                                                 **kwargs):
        stage = past_key_value.cache_kwargs[self.layer_idx]["stage"]
        r = None
        if position_ids is not None and hidden_states.is_cuda and self.q_proj.bias is None:
            router = {"prefill_stage1": "k", "prefill_stage2": "q"}.get(stage)
            q, k, v, r = self._project_fused(hidden_states, position_ids, router)   # [B, S, H, D] token-major
        else:
            q, k, v = self._project(hidden_states, position_embeddings)
        if stage == "prefill_stage1":
            return self._stage1(hidden_states, doc_ids, attention_mask, q, k, v, past_key_value, r)
        if stage == "prefill_stage2":
            return self._stage2(hidden_states, doc_ids, attention_mask, q, k, v, past_key_value, r)
        return self._generate(hidden_states, q, k, v, past_key_value, attention_mask)

    # ------------------------------------------------------------------------------------------ stage 1
    def _stage1(self, hidden_states, doc_ids, attention_mask, q, k, v, cache, router_k=None):
        """Encodes one packed block ``[template | doc 1 | doc 2 | ...]``: document-wise causal
        attention, and on router layers chunk-mean pooling of K (rotated), V and K_r
        (src/msa/memory_sparse_attention.py:137-243)."""
        B, T, _ = hidden_states.shape
        if B != 1:
            raise ValueError("stage 1 takes one packed block at a time (batch size 1)")
        Hq, Hkv, D, P = self.config.num_attention_heads, self.num_kv_heads, self.head_dim, self.pooling_kernel_size
        ids = doc_ids[0]
        n_template = int((ids == -2).sum())
        vals, counts = torch.unique_consecutive(ids[n_template:], return_counts=True)
        doc_lens = counts.tolist()
        if (vals <= 0).any() or (attention_mask is not None and int(attention_mask.sum()) != T):
            raise ValueError("stage 1 expects [template (-2) | documents (ids > 0)] with no padding")
        kwargs = {"template_prefix_kcache": k[:, :n_template].transpose(1, 2),          # [1, Hkv, n, D] views
                  "template_prefix_vcache": v[:, :n_template].transpose(1, 2)}
        if self.is_router_layer:
            table = ops.chunk_table(doc_lens, P, first_token=n_template, device=hidden_states.device)
            if not self.decouple_router:
                rk = None
            elif router_k is not None:                       # came out of the fused projection
                rk = router_k.reshape(T, Hkv, D)
            else:
                rk = self.router_k_proj(hidden_states).view(T, Hkv, D).contiguous()
            normalize = self.aux_loss_method == "INFONCE"
            pk, pv, prk = ops.pool_chunks(k[0], v[0], rk if rk is not None else k[0], table, normalize_kr=normalize)
            cache.update(pk.transpose(0, 1).unsqueeze(0), pv.transpose(0, 1).unsqueeze(0), self.layer_idx)
            if rk is not None or normalize:
                cache.update_router_kcache(prk.transpose(0, 1).unsqueeze(0), self.layer_idx)
            kwargs.update({"doc_id_bias": T, "pooled_doc_ids": table.chunk_doc.long() + 1,
                           "prefill_stage1_kvcache_size": cache.get_seq_length(self.layer_idx)})
        cache.record_kwargs(self.layer_idx, kwargs)

        # every document (and the template head) attends causally within itself
        seg = ([n_template] if n_template else []) + doc_lens
        cu = torch.tensor([0] + seg, dtype=torch.int64).cumsum(0)
        dev = hidden_states.device
        out = ops.sparse_attn(q[0], k[0], v[0], cu[:-1].to(dev), torch.tensor(seg, dtype=torch.int32, device=dev),
                              max(seg), cu_q=cu.to(torch.int32).to(dev), max_sq=max(seg), scale=self.scaling, causal=True)
        return self.o_proj(out.view(1, T, Hq * D)), None

    # ------------------------------------------------------------------------------------------ stage 2
    def _stage2(self, hidden_states, doc_ids, attention_mask, q, k, v, cache, router_q=None):
        """Routes the query batch, pulls the winners' pooled K / V, lays out
        ``[template prefix | selected chunks | query tokens]`` per sample and attends causally
        (src/msa/memory_sparse_attention.py:245-359)."""
        B, S, _ = hidden_states.shape
        dev, dtype = hidden_states.device, hidden_states.dtype
        Hq, Hkv, D = self.config.num_attention_heads, self.num_kv_heads, self.head_dim
        ck = cache.cache_kwargs[self.layer_idx]
        if self.memory_client is not None:
            if self.template_prefix_kcache is None:
                pk, pv = self.memory_client.get_template_prefix_kvcaches(self.layer_idx)
                self.template_prefix_kcache, self.template_prefix_vcache = pk.to(dev), pv.to(dev)
            pk, pv = self.template_prefix_kcache, self.template_prefix_vcache
        else:
            pk, pv = ck["template_prefix_kcache"].to(dev), ck["template_prefix_vcache"].to(dev)
        prefix_k = pk[0].transpose(0, 1).contiguous()                     # [n_prefix, Hkv, D]
        prefix_v = pv[0].transpose(0, 1).contiguous()
        n_prefix = prefix_k.shape[0]

        valid = attention_mask == 1
        n_q = valid.sum(dim=1)
        n_q_host = cache.meta.get("q_lens_host")              # the model computes it once per forward
        if n_q_host is None or len(n_q_host) != B:
            n_q_host = n_q.tolist()
        mem_k = mem_v = cu_sel = None
        max_sel = 0
        if self.is_router_layer:
            if not self.decouple_router:
                rq = q
            elif router_q is not None:                       # came out of the fused projection
                rq = router_q
            else:
                rq = self.router_q_proj(hidden_states).view(B, S, Hq, D)
            query_mask = (doc_ids == 0) & valid
            fused = self.aux_loss_method == "INFONCE"
            if hasattr(self.memory_client, "doc_query_device"):
                # native client: routing, gather plan and host->device gather are enqueued without any host sync
                mem_k, mem_v, cu_sel, scores, gids = self.memory_client.doc_query_device(rq.contiguous(), query_mask,
                                                                                         self.layer_idx, fused)
                # the same k the client sized its gather buffers from (its own top-k setting, not this layer's)
                max_sel = gids.shape[1] * self.memory_client.bank.max_doc_chunks
            else:
                mem_k, mem_v, scores, n_sel, gids = self.memory_client.doc_query(rq.transpose(1, 2), query_mask,
                                                                                 self.layer_idx)
                mem_k, mem_v = mem_k.permute(1, 0, 2).contiguous(), mem_v.permute(1, 0, 2).contiguous()
                cu_sel = F.pad(n_sel.cumsum(0), (1, 0)).to(torch.int32)
                max_sel = int(n_sel.max())
            if cache.meta.get("require_recall_topk", False):
                ck["recall_topk"] = [{"topk_doc_ids": gids[i].tolist(), "score": scores[i].float().tolist()} for i in range(B)]
        dense = min(n_q_host) == S                                        # no padding anywhere: the ragged rows are views
        if dense:
            local_k, local_v, q_rows = k.reshape(B * S, Hkv, D), v.reshape(B * S, Hkv, D), q.reshape(B * S, Hq, D)
        else:
            local_k, local_v, q_rows = k[valid], v[valid], q[valid]       # ragged [sum S_b, H, D]
        cu_local = F.pad(n_q.cumsum(0), (1, 0)).to(torch.int32)
        max_kv = n_prefix + max_sel + max(n_q_host)                       # upper bound of any sample's context rows
        Lcap = max_kv + self.decode_reserve
        kc, vc, kv_len = ops.assemble_context(prefix_k, prefix_v, mem_k, mem_v, cu_sel, local_k, local_v, cu_local, B, Lcap)
        kv_off = torch.arange(B, dtype=torch.int64, device=dev) * Lcap
        out_rows = ops.sparse_attn(q_rows, kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), kv_off, kv_len, max_kv,
                                   cu_q=cu_local, max_sq=max(n_q_host), scale=self.scaling, causal=True)
        if dense:
            attn = out_rows.view(B, S, Hq * D)
        else:
            attn = torch.zeros((B, S, Hq * D), device=dev, dtype=dtype)
            attn[valid] = out_rows.view(-1, Hq * D)
        ck.update({"compacked_key_cache": kc, "compacked_value_cache": vc, "kv_lengths": kv_len, "kv_offsets": kv_off,
                   "kv_capacity": Lcap, "rows_free": self.decode_reserve})
        cache.record_kwargs(self.layer_idx, ck)
        return self.o_proj(attn), None

    # ------------------------------------------------------------------------------------------ decode
    def _generate(self, hidden_states, q, k, v, cache, attention_mask=None):
        """One decode step over the compact cache, appended in place
        (src/msa/memory_sparse_attention.py:361-405).  With more than one token per sample (the source-context
        block the Memory-Interleave loop injects between rounds, src/msa/generate.py:190-259, left-padded) the
        valid tokens are appended as a ragged block and attend causally over ``[cache | block so far]``."""
        B, S, _ = hidden_states.shape
        ck = cache.cache_kwargs[self.layer_idx]
        if "compacked_key_cache" not in ck:
            raise ValueError("compact KV cache not found: did prefill stage 2 run?")
        kc, vc, kv_len = ck["compacked_key_cache"], ck["compacked_value_cache"], ck["kv_lengths"]
        Hq, Hkv, D = self.config.num_attention_heads, self.num_kv_heads, self.head_dim
        # qa_mode (:375-380): the step's attention mask decides which samples gain a key, so a sample that is
        # masked at this step (finished, or padding of an injected block) appends nothing.  The per-sample lengths
        # play the part of the reference's growing [B, L] mask; a masked sample's output row is zero here (the
        # reference computes a value nobody reads).
        masked_step = S == 1 and attention_mask is not None and bool(cache.meta.get("qa_mode", False))
        if S != 1 or masked_step:
            valid = attention_mask == 1 if attention_mask is not None else torch.ones((B, S), dtype=torch.bool, device=q.device)
            n_new = valid.sum(dim=1)
            n_host = None if masked_step else cache.meta.get("q_lens_host")
            if n_host is None or len(n_host) != B:
                n_host = n_new.tolist()
            if max(n_host) == 0:
                return self.o_proj(torch.zeros((B, S, Hq * D), device=q.device, dtype=q.dtype)), None
            cu_new = F.pad(n_new.cumsum(0), (1, 0)).to(torch.int32)
            self._claim_rows(ck, max(n_host))
            ops.cache_append_rows(k[valid], v[valid], cu_new, max(n_host), kc, vc, kv_len)
            rows = ops.sparse_attn(q[valid], kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), ck["kv_offsets"], kv_len,
                                   ck["kv_capacity"], cu_q=cu_new, max_sq=max(n_host), scale=self.scaling, causal=True)
            attn = torch.zeros((B, S, Hq * D), device=q.device, dtype=q.dtype)
            attn[valid] = rows.view(-1, Hq * D)
            return self.o_proj(attn), None
        self._claim_rows(ck, 1)
        ops.cache_append(k[:, 0].contiguous(), v[:, 0].contiguous(), kc, vc, kv_len)
        out = ops.sparse_attn(q[:, 0].contiguous(), kc.view(-1, Hkv, D), vc.view(-1, Hkv, D), ck["kv_offsets"], kv_len,
                              ck["kv_capacity"], scale=self.scaling, causal=True)
        return self.o_proj(out.view(B, 1, -1)), None
