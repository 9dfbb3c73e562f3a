"""Qwen3-shaped decoder hosting :class:`MemorySparseAttention` in every layer, with random-init
weights, for the end-to-end sparse-generation workload (no checkpoint can be fetched here).  The
dense parts (embedding, MLP, norms, LM head) are plain PyTorch-ROCm; they are the host model around
the hot path, mirroring src/msa/model.py:51-255 without losses or training code."""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .cache import CustomDynamicCache, create_cache
from .config import MSAConfig
from .memory_sparse_attention import MemorySparseAttention, RMSNorm, rotary_embedding
from .prefill import query_position_ids, source_block_position_ids


class MLP(nn.Module):
    def __init__(self, config: MSAConfig):
        super().__init__()
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)

        self._gate_up_weight = None
        self._gate_up_interleaved = None

    def decode_rows(self, residual, norm_weight, eps):
        """``residual + down(silu(gate(n)) * up(n))`` with ``n = rmsnorm(residual)`` for up to 16 bf16 rows:
        two weight-streaming launches, the norm folded into the first, silu-mul into its epilogue, the residual
        add into the second."""
        if self._gate_up_interleaved is None or self._gate_up_interleaved.device != residual.device:
            self._gate_up_interleaved = ops.interleave_gate_up(self.gate_proj.weight, self.up_proj.weight)
        act = ops.skinny_linear(residual, self._gate_up_interleaved, silu_mul=True, norm_weight=norm_weight, eps=eps)
        return ops.skinny_linear(act, self.down_proj.weight, residual=residual)

    def forward(self, x):
        if x.is_cuda and x.dtype in (torch.bfloat16, torch.float32):
            if self._gate_up_weight is None or self._gate_up_weight.device != x.device:
                self._gate_up_weight = torch.cat([self.gate_proj.weight, self.up_proj.weight], dim=0).contiguous()
            return self.down_proj(ops.silu_mul(F.linear(x, self._gate_up_weight)))
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class MSADecoderLayer(nn.Module):
    def __init__(self, config: MSAConfig, layer_idx: int):
        super().__init__()
        self.self_attn = MemorySparseAttention(config, layer_idx)
        self.mlp = MLP(config)
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, hidden_states, doc_ids, attention_mask, position_embeddings, past_key_value, position_ids=None):
        n1, n2 = self.input_layernorm, self.post_attention_layernorm
        if self._decode_rows_ok(hidden_states, past_key_value, position_ids):
            B = hidden_states.shape[0]
            h = self.self_attn.decode_rows(hidden_states.view(B, -1), n1.weight, n1.variance_epsilon, position_ids,
                                           past_key_value)
            return self.mlp.decode_rows(h, n2.weight, n2.variance_epsilon).view(B, 1, -1)
        if hidden_states.is_cuda and hidden_states.dtype in (torch.bfloat16, torch.float32):
            # HIP glue: norm kernels with the residual add folded in; hidden_states is updated in place
            h, _ = self.self_attn(ops.rmsnorm(hidden_states, n1.weight, n1.variance_epsilon), doc_ids, attention_mask,
                                  position_embeddings, past_key_value, position_ids=position_ids)
            x = ops.rmsnorm(h.contiguous(), n2.weight, n2.variance_epsilon, residual=hidden_states)
            return hidden_states.add_(self.mlp(x))
        h, _ = self.self_attn(self.input_layernorm(hidden_states), doc_ids, attention_mask, position_embeddings,
                              past_key_value)
        hidden_states = hidden_states + h
        return hidden_states + self.mlp(self.post_attention_layernorm(hidden_states))


    def _decode_rows_ok(self, hidden_states, cache, position_ids) -> bool:
        """One new token for at most 16 samples, bf16 on the GPU, no projection biases, hidden sizes the
        weight-streaming kernel takes: the decode step runs on it end to end."""
        if not (hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and position_ids is not None):
            return False
        B, S, H = hidden_states.shape
        if S != 1 or B > ops.SKINNY_MAX_ROWS or cache is None or not hidden_states.is_contiguous():
            return False
        if cache.meta.get("qa_mode", False):       # the step's attention mask decides who appends: generic path
            return False
        a = self.self_attn
        if cache.cache_kwargs[a.layer_idx].get("stage") != "generate" or a.q_proj.bias is not None:
            return False
        inter = self.mlp.gate_proj.weight.shape[0]
        return H % 128 == 0 and inter % 128 == 0 and (a.config.num_attention_heads * a.head_dim) % 128 == 0


class MSAModel(nn.Module):
    def __init__(self, config: MSAConfig):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList(MSADecoderLayer(config, i) for i in range(config.num_hidden_layers))
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, input_ids, attention_mask, position_ids, past_key_values, doc_ids, final_norm: bool = True):
        h = self.embed_tokens(input_ids)
        if past_key_values is not None and attention_mask is not None and input_ids.shape[1] > 1:
            past_key_values.meta["q_lens_host"] = attention_mask.sum(dim=1).tolist()   # one sync per forward, not per layer
            if h.is_cuda and position_ids is not None:
                # blocks of tokens (stage 1, stage 2, injected blocks) check their positions against the rotary
                # tables here; single-token decode steps are checked once by the generation loops
                self.layers[0].self_attn.check_positions(int(position_ids.max()))
        if h.is_cuda:
            for layer in self.layers:
                h = layer(h, doc_ids, attention_mask, None, past_key_values, position_ids=position_ids)
            if final_norm:
                return ops.rmsnorm(h, self.norm.weight, self.norm.variance_epsilon)
            return h
        pe = rotary_embedding(position_ids, self.config.head_dim, self.config.rope_theta, h.dtype)
        for layer in self.layers:
            h = layer(h, doc_ids, attention_mask, pe, past_key_values)
        return self.norm(h)


class MSAForCausalLM(nn.Module):
    def __init__(self, config: MSAConfig):
        super().__init__()
        self.config = config
        self.model = MSAModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)

    @torch.no_grad()
    def init_random(self, std: float = 0.02, seed: int = 0):
        g = torch.Generator(device="cpu").manual_seed(seed)
        for p in self.parameters():
            if p.dim() > 1:
                p.copy_(torch.randn(p.shape, generator=g).mul_(std).to(p.dtype))
        return self

    @torch.no_grad()
    def init_random_(self, std: float = 0.02, seed: int = 0):
        """In-place normal init on whatever device the parameters live on (fast for 4B parameters on
        the GPU); norm weights stay at one."""
        g = torch.Generator(device=next(self.parameters()).device).manual_seed(seed)
        for p in self.parameters():
            if p.dim() > 1:
                p.normal_(0.0, std, generator=g)
        return self

    @torch.no_grad()
    def generate_greedy(self, input_ids, attention_mask, doc_ids, max_new_tokens: int, top_k_docs: Optional[int] = None,
                        require_recall_topk: bool = False, past_key_values: Optional[CustomDynamicCache] = None,
                        timings: Optional[dict] = None, use_graph: bool = False):
        """Stage 2 on the (left-padded) query batch, then ``max_new_tokens`` greedy decode steps.
        Positions follow the reference: queries start at ``3 + top_k`` (src/msa_service.py:1823-1836),
        padding repeats the first position, each decode step advances by one
        (src/msa/generate.py:102-105).  With ``use_graph`` one decode step is captured as a HIP graph
        after two eager steps and replayed for the rest (the step is launch-bound in eager mode).
        Returns ``(tokens [B, max_new_tokens], cache)``."""
        B, S = input_ids.shape
        cfg = self.config
        k = cfg.msa_config.top_k_docs if top_k_docs is None else top_k_docs
        cache = past_key_values or create_cache()
        cache.meta["require_recall_topk"] = require_recall_topk
        for i in range(cfg.num_hidden_layers):
            cache.record_kwargs(i, {"stage": "prefill_stage2"})
        n_valid = attention_mask.sum(dim=1).tolist()
        pos = torch.tensor([query_position_ids(n, k, 3, S - n) for n in n_valid], dtype=torch.long, device=input_ids.device)
        self.model.layers[0].self_attn.check_positions(3 + k + max(n_valid) - 1 + max_new_tokens)
        if timings is not None:
            import time
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        h = self.model(input_ids, attention_mask, pos, cache, doc_ids)
        tok = self.lm_head(h[:, -1:]).argmax(-1)
        out = [tok]
        if timings is not None:
            torch.cuda.synchronize()
            timings["prefill_s"] = time.perf_counter() - t0
            t0 = time.perf_counter()
        for i in range(cfg.num_hidden_layers):
            cache.cache_kwargs[i]["stage"] = "generate"
        dev = input_ids.device
        n_steps = max_new_tokens - 1
        reserve = min(layer.self_attn.decode_reserve for layer in self.model.layers)
        if n_steps > reserve:
            raise RuntimeError(f"{n_steps} decode steps need decode_reserve >= {n_steps} (it is {reserve})")
        pos_buf = pos[:, -1:] + 1
        tok_buf = tok.clone()
        ones = torch.ones((B, 1), dtype=attention_mask.dtype, device=dev)
        gen_ids = torch.full((B, 1), -1, dtype=doc_ids.dtype, device=dev)
        out_buf = torch.zeros((B, max_new_tokens), dtype=tok.dtype, device=dev)
        out_buf[:, :1] = tok
        col = torch.ones((B, 1), dtype=torch.long, device=dev)

        fold_head = (dev.type == "cuda" and self.lm_head.weight.dtype == torch.bfloat16 and B <= ops.SKINNY_MAX_ROWS
                     and cfg.hidden_size % 128 == 0 and self.lm_head.bias is None)

        native_sample = (dev.type == "cuda" and tok_buf.is_contiguous() and pos_buf.is_contiguous()
                         and pos_buf.dtype == torch.int64 and pos_buf.numel() == B)
        sample_scratch = torch.empty(B * 32, dtype=torch.int64, device=dev) if native_sample else None

        def step():
            # everything is in-place on fixed buffers so the same launches can be replayed as a graph
            if fold_head:                          # final norm folded into the weight-streaming LM head
                h = self.model(tok_buf, ones, pos_buf, cache, gen_ids, final_norm=False)
                logits = ops.skinny_linear(h.view(B, -1), self.lm_head.weight, norm_weight=self.model.norm.weight,
                                           eps=self.model.norm.variance_epsilon).view(B, 1, -1)
            else:
                logits = self.lm_head(self.model(tok_buf, ones, pos_buf, cache, gen_ids))
            if native_sample:                      # argmax + token bookkeeping in two small launches
                ops.greedy_sample(logits.view(B, -1), tok_buf, pos_buf, out_buf, col, sample_scratch)
                return
            new_tok = logits.argmax(-1)
            tok_buf.copy_(new_tok)
            pos_buf.add_(1)
            out_buf.scatter_(1, col, new_tok)
            col.add_(1)

        done = 0
        if use_graph and n_steps > 3:
            for _ in range(2):                     # warm-up: workspaces and library handles exist before capture
                step()
                done += 1
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            done += 0                              # capture records the launches without running them
            while done < n_steps:
                graph.replay()
                done += 1
        else:
            while done < n_steps:
                step()
                done += 1
        if timings is not None:
            torch.cuda.synchronize()
            timings["decode_s"] = time.perf_counter() - t0
            timings["decode_steps"] = n_steps
        return out_buf, cache


@torch.no_grad()
def generate_interleaved(model: "MSAForCausalLM", input_ids, attention_mask, doc_ids, max_new_tokens: int, inject,
                         top_k_docs: Optional[int] = None, require_recall_topk: bool = False):
    """Greedy decoding with Memory-Interleave rounds (the control flow of src/msa/generate.py:190-259 without the
    tokenizer: text handling stays with the caller).  Stage 2 routes on the tokens whose ``doc_ids`` are 0.  After
    every new token ``inject(step, tokens [B, step])`` may return a list of ``B`` token-id lists; a non-empty list
    replaces the sample's just-generated token as the next model input (the reference feeds the retrieved
    documents' text instead of the round-end marker), an empty one lets the sample continue with its own token.
    The lists are fed as one left-padded block with the reference's positions (``source_block_position_ids``),
    appended to the compact caches by the ragged path of the decode stage, and the next token is read at the
    block's last position.  Returns ``(tokens [B, max_new_tokens], cache)``."""
    cfg = model.config
    B, S = input_ids.shape
    dev = input_ids.device
    k = cfg.msa_config.top_k_docs if top_k_docs is None else top_k_docs
    cache = create_cache()
    cache.meta["require_recall_topk"] = require_recall_topk
    for i in range(cfg.num_hidden_layers):
        cache.record_kwargs(i, {"stage": "prefill_stage2"})
    n_valid = attention_mask.sum(dim=1).tolist()
    pos = torch.tensor([query_position_ids(n, k, 3, S - n) for n in n_valid], dtype=torch.long, device=dev)
    h = model.model(input_ids, attention_mask, pos, cache, doc_ids)
    tok = model.lm_head(h[:, -1:]).argmax(-1)                 # [B, 1]
    for i in range(cfg.num_hidden_layers):
        cache.cache_kwargs[i]["stage"] = "generate"
    last_pos = [3 + k + n - 1 for n in n_valid]               # position of the last token each sample has fed
    attn0 = model.model.layers[0].self_attn
    rows_free = min(layer.self_attn.decode_reserve for layer in model.model.layers)
    out = [tok]
    for step in range(1, max_new_tokens):
        blocks = inject(step, torch.cat(out, dim=1)) if inject is not None else None
        blocks = [list(b) if b else [int(t)] for b, t in zip(blocks, tok[:, 0].tolist())] if blocks is not None else None
        # every sample's compact cache has decode_reserve free rows behind its stage-2 context: a step that would
        # not fit is refused here, before any kernel could drop rows
        widest = 1 if blocks is None else max(len(b) for b in blocks)
        if widest > rows_free:
            raise RuntimeError(f"step {step} appends {widest} rows per sample but only {rows_free} of the "
                               f"decode_reserve rows are left; raise decode_reserve on the layers before stage 2")
        rows_free -= widest
        lens = [1] * B if blocks is None else [len(b) for b in blocks]
        attn0.check_positions(max(p + n for p, n in zip(last_pos, lens)))
        if widest == 1:
            ids = tok if blocks is None else torch.tensor(blocks, dtype=torch.long, device=dev)
            p = torch.tensor([[x + 1] for x in last_pos], dtype=torch.long, device=dev)
            h = model.model(ids, torch.ones_like(ids), p, cache, torch.full_like(ids, -1))
        else:
            ids = torch.zeros((B, widest), dtype=torch.long)
            mask = torch.zeros((B, widest), dtype=torch.long)
            for b, blk in enumerate(blocks):
                ids[b, widest - len(blk):] = torch.tensor(blk)
                mask[b, widest - len(blk):] = 1
            p = torch.tensor(source_block_position_ids(last_pos, lens, widest), dtype=torch.long)
            h = model.model(ids.to(dev), mask.to(dev), p.to(dev), cache, torch.zeros((B, widest), dtype=torch.long, device=dev))
        last_pos = [x + n for x, n in zip(last_pos, lens)]
        tok = model.lm_head(h[:, -1:]).argmax(-1)
        out.append(tok)
    return torch.cat(out, dim=1), cache


@torch.no_grad()
def generate_with_hops(model: "MSAForCausalLM", input_ids, attention_mask, doc_ids, max_new_tokens: int, regenerate,
                       inject=None, max_hops: int = 4, top_k_docs: Optional[int] = None):
    """The multi-hop loop around generation (src/app/benchmark.py:202-212 with ``should_regenerate`` and
    src/msa_service.py:1734-1770 ``_apply_template_regenerate``): after a generation pass,
    ``regenerate(hop, tokens [B, T])`` may return a new batch ``(input_ids, attention_mask, doc_ids)`` — the
    regenerated prompt, in which ``doc_ids`` marks with 0 the regions that query the memory and with -1 the rest —
    or ``None`` to stop.  Every hop is a fresh stage-2 pass: the router scores the new prompt's marked tokens against
    the bank, the selected documents' K / V are fetched again and a new compact cache is built.  Returns the list of
    ``(tokens, cache)`` of all passes; the recalled documents of each pass are in its cache's ``recall_topk``."""
    passes = []
    batch = (input_ids, attention_mask, doc_ids)
    for hop in range(max_hops + 1):
        toks, cache = generate_interleaved(model, batch[0], batch[1], batch[2], max_new_tokens, inject,
                                           top_k_docs=top_k_docs, require_recall_topk=True)
        passes.append((toks, cache))
        if hop == max_hops or regenerate is None:
            break
        batch = regenerate(hop, toks)
        if batch is None:
            break
    return passes


def encode_block(model: MSAForCausalLM, block_input, device) -> CustomDynamicCache:
    """Runs stage 1 over one packed block and returns the cache holding its pooled K / V / K_r
    (the inference half of src/prefill.py:248-305)."""
    cache = create_cache()
    for i in range(model.config.num_hidden_layers):
        cache.record_kwargs(i, {"stage": "prefill_stage1"})
    with torch.no_grad():
        model.model(block_input.doc_input_ids.to(device), block_input.doc_attention_mask.to(device),
                    block_input.position_ids.to(device), cache, block_input.doc_ids.to(device))
    return cache
