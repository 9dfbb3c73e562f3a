"""Stage-1 input construction (src/prefill.py:75-91, 188-246) on pre-tokenised documents: packed
block = template head then the documents, document ids 1..n per block (-2 for the template),
position ids restarting at 0 for every document, ceil(len / P) chunks per document."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence

import torch


@dataclass
class Document:
    doc: str = ""
    doc_id: int = 0
    num_chunks: int = 0
    input_ids: Sequence[int] = ()      # pre-tokenised text (the reference tokenises `doc` on the fly)


@dataclass
class BlockModelInput:
    doc_input_ids: torch.Tensor
    doc_attention_mask: torch.Tensor
    doc_ids: torch.Tensor
    position_ids: torch.Tensor
    num_chunks: int
    chunk_sizes: List[int]
    doc_lens: List[int]
    template_len: int


def num_chunks(n_tokens: int, pooling_kernel_size: int) -> int:
    return (n_tokens + pooling_kernel_size - 1) // pooling_kernel_size


def split_docs(docs: List[Document], block_size: int) -> List[List[Document]]:
    """Greedy split into blocks of at most ``block_size`` chunks; a document never straddles blocks
    (src/prefill.py:75-91)."""
    blocks, cur, size = [], [], 0
    for d in docs:
        if size + d.num_chunks > block_size and cur:
            blocks.append(cur)
            cur, size = [], 0
        cur.append(d)
        size += d.num_chunks
    if cur:
        blocks.append(cur)
    return blocks


def prepare_block_inputs(block: List[Document], template_head_ids: Sequence[int], pooling_kernel_size: int,
                         template_id: int = -2) -> BlockModelInput:
    """src/prefill.py:188-246 with the tokenizer factored out."""
    head = list(template_head_ids)
    doc_ids = [template_id] * len(head)
    input_ids = list(head)
    positions = list(range(len(head)))
    chunk_sizes, doc_lens = [], []
    for i, item in enumerate(block):
        toks = list(item.input_ids)
        if not toks:
            raise ValueError(f"document {item.doc_id} has no tokens")
        n = len(toks)
        nch = num_chunks(n, pooling_kernel_size)
        if item.num_chunks and item.num_chunks != nch:
            raise AssertionError(f"pre calculated chunk {item.num_chunks} got {nch} for document {item.doc_id}")
        chunk_sizes.append(nch)
        doc_lens.append(n)
        doc_ids.extend([i + 1] * n)          # 1-based within the block: these become the pool ids
        input_ids.extend(toks)
        positions.extend(range(n))           # positions restart at 0 for every document
    t = lambda x: torch.tensor([x], dtype=torch.long)
    return BlockModelInput(t(input_ids), torch.ones(1, len(input_ids), dtype=torch.long), t(doc_ids), t(positions),
                           sum(chunk_sizes), chunk_sizes, doc_lens, len(head))


def query_position_ids(n_tokens: int, top_k: int, template_len: int = 3, left_pad: int = 0) -> List[int]:
    """Positions of a query: ``template_len + top_k + i``; left padding repeats the first position
    (src/msa_service.py:1823-1864)."""
    first = template_len + top_k
    return [first] * left_pad + [first + i for i in range(n_tokens)]


def source_block_position_ids(last_positions: Sequence[int], n_tokens: Sequence[int], width: int) -> List[List[int]]:
    """Positions of a left-padded block of source tokens injected between generation rounds
    (src/msa/generate.py:235-236): column ``j`` of sample ``b`` gets
    ``j + last_positions[b] + n_tokens[b] - width + 1``, so the sample's first real token (column
    ``width - n_tokens[b]``) continues at ``last_positions[b] + 1`` and the rest count up from there.  The same
    expression runs below that for the padding columns in front; those tokens are masked out everywhere, and their
    positions are floored at 0 here because the rotary tables start there."""
    out = []
    for last, n in zip(last_positions, n_tokens):
        out.append([max(0, j + int(last) + int(n) - width + 1) for j in range(width)])
    return out


class PrefillStage1Worker:
    """The encode worker with the reference's call surface (src/prefill.py:94-305), in process: no queues, no
    tokenizer (documents arrive tokenised), the model handed in instead of loaded from a path.

    ``inference(block)`` returns what the reference's worker sends back (:300-303, :142-157):
    ``{"chunk_sizes", "past_key_values", "nr_docs", "doc_ids", "nr_chunks"}`` with the pooled K / V / K_r of every
    router layer in ``past_key_values`` (getters ``get_kvcache`` / ``get_router_kcache``,
    ``cache_kwargs[layer]["pooled_doc_ids" | "template_prefix_kcache" | "template_prefix_vcache"]``)."""

    def __init__(self, gpu_id: int, model, template_head_ids: Sequence[int], pooling_kernel_size: int,
                 template_id: int = -2):
        self.gpu_id = gpu_id
        self.device = torch.device(f"cuda:{gpu_id}")
        self.model = model
        self.template_head_ids = list(template_head_ids)
        self.pooling_kernel_size = pooling_kernel_size
        self.template_id = template_id

    def num_model_layers(self) -> int:
        return self.model.config.num_hidden_layers

    @staticmethod
    def split_docs(docs: List[Document], block_size: int) -> List[List[Document]]:
        return split_docs(docs, block_size)

    def _prepare_block_inputs(self, block: List[Document]) -> BlockModelInput:
        return prepare_block_inputs(block, self.template_head_ids, self.pooling_kernel_size, self.template_id)

    def _inference(self, model_input: BlockModelInput) -> Dict:
        from .model import encode_block            # the model module imports this one
        cache = encode_block(self.model, model_input, self.device)
        return {"chunk_sizes": model_input.chunk_sizes, "past_key_values": cache}

    def inference(self, block: List[Document]) -> Dict:
        meta = self._inference(self._prepare_block_inputs(block))
        meta["nr_docs"] = len(block)
        meta["doc_ids"] = [item.doc_id for item in block]
        meta["nr_chunks"] = [item.num_chunks for item in block]
        return meta
