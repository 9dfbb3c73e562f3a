"""Memory bank and query service with the reference's call surface
(src/msa_service.py: ``BlockDesc`` :191-231, ``Memory`` :269-828, ``MSAService.doc_query`` :1133-1314),
single GPU, every tensor operation done by the HIP library.

Bank layout (differs from the reference on purpose): pooled tensors are chunk-major ``[C, Hkv, D]``
— K_r resident in HBM, K / V in pinned host memory — so a chunk's routing key is one contiguous
2 KB row for the scoring kernel and a document's K / V is one contiguous range for the gather.
Reference-shaped views (``[1, Hkv, C, D]``, ``[Hkv, n, D]``) are handed out where its API says so.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import ops
from .cache import CustomDynamicCache
from .config import GenerateConfig, MemoryConfig, ModelConfig, MSAConfig
from .prefill import Document


def cumulative_concat(tensors: Sequence[torch.Tensor]) -> torch.Tensor:
    """Concatenates per-block 1-based pool ids into bank-wide ids: each block is shifted by the last
    id of everything before it (src/utils/tools.py:34-55)."""
    out, shift = [], 0
    for t in tensors:
        out.append(t + shift)
        shift += int(t[-1])
    return torch.cat(out)


@dataclass
class BlockDesc:
    """Bank description (src/msa_service.py:191-231): tables carry a dummy slot 0."""
    docs: List[Document] = None
    tmp_doc_ids: List[torch.Tensor] = None
    pool_ids: torch.Tensor = None
    pool_ids_cpu: torch.Tensor = None
    doc_ids: torch.Tensor = None
    doc_ids_cpu: torch.Tensor = None
    doc_offsets_cpu: torch.Tensor = None
    doc_lens_cpu: torch.Tensor = None

    def init_docs(self, docs: List[Document], device):
        self.docs = docs
        self.doc_ids_cpu = torch.tensor([0] + [d.doc_id for d in docs], dtype=torch.long)
        self.doc_ids = self.doc_ids_cpu.to(device)
        self.tmp_doc_ids = []
        lens = [0] + [d.num_chunks for d in docs]
        self.doc_lens_cpu = torch.tensor(lens, dtype=torch.long)
        self.doc_offsets_cpu = torch.cumsum(torch.tensor([0] + lens[:-1], dtype=torch.long), dim=0)

    def create_global_doc_ids(self, local_doc_ids):
        return self.doc_ids[local_doc_ids]

    def merge_poolig_doc_id(self, device):
        self.pool_ids_cpu = cumulative_concat([t.cpu() for t in self.tmp_doc_ids])
        self.pool_ids = self.pool_ids_cpu.to(device)
        self.tmp_doc_ids.clear()

    def chunks(self) -> int:
        return sum(d.num_chunks for d in self.docs)

    @property
    def nr_docs(self) -> int:
        return len(self.docs)


class MemoryClientBase:
    """What the layer calls (src/msa_service.py:259-264)."""

    def get_template_prefix_kvcaches(self, layer_idx: int):
        raise NotImplementedError

    def doc_query(self, query_states: torch.Tensor, attention_mask: torch.Tensor, layer_idx: int):
        raise NotImplementedError


def _chunk_major(t: torch.Tensor) -> torch.Tensor:
    """``[1, Hkv, C, D]`` (reference) or ``[C, Hkv, D]`` (native) -> ``[C, Hkv, D]`` view."""
    return t[0].transpose(0, 1) if t.dim() == 4 else t


class Memory:
    """Tiered bank + scorer.  Fill it with :meth:`begin`, one :meth:`add_block` per stage-1 block and
    :meth:`finish`; then :meth:`prefill_stage2` scores queries against it."""

    def __init__(self, gpu_id: int, generate_config: GenerateConfig, model_config: ModelConfig,
                 memory_config: MemoryConfig, msa_model_config: Optional[MSAConfig] = None):
        self.gpu_id = gpu_id
        self.device = torch.device(f"cuda:{gpu_id}")
        self.generate_config, self.model_config, self.memory_config = generate_config, model_config, memory_config
        self.msa_model_config = msa_model_config or MSAConfig()
        cfg = self.msa_model_config
        n_layers = cfg.num_hidden_layers
        self.router_layer_ids = sorted(range(n_layers) if model_config.router_layer_idx == "all"
                                       else (int(x) for x in model_config.router_layer_idx.split(",")))
        self.num_key_value_groups = cfg.num_attention_heads // cfg.num_key_value_heads
        mc = cfg.msa_config
        self.head_reduce_method, self.query_reduce_method = mc.head_reduce_method, mc.query_reduce_method
        self.chunk_reduce_method, self.aux_loss_method = mc.chunk_reduce_method, mc.aux_loss_method
        self.decouple_router = mc.decouple_router
        # the reductions of src/msa_service.py:742-813: heads "mean" (the kernels sum a group's heads before the
        # scan, which a max over heads does not allow), tokens "max" / "mean" / "last", chunks "max" / "mean"
        if self.head_reduce_method != "mean":
            raise NotImplementedError(f"Unsupported head reduce method: {self.head_reduce_method}")
        if self.query_reduce_method not in ops.QUERY_REDUCE:
            raise NotImplementedError(f"Unsupported query reduce method: {self.query_reduce_method}")
        if self.chunk_reduce_method not in ops.CHUNK_REDUCE:
            raise ValueError(f"Invalid chunk reduction method: {self.chunk_reduce_method}")
        # -1 marks "already cosine, do not scale" exactly as the reference does (:318-321)
        self.scaling = -1.0 if (self.aux_loss_method == "INFONCE" and self.decouple_router) else cfg.head_dim ** -0.5
        self.block_desc = BlockDesc()
        self.template_prefix_kvcache: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.bank: Optional[ops.Bank] = None
        self._rk: Dict[int, torch.Tensor] = {}
        self._k: Dict[int, torch.Tensor] = {}
        self._v: Dict[int, torch.Tensor] = {}
        self._kv_offset = 0
        self._layer_slot = {layer: i for i, layer in enumerate(self.router_layer_ids)}

    def num_model_layers(self) -> int:
        return self.msa_model_config.num_hidden_layers

    # ---------------------------------------------------------------- bank fill (:497-582)
    def set_prefill_worker(self, worker) -> None:
        """The stage-1 worker :meth:`generate_blocks` drives (the reference starts one per GPU as a child process,
        :500-513; here it lives in this process and is handed in)."""
        self._prefill_worker = worker

    def generate_blocks(self, docs: List[Document], worker=None) -> None:
        """Builds the bank from documents exactly as the reference does (:497-582): an existing dump under
        ``$MEMORY_DATA_PATH/gpu<world>/<gpu_id>`` is loaded instead; otherwise the documents are split into blocks
        of at most ``memory_config.block_size`` chunks, every block is encoded by the worker's ``inference`` and its
        pooled K / V / K_r are copied into the bank at the running chunk offset, the pooled document ids are merged,
        and the bank is dumped when the variable is set."""
        path = os.environ.get("MEMORY_DATA_PATH", "")
        if path:
            path = os.path.join(path, f"gpu{self.generate_config.world}", str(self.gpu_id))
            if os.path.exists(path):
                self.deserialize(path, docs)
                assert len(docs) == self.block_desc.nr_docs
                return
        worker = worker or getattr(self, "_prefill_worker", None)
        if worker is None:
            raise ValueError("generate_blocks needs a stage-1 worker (set_prefill_worker or the worker argument)")
        self.begin(docs)
        recv = 0
        for block in worker.split_docs(docs, self.memory_config.block_size):
            meta = worker.inference(block)
            recv += meta["nr_docs"]
            self.add_block(meta["past_key_values"])
            meta["past_key_values"].clear_kvcache()
        assert recv == len(docs), f"encoded {recv} of {len(docs)} documents"
        self.finish()
        if path:
            self.serialize(path)

    def begin(self, docs: List[Document]) -> None:
        self.block_desc.init_docs(docs, self.device)
        self._kv_offset = 0

    def _init_block_data(self, Hkv: int, D: int, dtype: torch.dtype) -> None:
        C = self.block_desc.chunks()
        for layer in self.router_layer_ids:
            self._rk[layer] = torch.empty((C, Hkv, D), dtype=dtype, device=self.device)
            self._k[layer] = torch.empty((C, Hkv, D), dtype=dtype, pin_memory=True)
            self._v[layer] = torch.empty((C, Hkv, D), dtype=dtype, pin_memory=True)

    def add_block(self, past_key_values: CustomDynamicCache) -> None:
        """Copies one stage-1 block's pooled K / V / K_r into the bank at the running chunk offset
        and records its pooled document ids (:541-569)."""
        if not self.template_prefix_kvcache:
            kw = past_key_values.cache_kwargs
            self.template_prefix_kvcache = {
                layer: (kw[layer]["template_prefix_kcache"].to(self.device), kw[layer]["template_prefix_vcache"].to(self.device))
                for layer in range(self.num_model_layers()) if "template_prefix_kcache" in kw.get(layer, {})}
        meta_chunks = None
        for layer in self.router_layer_ids:
            k, v = past_key_values.get_kvcache(layer)
            rk = past_key_values.get_router_kcache(layer)
            if rk is None:
                raise ValueError("this bank needs decoupled routing keys (router_k_proj) for every router layer")
            k, v, rk = _chunk_major(k), _chunk_major(v), _chunk_major(rk)
            if not self._rk:
                self._init_block_data(k.shape[1], k.shape[2], k.dtype)
            if layer == self.router_layer_ids[0]:
                self.block_desc.tmp_doc_ids.append(past_key_values.cache_kwargs[layer]["pooled_doc_ids"])
            n = k.shape[0]
            if meta_chunks is None:
                meta_chunks = n
            assert meta_chunks == n, f"expect meta_chunks {meta_chunks} but got {n}"
            total = self.block_desc.chunks()
            assert self._kv_offset + n <= total, f"overflow: offset {self._kv_offset}, meta_chunks {n}, total_chunks {total}"
            s = slice(self._kv_offset, self._kv_offset + n)
            self._k[layer][s].copy_(k)
            self._v[layer][s].copy_(v)
            self._rk[layer][s].copy_(rk)
        self._kv_offset += meta_chunks or 0

    def finish(self) -> None:
        """Merges the pooled ids, checks them against the documents' chunk counts and creates the
        native bank handle (replaces ``_generate_slice``: no slices, no transposed views)."""
        self.block_desc.merge_poolig_doc_id(self.device)
        self._finish_bank()

    def _finish_bank(self) -> None:
        desc = self.block_desc
        counts = torch.bincount(desc.pool_ids_cpu, minlength=desc.nr_docs + 1)
        if not torch.equal(counts, desc.doc_lens_cpu):
            raise AssertionError("pooled document ids do not match the documents' chunk counts")
        if self._kv_offset != desc.chunks():
            raise AssertionError(f"bank holds {self._kv_offset} chunks, documents need {desc.chunks()}")
        off = torch.cat([desc.doc_offsets_cpu[1:], torch.tensor([desc.chunks()])])      # [n_docs + 1], 0-based docs
        ref = self._rk[self.router_layer_ids[0]]
        self.bank = ops.Bank(len(self.router_layer_ids), off.tolist(), desc.doc_ids_cpu[1:].tolist(), ref.shape[1],
                             ref.shape[2], ref.dtype)
        for layer, slot in self._layer_slot.items():
            self.bank.set_layer(slot, self._rk[layer], self._k[layer], self._v[layer])

    def load_pooled(self, docs: List[Document], rk: Dict[int, torch.Tensor], k: Dict[int, torch.Tensor],
                    v: Dict[int, torch.Tensor], template_prefix: Dict[int, Tuple[torch.Tensor, torch.Tensor]]) -> None:
        """Adopts an already pooled bank: per router layer ``rk`` on the device and ``k`` / ``v`` in
        pinned host memory, all chunk-major ``[C, Hkv, D]`` in document order, plus the template
        prefix K / V ``[1, Hkv, n, D]`` of every layer.  (Entry point for synthetic banks and for a
        bank read back from storage; :meth:`add_block` is the path that follows stage 1.)"""
        self.block_desc.init_docs(docs, self.device)
        lens = self.block_desc.doc_lens_cpu
        self.block_desc.pool_ids_cpu = torch.repeat_interleave(torch.arange(lens.numel()), lens)
        self.block_desc.pool_ids = self.block_desc.pool_ids_cpu.to(self.device)
        missing = [l for l in self.router_layer_ids if l not in rk or l not in k or l not in v]
        if missing:
            raise ValueError(f"router layers {missing} have no pooled tensors")
        self._rk, self._k, self._v = dict(rk), dict(k), dict(v)
        self._kv_offset = self.block_desc.chunks()
        self.template_prefix_kvcache = {l: (a.to(self.device), b.to(self.device)) for l, (a, b) in template_prefix.items()}
        self._finish_bank()

    # ---------------------------------------------------------------- storage (:351-479)
    def serialize(self, path: str) -> None:
        """Writes the bank as raw chunk-major arrays plus a JSON header (see ``bank_io``)."""
        from . import bank_io
        desc, mc = self.block_desc, self.msa_model_config.msa_config
        off = torch.cat([desc.doc_offsets_cpu[1:], torch.tensor([desc.chunks()])]).tolist()
        header = {"pooling_kernel_size": mc.pooling_kernel_size, "aux_loss_method": mc.aux_loss_method,
                  "head_reduce_method": mc.head_reduce_method, "query_reduce_method": mc.query_reduce_method,
                  "chunk_reduce_method": mc.chunk_reduce_method, "decouple_router": bool(mc.decouple_router)}
        os.makedirs(path, exist_ok=True)
        bank_io.save_docs(path, desc.docs)
        bank_io.save_bank(path, header, off, desc.doc_ids_cpu[1:].tolist(), self._rk, self._k, self._v,
                          self.template_prefix_kvcache)

    def deserialize(self, path: str, docs: Optional[List[Document]] = None) -> None:
        """Streams a stored bank back in: K_r to the device, K / V into freshly pinned host memory, one layer
        at a time.  ``docs`` restores the document texts; without it placeholders carry ids and chunk counts."""
        from . import bank_io
        files = bank_io.BankFiles(path)
        h = files.header
        if h["router_layers"] != self.router_layer_ids:
            raise ValueError(f"bank has router layers {h['router_layers']}, this model {self.router_layer_ids}")
        mc = self.msa_model_config.msa_config
        if h.get("aux_loss_method") != mc.aux_loss_method or h.get("pooling_kernel_size") != mc.pooling_kernel_size:
            raise ValueError("bank was built with different scoring / pooling hyper-parameters")
        counts = (files.doc_chunk_off[1:] - files.doc_chunk_off[:-1]).tolist()
        if docs is None:
            rows = bank_io.load_docs(path)
            if rows is not None:
                docs = [Document(doc=r["doc"], doc_id=r["doc_id"], num_chunks=r["num_chunks"]) for r in rows]
        if docs is None:
            docs = [Document(doc_id=int(g), num_chunks=int(n)) for g, n in zip(files.doc_global_id.tolist(), counts)]
        if [d.num_chunks for d in docs] != counts or [d.doc_id for d in docs] != files.doc_global_id.tolist():
            raise ValueError("documents do not match the stored bank")
        rk, k, v = {}, {}, {}
        for layer in self.router_layer_ids:
            rk[layer] = torch.empty(files.shape, dtype=files.torch_dtype, device=self.device)
            k[layer] = torch.empty(files.shape, dtype=files.torch_dtype, pin_memory=True)
            v[layer] = torch.empty(files.shape, dtype=files.torch_dtype, pin_memory=True)
            files.copy_into(layer, "rk", rk[layer])
            files.copy_into(layer, "k", k[layer])
            files.copy_into(layer, "v", v[layer])
        self.load_pooled(docs, rk, k, v, files.prefix())

    def load_reference_bank(self, path: str, docs: List[Document]) -> None:
        """Adopts a bank directory written by the reference's ``Memory.serialize`` (src/msa_service.py:351-404):
        ``layer_<i>_{k,v,rk}.pt`` and ``prefix_cache.pt`` are read as plain tensors (``weights_only=True``) and
        transposed to chunk-major; ``meta.pt`` pickles Document objects and is not opened, so the documents (ids
        and chunk counts, bank order) come from the caller.  K_r goes to the device, K / V into pinned host
        memory, whatever device the reference's own restore would have chosen (:447-461)."""
        from . import bank_io
        have = bank_io.reference_bank_layers(path)
        missing = [l for l in self.router_layer_ids if l not in have]
        if missing:
            raise ValueError(f"{path}: no pooled tensors for router layers {missing}")
        rk, k, v = {}, {}, {}
        for layer in self.router_layer_ids:
            r, kk, vv = bank_io.read_reference_layer(path, layer)
            rk[layer] = r.to(self.device)
            k[layer], v[layer] = kk.pin_memory(), vv.pin_memory()
        self.load_pooled(docs, rk, k, v, bank_io.read_reference_prefix(path))

    def get_max_local_pool_doc_id(self) -> int:
        return int(self.block_desc.pool_ids_cpu[-1])

    def get_template_prefix_kvcaches(self, layer_idx: int):
        return self.template_prefix_kvcache[layer_idx]

    # ---------------------------------------------------------------- scorer (:703-828)
    def _route(self, layer_idx: int, q_bshd: torch.Tensor, mask_bs: Optional[torch.Tensor], mode: str, scale: float):
        top_k = self.model_config.doc_top_k
        scores, doc, gid = ops.route_topk(self.bank, self._layer_slot[layer_idx], q_bshd, mask_bs, mode, scale, top_k,
                                          query_reduce=self.query_reduce_method, chunk_reduce=self.chunk_reduce_method)
        return scores, doc, gid

    def prefill_stage2(self, layer_idx: int, query_states: torch.Tensor, query_mask: torch.Tensor):
        """``query_states [B, Hkv, G, S, D]`` already scaled / normalised by the caller, ``query_mask
        [B, 1, 1, S, 1]`` -> ``(scores [B, k], local_ids [B, k] 1-based, global_ids [B, k])`` with
        ``k = min(doc_top_k, nr_docs + 1)``; when the bank has fewer than ``doc_top_k`` documents
        the dummy slot 0 fills the tail with the dtype's lowest value, as ``torch.topk`` over the
        reference's score table does."""
        B, Hkv, G, S, D = query_states.shape
        q = query_states.permute(0, 3, 1, 2, 4).reshape(B, S, Hkv * G, D).contiguous()
        mask = query_mask.reshape(B, S)
        scores, doc, gid = self._route(layer_idx, q, mask, "scaled_dot", 1.0)
        dtype = query_states.dtype
        k = min(self.model_config.doc_top_k, self.block_desc.nr_docs + 1)
        lowest = torch.finfo(dtype).min
        scores = scores[:, :k].clamp_min(lowest).to(dtype)
        local = (doc[:, :k].long() + 1)                      # -1 (no document) becomes the dummy slot 0
        scores = torch.where(local == 0, torch.full_like(scores, lowest), scores)
        return scores, local, self.block_desc.create_global_doc_ids(local)


class MSAService(Memory, MemoryClientBase):
    """Single-GPU service: the reference's collectives (src/msa_service.py:1098-1131, 1163-1198,
    1267-1283) are the identity at world size 1 and are not present."""

    def __init__(self, gpu_id: int, generate_config: GenerateConfig, model_config: ModelConfig,
                 memory_config: MemoryConfig, msa_model_config: Optional[MSAConfig] = None):
        super().__init__(gpu_id, generate_config, model_config, memory_config, msa_model_config)
        self.copy_stream = torch.cuda.Stream(device=self.device)
        self._ids_host: Optional[torch.Tensor] = None

    def setup_memory_client(self, model) -> None:
        for _, module in model.named_modules():
            if callable(getattr(module, "set_memory_client", None)):
                module.set_memory_client(self)

    def doc_query_device(self, q_bshd: torch.Tensor, query_mask: Optional[torch.Tensor], layer_idx: int,
                         fused_normalize: bool = True):
        """The sync-free form the native layer uses: ``q_bshd [B, S, Hq, D]`` contiguous.  Routing, plan and gather
        are all enqueued on the current stream; nothing is copied to the host.  Returns ``(K, V)`` buffers of
        ``B * k * max_doc_chunks`` rows ``[rows, Hkv, D]``, ``cu_sel`` (device int32 ``[B + 1]``: rows
        ``cu_sel[b] .. cu_sel[b + 1]`` are sample b's, documents in ascending bank order, each once), ``scores
        [B, k]`` fp32 and ``global_ids [B, k]`` (0 where nothing was selected)."""
        if fused_normalize:
            mode, scale = "cosine", 1.0
        else:
            mode, scale = "scaled_dot", (1.0 if self.scaling < 0 else self.scaling)
        scores, doc, gid = self._route(layer_idx, q_bshd, query_mask, mode, scale)
        if fused_normalize and self.scaling > 0:
            # normalised queries are still multiplied by head_dim^-0.5 unless the router is decoupled (:318-321, 1095-1096)
            scores = scores * self.scaling
        doc = torch.where(scores > -1e9, doc, torch.full_like(doc, -1))      # drop invalid picks (:1190-1191)
        B, k = doc.shape
        cap = B * k * self.bank.max_doc_chunks
        k_sel, v_sel, cu = ops.gather_kv_device(self.bank, self._layer_slot[layer_idx], doc.contiguous(), cap)
        return k_sel, v_sel, cu, scores, torch.where(doc >= 0, gid, torch.zeros_like(gid))

    def doc_query(self, query_states: torch.Tensor, query_mask: torch.Tensor, layer_idx: int,
                  fused_normalize: bool = False, native_layout: bool = False):
        """``query_states [B, Hq, S, D]`` (the layer's ``.transpose(1, 2)`` view, normalised by the
        caller in cosine mode unless ``fused_normalize``), ``query_mask [B, S]`` bool.

        Returns ``(K [Hkv, n, D], V [Hkv, n, D], scores [B, k], n_sel [B] int64, global_ids [B, k])``
        as src/msa_service.py:1314 does — K / V are views of chunk-major ``[n, Hkv, D]`` buffers
        (pass ``native_layout=True`` to get those).  Within a sample the selected documents'
        chunks come in ascending bank order, each document once; picks whose score is <= -1e9 are
        dropped (:1190-1191).  The host copies run on a side stream; the current stream waits for
        them before returning."""
        B, Hq, S, D = query_states.shape
        q = query_states.transpose(1, 2)
        if not q.is_contiguous():
            q = q.contiguous()
        if fused_normalize:
            mode, scale = "cosine", 1.0
        else:
            mode, scale = "scaled_dot", (1.0 if self.scaling < 0 else self.scaling)
        scores, doc, gid = self._route(layer_idx, q, query_mask, mode, scale)
        if fused_normalize and self.scaling > 0:
            scores = scores * self.scaling                   # (:318-321, 1095-1096: only a decoupled router skips the scale)
        valid = scores > -1e9
        doc = torch.where(valid, doc, torch.full_like(doc, -1))
        if self._ids_host is None or self._ids_host.shape != doc.shape:
            self._ids_host = torch.empty(doc.shape, dtype=torch.int32, pin_memory=True)
        self._ids_host.copy_(doc, non_blocking=True)
        torch.cuda.current_stream().synchronize()            # the ids must be on the host to address pinned K / V
        k_sel, v_sel, cu = ops.gather_kv(self.bank, self._layer_slot[layer_idx], self._ids_host, self.device,
                                         stream=self.copy_stream)
        torch.cuda.current_stream().wait_stream(self.copy_stream)
        k_sel.record_stream(torch.cuda.current_stream())
        v_sel.record_stream(torch.cuda.current_stream())
        n_sel = (cu[1:] - cu[:-1]).to(self.device)
        dtype = query_states.dtype
        scores = scores.clamp_min(torch.finfo(dtype).min).to(dtype)
        gid = torch.where(doc >= 0, gid, torch.zeros_like(gid))
        if native_layout:
            return k_sel, v_sel, scores, n_sel, gid
        return k_sel.permute(1, 0, 2), v_sel.permute(1, 0, 2), scores, n_sel, gid
