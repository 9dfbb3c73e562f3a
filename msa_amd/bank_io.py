"""On-disk format of a memory bank and its streaming loader.

Replaces ``Memory.serialize`` / ``Memory.deserialize`` (src/msa_service.py:351-479, a directory of
pickled ``.pt`` tensors).  A bank directory holds

* ``bank.json`` — version, dtype, ``Hkv``, ``D``, chunk and document counts, router layer ids,
  pooling size, scoring hyper-parameters, template length, every layer with a template prefix;
* ``doc_chunk_off.i32`` ``[n_docs + 1]``, ``doc_global_id.i64`` ``[n_docs]``, ``doc_num_chunks.i32``;
* per router layer ``layer_<i>.rk.bin``, ``.k.bin``, ``.v.bin`` — raw chunk-major ``[C, Hkv, D]``;
* ``docs.jsonl`` (optional) — one ``{"doc_id", "num_chunks", "doc"}`` object per document, bank order;
* ``prefix.bin`` — template-prefix K then V of every listed layer, ``[n_layers, 2, n_prefix, Hkv, D]``.

Raw little-endian arrays, so files can be memory-mapped and streamed layer by layer into pinned
host memory (K, V) and HBM (K_r) without ever holding more than one layer in pageable memory.
Nothing is unpickled.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Tuple

import numpy as np
import torch

FORMAT_VERSION = 1
_DTYPES = {"bfloat16": (torch.bfloat16, np.uint16), "float32": (torch.float32, np.float32)}


def _to_numpy(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    return t.view(torch.uint16).numpy() if t.dtype == torch.bfloat16 else t.numpy()


def _write(path: str, arr: np.ndarray) -> None:
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        arr.tofile(f)
    os.replace(tmp, path)


def save_bank(path: str, header: dict, doc_chunk_off, doc_global_id, rk: Dict[int, torch.Tensor],
              k: Dict[int, torch.Tensor], v: Dict[int, torch.Tensor],
              prefix: Dict[int, Tuple[torch.Tensor, torch.Tensor]]) -> None:
    """Writes a bank directory.  ``rk / k / v`` map router layer -> ``[C, Hkv, D]``; ``prefix`` maps
    layer -> ``(k, v) [1, Hkv, n_prefix, D]`` as the layer records them."""
    os.makedirs(path, exist_ok=True)
    layers = sorted(rk)
    ref = rk[layers[0]]
    name = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[ref.dtype]
    off = np.asarray(doc_chunk_off, dtype=np.int32)
    gid = np.asarray(doc_global_id, dtype=np.int64)
    C = int(off[-1])
    if tuple(ref.shape) != (C, ref.shape[1], ref.shape[2]):
        raise ValueError("pooled tensors must be [C, Hkv, D] with C = doc_chunk_off[-1]")
    _write(os.path.join(path, "doc_chunk_off.i32"), off)
    _write(os.path.join(path, "doc_global_id.i64"), gid)
    _write(os.path.join(path, "doc_num_chunks.i32"), np.diff(off).astype(np.int32))
    for layer in layers:
        for tag, store in (("rk", rk), ("k", k), ("v", v)):
            t = store[layer]
            if tuple(t.shape) != tuple(ref.shape) or t.dtype != ref.dtype:
                raise ValueError(f"layer {layer} {tag}: expected {tuple(ref.shape)} {ref.dtype}")
            _write(os.path.join(path, f"layer_{layer}.{tag}.bin"), _to_numpy(t))
    prefix_layers = sorted(prefix)
    n_prefix = prefix[prefix_layers[0]][0].shape[2] if prefix_layers else 0
    if prefix_layers:
        rows = [np.stack([_to_numpy(pk[0].transpose(0, 1)), _to_numpy(pv[0].transpose(0, 1))])
                for pk, pv in (prefix[l] for l in prefix_layers)]              # [2, n_prefix, Hkv, D] each
        _write(os.path.join(path, "prefix.bin"), np.stack(rows))
    meta = dict(header)
    meta.update({"format_version": FORMAT_VERSION, "dtype": name, "Hkv": int(ref.shape[1]), "D": int(ref.shape[2]),
                 "chunks": C, "docs": int(gid.shape[0]), "router_layers": layers, "prefix_layers": prefix_layers,
                 "n_prefix": int(n_prefix)})
    tmp = os.path.join(path, "bank.json.tmp")
    with open(tmp, "w") as f:
        json.dump(meta, f, indent=1)
    os.replace(tmp, os.path.join(path, "bank.json"))          # the header goes last: its presence marks a complete bank


class BankFiles:
    """Memory-mapped view of a bank directory."""

    def __init__(self, path: str):
        self.path = path
        with open(os.path.join(path, "bank.json")) as f:
            self.header = json.load(f)
        h = self.header
        if h.get("format_version") != FORMAT_VERSION:
            raise ValueError(f"unsupported bank format version {h.get('format_version')}")
        if h["dtype"] not in _DTYPES:
            raise ValueError(f"unsupported bank dtype {h['dtype']}")
        self.torch_dtype, self.np_dtype = _DTYPES[h["dtype"]]
        self.shape = (h["chunks"], h["Hkv"], h["D"])
        self.doc_chunk_off = np.fromfile(os.path.join(path, "doc_chunk_off.i32"), dtype=np.int32)
        self.doc_global_id = np.fromfile(os.path.join(path, "doc_global_id.i64"), dtype=np.int64)
        if self.doc_chunk_off.shape[0] != h["docs"] + 1 or int(self.doc_chunk_off[-1]) != h["chunks"]:
            raise ValueError("bank tables do not match the header")

    def layer(self, layer: int, tag: str) -> np.ndarray:
        f = os.path.join(self.path, f"layer_{layer}.{tag}.bin")
        want = int(np.prod(self.shape)) * np.dtype(self.np_dtype).itemsize
        if os.path.getsize(f) != want:
            raise ValueError(f"{f}: {os.path.getsize(f)} bytes, expected {want}")
        return np.memmap(f, dtype=self.np_dtype, mode="r", shape=self.shape)

    def copy_into(self, layer: int, tag: str, dst: torch.Tensor, rows_per_step: int = 1 << 16) -> None:
        """Streams one layer tensor into ``dst`` (pinned host or device) in slices of rows."""
        src = self.layer(layer, tag)
        for s in range(0, self.shape[0], rows_per_step):
            e = min(self.shape[0], s + rows_per_step)
            part = torch.from_numpy(np.array(src[s:e]))                 # a writable copy of the mapped slice
            if self.torch_dtype == torch.bfloat16:
                part = part.view(torch.bfloat16)
            dst[s:e].copy_(part)

    def prefix(self) -> Dict[int, Tuple[torch.Tensor, torch.Tensor]]:
        h = self.header
        if not h["prefix_layers"]:
            return {}
        arr = np.fromfile(os.path.join(self.path, "prefix.bin"), dtype=self.np_dtype).reshape(
            len(h["prefix_layers"]), 2, h["n_prefix"], h["Hkv"], h["D"])
        out = {}
        for i, layer in enumerate(h["prefix_layers"]):
            t = torch.from_numpy(arr[i].copy())
            if self.torch_dtype == torch.bfloat16:
                t = t.view(torch.bfloat16)
            out[layer] = (t[0].transpose(0, 1).unsqueeze(0), t[1].transpose(0, 1).unsqueeze(0))   # [1, Hkv, n, D]
        return out


def save_docs(path: str, docs) -> None:
    """Document texts and ids, one JSON object per line, in bank order."""
    tmp = os.path.join(path, "docs.jsonl.tmp")
    with open(tmp, "w") as f:
        for d in docs:
            f.write(json.dumps({"doc_id": int(d.doc_id), "num_chunks": int(d.num_chunks), "doc": d.doc}) + "\n")
    os.replace(tmp, os.path.join(path, "docs.jsonl"))


def load_docs(path: str):
    """Rows of ``docs.jsonl`` as dicts, or ``None`` when the bank was stored without texts."""
    f = os.path.join(path, "docs.jsonl")
    if not os.path.exists(f):
        return None
    with open(f) as fh:
        return [json.loads(line) for line in fh if line.strip()]


# --------------------------------------------------------------------------------------------------------------
# Banks the reference wrote (Memory.serialize, src/msa_service.py:351-404): a directory of ``layer_<i>_k.pt``,
# ``layer_<i>_v.pt``, ``layer_<i>_rk.pt`` (one pooled tensor each, ``[1, Hkv, C, D]``), ``prefix_cache.pt``
# (``{layer: (k, v)}``, ``[1, Hkv, n, D]``), ``meta.pt`` and ``stub.json``.  The tensor files are plain tensors and
# load with ``weights_only=True``; ``meta.pt`` pickles the reference's Document objects and is never opened here: the
# caller supplies the documents (ids and chunk counts, bank order), as the reference's own meta would.
# --------------------------------------------------------------------------------------------------------------
def _load_plain(path: str):
    return torch.load(path, map_location="cpu", weights_only=True)


def reference_bank_layers(path: str) -> List[int]:
    """Router layers a reference bank directory holds K_r for."""
    out = []
    for name in os.listdir(path):
        if name.startswith("layer_") and name.endswith("_rk.pt"):
            out.append(int(name[len("layer_"):-len("_rk.pt")]))
    return sorted(out)


def read_reference_layer(path: str, layer: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(rk, k, v)`` of one layer of a reference bank, chunk-major ``[C, Hkv, D]`` (the reference keeps
    ``[1, Hkv, C, D]``).  Whatever device the reference restored each of them to (its deserialize puts K on the
    GPU and leaves K_r on the host, :447-461, the reverse of where its scorer and gather read them), here all three
    come back as host tensors and the caller places them: K_r in HBM, K / V in pinned host memory."""
    out = []
    for tag in ("rk", "k", "v"):
        f = os.path.join(path, f"layer_{layer}_{tag}.pt")
        if not os.path.exists(f):
            raise FileNotFoundError(f"{f}: the reference bank has no {tag} for layer {layer}")
        t = _load_plain(f)
        if not isinstance(t, torch.Tensor) or t.dim() != 4 or t.shape[0] != 1:
            raise ValueError(f"{f}: expected one tensor [1, Hkv, C, D], got {type(t).__name__} "
                             f"{tuple(t.shape) if isinstance(t, torch.Tensor) else ''}")
        out.append(t[0].transpose(0, 1).contiguous())
    if not (out[0].shape == out[1].shape == out[2].shape):
        raise ValueError(f"layer {layer}: rk / k / v shapes differ: {[tuple(x.shape) for x in out]}")
    return out[0], out[1], out[2]


def read_reference_prefix(path: str) -> Dict[int, Tuple[torch.Tensor, torch.Tensor]]:
    """Template-prefix K / V of every layer, ``{layer: (k, v)}`` with ``[1, Hkv, n, D]`` tensors (empty if absent)."""
    f = os.path.join(path, "prefix_cache.pt")
    if not os.path.exists(f):
        return {}
    raw = _load_plain(f)
    return {int(layer): (kv[0], kv[1]) for layer, kv in raw.items()}


def convert_reference_bank(src: str, dst: str, docs, header: dict) -> None:
    """Converts a bank directory the reference wrote into this format (``save_bank``), one layer at a time.
    ``docs``: the documents in bank order (objects with ``doc_id``, ``num_chunks`` and optionally ``doc``);
    ``header``: the scoring / pooling hyper-parameters to record (see ``Memory.serialize``)."""
    counts = [int(d.num_chunks) for d in docs]
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    layers = reference_bank_layers(src)
    if not layers:
        raise ValueError(f"{src}: no layer_<i>_rk.pt files")
    rk, k, v = {}, {}, {}
    for layer in layers:
        rk[layer], k[layer], v[layer] = read_reference_layer(src, layer)
        if rk[layer].shape[0] != int(off[-1]):
            raise ValueError(f"layer {layer}: {rk[layer].shape[0]} chunks, the documents add up to {int(off[-1])}")
    os.makedirs(dst, exist_ok=True)
    save_docs(dst, docs)
    save_bank(dst, header, off.tolist(), [int(d.doc_id) for d in docs], rk, k, v, read_reference_prefix(src))
