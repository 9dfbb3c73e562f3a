"""Writes a small bank directory in the file layout of the reference's ``Memory.serialize``
(src/msa_service.py:384-404): ``layer_<i>_k.pt``, ``layer_<i>_v.pt``, ``layer_<i>_rk.pt`` holding one
``[1, Hkv, C, D]`` tensor each and ``prefix_cache.pt`` holding ``{layer: (k, v)}``.  The tensors come from a seeded
generator, so a reader can be checked against ``expected()``.  (``meta.pt`` is written as an opaque placeholder: a
reader must not need it.)

    python tests/golden/make_reference_style_bank.py <directory>
"""
import os
import sys

import torch

LAYERS = [18, 19]
HKV, D, N_PREFIX = 2, 128, 3
DOC_CHUNKS = [3, 1, 4, 2]
DOC_IDS = [11, 7, 42, 5]


def expected(dtype=torch.bfloat16):
    """``{layer: {"rk" | "k" | "v": [1, Hkv, C, D]}}`` and ``{layer: (k, v) [1, Hkv, n, D]}``."""
    g = torch.Generator().manual_seed(1234)
    C = sum(DOC_CHUNKS)
    layers = {l: {t: torch.randn((1, HKV, C, D), generator=g).to(dtype) for t in ("rk", "k", "v")} for l in LAYERS}
    prefix = {l: (torch.randn((1, HKV, N_PREFIX, D), generator=g).to(dtype),
                  torch.randn((1, HKV, N_PREFIX, D), generator=g).to(dtype)) for l in range(LAYERS[-1] + 1)}
    return layers, prefix


def write(path: str, dtype=torch.bfloat16) -> None:
    os.makedirs(path, exist_ok=True)
    layers, prefix = expected(dtype)
    for l, tensors in layers.items():
        for tag, t in tensors.items():
            torch.save(t, os.path.join(path, f"layer_{l}_{tag}.pt"))
    torch.save(prefix, os.path.join(path, "prefix_cache.pt"))
    with open(os.path.join(path, "meta.pt"), "wb") as f:
        f.write(b"not read by the converter")
    with open(os.path.join(path, "stub.json"), "w") as f:
        f.write('{"memory_file_path": "", "world": [0]}')


if __name__ == "__main__":
    write(sys.argv[1])
