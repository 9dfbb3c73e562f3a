"""Loads ``by_hand.json`` (see ``make_by_hand.py`` for how its numbers were derived) and builds its tensors."""
import json
import os

import numpy as np
import torch


def load():
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "by_hand.json")) as f:
        return json.load(f)


def _onehot(code: int, D: int, magnitude: float) -> torch.Tensor:
    v = torch.zeros(D)
    if code <= -100:                       # -100 - i means -e(i)
        v[-code - 100] = -magnitude
    else:
        v[code] = magnitude
    return v


def tensors(fx, dtype=torch.float32):
    """(q [B, S, Hq, D], mask [B, S] bool, kr [C, Hkv, D], doc_chunk_off np.int64)"""
    D, mag = fx["D"], fx["q_magnitude"]
    q = torch.stack([torch.stack([torch.stack([_onehot(c, D, mag) for c in tok]) for tok in qb]) for qb in fx["q_onehot"]])
    kr = torch.stack([torch.stack([_onehot(c, D, 1.0) for c in chunk]) for chunk in fx["kr_onehot"]])
    mask = torch.tensor(fx["mask"], dtype=torch.bool)
    return q.to(dtype), mask, kr.to(dtype), np.asarray(fx["doc_chunk_off"], dtype=np.int64)
