"""Writes ``by_hand.json``: a routing / pooling case small enough that every expected number below was
worked out with pencil and paper (one-hot unit vectors make every cosine 0, 1 or -1).  Nothing here calls
the oracle or the library: the file pins both from outside.  Re-run after editing: ``python make_by_hand.py``.

Layout.  Hkv = 2 KV heads, G = 2 query heads per KV head (Hq = 4), D = 128.  e(i) is the one-hot vector at i.
Bank: 3 documents with 2, 1, 3 chunks (doc_chunk_off 0, 2, 3, 6); chunk c has K_r = (e(a), e(b)) for KV heads 0, 1.
Query heads 0, 1 read KV head 0 and heads 2, 3 read KV head 1; a query head is 2 * e(i) or -2 * e(i).
score(b, c) = max over scored tokens of mean over the 4 heads of cos(q head, its K_r head).
"""
import json
import os

KR = [(0, 1), (2, 3), (0, 3), (4, 5), (2, 1), (6, 7)]          # chunk -> (index for KV head 0, for KV head 1)
DOC_CHUNK_OFF = [0, 2, 3, 6]
# query b, token t -> 4 signed indices (sign = direction of the one-hot); magnitude 2 everywhere
Q = [
    [[+0, +0, +1, +1], [+2, +9, +3, +9], [+6, +6, +7, +7]],      # query 0; its token 2 is masked out
    [[+4, +4, +5, +5], [+6, +0, +7, +3], [-100, -100, -101, -101]],   # -100 means -e(0), -101 means -e(1)
]
MASK = [[1, 1, 0], [1, 1, 1]]
# by hand: per token the mean of the four 0 / 1 / -1 cosines, then the max over the scored tokens
CHUNK_SCORES = [
    [1.0, 0.5, 0.5, 0.0, 0.5, 0.0],       # q0: t0 hits c0 fully, c2 and c4 by half; t1 gives c1 0.5 (c2, c4 0.25); t2 masked
    [0.25, 0.25, 0.5, 1.0, 0.0, 0.5],     # q1: t0 hits c3; t1 gives c5 0.5, c2 0.5, c0 and c1 0.25; t2 only gives negatives
]
DOC_SCORES = [[1.0, 0.5, 0.5], [0.25, 0.5, 1.0]]                # max over each document's chunks
TOP2 = [[0, 1], [2, 1]]                                          # q0: documents 1 and 2 tie at 0.5 -> the lower id
TOP3 = [[0, 1, 2], [2, 1, 0]]
SCALED_DOT_FACTOR = 2.0 * 128 ** -0.5                            # |q head| = 2, scale = D^-0.5: scores = cosines * this

# pooling: 2 documents of 3 and 5 tokens, chunk size 4, every element of token t equals t + 1
POOL = {"doc_lens": [3, 5], "P": 4, "chunk_start": [0, 3, 7], "chunk_len": [3, 4, 1], "chunk_doc": [0, 1, 1],
        "doc_chunk_off": [0, 1, 3], "chunk_mean": [2.0, 5.5, 8.0], "normalized_element": 128 ** -0.5}

# gather: a sample that selected documents (2, 0) gets the chunks of 0 then 2, each once
GATHER = {"selected": [[2, 0], [1, 1]], "chunks": [[0, 1, 3, 4, 5], [2]], "cu_sel": [0, 5, 6]}
# positions: 3 template tokens + top_k documents come first; left padding repeats the first position
POSITIONS = {"n_query": 3, "top_k": 2, "n_prefix": 3, "left_pad": 2, "position_ids": [5, 5, 5, 6, 7]}

if __name__ == "__main__":
    out = {"Hq": 4, "Hkv": 2, "D": 128, "kr_onehot": KR, "doc_chunk_off": DOC_CHUNK_OFF, "q_onehot": Q, "q_magnitude": 2.0,
           "mask": MASK, "chunk_scores_cosine": CHUNK_SCORES, "doc_scores_cosine": DOC_SCORES, "top2": TOP2, "top3": TOP3,
           "scaled_dot_factor": SCALED_DOT_FACTOR, "pool": POOL, "gather": GATHER, "positions": POSITIONS}
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "by_hand.json"), "w") as f:
        json.dump(out, f, indent=1)
