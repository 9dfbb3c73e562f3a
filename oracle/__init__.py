"""CPU oracle for the MSA routing / sparse-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``msa_amd``) may
import, call or link anything in this directory; only the tests, the smoke
check and the benchmark's ``cpu_baseline`` leg do, and there only as the
checker.

Two restatements of the reference algorithm live here:

``closed_form``
    fp64 definitions written from the mathematics of the path (segmented mean,
    half-split rotary, cosine / scaled-dot scoring with mean-over-heads,
    max-over-tokens, max-over-chunks, full-sort top-k, integer-exact gather,
    naive softmax attention).  This is the parity checker.

``reference_style``
    the same torch op sequence the reference executes (cumsum-difference
    pooling, matmul -> masked_fill -> mean -> max -> scatter_reduce -> topk,
    index_select gather with match-matrix regroup, cat + repeat_kv + SDPA
    decode).  This is the CPU baseline that gets timed, and a second reading
    of the semantics that must agree with ``closed_form``.

Pin status.  The reference ships no tests, golden vectors or fixtures for this
path, and its third-party arithmetic (torch matmul/topk/cumsum, flash-attn,
transformers rotary) is absent at the pinned versions.  Every function is
therefore pinned by mathematics instead (``tests/test_oracle_*.py``): library
special cases (``view(-1,P).mean`` for whole chunks, ``torch.sort`` for top-k,
``F.scaled_dot_product_attention`` for attention), closed forms (constant
input, planted needles, single key), invariants (RoPE relative-position
property, GQA pre-sum identity, permutation equivariance) and agreement of the
two independent restatements with each other.
"""
