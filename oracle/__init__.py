"""CPU oracle for the fused VQ-attention path.  TEST INFRASTRUCTURE ONLY.

Everything in this package is a plain fp32 PyTorch/numpy restatement of the
reference algorithms (each function cites the reference file:line it follows).
It exists to CHECK the HIP kernels, never to stand in for them: only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it.  The product package `vqtree_amd` must not import it and raises when its
HIP library is missing.

Pinning status (see tests/test_oracle_pins.py):
  * naive / windowed VQ attention, decode        : pinned (torch SDPA, per-query brute force, closed forms)
  * strict / loose / ReRoPE-local window masks   : pinned (SDPA with explicit masks, brute-force double loops)
  * full ReRoPE attention                        : pinned (window >= N reduces to SDPA; rotary shift identity)
  * base-2 LSE merge (third-party flashinfer op) : pinned by closed form only (merge of a key partition ==
                                                   softmax over the union); no reference vectors exist
  * count-based far kernel + sort preprocessing  : pinned (brute-force segment sums, M=1 identity with the
                                                   per-key formulation)
  * multi_head_single_quantize                   : pinned (brute-force argmax, first-max tie rule)
  * encode_residual (greedy additive encoder)    : pinned (brute-force nearest neighbour per stage; no reference
                                                   counterpart exists at run time)
"""
from .attention import (  # noqa: F401
    LOG2E,
    T_BLOCK,
    attend,
    attn_vq_decode,
    attn_vq_prefill,
    far_boundary,
    local_attn,
    local_visible_mask,
    merge_state,
    rerope_full,
    slow_reference,
    vq_scores_lut,
    vq_scores_reconstruct,
)
from .rope import apply_rope, rope_tables, rotate_half  # noqa: F401
from .vq import (  # noqa: F401
    encode_residual,
    multi_head_single_quantize,
    reconstruct_keys,
    sort_based_preprocess,
    vq_attn_forward,
    vq_count_forward,
)
