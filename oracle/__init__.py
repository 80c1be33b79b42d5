"""CPU oracles for the TileFusion hot path (TEST INFRASTRUCTURE, never a product path).

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
package.  The product (tilefusion_amd) never does: it fails loudly when the HIP library is
missing.

Every oracle works in fp32 on the CPU on the fp16-rounded inputs, so the GPU kernels and the
oracle consume bit-identical operands.

Pinning status (what independent check guards each function against a dropped term, wrong
sign/index or transposed operand):

* gemm_ref / fused_two_gemms_ref  - torch.matmul (library routine) cross-checked against the
  naive triple loop in oracle/naive_gemm.c (restating tests/cpp/cell/test_single_wmma.cu:20-33)
  and against hand-computed small cases.
* attention_ref - textbook softmax(scale QK^T + mask) V; pinned by invariants (rows of P sum
  to 1, causal row 0 == V[0], all-equal keys -> mean(V)) and by the blockwise online-softmax
  restatement (tests/python/test_flash_attn.py:85-134 as text, with -inf init and a global
  causal mask) which must agree to 1e-5.
* flash_decode_ref / split_kv_partials / combine_partials - q_len = 1 closed form; the
  split + log-sum-exp combine identity is pinned against the direct form for random split
  counts.  These have NO counterpart in the reference (it has no decoding kernel).
* scatter_nd_ref - torch index_put_(accumulate=True) (library routine), pinned against a
  hand-written loop on a tiny case in tests/test_oracle_numerics.py.
* layout oracles (oracle/layout.py) - pinned by the reference's integer known answers
  (tests/cpp/types/test_layout.cu, test_swizzle.cu, test_gtile_iterator.cu,
  test_warp_base_tile_shape.cu), restated in tests/test_oracle_layout.py.
"""

from .inputs import (  # noqa: F401
    make_c1_gemm_inputs,
    make_c2_gemm_inputs,
    make_c3_fused_inputs,
    make_c4_attention_inputs,
    make_c5_decode_slice,
    SEEDS,
)
from .numerics import (  # noqa: F401
    gemm_ref,
    fused_two_gemms_ref,
    fused_two_gemms_ref_rounded,
    attention_ref,
    scatter_nd_ref,
    attention_blockwise_ref,
    flash_decode_ref,
    split_kv_partials,
    combine_partials,
    rel_l2,
    max_abs,
    check_close,
    REL_L2_TOL,
    MAX_ABS_TOL,
)
