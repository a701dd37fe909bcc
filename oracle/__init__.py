"""CPU oracle for the paged-attention / FFN hot path.

TEST INFRASTRUCTURE ONLY.  Everything under ``oracle/`` is a CPU restatement
(plain torch on the host) of the torch golden functions that the reference
keeps next to its tile programs.  It is the checker the HIP path is compared
with; nothing in the product package imports it.  Allowed importers: the
``tests/`` tree, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``.

Pinning status (what fixes each function independently of its own formula):

* ``paged_gather``            — pinned: closed-form row-id known-answer case of
                                 the reference's own test plus permutation
                                 invariants (tests/test_oracle_attention.py).
* ``paged_attention_golden``  — pinned: fp64 brute-force loops on tiny shapes,
                                 ``torch.nn.functional.scaled_dot_product_attention``
                                 on gathered dense K/V, softmax invariants
                                 (uniform scores -> mean of V, dominant score ->
                                 that V row), partition independence.
* ``paged_attention_dynamic_golden`` / ``paged_attention_spmd_golden`` — the same
                                 block loop behind the reference's other two
                                 signatures; pinned: shape-derived config equals
                                 the explicit one, and an ``active_block_num`` of
                                 N equals contexts clipped to N blocks under the
                                 dense routine (tests/test_oracle_attention.py).
* ``stages.*``                — pinned: the reference's kernel-level known answers
                                 (all-ones scores -> m = scale, P = 1, l = block
                                 size; the four is_first / is_last cases on its
                                 constant state), and the block-by-block task
                                 loop built from them reproduces
                                 ``paged_attention_golden`` to 1e-4
                                 (tests/test_oracle_stages.py).
* ``ffn_swiglu`` / ``ffn_block`` — pinned: ``torch.nn.functional.silu`` form in
                                 fp64, committed seeded fixture.
* ``ffn_gelu`` / ``ffn_relu``  — pinned: the kernel's ``recip(1 + exp(-1.702 g))``
                                 form in fp64, the distance of that form to
                                 the erf GELU, ``clamp(min=0)``, and the two
                                 identities relu FFN(x) + relu FFN(-x) and
                                 gelu(g) - gelu(-g) = g
                                 (tests/test_oracle_ffn.py).
* ``rms_norm``                — pinned: ``torch.nn.functional.rms_norm``.
* ``rope_rotate_half``        — pinned: complex-rotation closed form, position-0
                                 identity, norm preservation, relative-position
                                 property.
* ``llama_mini_forward``      — pinned: dense causal attention against
                                 ``scaled_dot_product_attention(is_causal=True)``,
                                 first-token and zero-weight closed forms
                                 (tests/test_oracle_ffn.py).
* ``tile_ops.*``              — pinned: one meaning per op name of the hot
                                 programs (torch_codegen.py:954-1128), known
                                 answers for load padding, pad values, RNE casts,
                                 keepdim reductions and the 16-bit-rounded
                                 tile.matmul; the reference's kernels written op
                                 by op equal ``stages.*`` to the bit
                                 (tests/test_oracle_tile_ops.py).
* fp8-e4m3 KV and W8A16       — the reference has no such path; pinned by
                                 closed forms only (exhaustive 256-code table,
                                 integer matmul identity).
* ``quantize_rows_fp8`` / ``ffn_block_fp8`` — the reference has no 8-bit FFN:
                                 PARITY UNPINNED against it; pinned by the format
                                 only (rounding bound, row maximum on +-448,
                                 idempotence, exact small-integer case, distance
                                 to the 16-bit block; tests/test_oracle_ffn.py).
"""

from .attention import (  # noqa: F401
    decode_config,
    dequant_kv_fp8,
    paged_attention_dense,
    paged_attention_dynamic_golden,
    paged_attention_golden,
    paged_attention_spmd_golden,
    paged_attention_grouped_golden,
    paged_gather,
    quantize_kv_fp8,
)
from . import stages, tile_ops  # noqa: F401
from .ffn import (ffn_block, ffn_block_fp8, ffn_gelu, ffn_relu, ffn_swiglu, projection, quantize_rows_fp8, rms_norm,  # noqa: F401
                  swiglu)
from .layer import (  # noqa: F401
    decoder_layer_decode,
    kv_append_fp8,
    llama_mini_forward,
    quantize_w8,
    rope_cos_sin,
    rope_rotate_half,
    w8a16_matmul,
)
