"""flash_bla for AMD MI355X (gfx950): bidirectional linear-attention operators.

Same module paths and call signatures as fla-org/flash-bidirectional-linear-attention
(``flash_bla.ops.linear_attn.fused.linear_attention`` and friends); the kernels
underneath are hand-written HIP reached through the C ABI of ``libfbla_hip.so``.
"""
__version__ = "0.2+gfx950"
