"""MI355X (gfx950) implementation of BitMTP's packed low-bit GEMV hot path:
T2-g128 ternary and Q1-g128 sign weights times per-token INT8 activations."""
from . import contracts  # noqa: F401
from .ops import (  # noqa: F401
    OUT_BF16, OUT_F32, OUT_G32,
    init_kernels, last_kernel, launch_count, load_actq_kernel, load_q1_kernel, load_t2_kernel,
    packed_gemv_ex, packed_gemv_fused, packed_gemv_grouped, packed_int8_linear, q1g128_int8xint1_linear, q1g128_w1a16_linear,
    quant_input, t2g128_int8xint2_linear,
    add_rmsnorm, fused_add_norm_quant, fused_norm_quant, silu_mul_quant, fused_parts,
)
from .packing import (  # noqa: F401
    merge_packed_rows, pack_q1_g128, pack_t2_g128, unpack_q1_g128, unpack_t2_g128,
)

__all__ = [
    "contracts", "init_kernels", "last_kernel", "launch_count", "load_actq_kernel", "load_q1_kernel", "load_t2_kernel",
    "packed_gemv_ex", "packed_gemv_fused", "packed_gemv_grouped", "fused_parts", "packed_int8_linear", "q1g128_int8xint1_linear", "q1g128_w1a16_linear",
    "quant_input", "t2g128_int8xint2_linear", "pack_q1_g128", "pack_t2_g128",
    "unpack_q1_g128", "unpack_t2_g128", "OUT_BF16", "OUT_F32", "OUT_G32",
    "add_rmsnorm", "fused_add_norm_quant", "fused_norm_quant", "silu_mul_quant", "merge_packed_rows",
]
