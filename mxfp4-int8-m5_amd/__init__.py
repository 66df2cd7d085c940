"""scmx: MI355X-native SC-MXFP4 W4A8 linear-layer engine (dense prefill, grouped MoE GEMM, decode GEMV).

Modules keep the names of the reference's kernel call surface so model code can switch imports:
    sc_format   weight storage descriptor and bit packing
    sc_kernels  dense prefill kernels (unpack_i8, act_quant, mm_epi, rmsnorm_quant, ...)
    sc_moe      route_sort, moe_mm, moe_combine
    sc_decode   gemv
    sc_weights  PackedWeight, safetensors caches of packed weights, standard-MXFP4 scale export
    pack_format packing float weights into a member of the format family on the device
    fused_qwen3, fused_olmoe   model-level prefill / decode drivers (imported on demand)
All compute runs in libscmx.so (hand-written HIP for gfx950); importing the kernels without it raises."""
from . import _lib, sc_format, sc_kernels, sc_moe, sc_decode, sc_weights  # noqa: F401

__all__ = ["sc_format", "sc_kernels", "sc_moe", "sc_decode", "sc_weights"]
