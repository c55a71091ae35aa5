"""ctypes binding of libspark_shim_hip.so: the C ABI declared in include/spark_shim.h.

The library is the product; there is no CPU fallback.  Loading fails loudly when the shared object is missing.
"""
import ctypes as C
from pathlib import Path

PKG = Path(__file__).resolve().parent
SO = PKG / "libspark_shim_hip.so"

vp, i32, i64, f32, sz, ll = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t, C.c_longlong

# name -> (restype, argtypes); the stream argument (hipStream_t) is always last and passed as void*
SIGNATURES = {
    # dequantisation surfaces
    "spark_exl3_reconstruct": (i32, [vp, vp, i32, i32, i32, i32, vp]),
    "qwen_exl3_reconstruct": (i32, [vp, vp, i32, i32, i32, vp]),
    "spark_exl3_fold": (i32, [vp, vp, vp, i32, i32, i32, i32, vp, i64, vp]),
    "qwen_exl3_fold": (i32, [vp, vp, vp, i32, i32, i32, vp, i64, vp]),
    "qwen_exl3_had_in": (i32, [vp, i32, i64, vp, vp, i32, i32, vp]),
    "qwen_exl3_had_multi": (i32, [vp, i64, i32, i32, i32, vp, vp, vp]),
    "qwen_exl3_gemv": (i32, [vp, vp, vp, i32, i32, i32, i32, i32, vp]),
    "qwen_exl3_finish": (i32, [vp, i32, vp, vp, i32, i64, i32, i32, vp]),
    "qwen_exl3_finish_h": (i32, [vp, vp, vp, i64, i32, i32, vp]),
    "qwen_exl3_linear": (i32, [vp, i64, vp, vp, vp, vp, vp, i64, vp, i32, i32, i32, i32, i32, vp]),
    "qwen_exl3_multi": (i32, [vp, i64, vp, vp, vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp]),
    "spark_mxfp4_dequant": (i32, [vp, vp, vp, i32, i32, vp]),
    "spark_fp8_block_dequant": (i32, [vp, vp, vp, i32, i32, i32, vp]),
    "spark_fp8_e8m0_dequant": (i32, [vp, vp, vp, i32, i32, vp]),
    # activation quantisation and shared-expert glue
    "ds41_act_quant32": (i32, [vp, vp, ll, vp]),
    "ds41_act_quant_fp8": (i32, [vp, vp, vp, ll, vp]), "ds41_requant_fp8": (i32, [vp, vp, vp, vp, ll, vp]),
    "ds41_swiglu_quant": (i32, [vp, vp, i32, i32, f32, vp]),
    "qwen_moe_silu_mul": (i32, [vp, vp, vp, i32, vp]),
    "qwen_moe_gate_scale": (i32, [vp, i64, i32, vp, vp, i32, i32, vp]),
    # routers
    "spark_softmax_route": (i32, [vp, i64, i32, i32, i32, vp, vp, vp]),
    "qwen_moe_route": (i32, [vp, i32, vp, vp, vp]),
    "qwen_moe_route_ld": (i32, [vp, i64, i32, vp, vp, vp]),
    "ds41_route": (i32, [vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    "spark_sigmoid_route": (i32, [vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    "glm53_router_split": (i32, []),
    "glm53_router_fused_cuda": (i32, [vp, vp, i32, vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    "glm53_router_fused_h_cuda": (i32, [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, f32, vp]),
    # dense GEMVs
    "ds41_mxfp4_gemv": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "ds41_fp8_gemv": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "ds41_fp8_gemv_ex": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]),
    "ds41_fp8_gemv_bx": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]),
    "ds41_fp8_gemv_mx_init": (i32, []), "ds41_fp8_gemv_mx_smem_max": (sz, []),
    "ds41_fp8_gemv_mx_q": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "spark_fp8_block128_gemv": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "spark_fp8_t16_pack": (i32, [vp, vp, i32, i32, vp]),
    "spark_fp8_block128_gemv_t16": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "spark_fp8_e8m0_gemv_t16": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "spark_debug_rm_span": (None, [i32]),
    "ds41_bf16_gemv": (i32, [vp, vp, vp, i32, i32, i32, vp]), "ds41_bf16_gemv_mx": (i32, [vp, vp, vp, i32, i32, i32, vp]),
    # MXFP4 MoE
    "spark_mxfp4_packed_bytes": (sz, [ll, i32]),
    "spark_mxfp4_prepack": (i32, [vp, vp, vp, ll, i32, vp]),
    "spark_mxfp4_moe_ws_bytes": (sz, [i32, i32, i32, i32, i32, i32]),
    "spark_mxfp4_moe_q": (i32, [vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp]),
    "spark_mxfp4_moe": (i32, [vp, vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp]),
    "spark_mxfp4_moe_ws_init": (i32, [vp, sz, vp]),
    "spark_mxfp4_moe_x": (i32, [vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp, i32, vp]),
    "ds41_moe_mx_set_s2": (None, [i32]), "ds41_moe_mx_get_s2": (i32, []), "ds41_moe_gr16_max": (None, [i32]),
    "ds41_moe_mx_col_passes": (i32, [i32, i32, i32]), "ds41_moe_mx_pair_b16": (i32, [i32, i32, i32]),
    "ds41_moe_mx_ws_bytes": (sz, [i32, i32, i32, i32]), "ds41_moe_ws_bytes": (sz, [i32, i32, i32, i32]),
    "ds41_moe_mx_ex": (i32, [vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, i32, i32, vp]),
    "ds41_moe_mx": (i32, [vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, i32, vp]),
    "ds41_moe_mx_combine_rows": (i32, [vp, i32, i32, i32, i32, vp, vp, i32, i32, vp]),
    "ds41_moe_mx_combine": (i32, [vp, i32, i32, i32, i32, vp, vp, vp]),
    "ds41_moe_mx_ws_ptrs": (i32, [vp, i32, i32, i32, i32, C.POINTER(vp), C.POINTER(vp)]),
    "ds41_moe": (i32, [vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, i32, vp]),
    # EXL3 MoE
    "spark_exl3_moe_ws_bytes": (sz, [i32, i32, i32, i32, i32]),
    "spark_exl3_moe": (i32, [vp, i32, i64, i32, vp, i32, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp]),
    "spark_exl3_moe_ws_init": (i32, [vp, sz, vp]),
    "spark_exl3_moe_static": (i32, [vp, i32, i64, i32, vp, i32, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]),
    "qwen_moe_ws_bytes": (sz, [i32, i32]),
    "qwen_moe_experts": (i32, [vp, i64, i32, vp, vp, vp, vp, vp, vp, i32, vp]),
    "glm_moe_ws_bytes": (sz, [i32, i32]),
    "glm_moe_experts": (i32, [vp, i64, i32, vp, vp, vp, vp, vp, vp, i32, vp, i32, vp]),
    "glm_moe3_ws_bytes": (sz, [i32, i32]),
    "glm_moe3_experts": (i32, [vp, i64, i32, vp, vp, vp, vp, vp, vp, i32, i32, vp]),
    # weight-only FP8 with a scale per output row (the GLM dense projections)
    "glm53_fp8_dense_cuda": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]),
    "glm53_fp8_bf16_cuda": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "glm53_fp8_bf16_skinny_cuda": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    # single-launch workspaces
    "spark_moe_ws_status": (i32, [vp, vp]), "spark_exl3_moe_static_status": (i32, [vp]),
    "spark_moe_ws_release": (None, [vp]),
    # diagnostics
    "spark_debug_mx_pair_b16": (None, [i32]),
    "spark_debug_stream_read": (i32, [vp, sz, vp, vp]),
    "spark_debug_mx_ws_h": (i32, [vp, i32, i32, i32, i32, i32, i32, vp, vp, vp]),
    "spark_debug_exl3_local": (None, [i32]), "spark_debug_mx_local": (None, [i32]), "spark_debug_exl3_twa": (None, [i32]),
    "spark_debug_mx_out_cap": (None, [sz]), "spark_debug_validate_routes": (None, [i32]), "spark_mxfp4_moe_path": (i32, [i32] * 7), "spark_exl3_moe_path": (i32, [i32] * 6), "spark_debug_mx_fused_rows": (None, [i32]), "spark_debug_placement": (i32, []), "spark_debug_gemv_rows": (None, [i32]), "spark_debug_fp8q_rowmajor": (None, [i32]),
}

_lib = None


def load():
    """The loaded library with every declared symbol typed.  Raises if the shared object or a symbol is missing."""
    global _lib
    if _lib is None:
        if not SO.exists():
            raise RuntimeError(f"{SO} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` (hipcc, gfx950) first")
        lib = C.CDLL(str(SO))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)          # AttributeError names a missing export
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib
