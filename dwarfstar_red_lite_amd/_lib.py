"""Loads libredmetal_hip.so and declares the C ABI (include/*.h). There is no fallback: without the built HIP
library every entry point of this package raises."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# REDHIP_LIBRARY: another build of the same library (the one with phase stamps, build.py --timeline)
LIB_PATH = os.environ.get("REDHIP_LIBRARY") or os.path.join(HERE, "libredmetal_hip.so")


class RedHipError(RuntimeError):
    pass


class RouterTensorInfo(C.Structure):      # include/redmetal_router.h
    _fields_ = [("layer", C.c_uint32), ("ggml_type", C.c_uint32), ("n_dims", C.c_uint32), ("shape", C.c_uint64 * 8),
                ("tensor_offset", C.c_uint64), ("tensor_span_bytes", C.c_uint64)]


class RouterTelemetry(C.Structure):
    _fields_ = [("read_ms", C.c_double), ("compute_ms", C.c_double)]


class MoeConfig(C.Structure):             # include/redhip_moe.h
    _fields_ = [(n, C.c_uint32) for n in ("hidden", "ffn", "n_expert", "top_k", "n_layer", "max_tokens", "router_type",
                                          "expert_type_word", "shared_type_word", "reserved")]


class GgufExpertLayout(C.Structure):      # include/redhip_moe.h; the reference's rl_expert_layout (native/redlite_native_gguf.h:47-59)
    _fields_ = [(n, C.c_uint32) for n in ("layer", "expert", "ggml_type", "down_type")] + \
               [(n, C.c_uint64) for n in ("gate_offset", "gate_bytes", "up_offset", "up_bytes", "down_offset", "down_bytes", "total_bytes")]


# every symbol the headers declare: name -> (restype, argtypes)
u32, u64, vp, dbl, i32 = C.c_uint32, C.c_uint64, C.c_void_p, C.c_double, C.c_int
ABI = {
    "redmetal_ffn_abi_version": (u32, []),
    "redmetal_ffn_last_error": (C.c_char_p, []),
    "redmetal_ffn_pool_create": (vp, [C.c_char_p, u64, u64, u32, vp, u32, vp, u32]),
    "redmetal_ffn_pool_destroy": (None, [vp]),
    "redmetal_ffn_pool_capacity": (u32, [vp]),
    "redmetal_ffn_pool_slab_count": (u32, [vp]),
    "redmetal_ffn_pool_allocated_bytes": (u64, [vp]),
    "redmetal_ffn_pool_bytes_read": (u64, [vp]),
    "redmetal_ffn_pool_read_calls": (u64, [vp]),
    "redmetal_ffn_pool_read_ms": (dbl, [vp]),
    "redmetal_ffn_pool_slot_inflight": (i32, [vp, u32]),
    "redmetal_ffn_pool_load_expert": (i32, [vp, u32, u64, u64, u64, u64, u64, u64, C.POINTER(u64), C.POINTER(dbl)]),
    "redmetal_ffn_pool_slot_addresses": (i32, [vp, u32, u64, u64, u64, C.POINTER(u64), C.POINTER(u64), C.POINTER(u64)]),
    "redmetal_ffn_pool_execute_expert": (i32, [vp, u32, u32, u64, u64, u64, u32, u32, u32, u32, vp, u32, vp, u32, C.POINTER(dbl)]),
    "redmetal_ffn_pool_execute_expert_noalloc": (i32, [vp, u32, u32, u64, u64, u64, u32, u32, u32, u32, vp, u32, vp, u32, vp]),
    "redmetal_quant_abi_version": (u32, []),
    "redmetal_quant_last_error": (C.c_char_p, []),
    "redmetal_quant_rows": (i32, [C.c_char_p, u64, u64, u32, u32, u32, u32, u32, vp, u32, vp, u32, vp, u32, C.POINTER(dbl), C.POINTER(dbl)]),
    "rl_native_router_gpu_f32": (i32, [C.c_char_p, C.POINTER(RouterTensorInfo), vp, u32, vp, u32, C.POINTER(RouterTelemetry), C.c_char_p, C.c_size_t]),
    "rl_native_router_select_softmax_topk": (i32, [vp, u32, u32, vp, vp, vp, C.c_char_p, C.c_size_t]),
    "redhip_moe_abi_version": (u32, []),
    "redhip_moe_last_error": (C.c_char_p, []),
    "redhip_moe_create": (vp, [C.POINTER(MoeConfig)]),
    "redhip_moe_destroy": (None, [vp]),
    "redhip_moe_resident_bytes": (u64, [vp]),
    "redhip_moe_load_router": (i32, [vp, u32, vp, u64]),
    "redhip_moe_load_shared": (i32, [vp, u32, vp, vp, u64, vp, u64, vp, u64]),
    "redhip_moe_load_experts": (i32, [vp, u32, u32, u32, vp, vp, vp]),
    "redhip_gguf_last_error": (C.c_char_p, []),
    "redhip_gguf_moe_config": (i32, [C.c_char_p, u32, C.POINTER(MoeConfig)]),
    "redhip_moe_load_gguf": (i32, [vp, C.c_char_p, u32, u32, C.POINTER(MoeConfig)]),
    "redhip_gguf_expert_layout": (i32, [C.c_char_p, u32, u32, u32, C.POINTER(GgufExpertLayout)]),
    "redhip_moe_forward": (i32, [vp, u32, vp, u32, vp, vp]),
    "redhip_moe_forward_block": (i32, [vp, u32, vp, vp, vp, C.c_float, u32, vp, vp]),
    "redhip_moe_route": (i32, [vp, u32, vp, u32, vp, vp, vp, vp]),
    "redhip_moe_experts": (i32, [vp, u32, vp, u32, vp, vp, vp, vp]),
    "redhip_moe_last_route": (i32, [vp, u32, vp, vp, vp, vp]),
    "redhip_moe_group": (i32, [vp, vp, vp, u32, vp, vp, vp, vp, vp, vp, vp]),
    "redhip_set_codebooks": (i32, [vp, u32, vp, u32]),
    "redhip_dequant_rows": (i32, [u32, vp, u32, u32, vp, vp]),
    "redhip_moe_dequant_resident": (i32, [vp, u32, u32, u32, vp, vp]),
    "redhip_gemv_rows": (i32, [u32, vp, u32, u32, u32, vp, vp, vp]),
    "redhip_profile_stage_count": (u32, []),
    "redhip_profile_stage_name": (C.c_char_p, [u32]),
    "redhip_profile_begin": (i32, []),
    "redhip_profile_end": (i32, [C.POINTER(dbl), C.POINTER(u32), u32]),
    "redhip_timeline_read": (i32, [C.POINTER(u64), u32, u32]),
    "redhip_calibration_copy": (i32, [vp, vp, u64, vp]),
    "redhip_calibration_empty": (i32, [u32, u32, vp]),
    "redhip_calibration_read": (i32, [vp, u64, vp, vp]),
    "redhip_calibration_mfma": (i32, [u32, u32, vp, C.POINTER(C.c_uint64), vp]),
    # include/redmetal_topk.h
    "redmetal_topk_abi_version": (u32, []),
    "redmetal_topk_last_error": (C.c_char_p, []),
    "redmetal_topk_pool_create": (vp, [C.c_char_p, u64, u64, u32, vp, u32, vp, u32]),
    "redmetal_topk_pool_destroy": (None, [vp]),
    "redmetal_topk_pool_set_classes": (i32, [vp, u32, vp, vp]),
    "redhip_topk_pool_enable_fast_path": (i32, [vp, u32, u32, u32, u32]),
    "redmetal_topk_pool_capacity": (u32, [vp]),
    "redmetal_topk_pool_slab_count": (u32, [vp]),
    "redmetal_topk_pool_allocated_bytes": (u64, [vp]),
    "redmetal_topk_pool_bytes_read": (u64, [vp]),
    "redmetal_topk_pool_read_calls": (u64, [vp]),
    "redmetal_topk_pool_read_ms": (dbl, [vp]),
    "redmetal_topk_pool_slot_generation": (u32, [vp, u32]),
    "redmetal_topk_pool_slot_inflight": (i32, [vp, u32]),
    "redmetal_topk_pool_load_expert": (i32, [vp, u32, u64, u64, u64, u64, u64, u64, C.POINTER(u64), C.POINTER(dbl)]),
    "redmetal_topk_pool_slot_addresses": (i32, [vp, u32, u64, u64, u64, C.POINTER(u64), C.POINTER(u64), C.POINTER(u64)]),
    "redmetal_topk_pool_execute": (i32, [vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp, u32, vp, u32, C.POINTER(dbl)]),
    "redmetal_topk_pool_encode": (i32, [vp, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp, u64, vp, u64]),
    "redmetal_topk_pool_release": (None, [vp, vp, u32]),
    "redmetal_topk_pool_residency_table_init": (i32, [vp, u32, u32]),
    "redmetal_topk_pool_residency_table": (vp, [vp]),
    "redmetal_topk_pool_residency_set": (i32, [vp, u32, u32, u32]),
    "redmetal_topk_pool_residency_clear": (None, [vp, u32, u32]),
    "redmetal_topk_pool_slab_residency_set": (vp, [vp]),
    "redmetal_topk_pool_allocate_all": (i32, [vp]),
    "redmetal_topk_pool_use_all_slabs": (None, [vp, vp]),
    "redmetal_topk_pool_tmp_buffer": (vp, [vp]),
    "redmetal_topk_pool_encode_device": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, u32, u32, u64, u64, vp, u64, vp, u64]),
    "redmetal_topk_pool_encode_device_into": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, u32, u32, u64, u64, vp, u64, vp, u64]),
    "redmetal_topk_pool_encode_device_into2": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, u32, u32, u64, u64, vp, u64, vp, u64, vp, u64, u32]),
    "redmetal_topk_pool_encode_device_tail": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, u32, u32, u64, u64, vp, u64, vp, vp, vp, vp, vp, u64]),
    "redmetal_topk_pool_encode_batched": (i32, [vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, u32, u32, vp, vp, vp, vp, vp, u64, vp, u64]),
    "redmetal_topk_pool_encode_mapped": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u64, u64, u64, vp, u32, u32, u32, u32, u32, u32, u32, u32, vp, vp, vp, vp, vp, u64, vp, u64]),
}

_lib = None


def load():
    """The shared library with argtypes set. Raises RedHipError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.isfile(LIB_PATH):
            raise RedHipError("HIP library not found at %s: run `python -m dwarfstar_red_lite_amd.build`" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in ABI.items():
            fn = getattr(lib, name)          # AttributeError here = header/library mismatch
            fn.restype = res
            fn.argtypes = args
        for fam in ("redmetal_ffn", "redmetal_quant", "redmetal_topk", "redhip_moe"):
            if getattr(lib, fam + "_abi_version")() != 1:
                raise RedHipError("unsupported %s ABI version" % fam)
        _lib = lib
    return _lib
