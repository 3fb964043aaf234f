"""ctypes binding of the C-ABI library (include/xlite_hip.h). No fallback: if the shared object
is missing the import of any operator fails loudly."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libxlite_hip.so")

_vp, _u32, _u64, _i32, _f32, _sz = (ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int,
                                    ctypes.c_float, ctypes.c_size_t)

# name -> (restype, argtypes); the exported symbols of include/xlite_hip.h
SIGNATURES = {
    "xlite_hip_last_error": (ctypes.c_char_p, []),
    "xlite_hip_version": (_i32, []),
    "xlite_hip_device_info": (_i32, [_i32, _vp, _vp, _vp, _sz]),
    "xlite_hip_rope_and_cache": (_i32, [_vp] * 7 + [_u32] * 6 + [_i32, _u64, _u64, _i32]),
    "xlite_hip_attention_workspace_bytes": (_sz, [_u32] * 7),
    "xlite_hip_attention_workspace_bytes_kv": (_sz, [_u32] * 7 + [_i32]),
    "xlite_hip_attention": (_i32, [_vp] * 9 + [_u32] * 7 + [_i32, _i32, _vp, _vp, _vp, _sz]),
    "xlite_hip_set_clock_probe": (_i32, [_vp]),
    "xlite_hip_decode_step": (_i32, [_vp] * 12 + [_u32] * 8 + [_i32, _u64, _u64, _i32, _vp, _sz]),
    "xlite_hip_attention_noalloc_scratch_bytes": (_sz, []),
    "xlite_hip_attention_noalloc": (_i32, [_vp] * 9 + [_u32] * 7 + [_i32, _i32, _vp, _vp]),
    "xlite_hip_mla_workspace_bytes": (_sz, [_u32] * 8),
    "xlite_hip_mla_attention": (_i32, [_vp] * 10 + [_u32] * 7 + [_f32, _vp, _u32, _i32, _vp, _sz]),
    "xlite_hip_mla_v3": (_i32, [_vp] * 9 + [_u32] * 6 + [_f32, _i32, _vp, _sz]),
    "xlite_hip_gather_sparse_kv_cache": (_i32, [_vp] * 9 + [_u32] * 7 + [_i32]),
    "xlite_hip_rope_complex": (_i32, [_vp] + [_u32] * 4 + [_vp] * 4 + [_i32]),
    "xlite_hip_mla_prepare": (_i32, [_vp] * 10 + [_u32] * 5 + [_vp] * 3 + [_f32, _i32]),
    "xlite_hip_einsum_mht_mhd": (_i32, [_vp] * 4 + [_u32] * 5 + [_i32, _i32]),
    "xlite_hip_get_tile_size_of_cached_kv": (_i32, [_vp, _vp] + [_u32] * 5),
    "xlite_hip_prepare_attn": (_i32, [_vp, _vp, _u32, _vp, _vp, _u32, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp]),
    "xlite_hip_quantize_kv": (_i32, [_vp] * 4 + [_u64, _u32, _i32, _i32]),
    "xlite_hip_quantize_kv_int8": (_i32, [_vp] * 4 + [_u64, _u32, _i32]),
    "xlite_hip_rope_and_cache_quant": (_i32, [_vp] * 9 + [_u32] * 6 + [_i32, _u64, _u64, _i32, _i32]),
    "xlite_hip_rope_and_cache_int8": (_i32, [_vp] * 9 + [_u32] * 6 + [_i32, _u64, _u64, _i32]),
    "xlite_hip_qk_rms_norm": (_i32, [_vp] * 7 + [_u32] * 7 + [_f32, _i32]),
    "xlite_hip_indexer_scores": (_i32, [_vp] * 9 + [_u32] * 6 + [_i32]),
    "xlite_hip_indexer_topk_workspace_bytes": (_sz, [_u32] * 3),
    "xlite_hip_indexer_topk": (_i32, [_vp] * 10 + [_u32] * 7 + [_i32, _vp, _sz]),
    "xlite_hip_layernorm": (_i32, [_vp] * 5 + [_u32] * 4 + [_f32, _i32]),
    "xlite_hip_muls": (_i32, [_vp] * 3 + [_u32] * 4 + [_f32, _i32]),
    "xlite_hip_rope_complex_and_cache": (_i32, [_vp] + [_u32] * 6 + [_vp, _vp, _u32, _u32, _vp, _vp, _u32, _vp, _vp, _i32]),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "gvirt_amd: %s is not built; run `python -m gvirt_amd.build` (needs hipcc)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the library misses a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int) -> None:
    """Turn a negative return code into the RuntimeError the reference raises from C++."""
    if rc != 0:
        msg = load().xlite_hip_last_error()
        raise RuntimeError(msg.decode() if msg else "xlite_hip error %d" % rc)
