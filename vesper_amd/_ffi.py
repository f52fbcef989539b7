"""ctypes binding of libvsp_attn.so (the C ABI declared in include/vsp_attn.h).

The library must have been built (python -c "import __graft_entry__ as g; g.build()" or
`make -C vesper_amd/csrc`); there is no fallback: importing this module without it raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libvsp_attn.so")

# vsp_status
OK = 0
ERR_NDIM, ERR_SHAPE, ERR_DTYPE, ERR_DROPOUT, ERR_NUMEL, ERR_COPY_DTYPE = 1, 2, 3, 4, 5, 6
ERR_REPEAT_NDIM, ERR_GQA_HEADS, ERR_GQA_EMBED, ERR_BROADCAST = 7, 8, 9, 10
ERR_NULL, ERR_UNSUPPORTED, ERR_STRIDE, ERR_ALIGN, ERR_WORKSPACE, ERR_ARG, ERR_LAUNCH = 32, 33, 34, 35, 36, 37, 38
# vsp_dtype
F32, BF16, F16, I8, I32 = 0, 1, 2, 3, 4
# vsp_kv_format / planes
KV_F32, KV_BF16, KV_Q8_0 = 0, 1, 2
PLANE_K, PLANE_V, PLANE_K_SCALE, PLANE_V_SCALE = 0, 1, 2, 3


class VspTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("ndim", C.c_int32),
                ("shape", C.c_int64 * 4), ("stride", C.c_int64 * 4)]


class VspKVCache(C.Structure):
    _fields_ = [("format", C.c_int32), ("B", C.c_int32), ("Hkv", C.c_int32), ("S_max", C.c_int32), ("D", C.c_int32),
                ("k", C.c_void_p), ("v", C.c_void_p), ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
                ("len", C.c_int32),
                ("page_table", C.c_void_p), ("page_tokens", C.c_int32), ("pages_per_seq", C.c_int32),
                ("n_pages", C.c_int32)]


# every symbol include/vsp_attn.h declares: name -> (restype, argtypes)
_TP, _KP = C.POINTER(VspTensor), C.POINTER(VspKVCache)
SYMBOLS = {
    "vsp_kv_plane_bytes": (C.c_size_t, [C.c_int32] * 6),
    "vsp_kv_cache_reset": (C.c_int, [_KP, C.c_void_p]),
    "vsp_kv_append": (C.c_int, [_KP, _TP, _TP, C.c_int64, C.c_void_p, C.c_void_p]),
    "vsp_rope_kv_append": (C.c_int, [_KP, _TP, _TP, _TP, _TP, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
    "vsp_kv_read": (C.c_int, [_KP, C.c_int64, C.c_int64, _TP, _TP, C.c_void_p]),
    "vsp_kv_read_q8_0": (C.c_int, [_KP, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]),
    "vsp_kv_view_f32": (C.c_int, [_KP, _TP, _TP]),
    "vsp_attn_prefill": (C.c_int, [_TP, _TP, _TP, _TP, _TP, C.c_float, C.c_int, C.c_float, C.c_int, C.c_void_p]),
    "vsp_attn_prefill_split_workspace_bytes": (C.c_size_t, [C.c_int32] * 6),
    "vsp_attn_prefill_split": (C.c_int, [_TP] * 5 + [C.c_float, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vsp_attn_backward_workspace_bytes": (C.c_size_t, [C.c_int32] * 3),
    "vsp_attn_backward_fast_workspace_bytes": (C.c_size_t, [C.c_int32] * 3),
    "vsp_attn_prefill_backward": (C.c_int, [_TP] * 9 + [C.c_float, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vsp_attn_backward_split_workspace_bytes": (C.c_size_t, [C.c_int32] * 5),
    "vsp_attn_prefill_backward_split": (C.c_int, [_TP] * 9 + [C.c_float, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vsp_attn_prefill_cached_workspace_bytes": (C.c_size_t, [_KP, C.c_int, C.c_int32]),
    "vsp_attn_prefill_cached_split_workspace_bytes": (C.c_size_t, [_KP, C.c_int, C.c_int32, C.c_int32, C.c_int32]),
    "vsp_attn_prefill_cached": (C.c_int, [_TP, _KP, C.c_void_p, C.c_int32, C.c_void_p, _TP, _TP, C.c_float, C.c_int, C.c_void_p,
                                          C.c_size_t, C.c_void_p]),
    "vsp_seq_lens_advance": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "vsp_attn_decode_workspace_bytes": (C.c_size_t, [C.c_int32] * 4),
    "vsp_attn_decode": (C.c_int, [_TP, _KP, C.c_void_p, C.c_int32, _TP, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vsp_attn_decode_multi": (C.c_int, [_TP, _KP, C.c_void_p, C.c_int32, _TP, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vsp_attn_decode_noalloc": (C.c_int, [_TP, _KP, C.c_void_p, C.c_int32, _TP, C.c_float, C.c_void_p]),
    "vsp_attn_decode_proj_workspace_bytes": (C.c_size_t, [C.c_int32] * 5),
    "vsp_attn_decode_proj": (C.c_int, [_TP, _KP, C.c_void_p, C.c_int32, _TP, _TP, _TP, C.c_float, C.c_void_p, C.c_size_t,
                                       C.c_void_p]),
    "vsp_f32_to_bf16": (C.c_uint16, [C.c_float]),
    "vsp_bf16_to_f32": (C.c_float, [C.c_uint16]),
    "vsp_f32_to_f16": (C.c_uint16, [C.c_float]),
    "vsp_f16_to_f32": (C.c_float, [C.c_uint16]),
    "vsp_q8_0_quantize_row": (None, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "vsp_q8_0_dequantize_row": (None, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "vsp_rope_fill_table": (None, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_float]),
    "vsp_slice_bounds": (None, [C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "vsp_gqa_config": (C.c_int, [C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "vsp_status_str": (C.c_char_p, [C.c_int]),
    "vsp_last_hip_error": (C.c_char_p, []),
    "vsp_attn_abi_version": (C.c_int, []),
}


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP extension has not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'`). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = load()


class VspError(RuntimeError):
    """A non-zero vsp_status; .status holds the code, the text is the reference's exception message
    where the reference has one."""

    def __init__(self, status):
        self.status = status
        msg = lib.vsp_status_str(status).decode()
        if status == ERR_LAUNCH:
            msg += ": " + lib.vsp_last_hip_error().decode()
        super().__init__(msg)


def check(status):
    if status != OK:
        raise VspError(status)
