"""ctypes binding of libmigemm.so (declarations: include/mi_gemm.h)."""

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("VKGRAD_AMD_LIB") or os.path.join(_HERE, "libmigemm.so")

MG_OK, MG_ERR_ARG, MG_ERR_HIP, MG_ERR_STATE, MG_ERR_NOMEM, MG_ERR_NODEVICE = range(6)
MG_NN, MG_NT, MG_TN = 0, 1, 2
MG_F16, MG_BF16 = 0, 1
MG_DEVICE, MG_SHARED, MG_CACHED, MG_BAR = 0, 1, 2, 3
MG_ACT_NONE, MG_ACT_GELU, MG_ACT_RELU = 0, 1, 2
MG_FLAG_TIGHT_BUFFERS = 1
MG_FLAG_SPLITK_ATOMIC = 2
MG_FLAG_SIDE_STREAM = 4
MG_FLAG_XCD_ROTATE = 8
MG_FLAG_XCD_IN_STEP = 16
MG_STATIC_WS_BYTES = 32 << 20
MG_STATIC_MAX_TILES = 16384

DTYPES = {"f16": MG_F16, "bf16": MG_BF16}
KINDS = {"device": MG_DEVICE, "shared": MG_SHARED, "cached": MG_CACHED, "bar": MG_BAR}
MG_ACT_GELU_GRAD, MG_ACT_RELU_GRAD, MG_ACT_SOFTMAX_GRAD = 3, 4, 5
TRI = {None: 0, "c_lower": 1, "a_lower": 2, "a_upper": 3}
ACTS = {None: MG_ACT_NONE, "none": MG_ACT_NONE, "gelu": MG_ACT_GELU, "relu": MG_ACT_RELU,
        "gelu_grad": MG_ACT_GELU_GRAD, "relu_grad": MG_ACT_RELU_GRAD, "softmax_grad": MG_ACT_SOFTMAX_GRAD}


class GemmArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_int32), ("layout", C.c_int32), ("dtype", C.c_int32), ("beta", C.c_int32),
        ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
        ("a", C.c_void_p), ("lda", C.c_int64),
        ("b", C.c_void_p), ("ldb", C.c_int64),
        ("c", C.c_void_p), ("ldc", C.c_int64),
        ("bias", C.c_void_p),
        ("nbatch", C.c_int32), ("tile", C.c_int32),
        ("sa", C.c_int64), ("sb", C.c_int64), ("sc", C.c_int64),
        ("split_k", C.c_int32), ("group_m", C.c_int32),
        ("flags", C.c_int32), ("act", C.c_int32),
        ("y16", C.c_void_p), ("ldy", C.c_int64),
        ("z", C.c_void_p), ("ldz", C.c_int64), ("colsum", C.c_void_p),
        ("res", C.c_void_p), ("ldr", C.c_int64),
        ("tri", C.c_int32), ("reserved", C.c_int32),
        ("p16", C.c_void_p), ("ldp", C.c_int64), ("rowsub", C.c_void_p),
        ("scale", C.c_float), ("reserved2", C.c_int32),
    ]


class AdamWEntry(C.Structure):
    _fields_ = [("w", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("w16", C.c_void_p),
                ("n", C.c_int64), ("first_block", C.c_int64), ("wd", C.c_float), ("vec", C.c_int32)]


class Tile(C.Structure):
    _fields_ = [
        ("id", C.c_int32), ("bm", C.c_int32), ("bn", C.c_int32), ("bk", C.c_int32),
        ("waves_m", C.c_int32), ("waves_n", C.c_int32), ("threads", C.c_int32),
        ("lds_bytes", C.c_int32), ("min_m", C.c_int32), ("stages", C.c_int32), ("fallback", C.c_int32),
        ("persistent", C.c_int32), ("reserved", C.c_int32), ("name", C.c_char * 48),
    ]


class KernelStats(C.Structure):
    _fields_ = [
        ("vgprs", C.c_int32), ("scratch_bytes", C.c_int32), ("static_lds_bytes", C.c_int32),
        ("dynamic_lds_bytes", C.c_int32), ("threads", C.c_int32), ("wgs_per_cu", C.c_int32),
        ("waves_per_simd", C.c_int32), ("max_threads", C.c_int32),
    ]


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128), ("arch", C.c_char * 64),
        ("compute_units", C.c_int32), ("clock_khz", C.c_int32), ("mem_clock_khz", C.c_int32),
        ("mem_bus_bits", C.c_int32), ("l2_bytes", C.c_int32), ("lds_bytes_per_cu", C.c_int32),
        ("wavefront", C.c_int32), ("reserved", C.c_int32), ("total_mem", C.c_int64),
    ]


# name -> (restype, argtypes); every symbol include/mi_gemm.h declares.
_P = C.c_void_p
_I = C.c_int64
SIGNATURES = {
    "mg_init": (C.c_int, [C.c_int, C.POINTER(_P)]),
    "mg_destroy": (C.c_int, [_P]),
    "mg_get_device_info": (C.c_int, [_P, C.POINTER(DeviceInfo)]),
    "mg_alloc": (C.c_int, [_P, C.c_size_t, C.c_int, C.POINTER(_P), C.POINTER(_P)]),
    "mg_free": (C.c_int, [_P, _P, C.c_int]),
    "mg_copy": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "mg_upload": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "mg_download": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "mg_sync": (C.c_int, [_P]),
    "mg_last_error": (C.c_char_p, []),
    "mg_gemm_check": (C.c_int, [C.POINTER(GemmArgs)]),
    "mg_gemm": (C.c_int, [_P, C.POINTER(GemmArgs)]),
    "mg_gemm_static": (C.c_int, [C.c_int, _P, C.POINTER(GemmArgs)]),
    "mg_gemm_static_launches": (C.c_int, [C.c_int, C.POINTER(GemmArgs), C.POINTER(C.c_int)]),
    "mg_launch_count": (C.c_int, [C.POINTER(GemmArgs), C.c_int, C.c_int64, C.c_int64, C.c_int, C.POINTER(C.c_int)]),
    "mg_side_fork": (C.c_int, [_P]),
    "mg_side_join": (C.c_int, [_P]),
    "mg_gemm_time": (C.c_int, [_P, C.POINTER(GemmArgs), C.c_int, C.POINTER(C.c_double)]),
    "mg_gemm_time_rotating": (C.c_int, [_P, C.POINTER(GemmArgs), C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "mg_gemm_time_each": (C.c_int, [_P, C.POINTER(GemmArgs), C.c_int, C.POINTER(C.c_double)]),
    "mg_probe_mfma": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "mg_probe_stream": (C.c_int, [_P, C.c_int64, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "mg_tile_count": (C.c_int, []),
    "mg_tile_info": (C.c_int, [C.c_int, C.POINTER(Tile)]),
    "mg_tile_fits": (C.c_int, [C.c_int, C.POINTER(GemmArgs)]),
    "mg_kernel_stats_for": (C.c_int, [_P, C.POINTER(GemmArgs), C.POINTER(C.c_int), C.POINTER(KernelStats)]),
    "mg_tile_kernel_stats": (C.c_int, [_P, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(KernelStats)]),
    "mg_pick": (C.c_int, [C.POINTER(GemmArgs), C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mg_graph_begin": (C.c_int, [_P]),
    "mg_graph_end": (C.c_int, [_P, C.POINTER(_P)]),
    "mg_graph_launch": (C.c_int, [_P, _P, C.POINTER(C.c_double)]),
    "mg_graph_enqueue": (C.c_int, [_P, _P]),
    "mg_graph_time": (C.c_int, [_P, _P, C.c_int, C.POINTER(C.c_double)]),
    "mg_graph_kernel_count": (C.c_int, [_P, _P, C.POINTER(C.c_int)]),
    "mg_graph_destroy": (C.c_int, [_P, _P]),
    "mg_ew_bias_act": (C.c_int, [_P, _P, _P, _P, _P, C.c_int64, C.c_int64, C.c_int, C.c_int]),
    "mg_ew_act_bwd": (C.c_int, [_P, _P, _P, _P, _P, C.c_int64, C.c_int, C.c_int]),
    "mg_ew_col_sum": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int64, C.c_int]),
    "mg_ew_softmax_ce": (C.c_int, [_P, _P, _P, _P, _P, _P, C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "mg_ew_adamw": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, C.c_int64, C.c_float, C.c_int]),
    "mg_ew_adamw_multi": (C.c_int, [_P, _P, C.c_int, C.c_int64, _P, C.c_int]),
    "mg_ew_zero_multi": (C.c_int, [_P, _P, C.c_int, C.c_int64]),
    "mg_ew_zero": (C.c_int, [_P, _P, C.c_int64]),
    "mg_ew_copy": (C.c_int, [_P, _P, _P, C.c_int64]),
    "mg_ew_cast16": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int]),
    "mg_ew_grad_add": (C.c_int, [_P, _P, _P, C.c_int64]),
    "mg_ew_scale_copy": (C.c_int, [_P, _P, _P, C.c_int64, C.c_float]),
    "mg_ew_fill_uniform16": (C.c_int, [_P, _P, C.c_int64, C.c_uint32, C.c_int]),
    "mg_tk_layernorm": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _I, _I, C.c_int]),
    "mg_tk_layernorm_bwd": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, C.c_int]),
    "mg_tk_attn_softmax": (C.c_int, [_P, _P, _P, _P, _I, _I, _I, C.c_float, C.c_int]),
    "mg_tk_attn_softmax_bwd": (C.c_int, [_P, _P, _P, _P, _I, _I, C.c_float, C.c_int]),
    "mg_tk_attn_rowdot": (C.c_int, [_P, _P, _P, _P, _I, _I, C.c_int]),
    "mg_tk_attn_p_supported": (C.c_int, [_I, _I]),
    "mg_tk_attn_p": (C.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, C.c_float, C.c_int, C.c_int]),
    "mg_tk_attn_fwd_supported": (C.c_int, [_I, _I]),
    "mg_tk_attn_fwd": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, C.c_float, C.c_int, C.c_int]),
    "mg_tk_attn_ds_supported": (C.c_int, [_I, _I]),
    "mg_tk_attn_ds": (C.c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, C.c_float, C.c_int, C.c_int]),
    "mg_tk_split_qkv": (C.c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, C.c_int]),
    "mg_tk_merge_qkv_grad": (C.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, C.c_int]),
    "mg_tk_merge_heads": (C.c_int, [_P, _P, _P, _I, _I, _I, _I, _I, C.c_int]),
    "mg_tk_split_heads": (C.c_int, [_P, _P, _P, _I, _I, _I, _I, _I, C.c_int]),
    "mg_tk_embed": (C.c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I]),
    "mg_tk_embed_bwd": (C.c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I]),
    "mg_tk_residual": (C.c_int, [_P, _P, _P, _P, _P, _I, _I]),
    "mg_tk_add": (C.c_int, [_P, _P, _P, _P, _I]),
    "mg_tk_add16": (C.c_int, [_P, _P, _P, _P, _P, _I, C.c_int]),
    "mg_tk_add_bias": (C.c_int, [_P, _P, _P, _I, _I]),
    "mg_tk_col_sum16": (C.c_int, [_P, _P, _P, _I, _I, C.c_int, C.c_int]),
    "mg_tk_softmax_ce": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, C.c_int]),
}

_lib = None


def load():
    """Load libmigemm.so and declare every entry point.  Raises OSError with
    build instructions if the library is missing: there is no fallback."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OSError(f"{LIB_PATH} not found: build it with "
                      f"`make -C {os.path.join(_HERE, 'csrc')} -j8` "
                      "(or python -c 'import __graft_entry__ as g; g.build()')")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error():
    msg = load().mg_last_error()
    return msg.decode(errors="replace") if msg else ""
