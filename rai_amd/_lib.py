"""ctypes binding of librai_hip.so (the C ABI declared in include/rai_hip.h).

There is no CPU fallback: if the shared library is missing or a call fails, a
RaiHipError is raised.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "librai_hip.so"
MAX_RANK = 8

U8, U32, I64, F16, BF16, F32, F64 = range(7)
DTYPE_NAMES = ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"]
DTYPE_BY_NAME = {n: i for i, n in enumerate(DTYPE_NAMES)}
DTYPE_SIZE = [1, 4, 8, 2, 2, 4, 8]

UNARY = {n: i for i, n in enumerate(
    ["sin", "cos", "neg", "square", "sqrt", "rsqrt", "abs", "exp", "log", "log2", "log10", "erf", "tanh", "powf",
     "sign", "gelu", "new_gelu", "silu", "relu"])}
BINARY = {n: i for i, n in enumerate(
    ["add", "sub", "mul", "div", "maximum", "minimum", "eq", "ne", "gt", "ge", "lt", "le"])}
REDUCE = {"sum": 0, "max": 1, "min": 2}
ARCH = {"phi2": 0, "qwen2": 1, "gemma": 2, "phi3": 3}


class RaiHipError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"rai_hip status {status}: {msg}")
        self.status = status


class TensorDesc(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("dtype", C.c_int32),
        ("rank", C.c_int32),
        ("shape", C.c_int64 * MAX_RANK),
        ("stride", C.c_int64 * MAX_RANK),
        ("offset", C.c_int64),
    ]


class DecoderConfig(C.Structure):
    _fields_ = [
        ("arch", C.c_int32),
        ("dtype", C.c_int32),
        ("vocab_size", C.c_int32),
        ("hidden_size", C.c_int32),
        ("intermediate_size", C.c_int32),
        ("num_hidden_layers", C.c_int32),
        ("num_attention_heads", C.c_int32),
        ("num_key_value_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("rotary_dim", C.c_int32),
        ("max_position_embeddings", C.c_int32),
        ("hidden_act", C.c_int32),
        ("tie_word_embeddings", C.c_int32),
        ("max_batch", C.c_int32),
        ("max_context", C.c_int32),
        ("rope_tables_f32", C.c_int32),
        ("qk_layernorm", C.c_int32),
        ("rope_theta", C.c_double),
        ("norm_eps", C.c_double),
    ]


_TP = C.POINTER(TensorDesc)
_vp = C.c_void_p
_i32 = C.c_int32
_i64 = C.c_int64
_dbl = C.c_double

# name -> argtypes (every function returns int status except last_error)
PROTOTYPES = {
    "rai_hip_device_count": [C.POINTER(C.c_int)],
    "rai_hip_init": [C.c_int],
    "rai_hip_sync": [C.c_int],
    "rai_hip_alloc": [C.c_int, C.c_size_t, C.POINTER(_vp)],
    "rai_hip_retain": [_vp],
    "rai_hip_release": [_vp],
    "rai_hip_mem_stats": [C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "rai_hip_trim": [C.c_int],
    "rai_hip_h2d": [C.c_int, _vp, _vp, C.c_size_t],
    "rai_hip_d2h": [C.c_int, _vp, _vp, C.c_size_t],
    "rai_hip_d2d": [C.c_int, _vp, _vp, C.c_size_t],
    "rai_hip_to_device": [C.c_int, _TP, C.c_int, _TP],
    "rai_hip_timer_create": [C.c_int, C.POINTER(_vp)],
    "rai_hip_timer_start": [_vp],
    "rai_hip_timer_stop": [_vp],
    "rai_hip_timer_elapsed_ms": [_vp, C.POINTER(C.c_float)],
    "rai_hip_timer_destroy": [_vp],
    "rai_hip_fill": [C.c_int, _TP, _dbl],
    "rai_hip_arange": [C.c_int, _TP, _dbl, _dbl],
    "rai_hip_cast": [C.c_int, _TP, _TP],
    "rai_hip_copy": [C.c_int, _TP, _TP],
    "rai_hip_unary": [C.c_int, C.c_int, _TP, _TP, _dbl],
    "rai_hip_binary": [C.c_int, C.c_int, _TP, _TP, _TP],
    "rai_hip_where": [C.c_int, _TP, _TP, _TP, _TP],
    "rai_hip_reduce": [C.c_int, C.c_int, _TP, C.POINTER(_i32), _i32, _i32, _TP],
    "rai_hip_softmax": [C.c_int, _TP, _i32, _TP],
    "rai_hip_log_softmax": [C.c_int, _TP, _i32, _TP],
    "rai_hip_argmax": [C.c_int, _TP, _i32, _i32, _TP],
    "rai_hip_argmin": [C.c_int, _TP, _i32, _i32, _TP],
    "rai_hip_argmax_static": [C.c_int, _TP, _i32, _i32, _TP],
    "rai_hip_index_select": [C.c_int, _TP, _TP, _i32, _TP],
    "rai_hip_gather": [C.c_int, _TP, _TP, _i32, _TP],
    "rai_hip_index_add": [C.c_int, _TP, _TP, _TP, _i32, _TP],
    "rai_hip_scatter_add": [C.c_int, _TP, _TP, _TP, _i32, _TP],
    "rai_hip_index_errors": [C.c_int, C.POINTER(C.c_uint64)],
    "rai_hip_matmul": [C.c_int, _TP, _TP, _TP],
    "rai_hip_linear": [C.c_int, _TP, _TP, _TP, _i32, _TP, _TP],
    "rai_hip_linear_packed": [C.c_int, _TP, _TP, _TP, _TP, _i32, _i32, _TP, _i32, _i32, _TP, _TP],
    "rai_hip_layer_norm": [C.c_int, _TP, _TP, _TP, _dbl, _TP],
    "rai_hip_rms_norm": [C.c_int, _TP, _TP, _dbl, _i32, _TP],
    "rai_hip_rope": [C.c_int, _TP, _TP, _TP, _i32, _i64, _TP],
    "rai_hip_rope_tables": [C.c_int, _dbl, _i32, _i32, _TP, _TP],
    "rai_hip_attention": [C.c_int, _TP, _TP, _TP, _dbl, _i32, _i32, _TP],
    "rai_hip_decoder_create": [C.c_int, C.POINTER(DecoderConfig), C.POINTER(_vp)],
    "rai_hip_decoder_destroy": [_vp],
    "rai_hip_decoder_load_param": [_vp, C.c_char_p, _vp, C.c_size_t],
    "rai_hip_decoder_load_safetensors": [_vp, C.POINTER(C.c_char_p), _i32],
    "rai_hip_safetensors_index_files": [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(_i32)],
    "rai_hip_decoder_dtype": [_vp, C.POINTER(_i32)],
    "rai_hip_decoder_param_count": [_vp, C.POINTER(_i32)],
    "rai_hip_decoder_param_name": [_vp, _i32, C.c_char_p, C.c_size_t, C.POINTER(_i64)],
    "rai_hip_decoder_param_shape": [_vp, _i32, C.POINTER(_i64), C.POINTER(_i64)],
    "rai_hip_decoder_forward": [_vp, C.POINTER(C.c_uint32), _i32, _i32, C.POINTER(C.c_float), C.POINTER(C.c_uint32)],
    "rai_hip_decoder_forward_hidden": [_vp, C.POINTER(C.c_uint32), _vp, _i32, _i32, C.POINTER(C.c_float), C.POINTER(C.c_float),
                                       C.POINTER(C.c_uint32)],
    "rai_hip_decoder_generate": [_vp, C.POINTER(C.c_uint32), _i32, _i32, _i32, C.POINTER(C.c_uint32),
                                 C.POINTER(C.c_float), C.POINTER(C.c_float)],
    "rai_hip_decoder_generate_sampled": [_vp, C.POINTER(C.c_uint32), _i32, _i32, _i32, C.c_float, _i32, _i64,
                                         C.POINTER(C.c_uint32), C.POINTER(_i32), C.POINTER(C.c_float),
                                         C.POINTER(C.c_float)],
    "rai_hip_sample_argmax": [C.c_int, _TP, _TP, C.c_float, _TP],
    "rai_hip_decoder_time_decode_linear": [_vp, _i32, C.POINTER(C.c_float), C.POINTER(C.c_double)],
    "rai_hip_decoder_time_decode_step": [_vp, _i32, C.POINTER(C.c_float), C.POINTER(C.c_double)],
    "rai_hip_decoder_clear_kv_cache": [_vp],
    "rai_hip_decoder_context_len": [_vp, C.POINTER(_i32)],
}

class GraphStats(C.Structure):
    _fields_ = [("nodes_evaluated", C.c_uint64), ("kernel_launches", C.c_uint64), ("fused_regions", C.c_uint64),
                ("fused_nodes", C.c_uint64), ("composed_regions", C.c_uint64), ("composed_nodes", C.c_uint64),
                ("plan_ns", C.c_uint64), ("run_ns", C.c_uint64)]


_T = C.c_void_p  # rai_tensor *
_I64P = C.POINTER(_i64)
_I32P = C.POINTER(_i32)
# include/rai_graph.h: name -> (restype, argtypes)
# include/rai_hip_peaks.h (measurement aid)
PEAK_PROTOTYPES = {
    "rai_hip_measure_peak": [C.c_int, C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_double)],
}
PEAK_KINDS = {"mfma_bf16": 0, "mfma_bf16_lds": 1, "lds_read": 2, "hbm_read": 3, "hbm_copy": 4, "stage_dma": 5, "stage_vgpr": 6, "gemm_loop": 7}

GRAPH_PROTOTYPES = {
    "rai_full": (_T, [_dbl, _i32, _I64P, _i32, _i32]),
    "rai_arange": (_T, [_dbl, _dbl, _dbl, _i32, _i32]),
    "rai_from_array": (_T, [_vp, _i32, _I64P, _i32, _i32]),
    "rai_to_dtype": (_T, [_T, _i32]),
    "rai_unary": (_T, [_i32, _T, _dbl]),
    "rai_binary": (_T, [_i32, _T, _T]),
    "rai_matmul": (_T, [_T, _T]),
    "rai_softmax": (_T, [_T, _i32]),
    "rai_log_softmax": (_T, [_T, _i32]),
    "rai_reduce": (_T, [_i32, _T, _I32P, _i32, _i32]),
    "rai_argmax": (_T, [_T, _i32, _i32]),
    "rai_argmin": (_T, [_T, _i32, _i32]),
    "rai_index_select": (_T, [_T, _i32, _T]),
    "rai_gather": (_T, [_T, _i32, _T]),
    "rai_index_add": (_T, [_T, _i32, _T, _T]),
    "rai_scatter_add": (_T, [_T, _i32, _T, _T]),
    "rai_narrow": (_T, [_T, _i32, _i64, _i64]),
    "rai_concatenate": (_T, [C.POINTER(_T), _i32, _i32]),
    "rai_where": (_T, [_T, _T, _T]),
    "rai_transpose": (_T, [_T, _i32, _i32]),
    "rai_reshape": (_T, [_T, _I64P, _i32]),
    "rai_permute": (_T, [_T, _I32P, _i32]),
    "rai_broadcast_to": (_T, [_T, _I64P, _i32]),
    "rai_to_contiguous": (_T, [_T]),
    "rai_to_device": (_T, [_T, _i32]),
    "rai_tensor_retain": (None, [_T]),
    "rai_tensor_release": (None, [_T]),
    "rai_tensor_rank": (_i32, [_T]),
    "rai_tensor_dtype": (_i32, [_T]),
    "rai_tensor_device": (_i32, [_T]),
    "rai_tensor_op": (_i32, [_T]),
    "rai_tensor_shape": (_i32, [_T, _I64P]),
    "rai_tensor_is_evaluated": (_i32, [_T]),
    "rai_tensor_num_inputs": (_i32, [_T]),
    "rai_tensor_id": (C.c_uint64, [_T]),
    "rai_tensor_error": (C.c_char_p, [_T]),
    "rai_tensor_storage": (C.c_int, [_T, _TP]),
    "rai_from_storage": (_T, [_TP, _vp, _i32]),
    "rai_tensor_buffer": (_vp, [_T]),
    "rai_eval": (C.c_int, [C.POINTER(_T), _i32, _i32]),
    "rai_graph_eval_order": (C.c_int, [C.POINTER(_T), _i32, C.POINTER(C.c_uint64), _i32, _I32P]),
    "rai_tensor_to_host": (C.c_int, [_T, _vp, C.c_size_t]),
    "rai_dispatch_unregister": (C.c_int, [_i32]),
    "rai_dispatch_register_builtin": (C.c_int, [_i32]),
    "rai_dispatch_has_rule": (_i32, [_i32]),
    "rai_graph_set_fusion": (C.c_int, [_i32]),
    "rai_graph_set_compose": (C.c_int, [_i32]),
    "rai_graph_get_stats": (C.c_int, [C.POINTER(GraphStats), _i32]),
}

_lib = None


def load():
    """Load librai_hip.so (built by rai_amd.build); raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RaiHipError(-5, f"{LIB_PATH} not built; run `python -m rai_amd.build`")
    lib = C.CDLL(str(LIB_PATH))
    lib.rai_hip_last_error.restype = C.c_char_p
    lib.rai_hip_last_error.argtypes = []
    for name, args in list(PROTOTYPES.items()) + list(PEAK_PROTOTYPES.items()):
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = C.c_int
        fn.argtypes = args
    for name, (res, args) in GRAPH_PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status):
    if status != 0:
        raise RaiHipError(status, load().rai_hip_last_error().decode("utf-8", "replace"))


def call(name, *args):
    check(getattr(load(), name)(*args))
