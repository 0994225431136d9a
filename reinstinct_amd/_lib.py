"""ctypes loader for librein.so.  Fails loudly when the library is missing."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "librein.so")
HSACO_PATH = os.path.join(_HERE, "rein_gfx950.hsaco")


class ReinError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"{msg} [rc={code}]")
        self.code = code


class MoeShape(C.Structure):
    _fields_ = [("n_tok", C.c_uint), ("hidden", C.c_uint), ("n_expert", C.c_uint), ("n_used", C.c_uint),
                ("expert_ff", C.c_uint), ("gate_up_fmt", C.c_int), ("down_fmt", C.c_int)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_type", C.c_int), ("n_dims", C.c_uint), ("dims", C.c_uint64 * 4),
                ("offset", C.c_uint64), ("byte_size", C.c_uint64), ("data", C.c_void_p)]


class GgufDims(C.Structure):
    _fields_ = [("in_dim", C.c_uint), ("out_dim", C.c_uint), ("n_expert", C.c_uint), ("bytes_per_expert", C.c_size_t)]


_vp, _u, _i, _sz = C.c_void_p, C.c_uint, C.c_int, C.c_size_t
_u64 = C.c_uint64
_P = C.POINTER

# name -> (restype, argtypes); every symbol declared in include/rein.h
SIGNATURES = {
    "rein_last_error": (C.c_char_p, []),
    "rein_init": (_i, [C.c_char_p]),
    "rein_is_loaded": (_i, []),
    "rein_set_option": (_i, [C.c_char_p, C.c_char_p]),
    "rein_get_option": (_i, [C.c_char_p, _P(_u), _P(_i)]),
    "rein_reset_options": (_i, []),
    "rein_option_count": (_i, []),
    "rein_option_name": (C.c_char_p, [_i]),
    "rein_device_count": (_i, [_P(_i)]),
    "rein_set_device": (_i, [_i]),
    "rein_get_device": (_i, [_P(_i)]),
    "rein_device_name": (_i, [_i, C.c_char_p, _i]),
    "rein_device_total_mem": (_i, [_i, _P(_sz)]),
    "rein_mem_info": (_i, [_P(_sz), _P(_sz)]),
    "rein_device_synchronize": (_i, []),
    "rein_malloc": (_i, [_P(_vp), _sz]),
    "rein_free": (_i, [_vp]),
    "rein_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "rein_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "rein_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "rein_memcpy_h2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "rein_memcpy_d2h_async": (_i, [_vp, _vp, _sz, _vp]),
    "rein_memcpy_d2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "rein_stream_create": (_i, [_P(_vp)]),
    "rein_stream_destroy": (_i, [_vp]),
    "rein_stream_synchronize": (_i, [_vp]),
    "rein_stream_wait_event": (_i, [_vp, _vp]),
    "rein_event_create": (_i, [_P(_vp)]),
    "rein_event_record": (_i, [_vp, _vp]),
    "rein_event_synchronize": (_i, [_vp]),
    "rein_event_elapsed_ms": (_i, [_P(C.c_float), _vp, _vp]),
    "rein_event_destroy": (_i, [_vp]),
    "rein_stream_begin_capture": (_i, [_vp]),
    "rein_stream_end_capture": (_i, [_vp, _P(_vp)]),
    "rein_graph_instantiate": (_i, [_P(_vp), _vp]),
    "rein_graph_launch": (_i, [_vp, _vp]),
    "rein_graph_destroy": (_i, [_vp]),
    "rein_graph_exec_destroy": (_i, [_vp]),
    "rein_module_load": (_i, [_P(_vp), C.c_char_p]),
    "rein_module_unload": (_i, [_vp]),
    "rein_module_get_function": (_i, [_P(_vp), _vp, C.c_char_p]),
    "rein_builtin_module": (_i, [_P(_vp)]),
    "rein_launch_kernel": (_i, [_vp, _u, _u, _u, _u, _u, _u, _u, _vp, _P(_vp)]),
    "rein_repacked_n_sub_padded": (_sz, [_sz]),
    "rein_repacked_len": (_sz, [_i, _sz, _sz]),
    "rein_block_size": (_i, [_i]),
    "rein_bytes_per_block": (_i, [_i]),
    "rein_repack_for_matvec": (_i, [_i, _vp, _sz, _sz, _vp]),
    "rein_quantize_weights": (_i, [_i, _vp, _sz, _vp]),
    "rein_quantize_q8": (_i, [_vp, _vp, _u, _u, _vp]),
    "rein_matvec_xq8": (_i, [_i, _vp, _vp, _vp, _u, _u, _vp]),
    "rein_matvec_batched_xq8": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_matvec_kernel_name": (_i, [_i, _u, _u, _u, C.c_char_p, _sz]),
    "rein_matvec_multi_xq8": (_i, [_u, C.POINTER(_i), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_u), _vp, _u, _u, _vp]),
    "rein_mmq_xq8": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_matmul": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp, _vp]),
    "rein_mmq_workspace_bytes": (_sz, [_i, _u, _u]),
    "rein_mmq_workspace_min_bytes": (_sz, [_i, _u, _u]),
    "rein_mmq_form_ws": (_i, [_i, _u, _u, _u, _sz]),
    "rein_mmq_xq8_ws": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp, _sz, _vp]),
    "rein_noalloc_prepare": (_i, []),
    "rein_mmq_xq8_noalloc": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_mmq_tile_plan_ws": (_i, [_i, _u, _u, _vp, _vp]),
    "rein_mmq_block_dots_ws": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp, _sz, _vp]),
    "rein_matmul_scratch_bytes": (_sz, [_i, _u, _u]),
    "rein_matmul_ws": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _vp, _sz, _vp]),
    "rein_matmul_path": (_i, [_i, _u]),
    "rein_mmq_tile_plan": (_i, [_i, _u, _u, _u]),
    "rein_block_dot_parts": (_i, [_i]),
    "rein_block_dots": (_i, [_i, _vp, _vp, _vp, _u, _u, _u, _i, _vp]),
    "rein_moe_topk": (_i, [_vp, _u, _u, _u, _vp, _vp, _vp]),
    "rein_moe_sort": (_i, [_vp, _u, _u, _u, _vp, _vp, _vp, _vp, _vp, _vp]),
    "rein_moe_gather_xq": (_i, [_vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_moe_quantize_scatter": (_i, [_vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_moe_scatter_rows": (_i, [_vp, _vp, _vp, _u, _u, _vp]),
    "rein_moe_grouped_gemm": (_i, [_i, _vp, _u, _vp, _vp, _u, _vp, _vp, _u, _u, _u, _vp]),
    "rein_moe_grouped_swiglu_q8": (_i, [_i, _vp, _vp, _u, _vp, _vp, _u, _vp, _vp, _u, _u, _u, _vp]),
    "rein_swiglu_mul": (_i, [_vp, _vp, _vp, _u, _vp]),
    "rein_ingest_format": (_i, [_i]),
    "rein_ingest_expert_format": (_i, [_i]),
    "rein_ingest_src_len": (_sz, [_i, _sz, _sz]),
    "rein_ingest_for_matvec": (_i, [_i, _vp, _sz, _sz, _vp, _P(_i)]),
    "rein_transcode_q3_k_to_q6_k": (_i, [_vp, _sz, _vp]),
    "rein_gguf_open": (_i, [C.c_char_p, _P(_vp)]),
    "rein_gguf_from_bytes": (_i, [_vp, _sz, _P(_vp)]),
    "rein_gguf_close": (None, [_vp]),
    "rein_gguf_header": (_i, [_vp, _P(C.c_uint32), _P(_u64), _P(_u64), _P(_u64), _P(_u64)]),
    "rein_gguf_align_up": (_u64, [_u64, _u64]),
    "rein_gguf_tensor_at": (_i, [_vp, _u64, _P(GgufTensor)]),
    "rein_gguf_tensor_by_name": (_i, [_vp, C.c_char_p, _P(GgufTensor)]),
    "rein_gguf_meta_at": (_i, [_vp, _u64, _P(C.c_char_p), _P(_i)]),
    "rein_gguf_meta_type": (_i, [_vp, C.c_char_p, _P(_i)]),
    "rein_gguf_meta_raw": (_i, [_vp, C.c_char_p, _P(_i), _P(_vp)]),
    "rein_gguf_meta_u64": (_i, [_vp, C.c_char_p, _P(_u64)]),
    "rein_gguf_meta_f32": (_i, [_vp, C.c_char_p, _P(C.c_float)]),
    "rein_gguf_meta_bool": (_i, [_vp, C.c_char_p, _P(_i)]),
    "rein_gguf_meta_str": (_i, [_vp, C.c_char_p, _P(_vp), _P(_sz)]),
    "rein_gguf_meta_array": (_i, [_vp, C.c_char_p, _P(_i), _P(_u64), _P(_vp)]),
    "rein_gguf_load_for_matvec": (_i, [_vp, C.c_char_p, _vp, _sz, _P(_i), _P(GgufDims)]),
    "rein_matvec_ondisk_xq8": (_i, [_i, _vp, _vp, _vp, _u, _u, _vp]),
    "rein_matvec_q8_0_splitk": (_i, [_vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_moe_expert_matvec": (_i, [_i, _vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, _vp]),
    "rein_moe_down": (_i, [_i, _vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, _vp]),
    "rein_moe_gate_up_swiglu": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, _vp]),
    "rein_moe_gate_up_swiglu_q8": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, _vp]),
    "rein_moe_down_combine": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, _vp]),
    "rein_rmsnorm_q8": (_i, [_vp, _vp, _vp, _u, _u, C.c_float, _vp]),
    "rein_add_rmsnorm_q8": (_i, [_vp, _vp, _vp, _vp, _vp, _u, _u, C.c_float, _vp]),
    "rein_swiglu_q8": (_i, [_vp, _vp, _vp, _vp, _u, _vp]),
    "rein_sigmoid_mul_q8": (_i, [_vp, _vp, _vp, _u, _vp]),
    "rein_rmsnorm_gated_q8": (_i, [_vp, _vp, _vp, _vp, _vp, _u, _u, C.c_float, _vp]),
    "rein_moe_geglu_q8": (_i, [_vp, _vp, _u, _u, _vp]),
    "rein_moe_combine": (_i, [_vp, _vp, _vp, _vp, _vp, _u, _u, _u, _vp]),
    "rein_moe_gemm_bn": (_u, []),
    "rein_moe_workspace_bytes": (_sz, [_P(MoeShape)]),
    "rein_moe_ffn": (_i, [_P(MoeShape), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
}

_lib = None


def load():
    """dlopen librein.so and type every entry point (no GPU needed for this)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ReinError(-1, f"{SO_PATH} is not built: run `make -C reinstinct_amd/csrc` "
                            "(or __graft_entry__.build()); there is no fallback path")
    handle = C.CDLL(SO_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    _lib = handle
    return _lib


class _Lazy:
    def __getattr__(self, name):
        return getattr(load(), name)


lib = _Lazy()


def check(rc):
    """Turn a non-zero status into ReinError carrying rein_last_error()."""
    if rc != 0:
        msg = load().rein_last_error()
        raise ReinError(rc, msg.decode() if msg else "unknown error")
    return rc


def init():
    """Bind libamdhip64.so and load the gfx950 code object (needs a GPU)."""
    check(load().rein_init(HSACO_PATH.encode()))


def set_option(name, value):
    """rein_set_option: pin a launch choice (value None: hand it back to the library)."""
    check(load().rein_set_option(name.encode(), None if value is None else str(value).encode()))


def get_option(name):
    """-> the option's value, or None while it is unset"""
    v, on = _u(0), _i(0)
    check(load().rein_get_option(name.encode(), C.byref(v), C.byref(on)))
    return v.value if on.value else None


def reset_options():
    check(load().rein_reset_options())
