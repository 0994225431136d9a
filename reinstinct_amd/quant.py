"""Mirror of the reference's src/quant for the six formats of the path:
layout sizes, repack_for_matvec, and synthetic-weight quantizers (host code)."""
import ctypes as C

import numpy as np

from ._lib import check, lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def block_size(fmt):
    return lib.rein_block_size(fmt)


def bytes_per_block(fmt):
    return lib.rein_bytes_per_block(fmt)


def repacked_n_sub_padded(in_dim):
    """src/quant/q4_k.rs:92-95"""
    return lib.rein_repacked_n_sub_padded(in_dim)


def repacked_len(fmt, in_dim, out_dim):
    """<fmt>::repacked_len, e.g. src/quant/q4_k.rs:98-102"""
    return lib.rein_repacked_len(fmt, in_dim, out_dim)


def repack_for_matvec(fmt, raw, in_dim, out_dim):
    """<fmt>::repack_for_matvec (src/quant/q4_k.rs:126-176 and twins): on-disk
    blocks [out_dim, in_dim] -> repacked-v2 slab (uint8 array)."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    bs, bb = block_size(fmt), bytes_per_block(fmt)
    if bs == 0:
        check(lib.rein_repack_for_matvec(fmt, None, in_dim, out_dim, None))
    if in_dim % bs == 0 and raw.size < out_dim * (in_dim // bs) * bb:
        raise ValueError("raw weight buffer too small for the shape")
    out = np.empty(max(repacked_len(fmt, in_dim, out_dim), 1), np.uint8)
    check(lib.rein_repack_for_matvec(fmt, _ptr(raw), in_dim, out_dim, _ptr(out)))
    return out[: repacked_len(fmt, in_dim, out_dim)]


def quantize_weights(fmt, w):
    """fp32 weights (any shape, row-major, last dim a block multiple) -> on-disk
    blocks.  Q8_0 is q8_0::quantize_from_f32 (src/quant/q8_0.rs:45-61)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    bs, bb = block_size(fmt), bytes_per_block(fmt)
    out = np.empty(max(w.size // max(bs, 1) * bb, 1), np.uint8)
    check(lib.rein_quantize_weights(fmt, _ptr(w), w.size, _ptr(out)))
    return out[: w.size // bs * bb]


GGML_Q3_K, GGML_IQ4_NL, GGML_BF16 = 11, 20, 30


def ingest_for_matvec(ggml_type, raw, in_dim, out_dim):
    """GpuMatvecTensor::from_bytes_matvec (src/runtime/qwen35.rs:251-331): GGUF tensor bytes ->
    (repacked slab, format id of the kernels that read it)."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    label = lib.rein_ingest_format(ggml_type)
    if label == 0:
        check(lib.rein_ingest_for_matvec(ggml_type, _ptr(raw), in_dim, out_dim, None, None))
    if raw.size < lib.rein_ingest_src_len(ggml_type, in_dim, out_dim):
        raise ValueError("tensor bytes too short for the shape")
    out = np.empty(max(repacked_len(label, in_dim, out_dim), 1), np.uint8)
    fmt = C.c_int(0)
    check(lib.rein_ingest_for_matvec(ggml_type, _ptr(raw), in_dim, out_dim, _ptr(out), C.byref(fmt)))
    return out[: repacked_len(label, in_dim, out_dim)], fmt.value


def transcode_q3_k_to_q6_k(raw, n_weights):
    """q3_k::transcode_to_q6_k (src/quant/q3_k.rs:85-122)"""
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(n_weights // 256 * 210, np.uint8)
    check(lib.rein_transcode_q3_k_to_q6_k(_ptr(raw), n_weights, _ptr(out)))
    return out
