"""ctypes binding of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark — never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS = 2, 8, 12, 13, 14, 23
Q5_1, IQ3_S = 7, 21          # relabelled onto the Q5_K / IQ4_XS kernels (src/quant/q5_1.rs, iq3_s.rs)
FORMATS = {"q4_0": Q4_0, "q8_0": Q8_0, "q4_k": Q4_K, "q5_k": Q5_K, "q6_k": Q6_K, "iq4_xs": IQ4_XS}


def build():
    """Compile liboracle.so from oracle.c (gcc, a second or two)."""
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle.so"])


def _load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    u8p, f32p, i32p = C.c_void_p, C.c_void_p, C.c_void_p
    sz = C.c_size_t
    sig = {
        "orc_f16_to_f32": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [C.c_float]),
        "orc_block_size": (C.c_int, [C.c_int]),
        "orc_bytes_per_block": (C.c_int, [C.c_int]),
        "orc_get_scale_min_k4": (None, [C.c_int, u8p, u8p, u8p]),
        "orc_dequantize_to_f32": (C.c_int, [C.c_int, u8p, f32p, sz]),
        "orc_repacked_n_sub_padded": (sz, [sz]),
        "orc_repacked_len": (sz, [C.c_int, sz, sz]),
        "orc_repack_for_matvec": (C.c_int, [C.c_int, u8p, sz, sz, u8p]),
        "orc_decode_repacked_to_f32": (C.c_int, [C.c_int, u8p, sz, sz, f32p]),
        "orc_q8_0_quantize_from_f32": (None, [f32p, sz, u8p]),
        "orc_quantize_q8": (None, [f32p, sz, sz, u8p]),
        "orc_block_dot_parts": (C.c_int, [C.c_int]),
        "orc_block_dots": (C.c_int, [C.c_int, u8p, sz, sz, u8p, sz, i32p]),
        "orc_matvec_q8": (C.c_int, [C.c_int, u8p, sz, sz, u8p, sz, f32p, C.c_int]),
        "orc_matvec_f32": (None, [f32p, f32p, sz, sz, f32p, C.c_int]),
        "orc_moe_topk": (None, [f32p, C.c_int, C.c_int, C.c_int, i32p, f32p]),
        "orc_moe_sort": (None, [i32p, C.c_int, C.c_int, C.c_int, i32p, i32p, i32p]),
        "orc_moe_gather_xq": (None, [u8p, i32p, u8p, C.c_int, C.c_int, C.c_int]),
        "orc_moe_scatter_rows": (None, [f32p, i32p, f32p, C.c_int, C.c_int]),
        "orc_moe_combine": (None, [f32p, i32p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]),
        "orc_swiglu_mul": (None, [f32p, f32p, f32p, sz]),
        "orc_q3_k_dequantize": (None, [u8p, f32p, sz]),
        "orc_iq4_nl_dequantize": (None, [u8p, f32p, sz]),
        "orc_iq3s_grid_entry": (C.c_uint32, [C.c_int]),
        "orc_bf16_to_f32": (None, [u8p, f32p, sz]),
        "orc_map_det": (None, [C.c_int, f32p, f32p, sz]),
        "orc_map_ref": (None, [C.c_int, f32p, f32p, sz]),
        "orc_sumsq_det": (C.c_float, [f32p, sz]),
        "orc_add_rmsnorm": (None, [f32p, f32p, f32p, f32p, sz, sz, C.c_float]),
        "orc_rmsnorm_gated": (None, [f32p, f32p, f32p, f32p, sz, sz, C.c_float]),
        "orc_swiglu_det": (None, [f32p, f32p, f32p, sz]),
        "orc_sigmoid_mul_det": (None, [f32p, f32p, f32p, sz]),
        "orc_geglu_det": (None, [f32p, f32p, sz, sz]),
        "orc_rmsnorm_ref": (None, [f32p, f32p, C.c_float, f32p, sz]),
        "orc_rmsnorm_gated_ref": (None, [f32p, f32p, f32p, C.c_float, f32p, sz]),
        "orc_grouped_gemm": (C.c_int, [C.c_int, u8p, sz, i32p, C.c_int, u8p, f32p, sz, sz, C.c_int]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def f16_to_f32(bits):
    return lib.orc_f16_to_f32(int(bits))


def f32_to_f16(v):
    return lib.orc_f32_to_f16(float(np.float32(v)))


def block_size(fmt):
    return lib.orc_block_size(fmt)


def bytes_per_block(fmt):
    return lib.orc_bytes_per_block(fmt)


def get_scale_min_k4(j, q12):
    q = _u8(np.asarray(q12, dtype=np.uint8))
    sc = np.zeros(1, np.uint8)
    m = np.zeros(1, np.uint8)
    lib.orc_get_scale_min_k4(j, _p(q), _p(sc), _p(m))
    return int(sc[0]), int(m[0])


def dequantize_to_f32(fmt, raw, n_elems):
    raw = _u8(raw)
    assert raw.size >= n_elems // block_size(fmt) * bytes_per_block(fmt)
    out = np.empty(n_elems, np.float32)
    rc = lib.orc_dequantize_to_f32(fmt, _p(raw), _p(out), n_elems)
    assert rc == 0
    return out


def repacked_n_sub_padded(in_dim):
    return lib.orc_repacked_n_sub_padded(in_dim)


def repacked_len(fmt, in_dim, out_dim):
    return lib.orc_repacked_len(fmt, in_dim, out_dim)


def repack_for_matvec(fmt, raw, in_dim, out_dim):
    raw = _u8(raw)
    assert raw.size >= out_dim * (in_dim // block_size(fmt)) * bytes_per_block(fmt)
    out = np.empty(repacked_len(fmt, in_dim, out_dim), np.uint8)
    rc = lib.orc_repack_for_matvec(fmt, _p(raw), in_dim, out_dim, _p(out))
    assert rc == 0
    return out


def decode_repacked_to_f32(fmt, packed, in_dim, out_dim):
    packed = _u8(packed)
    assert packed.size == repacked_len(fmt, in_dim, out_dim)
    out = np.empty((out_dim, in_dim), np.float32)
    rc = lib.orc_decode_repacked_to_f32(fmt, _p(packed), in_dim, out_dim, _p(out))
    assert rc == 0
    return out


def q8_0_quantize_from_f32(vals):
    vals = _f32(vals).ravel()
    assert vals.size % 32 == 0
    out = np.empty(vals.size // 32 * 34, np.uint8)
    lib.orc_q8_0_quantize_from_f32(_p(vals), vals.size, _p(out))
    return out


def quantize_q8(x, in_dim=None):
    """x: [n_vec, in_dim] (or 1-D) fp32 -> uint8 [n_vec * in_dim/32 * 40]."""
    x = _f32(x)
    if x.ndim == 1:
        x = x[None, :]
    n_vec, k = x.shape
    assert k % 32 == 0
    out = np.empty(n_vec * (k // 32) * 40, np.uint8)
    lib.orc_quantize_q8(_p(x), k, n_vec, _p(out))
    return out


def block_dots(fmt, packed, in_dim, out_dim, xq, n_rows):
    packed, xq = _u8(packed), _u8(xq)
    assert packed.size == repacked_len(fmt, in_dim, out_dim)
    assert xq.size == n_rows * (in_dim // 32) * 40
    parts = lib.orc_block_dot_parts(fmt)
    out = np.empty((n_rows, out_dim, in_dim // 32, parts), np.int32)
    rc = lib.orc_block_dots(fmt, _p(packed), in_dim, out_dim, _p(xq), n_rows, _p(out))
    assert rc == 0
    return out


def matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows=1, n_threads=8):
    packed, xq = _u8(packed), _u8(xq)
    assert packed.size == repacked_len(fmt, in_dim, out_dim)
    assert xq.size == n_rows * (in_dim // 32) * 40
    y = np.empty((n_rows, out_dim), np.float32)
    rc = lib.orc_matvec_q8(fmt, _p(packed), in_dim, out_dim, _p(xq), n_rows, _p(y), n_threads)
    assert rc == 0
    return y


def matvec_f32(x, w, n_threads=8):
    """w: [out_dim, in_dim] fp32, x: [in_dim] -> y [out_dim]."""
    w, x = _f32(w), _f32(x)
    out_dim, in_dim = w.shape
    assert x.shape == (in_dim,)
    y = np.empty(out_dim, np.float32)
    lib.orc_matvec_f32(_p(x), _p(w), in_dim, out_dim, _p(y), n_threads)
    return y


def moe_topk(logits, n_used):
    logits = _f32(logits)
    n_tok, n_expert = logits.shape
    ids = np.empty((n_tok, n_used), np.int32)
    w = np.empty((n_tok, n_used), np.float32)
    lib.orc_moe_topk(_p(logits), n_tok, n_expert, n_used, _p(ids), _p(w))
    return ids, w


def moe_sort(ids, n_expert, bn):
    ids = _i32(ids).ravel()
    n = ids.size
    perm = np.full(n, -1, np.int32)
    eoff = np.empty(n_expert + 1, np.int32)
    toff = np.empty(n_expert + 1, np.int32)
    lib.orc_moe_sort(_p(ids), n, n_expert, bn, _p(perm), _p(eoff), _p(toff))
    return perm, eoff, toff


def moe_gather_xq(xq_src, perm, nsub, n_used):
    xq_src, perm = _u8(xq_src), _i32(perm)
    out = np.empty(perm.size * nsub * 40, np.uint8)
    lib.orc_moe_gather_xq(_p(xq_src), _p(perm), _p(out), nsub, n_used, perm.size)
    return out


def moe_scatter_rows(src, perm, dim):
    src, perm = _f32(src), _i32(perm)
    out = np.zeros((perm.size, dim), np.float32)
    lib.orc_moe_scatter_rows(_p(src), _p(perm), _p(out), dim, perm.size)
    return out


def moe_combine(experts, ids, weights, down_exps_s):
    experts, ids, weights, s = _f32(experts), _i32(ids), _f32(weights), _f32(down_exps_s)
    n_tok, n_used, hidden = experts.shape
    out = np.empty((n_tok, hidden), np.float32)
    lib.orc_moe_combine(_p(experts), _p(ids), _p(weights), _p(s), _p(out), n_tok, hidden, n_used)
    return out


def swiglu_mul(gate, up):
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    lib.orc_swiglu_mul(_p(gate), _p(up), _p(out), gate.size)
    return out


# ---- relabelled GGUF types
def q3_k_dequantize(raw, n):
    """src/quant/q3_k.rs:124-165"""
    raw = _u8(raw)
    out = np.empty(n, np.float32)
    lib.orc_q3_k_dequantize(_p(raw), _p(out), n)
    return out


def iq4_nl_dequantize(raw, n):
    """src/quant/iq4_nl.rs:34-50"""
    raw = _u8(raw)
    out = np.empty(n, np.float32)
    lib.orc_iq4_nl_dequantize(_p(raw), _p(out), n)
    return out


def iq3s_grid_entry(idx):
    return int(lib.orc_iq3s_grid_entry(idx))


def bf16_to_f32(bits):
    """src/quant/half.rs:42-46"""
    bits = np.ascontiguousarray(bits, np.uint16)
    out = np.empty(bits.size, np.float32)
    lib.orc_bf16_to_f32(_p(bits), _p(out), bits.size)
    return out


# ---- fused BlockQ8 producers: fp32 results (BlockQ8 form = quantize_q8 of them)
_DET = {"exp": 0, "silu": 1, "sigmoid": 2, "gelu": 4}


def map_det(which, x):
    """the deterministic elementwise functions the fused producers use"""
    x = _f32(x)
    out = np.empty_like(x)
    lib.orc_map_det(_DET[which], _p(x), _p(out), x.size)
    return out


def map_ref(which, x):
    """the reference CPU forms with libm (src/cpu/ops.rs:14-36)"""
    x = _f32(x)
    out = np.empty_like(x)
    lib.orc_map_ref(_DET[which], _p(x), _p(out), x.size)
    return out


def sumsq_det(x):
    x = _f32(x)
    return float(lib.orc_sumsq_det(_p(x), x.size))


def add_rmsnorm(hidden, add, w, eps):
    """-> (hidden after the add, y); hidden/add [n_vec, n], w [n]"""
    hidden = np.array(_f32(hidden), copy=True)
    n_vec, n = hidden.shape
    w = _f32(w)
    y = np.empty_like(hidden)
    a = _f32(add) if add is not None else None
    lib.orc_add_rmsnorm(_p(hidden), _p(a) if a is not None else None, _p(w), _p(y), n, n_vec, eps)
    return hidden, y


def rmsnorm_gated(x, z, w, eps):
    x, z, w = _f32(x), _f32(z), _f32(w)
    n_heads, head_dim = x.shape
    y = np.empty_like(x)
    lib.orc_rmsnorm_gated(_p(x), _p(z), _p(w), _p(y), n_heads, head_dim, eps)
    return y


def swiglu_det(gate, up):
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    lib.orc_swiglu_det(_p(gate), _p(up), _p(out), gate.size)
    return out


def sigmoid_mul_det(x, gate):
    x, gate = _f32(x), _f32(gate)
    out = np.empty_like(x)
    lib.orc_sigmoid_mul_det(_p(x), _p(gate), _p(out), x.size)
    return out


def geglu_det(gu):
    """gu [n_slot, 2*ff] -> [n_slot, ff]"""
    gu = _f32(gu)
    n_slot, two_ff = gu.shape
    out = np.empty((n_slot, two_ff // 2), np.float32)
    lib.orc_geglu_det(_p(gu), _p(out), two_ff // 2, n_slot)
    return out


def rmsnorm_ref(x, w, eps):
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    lib.orc_rmsnorm_ref(_p(x), _p(w), eps, _p(out), x.size)
    return out


def rmsnorm_gated_ref(x, gate, w, eps):
    x, gate, w = _f32(x), _f32(gate), _f32(w)
    out = np.empty_like(x)
    lib.orc_rmsnorm_gated_ref(_p(x), _p(gate), _p(w), eps, _p(out), x.size)
    return out


def grouped_gemm(fmt, slab, bytes_per_expert, expert_off, xq, in_dim, out_dim, n_threads=8):
    slab, xq, expert_off = _u8(slab), _u8(xq), _i32(expert_off)
    n_expert = expert_off.size - 1
    n_entries = int(expert_off[-1])
    y = np.zeros((n_entries, out_dim), np.float32)
    rc = lib.orc_grouped_gemm(fmt, _p(slab), bytes_per_expert, _p(expert_off), n_expert, _p(xq),
                              _p(y), in_dim, out_dim, n_threads)
    assert rc == 0
    return y
