"""Launch sites of the path, as thin wrappers over the C ABI.  Arguments are
device pointers (ints or DeviceBuf) exactly as the C functions take them."""
import ctypes as C

from ._lib import MoeShape, check, lib
from .hip import DeviceBuf


def _p(x):
    if isinstance(x, DeviceBuf):
        return x.ptr
    return x


def _s(stream):
    return stream.raw if stream is not None else None


def quantize_q8(x, xq, in_dim, n_vec=1, stream=None):
    """launch_quantize_q8 (src/runtime/qwen35.rs:3202-3211)"""
    check(lib.rein_quantize_q8(_p(x), _p(xq), in_dim, n_vec, _s(stream)))


def rmsnorm_q8(x, w, xq, n, n_vec=1, eps=1e-6, stream=None):
    """rmsnorm_q8_f32 (kernels/rmsnorm_q8.cpp:38-103): xq = q8(rmsnorm(x) * w)"""
    check(lib.rein_rmsnorm_q8(_p(x), _p(w), _p(xq), n, n_vec, eps, _s(stream)))


def add_rmsnorm_q8(hidden, add, w, y, xq, n, n_vec=1, eps=1e-6, stream=None):
    """add_rmsnorm_q8_f32 (kernels/qwen35_fused.cpp:66-121): hidden += add; y, xq = rmsnorm(hidden) * w"""
    check(lib.rein_add_rmsnorm_q8(_p(hidden), _p(add), _p(w), _p(y), _p(xq), n, n_vec, eps, _s(stream)))


def swiglu_q8(gate, up, out, xq, n, stream=None):
    """swiglu_q8_f32 (kernels/qwen35_fused.cpp:132-146): out, xq = silu(gate) * up"""
    check(lib.rein_swiglu_q8(_p(gate), _p(up), _p(out), _p(xq), n, _s(stream)))


def sigmoid_mul_q8(x, gate, xq, n, stream=None):
    """sigmoid_mul_q8_f32 (kernels/qwen35_fused.cpp:149-162): x *= sigmoid(gate); xq = q8(x)"""
    check(lib.rein_sigmoid_mul_q8(_p(x), _p(gate), _p(xq), n, _s(stream)))


def rmsnorm_gated_q8(x, z, w, y, xq, n_heads, head_dim, eps=1e-6, stream=None):
    """rmsnorm_gated_q8_f32 (kernels/qwen35_fused.cpp:195-217)"""
    check(lib.rein_rmsnorm_gated_q8(_p(x), _p(z), _p(w), _p(y), _p(xq), n_heads, head_dim, eps, _s(stream)))


def moe_geglu_q8(gu, xq, ff_exp, n_slot, stream=None):
    """moe_geglu_q8_f32 (kernels/moe_geglu_q8.cpp:31-66): xq = q8(gelu(gate) * up)"""
    check(lib.rein_moe_geglu_q8(_p(gu), _p(xq), ff_exp, n_slot, _s(stream)))


def matvec_xq8(fmt, w, xq, y, in_dim, out_dim, stream=None):
    """launch_matvec_repacked_xq8 (src/runtime/qwen35.rs:2232-2280)"""
    check(lib.rein_matvec_xq8(fmt, _p(w), _p(xq), _p(y), in_dim, out_dim, _s(stream)))


def matvec_batched_xq8(fmt, w, xq, y, in_dim, out_dim, n_rows, stream=None):
    """matmul_kquant_batched_into minus its quantize (src/runtime/prefill.rs:448-508)"""
    check(lib.rein_matvec_batched_xq8(fmt, _p(w), _p(xq), _p(y), in_dim, out_dim, n_rows, _s(stream)))


def matvec_multi_xq8(fmts, ws, ys, out_dims, xq, in_dim, n_rows=1, stream=None):
    """the decode step's consecutive matvecs on the same activations (Q / K / V, gate / up; src/runtime/qwen35.rs:2670-2672,
    2702-2703) as one launch: ys[i][n_rows][out_dims[i]] = xq . ws[i]^T, up to four matrices and four rows"""
    n = len(fmts)
    check(lib.rein_matvec_multi_xq8(n, (C.c_int * n)(*fmts), (C.c_void_p * n)(*[_p(w) for w in ws]),
                                    (C.c_void_p * n)(*[_p(y) for y in ys]), (C.c_uint * n)(*out_dims), _p(xq), in_dim,
                                    n_rows, _s(stream)))


def matvec_kernel_name(fmt, in_dim, out_dim, n_rows):
    """the kernel a product of 1..32 activation rows launches for this shape ('' where rein_mmq_xq8 launches token tiles)"""
    buf = C.create_string_buffer(64)
    check(lib.rein_matvec_kernel_name(fmt, in_dim, out_dim, n_rows, buf, len(buf)))
    return buf.value.decode()


def matvec_ondisk_xq8(fmt, w_blocks, xq, y, in_dim, out_dim, stream=None):
    """the on-disk-layout dp4a matvec (src/runtime/qwen35.rs:2209-2229)"""
    check(lib.rein_matvec_ondisk_xq8(fmt, _p(w_blocks), _p(xq), _p(y), in_dim, out_dim, _s(stream)))


def matvec_q8_0_splitk(w, xq, y_partials, in_dim, out_dim, n_split, stream=None):
    """matvec_q8_0_repacked_splitk_f32 (kernels/matvec_q8_0_repacked.cpp:117-176)"""
    check(lib.rein_matvec_q8_0_splitk(_p(w), _p(xq), _p(y_partials), in_dim, out_dim, n_split, _s(stream)))


def mmq_xq8(fmt, w, xq, y, in_dim, out_dim, p_rows, stream=None):
    """matmul_mmq_into minus its quantize (src/runtime/prefill.rs:512-567)"""
    check(lib.rein_mmq_xq8(fmt, _p(w), _p(xq), _p(y), in_dim, out_dim, p_rows, _s(stream)))


def mmq_workspace_bytes(fmt, in_dim, p_rows):
    """bytes of workspace mmq_xq8_ws wants for this shape (0: none)"""
    return int(lib.rein_mmq_workspace_bytes(fmt, in_dim, p_rows))


def mmq_form_ws(fmt, in_dim, out_dim, p_rows, workspace_bytes):
    """0: int8 launch, 1: fp6 with one token group per workgroup, 2: fp6 split-tail, 3: int8 split-tail,
    4: fp16 with superblocks summed in the matrix unit (REIN_MMQ16=1)"""
    return int(lib.rein_mmq_form_ws(fmt, in_dim, out_dim, p_rows, workspace_bytes))


def mmq_workspace_min_bytes(fmt, in_dim, p_rows):
    """the smallest workspace rein_mmq_xq8_ws accepts: the activation image alone (no split-tail launch)"""
    return int(lib.rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows))


def mmq_xq8_ws(fmt, w, xq, y, in_dim, out_dim, p_rows, workspace, workspace_bytes, stream=None):
    """mmq_xq8 with the caller's workspace (the scratch PrefillGemm keeps, prefill.rs:479-495)"""
    check(lib.rein_mmq_xq8_ws(fmt, _p(w), _p(xq), _p(y), in_dim, out_dim, p_rows, _p(workspace), workspace_bytes,
                              _s(stream)))


def noalloc_prepare():
    """rein_noalloc_prepare: place the fixed scratch array on the current device; outside any capture."""
    check(lib.rein_noalloc_prepare())


def mmq_xq8_noalloc(fmt, w, xq, y, in_dim, out_dim, p_rows, stream=None):
    """mmq_xq8_ws on the library's fixed 48 MiB device array: allocates nothing"""
    check(lib.rein_mmq_xq8_noalloc(fmt, _p(w), _p(xq), _p(y), in_dim, out_dim, p_rows, _s(stream)))


def mmq_tile_plan_ws(fmt, out_dim, p_rows):
    """(n4, n2): token groups of four and of two 32-token tiles per 128-row block in mmq_xq8_ws"""
    n4, n2 = C.c_uint(0), C.c_uint(0)
    check(lib.rein_mmq_tile_plan_ws(fmt, out_dim, p_rows, C.byref(n4), C.byref(n2)))
    return n4.value, n2.value


def mmq_block_dots_ws(fmt, w, xq, out, in_dim, out_dim, n_rows, workspace, workspace_bytes, stream=None):
    check(lib.rein_mmq_block_dots_ws(fmt, _p(w), _p(xq), _p(out), in_dim, out_dim, n_rows, _p(workspace),
                                     workspace_bytes, _s(stream)))


def matmul_scratch_bytes(fmt, in_dim, n_rows):
    return int(lib.rein_matmul_scratch_bytes(fmt, in_dim, n_rows))


def matmul_ws(fmt, w, x, y, in_dim, out_dim, n_rows, scratch, scratch_bytes, stream=None):
    """matmul with one scratch buffer for the quantized activations and the MMQ workspace"""
    check(lib.rein_matmul_ws(fmt, _p(w), _p(x), _p(y), in_dim, out_dim, n_rows, _p(scratch), scratch_bytes, _s(stream)))


def matmul(fmt, w, x, y, in_dim, out_dim, n_rows, xq_scratch, stream=None):
    """PrefillGemm::matmul_into_raw (src/runtime/prefill.rs:343-384)"""
    check(lib.rein_matmul(fmt, _p(w), _p(x), _p(y), in_dim, out_dim, n_rows, _p(xq_scratch), _s(stream)))


def matmul_path(fmt, n_rows):
    rc = lib.rein_matmul_path(fmt, n_rows)
    if rc < 0:
        check(rc)
    return ("matvec", "batched_matvec", "mmq")[rc]


def mmq_tile_plan(fmt, in_dim, out_dim, p_rows):
    """64-token tiles per 128-row block that mmq_xq8 launches for this shape (0: 32-token tiles only)"""
    rc = lib.rein_mmq_tile_plan(fmt, in_dim, out_dim, p_rows)
    if rc < 0:
        check(rc)
    return rc


def block_dots(fmt, w, xq, out, in_dim, out_dim, n_rows, via_mfma=False, stream=None):
    check(lib.rein_block_dots(fmt, _p(w), _p(xq), _p(out), in_dim, out_dim, n_rows, int(via_mfma), _s(stream)))


def moe_topk(logits, n_tok, n_expert, n_used, out_ids, out_weights, stream=None):
    check(lib.rein_moe_topk(_p(logits), n_tok, n_expert, n_used, _p(out_ids), _p(out_weights), _s(stream)))


def moe_sort(ids, n_entries, n_expert, bn, count, cursor, perm, expert_off, tile_off, stream=None):
    check(lib.rein_moe_sort(_p(ids), n_entries, n_expert, bn, _p(count), _p(cursor), _p(perm),
                            _p(expert_off), _p(tile_off), _s(stream)))


def moe_gather_xq(xq_src, perm, xq_dst, nsub, n_used, n_entries, stream=None):
    check(lib.rein_moe_gather_xq(_p(xq_src), _p(perm), _p(xq_dst), nsub, n_used, n_entries, _s(stream)))


def moe_quantize_scatter(x, inv, xq_dst, in_dim, n_used, n_tok, stream=None):
    """quantize_q8 + moe_gather_xq in one launch (inv = inverse of the sort's perm)"""
    check(lib.rein_moe_quantize_scatter(_p(x), _p(inv), _p(xq_dst), in_dim, n_used, n_tok, _s(stream)))


def moe_scatter_rows(src, perm, dst, dim, n_entries, stream=None):
    check(lib.rein_moe_scatter_rows(_p(src), _p(perm), _p(dst), dim, n_entries, _s(stream)))


def moe_grouped_gemm(fmt, slab, bytes_per_expert, expert_off, tile_off, n_expert, xq, y, in_dim, out_dim,
                     n_entries, stream=None):
    check(lib.rein_moe_grouped_gemm(fmt, _p(slab), bytes_per_expert, _p(expert_off), _p(tile_off), n_expert,
                                    _p(xq), _p(y), in_dim, out_dim, n_entries, _s(stream)))


def moe_grouped_swiglu_q8(fmt, gate_slab, up_slab, bytes_per_expert, expert_off, tile_off, n_expert, xq, xq_out,
                          in_dim, out_dim, n_entries, stream=None):
    """gate + up grouped GEMM with SwiGLU and the BlockQ8 quantizer in the epilogue"""
    check(lib.rein_moe_grouped_swiglu_q8(fmt, _p(gate_slab), _p(up_slab), bytes_per_expert, _p(expert_off),
                                         _p(tile_off), n_expert, _p(xq), _p(xq_out), in_dim, out_dim, n_entries,
                                         _s(stream)))


def moe_expert_matvec(fmt, slab, ids, xq, y, in_dim, out_dim, bytes_per_expert, xq_tok_stride, xq_slot_stride,
                      n_used, n_tok=1, stream=None):
    """launch_moe_expert_matvec (src/runtime/qwen35.rs:3071-3100)"""
    check(lib.rein_moe_expert_matvec(fmt, _p(slab), _p(ids), _p(xq), _p(y), in_dim, out_dim, bytes_per_expert,
                                     xq_tok_stride, xq_slot_stride, n_used, n_tok, _s(stream)))


def moe_down(fmt, slab, ids, xq, y, in_dim, out_dim, bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used,
             n_tok=1, stream=None):
    """launch_moe_down (src/runtime/qwen35.rs:3102-3139)"""
    check(lib.rein_moe_down(fmt, _p(slab), _p(ids), _p(xq), _p(y), in_dim, out_dim, bytes_per_expert,
                            xq_tok_stride, xq_slot_stride, n_used, n_tok, _s(stream)))


def moe_gate_up_swiglu(fmt, gate_slab, up_slab, ids, xq, y, in_dim, out_dim, bytes_per_expert, xq_tok_stride,
                       xq_slot_stride, n_used, n_tok=1, stream=None):
    """launch_moe_gate_up_swiglu (src/runtime/qwen35.rs:3141-3167)"""
    check(lib.rein_moe_gate_up_swiglu(fmt, _p(gate_slab), _p(up_slab), _p(ids), _p(xq), _p(y), in_dim, out_dim,
                                      bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used, n_tok, _s(stream)))


def moe_gate_up_swiglu_q8(fmt, gate_slab, up_slab, ids, xq, xq_out, in_dim, out_dim, bytes_per_expert, xq_tok_stride,
                          xq_slot_stride, n_used, n_tok=1, stream=None):
    """moe_gate_up_swiglu followed by quantize_q8 in one launch (BlockQ8 rows of the down projection's input)"""
    check(lib.rein_moe_gate_up_swiglu_q8(fmt, _p(gate_slab), _p(up_slab), _p(ids), _p(xq), _p(xq_out), in_dim, out_dim,
                                         bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used, n_tok, _s(stream)))


def moe_down_combine(fmt, slab, ids, weights, down_exps_s, xq, out, in_dim, out_dim, bytes_per_expert, xq_tok_stride,
                     xq_slot_stride, n_used, n_tok=1, stream=None):
    """moe_down followed by moe_combine in one launch"""
    check(lib.rein_moe_down_combine(fmt, _p(slab), _p(ids), _p(weights), _p(down_exps_s), _p(xq), _p(out), in_dim,
                                    out_dim, bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used, n_tok,
                                    _s(stream)))


def swiglu_mul(gate, up, out, n, stream=None):
    check(lib.rein_swiglu_mul(_p(gate), _p(up), _p(out), n, _s(stream)))


def moe_combine(experts, ids, weights, down_exps_s, out, n_tok, hidden, n_used, stream=None):
    check(lib.rein_moe_combine(_p(experts), _p(ids), _p(weights), _p(down_exps_s), _p(out), n_tok, hidden,
                               n_used, _s(stream)))


def moe_gemm_bn():
    return lib.rein_moe_gemm_bn()


def moe_shape(n_tok, hidden, n_expert, n_used, expert_ff, gate_up_fmt, down_fmt):
    return MoeShape(n_tok, hidden, n_expert, n_used, expert_ff, gate_up_fmt, down_fmt)


def moe_workspace_bytes(shape):
    return lib.rein_moe_workspace_bytes(C.byref(shape))


def moe_ffn(shape, x, logits, gate_exps, up_exps, down_exps, down_exps_s, workspace, out, stream=None):
    """routed-expert part of step_moe_ffn_batched (src/runtime/qwen35.rs:2788-2870)"""
    check(lib.rein_moe_ffn(C.byref(shape), _p(x), _p(logits), _p(gate_exps), _p(up_exps), _p(down_exps),
                           _p(down_exps_s), _p(workspace), _p(out), _s(stream)))
