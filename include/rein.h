/*
 * librein — C ABI of the MI355X (gfx950) quantized-weight matmul path.
 *
 * Drop-in boundary for sixvolts/reinstinct's `src/quant` (repacked-v2 layouts)
 * and `src/hip` (module / launch surface) for this one path.  Plain pointers
 * and sizes only; every `void*` that is not marked "host" is a device pointer;
 * `rein_stream_t` is a `hipStream_t` (NULL = the default stream).
 *
 * Error model (reference: src/hip/mod.rs:17-22): every call returns 0 on
 * success, a positive `hipError_t` when a HIP call failed, or a negative
 * REIN_E_* code for argument / library errors.  `rein_last_error()` returns a
 * thread-local message of the form "<context>: <hipGetErrorString> (code N)".
 * Nothing throws across the boundary.  There is no CPU fallback: if the HIP
 * runtime or the gfx950 code object cannot be loaded, every compute call fails.
 *
 * Format ids are the reference's GgmlType discriminants
 * (src/gguf/types.rs:16-35).
 */
#ifndef REIN_H
#define REIN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    REIN_TYPE_Q4_0   = 2,
    REIN_TYPE_Q8_0   = 8,
    REIN_TYPE_Q4_K   = 12,
    REIN_TYPE_Q5_K   = 13,
    REIN_TYPE_Q6_K   = 14,
    REIN_TYPE_IQ4_XS = 23,
    /* relabelled: own repack, the kernels of another format compiled with another scale
     * source / codebook (src/quant/q5_1.rs:12-20, src/quant/iq3_s.rs:13-19).  Q5_1 has MoE
     * expert kernels only, IQ3_S dense kernels only, as in the reference. */
    REIN_TYPE_Q5_1   = 7,
    REIN_TYPE_IQ3_S  = 21
};
/* ggml types that have no kernels of their own but load onto one of the layouts above
 * (rein_ingest_for_matvec) */
enum {
    REIN_GGML_Q3_K   = 11,   /* -> Q6_K, exact */
    REIN_GGML_IQ4_NL = 20,   /* -> IQ4_XS, exact */
    REIN_GGML_BF16   = 30    /* -> Q8_0, one quantization step */
};

enum {
    REIN_OK            = 0,
    REIN_E_NOT_LOADED  = -1,   /* libamdhip64.so or the code object is not loaded */
    REIN_E_BAD_FORMAT  = -2,   /* unknown / unsupported format id */
    REIN_E_BAD_SHAPE   = -3,   /* dimension not a block multiple, zero, or out of range */
    REIN_E_BAD_POINTER = -4,   /* NULL or misaligned pointer */
    REIN_E_NO_KERNEL   = -5,   /* symbol missing from the code object */
    REIN_E_TOO_LARGE   = -6,   /* exceeds a documented fixed limit */
    REIN_E_BAD_FILE    = -7,   /* GGUF container: io error, bad magic / version, truncated, bad type or shape */
    REIN_E_NOT_FOUND   = -8    /* no tensor / metadata key of that name, or index out of range */
};

typedef void *rein_stream_t;   /* hipStream_t   */
typedef void *rein_event_t;    /* hipEvent_t    */
typedef void *rein_graph_t;    /* hipGraph_t    */
typedef void *rein_graph_exec_t; /* hipGraphExec_t */
typedef void *rein_module_t;   /* hipModule_t   */
typedef void *rein_function_t; /* hipFunction_t */

/* ------------------------------------------------------------------ errors */
const char *rein_last_error(void);

/* ---------------------------------------------------------- runtime / init */
/* dlopen libamdhip64.so (candidates as src/hip/sys.rs:128-135), resolve the
 * entry points of src/hip/sys.rs:57-101, and load the gfx950 code object.
 * `hsaco_path` NULL = "rein_gfx950.hsaco" next to librein.so.  Idempotent;
 * thread-safe (reference: OnceLock, sys.rs:122-127). */
int rein_init(const char *hsaco_path);
/* 1 when rein_init has succeeded in this process */
int rein_is_loaded(void);

/* ----------------------------------------------------------------- options */
/* The switches that pin a launch choice (which kernel family, which tiling) instead of
 * leaving it to the library's cost models.  No counterpart in the reference, whose launch
 * shapes are fixed; the tests use them to reach every kernel family, and a host may pin a
 * choice it has measured.  An option is unset (the library decides) or set to an unsigned
 * decimal number.  The environment variables of the same names are read ONCE per process, when
 * the table is first looked at (rein_init looks); after that only these calls change it, so
 * what an entry point launches depends on its arguments and on this table alone.  A set option
 * pins its choice whatever its value: several cost models step aside as soon as the option that
 * overrides them is set, and setting it back to NULL / "" hands the choice back.  Entries are
 * single atomic words; changing one while another thread launches is safe.
 * Names (rein_option_name enumerates them): REIN_MV_ROWS, REIN_MV_WPB (decode matvec rows per
 * wavefront 1/2/4, wavefronts per workgroup 1/2/4; 1..16 for the LDS-staged kernel), REIN_MV_LDS
 * (batched decode of 2..4 rows on the kernel that stages the activation rows in LDS: 0 never,
 * 1 whenever the rows fit), REIN_QUAD_LDS (the same for the 4x4x4 kernel, 3..8 rows),
 * REIN_QUAD_SLICES, REIN_QUAD_DEPTH (wavefronts that share a row group of that kernel, 1..8;
 * trips of weights in flight per wavefront, 1 or 2), REIN_QUAD_WIDE32 (17..32 rows on that kernel:
 * 1 the build for sixteen wavefronts per workgroup, 0 the build for eight),
 * REIN_SKINNY_FROM, REIN_SKINNY_KS,
 * REIN_QUAD_FROM (batched decode: row count from which the skinny MMQ / the 4x4x4 kernel run,
 * wavefronts per row tile), REIN_GROUPED_STRIDED (1: the reference-named strided grouped
 * kernel), REIN_MMQ_TM, REIN_MMQ_N64 (int8 GEMM tile: 32 forces 32-token tiles; 64-token tiles
 * per row block), REIN_MMQ_SK, REIN_MMQ_SK_GRID, REIN_MMQ_SK_SPLIT, REIN_MMQ_SK_TM (split-tail
 * launch of the int8 tile: 0 off / 2 forced, resident workgroups, ranges per tail unit, unit
 * width), REIN_MMQ6, REIN_MMQ6_FROM, REIN_MMQ6_N4, REIN_MMQ6_N2, REIN_MMQ6_SK,
 * REIN_MMQ6_SK_GRID, REIN_MMQ6_SK_SPLIT (Q4_K fp6 launch: 0 off, first row count, token groups
 * of four / two tiles per row block, split-tail 0 off / 2 forced, its grid and ranges),
 * REIN_MMQ16 (1: the fp16 formulation where the code object holds it), REIN_TOPK_WAVE,
 * REIN_MOE_SORT_SPLIT, REIN_MOE_CHAIN, REIN_MOE_FUSED, REIN_MOE_GU_ROWS, REIN_MOE_DC_ROWS (MoE
 * glue: 0 = the workgroup router, 1 = the four-launch sort, 0 = no decode chain for few
 * tokens, 0 = unfused gate/up, rows per workgroup of the two decode launches).
 * Unknown name: REIN_E_NOT_FOUND; a value that is not an unsigned 32-bit decimal:
 * REIN_E_BAD_SHAPE. */
int rein_set_option(const char *name, const char *value);   /* value NULL or "": unset */
int rein_get_option(const char *name, unsigned *value, int *is_set);
int rein_reset_options(void);                                /* every option unset (the environment is not read again) */
int rein_option_count(void);
const char *rein_option_name(int index);                     /* NULL outside [0, rein_option_count()) */

/* src/hip/mod.rs:25-58, 88-131 */
int rein_device_count(int *n);
int rein_set_device(int device);
int rein_get_device(int *device);
int rein_device_name(int device, char *buf, int buf_len);   /* buf: host */
int rein_device_total_mem(int device, size_t *bytes);
int rein_mem_info(size_t *free_bytes, size_t *total_bytes);
int rein_device_synchronize(void);

/* DeviceBuf (src/hip/mod.rs:170-330) */
int rein_malloc(void **dptr, size_t bytes);
int rein_free(void *dptr);
int rein_memcpy_h2d(void *dst, const void *src_host, size_t bytes);
int rein_memcpy_d2h(void *dst_host, const void *src, size_t bytes);
int rein_memcpy_d2d(void *dst, const void *src, size_t bytes);
int rein_memcpy_h2d_async(void *dst, const void *src_host, size_t bytes, rein_stream_t s);
int rein_memcpy_d2h_async(void *dst_host, const void *src, size_t bytes, rein_stream_t s);
int rein_memcpy_d2d_async(void *dst, const void *src, size_t bytes, rein_stream_t s);

/* Stream / Event / Graph (src/hip/mod.rs:133-168, 332-435) */
int rein_stream_create(rein_stream_t *s);
int rein_stream_destroy(rein_stream_t s);
int rein_stream_synchronize(rein_stream_t s);
int rein_stream_wait_event(rein_stream_t s, rein_event_t e);
int rein_event_create(rein_event_t *e);
int rein_event_record(rein_event_t e, rein_stream_t s);
int rein_event_synchronize(rein_event_t e);
int rein_event_elapsed_ms(float *ms, rein_event_t start, rein_event_t stop);
int rein_event_destroy(rein_event_t e);
int rein_stream_begin_capture(rein_stream_t s);              /* mode Global, as the reference */
int rein_stream_end_capture(rein_stream_t s, rein_graph_t *g);
int rein_graph_instantiate(rein_graph_exec_t *ge, rein_graph_t g);
int rein_graph_launch(rein_graph_exec_t ge, rein_stream_t s);
int rein_graph_destroy(rein_graph_t g);
int rein_graph_exec_destroy(rein_graph_exec_t ge);

/* Module / Function::launch (src/hip/mod.rs:437-502): load any .hsaco, look a
 * kernel up by name, launch with an array of pointers-to-values (kernelParams). */
int rein_module_load(rein_module_t *m, const char *path);
int rein_module_unload(rein_module_t m);
int rein_module_get_function(rein_function_t *f, rein_module_t m, const char *name);
/* the code object rein_init loaded, for looking up the reference-named kernels */
int rein_builtin_module(rein_module_t *m);
int rein_launch_kernel(rein_function_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                       unsigned by, unsigned bz, unsigned shared_bytes, rein_stream_t s,
                       void **args);

/* ------------------------------------------------------- src/quant mirror */
/* repacked_n_sub_padded (src/quant/q4_k.rs:92-95 and per-format twins) */
size_t rein_repacked_n_sub_padded(size_t in_dim);
/* <fmt>::repacked_len (q4_k.rs:98-102, q5_k.rs, q6_k.rs, q8_0.rs:74-77,
 * q4_0.rs:66-69, iq4_xs.rs:85-88); 0 for an unknown format */
size_t rein_repacked_len(int fmt, size_t in_dim, size_t out_dim);
/* on-disk geometry: weights per block / bytes per block (0 = unknown format) */
int rein_block_size(int fmt);
int rein_bytes_per_block(int fmt);
/* <fmt>::repack_for_matvec (q4_k.rs:126-176, q5_k.rs:97-151, q6_k.rs:86-148,
 * q8_0.rs:93-119, q4_0.rs:86-104, iq4_xs.rs:106-136).  Host to host:
 * `src` holds out_dim*in_dim/block on-disk blocks, `dst` rein_repacked_len
 * bytes.  The reference asserts on a bad in_dim; this returns REIN_E_BAD_SHAPE. */
int rein_repack_for_matvec(int fmt, const uint8_t *src, size_t in_dim, size_t out_dim,
                           uint8_t *dst);
/* GpuMatvecTensor::from_bytes_matvec (src/runtime/qwen35.rs:251-331): GGUF tensor bytes of
 * `ggml_type` -> repacked slab in `dst`, *out_fmt = the format id whose kernels read it.
 * The six kernel formats repack as they are; IQ4_NL -> IQ4_XS and Q3_K -> Q6_K relabel
 * without rounding (src/quant/iq4_nl.rs:52-75, q3_k.rs:85-122); IQ3_S keeps its id on the
 * IQ4_XS planes (src/quant/iq3_s.rs:186-207); BF16 -> Q8_0.  `dst` holds
 * rein_repacked_len(rein_ingest_format(ggml_type), in_dim, out_dim) bytes, `src`
 * rein_ingest_src_len(...).  Other types: REIN_E_BAD_FORMAT. */
int rein_ingest_format(int ggml_type);                 /* 0 when the type has no layout here */
/* the types GpuExpertTensor::from_gguf accepts (qwen35.rs:415-425): Q4_K, Q5_K, Q6_K, Q8_0, Q5_1 */
int rein_ingest_expert_format(int ggml_type);
size_t rein_ingest_src_len(int ggml_type, size_t in_dim, size_t out_dim);
int rein_ingest_for_matvec(int ggml_type, const uint8_t *src, size_t in_dim, size_t out_dim,
                           uint8_t *dst, int *out_fmt);
/* q3_k::transcode_to_q6_k (src/quant/q3_k.rs:85-122): n_weights/256 blocks of 110 bytes ->
 * blocks of 210 bytes that dequantize to the same values bit for bit. */
int rein_transcode_q3_k_to_q6_k(const uint8_t *src, size_t n_weights, uint8_t *dst);
/* ------------------------------------------------------- src/gguf mirror */
/* GGUF v3 container (src/gguf/mod.rs:97-217).  The handle owns a read-only mapping of
 * the file (or borrows the caller's bytes); every pointer handed out points into it and
 * dies with rein_gguf_close.  Parse errors are REIN_E_BAD_FILE with the reference's
 * error text (src/gguf/error.rs:4-47) in rein_last_error(). */
typedef struct rein_gguf rein_gguf;
typedef struct rein_gguf_tensor {        /* TensorInfo (src/gguf/tensor_info.rs:7-17) + its payload */
    const char    *name;                 /* NUL-terminated, owned by the handle */
    int            ggml_type;            /* types.rs:37-59 */
    unsigned       n_dims;               /* 1..4 */
    uint64_t       dims[4];              /* fastest first; unused trailing dims are 1 */
    uint64_t       offset;               /* from the start of the data section */
    uint64_t       byte_size;            /* TensorInfo::byte_size (tensor_info.rs:34-46) */
    const uint8_t *data;                 /* GgufFile::tensor_data (mod.rs:196-201) */
} rein_gguf_tensor;
typedef struct rein_gguf_dims {
    unsigned in_dim, out_dim, n_expert;  /* dims[0], dims[1], dims[2] (1 for a 2-D tensor) */
    size_t   bytes_per_expert;           /* repacked bytes of one [in_dim, out_dim] slab */
} rein_gguf_dims;
/* GgufFile::open (mod.rs:97-102) / from_mmap (mod.rs:104-177) */
int rein_gguf_open(const char *path, rein_gguf **out);
int rein_gguf_from_bytes(const uint8_t *bytes, size_t len, rein_gguf **out);   /* caller keeps bytes alive */
void rein_gguf_close(rein_gguf *g);
/* Header, alignment, data_section_offset (mod.rs:45-49,64-68); any out pointer may be NULL */
int rein_gguf_header(const rein_gguf *g, uint32_t *version, uint64_t *tensor_count,
                     uint64_t *metadata_kv_count, uint64_t *alignment, uint64_t *data_section_offset);
/* align_up (mod.rs:208-210): align <= 1 leaves v as it is */
uint64_t rein_gguf_align_up(uint64_t v, uint64_t align);
/* GgufFile::tensors[i] / tensor(name) (mod.rs:186-188); REIN_E_NOT_FOUND when absent */
int rein_gguf_tensor_at(const rein_gguf *g, uint64_t index, rein_gguf_tensor *out);
int rein_gguf_tensor_by_name(const rein_gguf *g, const char *name, rein_gguf_tensor *out);
/* GgufFile::metadata[i] / metadata_get(key) (mod.rs:181-183) with MetaValue's coercions
 * (src/gguf/value.rs:50-101): u64 from any non-negative integer variant, f32 from F32 / F64.
 * value_type is gguf_metadata_value_type (types.rs:108-113).  A wrong variant is
 * REIN_E_BAD_FORMAT, an absent key REIN_E_NOT_FOUND.  Strings are not NUL-terminated.
 * rein_gguf_meta_raw points at the value's little-endian bytes in the mapping, whatever
 * its type.  For an array `first` points at its packed payload: count fixed-width little-endian
 * elements, or (u64 length, bytes) strings back to back. */
int rein_gguf_meta_at(const rein_gguf *g, uint64_t index, const char **key, int *value_type);
int rein_gguf_meta_type(const rein_gguf *g, const char *key, int *value_type);
int rein_gguf_meta_raw(const rein_gguf *g, const char *key, int *value_type, const uint8_t **value);
int rein_gguf_meta_u64(const rein_gguf *g, const char *key, uint64_t *out);
int rein_gguf_meta_f32(const rein_gguf *g, const char *key, float *out);
int rein_gguf_meta_bool(const rein_gguf *g, const char *key, int *out);
int rein_gguf_meta_str(const rein_gguf *g, const char *key, const char **s, size_t *len);
int rein_gguf_meta_array(const rein_gguf *g, const char *key, int *elem_type, uint64_t *count,
                         const uint8_t **first);
/* GpuMatvecTensor::from_gguf_matvec (src/runtime/qwen35.rs:235-245) for a 2-D tensor and
 * GpuExpertTensor::from_gguf (qwen35.rs:397-431) for a 3-D one: repack tensor `name` into
 * `dst` through rein_ingest_for_matvec, expert slabs back to back.  With dst == NULL only
 * *out_fmt and *dims are filled (dims->bytes_per_expert * dims->n_expert bytes are needed). */
int rein_gguf_load_for_matvec(const rein_gguf *g, const char *name, uint8_t *dst, size_t dst_len,
                              int *out_fmt, rein_gguf_dims *dims);

/* fp32 -> on-disk blocks, host to host, for building synthetic weights.  Q8_0
 * follows q8_0::quantize_from_f32 (q8_0.rs:45-61); the reference has no
 * quantizer for the other five formats, these follow ggml's reference
 * quantizers in structure and produce valid blocks. n must be a block multiple. */
int rein_quantize_weights(int fmt, const float *src, size_t n, uint8_t *dst);

/* ------------------------------------------------------------- hot path */
/* quantize_q8_f32 (kernels/quantize_q8.cpp:23-54; launcher qwen35.rs:3202-3211):
 * x [n_vec][in_dim] fp32 -> xq [n_vec][in_dim/32] 40-byte BlockQ8. */
int rein_quantize_q8(const float *x, void *xq, unsigned in_dim, unsigned n_vec, rein_stream_t s);

/* ---- fused BlockQ8 producers: the step in front of a quantized matvec writes
 * the matvec's input blocks itself.  All dimensions are multiples of 32; every
 * BlockQ8 output is byte-identical to rein_quantize_q8 of the fp32 result.
 *
 * rmsnorm_q8_f32 (kernels/rmsnorm_q8.cpp:38-103; launcher gemma4.rs:1303-1316):
 * xq[v] = q8(x[v] * rsqrt(mean(x[v]^2) + eps) * w) for n_vec vectors of n values,
 * n <= 32768.  w [n] is shared by the vectors. */
int rein_rmsnorm_q8(const float *x, const float *w, void *xq, unsigned n, unsigned n_vec, float eps,
                    rein_stream_t s);
/* add_rmsnorm_q8_f32 (kernels/qwen35_fused.cpp:66-121; launcher qwen35.rs:2036-2054):
 * hidden += add (add may be NULL), y = rmsnorm(hidden) * w as fp32 (y may be NULL)
 * and as BlockQ8.  The reference handles one vector of n % 1024 == 0, n <= 8192;
 * here n_vec vectors of any n % 32 == 0, n <= 32768. */
int rein_add_rmsnorm_q8(float *hidden, const float *add, const float *w, float *y, void *xq,
                        unsigned n, unsigned n_vec, float eps, rein_stream_t s);
/* swiglu_q8_f32 (kernels/qwen35_fused.cpp:132-146; launcher qwen35.rs:2056-2069):
 * out = silu(gate) * up as fp32 (out may be NULL or alias gate) and as BlockQ8. */
int rein_swiglu_q8(const float *gate, const float *up, float *out, void *xq, unsigned n,
                   rein_stream_t s);
/* sigmoid_mul_q8_f32 (kernels/qwen35_fused.cpp:149-162; launcher qwen35.rs:2071-2079):
 * x *= sigmoid(gate) in place, plus BlockQ8. */
int rein_sigmoid_mul_q8(float *x, const float *gate, void *xq, unsigned n, rein_stream_t s);
/* rmsnorm_gated_q8_f32 (kernels/qwen35_fused.cpp:195-217): per head of head_dim values,
 * y = rmsnorm(x) * w * silu(z) as fp32 (y may be NULL) and as BlockQ8; w [head_dim]. */
int rein_rmsnorm_gated_q8(const float *x, const float *z, const float *w, float *y, void *xq,
                          unsigned n_heads, unsigned head_dim, float eps, rein_stream_t s);
/* moe_geglu_q8_f32 (kernels/moe_geglu_q8.cpp:31-66; launcher gemma4.rs:1781-1796):
 * gu [n_slot][2*ff_exp] (gate half, up half) -> xq [n_slot][ff_exp/32] =
 * q8(gelu_tanh(gate) * up). */
int rein_moe_geglu_q8(const float *gu, void *xq, unsigned ff_exp, unsigned n_slot, rein_stream_t s);

/* launch_matvec_repacked_xq8 (src/runtime/qwen35.rs:2232-2280): y[out_dim] =
 * W . xq for one pre-quantized activation row. */
int rein_matvec_xq8(int fmt, const void *w, const void *xq, float *y, unsigned in_dim,
                    unsigned out_dim, rein_stream_t s);
/* matmul_kquant_batched_into without its quantize step (src/runtime/prefill.rs:
 * 448-508): y[n_rows][out_dim], 1 <= n_rows <= 8; the weights are streamed once. */
int rein_matvec_batched_xq8(int fmt, const void *w, const void *xq, float *y, unsigned in_dim,
                            unsigned out_dim, unsigned n_rows, rein_stream_t s);
/* The consecutive launch_matvec_prequant calls of the decode step that share their activations --
 * attn_q / attn_k / attn_v (src/runtime/qwen35.rs:2670-2672, 3612-3614), the dense FFN's gate / up
 * (qwen35.rs:2702-2703, 3662-3663), ssm_alpha / ssm_beta (qwen35.rs:2465-2466) -- as one launch:
 * ys[i][n_rows][out_dims[i]] = xq[n_rows] . ws[i]^T for i < n_mat, 1 <= n_mat <= 4, 1 <= n_rows <= 4
 * (the two to four rows of the speculative-decode verify step, prefill.rs:448-508).  The matrices
 * share in_dim and may differ in format and in out_dims[i]; with one row every output is bit for
 * bit what rein_matvec_xq8 gives for that matrix, with more rows what the dot4 kernels behind
 * rein_matvec_batched_xq8 give (three and four rows against matrices of an FFN's size go out as
 * the launches of rein_matvec_batched_xq8 one by one, which are faster there).  The four tables are
 * host arrays, read before the call returns. */
int rein_matvec_multi_xq8(unsigned n_mat, const int *fmts, const void *const *ws, float *const *ys,
                          const unsigned *out_dims, const void *xq, unsigned in_dim, unsigned n_rows,
                          rein_stream_t s);
/* Which kernel a product of few activation rows launches, given the shape and the option table
 * (host logic only, nothing is launched): 1..8 rows as rein_matvec_xq8 / rein_matvec_batched_xq8
 * dispatch them, 9..32 rows the few-row kernels behind rein_mmq_xq8, "" where that entry point
 * launches token tiles.  The reference picks its kernels in qwen35.rs:2232-2280 by format alone;
 * here the choice also depends on the shape, and this call makes it visible. */
int rein_matvec_kernel_name(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows, char *name,
                            size_t name_len);
/* The on-disk-layout matvec (src/runtime/qwen35.rs:2209-2229; kernels/matvec_q4_k_dp4a.cpp
 * and its Q5_K / Q6_K / Q8_0 siblings): `w_blocks` holds out_dim rows of GGUF blocks as
 * they are on disk (not repacked) -- the path a tied token_embd / output matrix takes.
 * Formats Q4_K, Q5_K, Q6_K, Q8_0; w_blocks 16-byte aligned. */
int rein_matvec_ondisk_xq8(int fmt, const void *w_blocks, const void *xq, float *y, unsigned in_dim,
                           unsigned out_dim, rein_stream_t s);
/* matvec_q8_0_repacked_splitk_f32 (kernels/matvec_q8_0_repacked.cpp:117-176): repacked
 * Q8_0, the contraction split into n_split ranges of ceil(n_sub/n_split) sub-blocks;
 * y_partials [n_split][out_dim] receives one partial sum per range, the caller adds
 * them.  For projections whose out_dim is too small to fill the machine. */
int rein_matvec_q8_0_splitk(const void *w, const void *xq, float *y_partials, unsigned in_dim,
                            unsigned out_dim, unsigned n_split, rein_stream_t s);
/* matmul_mmq_into without its quantize step (src/runtime/prefill.rs:512-567):
 * Y[p_rows][out_dim] = Xq . W^T on the int8 MFMA path.  Few rows take the batched-decode
 * kernels instead of token tiles: up to 8 rows what rein_matvec_batched_xq8 launches, up to 16
 * the skinny MMQ or the LDS-staged 4x4x4 kernel, up to 32 rows against at most 8192 output
 * rows that kernel as well (the tile launch would hand out one workgroup per 128 rows). */
int rein_mmq_xq8(int fmt, const void *w, const void *xq, float *y, unsigned in_dim,
                 unsigned out_dim, unsigned p_rows, rein_stream_t s);
/* The same product with a caller-provided workspace of rein_mmq_workspace_bytes(fmt, in_dim,
 * p_rows) bytes (16-byte aligned; 0 = the row count has no use for one, and NULL
 * falls back to rein_mmq_xq8).  With it Q4_K from 128 rows up runs on the block-scaled fp6
 * matrix instruction: the activations are first brought into operand form in the workspace
 * (one extra launch), then the GEMM streams them from there (GEMMs of less than 2.8e10 operations
 * 2 M N K, about 50 us, and GEMMs with fewer than 1.25 four-tile token groups per CU that do not
 * take the split-tail form below stay on the int8 tile).  The reference keeps such
 * scratch in its PrefillGemm object (src/runtime/prefill.rs:479-495); here the caller owns
 * it, so nothing allocates and the call can be captured into a graph.  Calls that share a
 * workspace must be ordered on one stream.
 * Two sizes: rein_mmq_workspace_min_bytes holds the activation image alone; with
 * rein_mmq_workspace_bytes (the image and one partial tile per resident workgroup, 32 MiB
 * more) the GEMM may run as a split-tail launch -- one workgroup per resident slot, whole tiles
 * in rounds, the tiles left over after the last whole round split along the contraction and
 * their partial tiles summed in a fixed order by a second launch -- which is what evens out shapes
 * such as 512 x 17408 whose tiles do not divide over the CUs.  Any size from the minimum on is
 * accepted; below the full size the GEMM runs its one-tile-group-per-workgroup launch.  Results
 * of the two launches can differ in the order of fp32 additions across superblocks (both within
 * the parity bar); each is reproducible from run to run.
 * Every other dense format, and Q4_K below the fp6 launch's row count, needs no workspace
 * (rein_mmq_workspace_min_bytes = 0) and can use one: rein_mmq_workspace_bytes is then 16 MiB,
 * room for the partial tiles of the same split-tail scheme on the int8 tile (64-token units, or
 * 32-token units where those would be half empty).  The library takes that launch where a GEMM
 * has too few workgroup tiles for the machine or a tail that splits well -- 17408 -> 5120 at 64
 * tokens is 40 workgroup tiles on 256 CUs -- and its own estimate puts it ahead of the plain
 * launch with the second launch counted; the plain launch of rein_mmq_xq8 everywhere else, and
 * whenever the workspace is smaller. */
size_t rein_mmq_workspace_bytes(int fmt, unsigned in_dim, unsigned p_rows);
size_t rein_mmq_workspace_min_bytes(int fmt, unsigned in_dim, unsigned p_rows);
/* Which launch rein_mmq_xq8_ws takes for this shape and workspace size: 0 = the int8 launch of
 * rein_mmq_xq8, 1 = fp6 with one token group per workgroup, 2 = fp6 split-tail, 3 = int8
 * split-tail, 4 = the fp16 formulation that sums whole superblocks in the matrix unit (only
 * with the option REIN_MMQ16 set to 1 and a code object built with it: slower than the others,
 * kept for study). */
int rein_mmq_form_ws(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows, size_t workspace_bytes);
int rein_mmq_xq8_ws(int fmt, const void *w, const void *xq, float *y, unsigned in_dim,
                    unsigned out_dim, unsigned p_rows, void *workspace, size_t workspace_bytes,
                    rein_stream_t s);
/* rein_mmq_xq8_ws without the workspace argument and without any allocation, for callers that
 * cannot allocate device memory: code under graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  The workspace is a fixed array of
 * 48 MiB in device memory that every GPU the process uses holds until the process ends
 * (librein_scratch.so, loaded from the directory of librein.so on the first call); the call
 * launches what rein_mmq_xq8_ws launches for a workspace of that size, the split-tail forms
 * included (rein_mmq_form_ws tells which).  Shapes whose rein_mmq_workspace_min_bytes exceeds
 * 48 MiB are refused with REIN_E_TOO_LARGE (at in_dim 5120 that is above 4608 rows; the
 * split-tail form of the fp6 launch fits to 1536 rows).  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race.
 * "Allocates nothing" holds once the array's address is known on the current device: the first
 * look loads librein_scratch.so and asks the runtime for the symbol's address, which makes the
 * runtime place (and zero) the array on that device.  That step must not fall into a stream
 * capture: call rein_noalloc_prepare() once per device, with that device current and nothing
 * capturing (it also looks up the kernel handles the entry point launches), or make the first
 * call of rein_mmq_xq8_noalloc on the device outside any capture.  Neither this entry point nor
 * rein_noalloc_prepare has a counterpart in the reference; both are for callers that cannot
 * allocate. */
int rein_noalloc_prepare(void);
int rein_mmq_xq8_noalloc(int fmt, const void *w, const void *xq, float *y, unsigned in_dim,
                         unsigned out_dim, unsigned p_rows, rein_stream_t s);
/* How rein_mmq_xq8_ws cuts the tokens of a 128-row block: n4 groups of four 32-token tiles,
 * n2 groups of two, single tiles for the rest.  No counterpart in the reference. */
int rein_mmq_tile_plan_ws(int fmt, unsigned out_dim, unsigned p_rows, unsigned *n4, unsigned *n2);
/* PrefillGemm::matmul_into_raw (src/runtime/prefill.rs:343-384): quantize x
 * [n_rows][in_dim] into the caller's `xq_scratch` (n_rows*in_dim/32*40 bytes),
 * then dispatch by row count: 1 -> matvec, 2..8 -> batched matvec (the reference
 * switches to its narrow MMQ at 5), above -> MMQ. */
int rein_matmul(int fmt, const void *w, const float *x, float *y, unsigned in_dim,
                unsigned out_dim, unsigned n_rows, void *xq_scratch, rein_stream_t s);
/* rein_matmul with one scratch buffer of rein_matmul_scratch_bytes(fmt, in_dim, n_rows) bytes
 * (16-byte aligned) that holds the quantized activations and, for the MMQ path, the workspace
 * of rein_mmq_xq8_ws.  A scratch that only holds the activations runs rein_matmul. */
size_t rein_matmul_scratch_bytes(int fmt, unsigned in_dim, unsigned n_rows);
int rein_matmul_ws(int fmt, const void *w, const float *x, float *y, unsigned in_dim,
                   unsigned out_dim, unsigned n_rows, void *scratch, size_t scratch_bytes,
                   rein_stream_t s);
/* Which path rein_matmul takes: 0 matvec, 1 batched matvec, 2 MMQ; <0 on error. */
int rein_matmul_path(int fmt, unsigned n_rows);
/* How rein_mmq_xq8 tiles the tokens of a P-row GEMM above 16 rows: the number of 64-token
 * tiles per 128-row block; the remaining tokens run in 32-token tiles (0: all of them).
 * The reference launches one fixed tile shape (prefill.rs:536-560); this choice has no
 * counterpart there.  <0 on error. */
int rein_mmq_tile_plan(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows);

/* Debug / parity: per-block int32 dots exactly as the kernels form them.
 * out [n_rows][out_dim][in_dim/32][parts], parts = rein_block_dot_parts(fmt)
 * (2 for Q6_K: one per 16-weight half, each minus 32*sum(q8); Q4_0: dot minus
 * 8*sum(q8); otherwise the raw dot).  via_mfma != 0 takes the dots from the MMQ
 * kernel's MFMA tiles instead of the matvec's v_dot4 path. */
int rein_block_dot_parts(int fmt);
int rein_block_dots(int fmt, const void *w, const void *xq, int32_t *out, unsigned in_dim,
                    unsigned out_dim, unsigned n_rows, int via_mfma, rein_stream_t s);

/* The per-block dots of the workspace launch of rein_mmq_xq8_ws (Q4_K): out [n_rows][out_dim]
 * [in_dim/32] int32, converted from the fp32 results of the fp6 matrix instruction, which are
 * exact integers.  workspace as for rein_mmq_xq8_ws (any n_rows). */
int rein_mmq_block_dots_ws(int fmt, const void *w, const void *xq, int32_t *out, unsigned in_dim,
                           unsigned out_dim, unsigned n_rows, void *workspace,
                           size_t workspace_bytes, rein_stream_t s);

/* ------------------------------------------------------------------- MoE */
/* moe_topk_f32 (kernels/moe_topk.cpp:17-108; launcher qwen35.rs:2873-2886).  Up to 256 experts
 * run on rein_moe_topk_wave (one wavefront per token, same ids and weight bits); the
 * reference-named kernel serves larger expert counts and stays in the code object. */
int rein_moe_topk(const float *logits, unsigned n_tok, unsigned n_expert, unsigned n_used,
                  int32_t *out_ids, float *out_weights, rein_stream_t s);
/* launch_moe_sort (qwen35.rs:2892-2938; kernels/moe_expert_sort.cpp:27-75):
 * counting sort of ids [n_entries] by expert.  count/cursor: n_expert ints of
 * scratch; perm [n_entries]; expert_off/tile_off [n_expert+1]; bn = tokens per
 * GEMM tile used for tile_off. */
int rein_moe_sort(const int32_t *ids, unsigned n_entries, unsigned n_expert, unsigned bn,
                  int32_t *count, int32_t *cursor, int32_t *perm, int32_t *expert_off,
                  int32_t *tile_off, rein_stream_t s);
/* moe_gather_xq / moe_scatter_rows (kernels/moe_expert_sort.cpp:81-110) */
int rein_moe_gather_xq(const void *xq_src, const int32_t *perm, void *xq_dst, unsigned nsub,
                       unsigned n_used, unsigned n_entries, rein_stream_t s);
/* quantize_q8_f32 followed by moe_gather_xq in one launch (no single counterpart in the
 * reference): every row of x [n_tok][in_dim] is quantized once and written to the places
 * inv[tok * n_used + j] of its routing entries in the expert-sorted order (inv = the inverse
 * of the sort's perm; negative = dropped entry); xq_dst [n_tok * n_used][in_dim/32] blocks.
 * The same bytes as the two launches, without the quantized table between them. */
int rein_moe_quantize_scatter(const float *x, const int32_t *inv, void *xq_dst, unsigned in_dim,
                              unsigned n_used, unsigned n_tok, rein_stream_t s);
int rein_moe_scatter_rows(const float *src, const int32_t *perm, float *dst, unsigned dim,
                          unsigned n_entries, rein_stream_t s);
/* launch_moe_grouped_gemm (qwen35.rs:3036-3064; kernels/mmq_gemm_*_grouped.cpp):
 * rows expert_off[e]..expert_off[e+1] of the sorted xq / y against
 * slab + e*bytes_per_expert.  n_entries = total sorted rows (upper bound for the
 * launch). Formats: Q4_K, Q5_K, Q6_K, Q8_0. */
int rein_moe_grouped_gemm(int fmt, const void *slab, unsigned bytes_per_expert,
                          const int32_t *expert_off, const int32_t *tile_off, unsigned n_expert,
                          const void *xq, float *y, unsigned in_dim, unsigned out_dim,
                          unsigned n_entries, rein_stream_t s);
/* Gate and up projection of an expert FFN with SwiGLU and the BlockQ8 quantizer in the GEMM's
 * epilogue: xq_out [n_entries][out_dim/32] blocks = the bytes that rein_moe_grouped_gemm on
 * gate_slab and on up_slab followed by rein_swiglu_q8 (swiglu_q8_f32,
 * kernels/qwen35_fused.cpp:132-146) produce, without the two fp32 matrices between them.
 * out_dim (the expert's ff width) a multiple of 32.  Formats: Q4_K, Q5_K, Q6_K, Q8_0. */
int rein_moe_grouped_swiglu_q8(int fmt, const void *gate_slab, const void *up_slab,
                               unsigned bytes_per_expert, const int32_t *expert_off,
                               const int32_t *tile_off, unsigned n_expert, const void *xq,
                               void *xq_out, unsigned in_dim, unsigned out_dim,
                               unsigned n_entries, rein_stream_t s);
/* ---- MoE decode: expert matvecs, the expert id is read on the device.
 * launch_moe_expert_matvec (qwen35.rs:3071-3100; kernels/moe_matvec_*_repacked.cpp):
 * y[tok][slot][out_dim] = W[ids[tok*n_used+slot]] . xq row at
 * xq + tok*xq_tok_stride + slot*xq_slot_stride (strides in BlockQ8 blocks; slot
 * stride 0 = every slot reads the token's row).  Formats Q4_K, Q5_K, Q6_K, Q8_0. */
int rein_moe_expert_matvec(int fmt, const void *slab, const int32_t *ids, const void *xq, float *y,
                           unsigned in_dim, unsigned out_dim, unsigned bytes_per_expert,
                           unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used,
                           unsigned n_tok, rein_stream_t s);
/* launch_moe_down (qwen35.rs:3102-3139; kernels/moe_matvec_{q5k,q6k}_down.cpp): the same
 * product for the down projection, whose short contraction (expert_ff) is walked by
 * half-wavefronts. */
int rein_moe_down(int fmt, const void *slab, const int32_t *ids, const void *xq, float *y,
                  unsigned in_dim, unsigned out_dim, unsigned bytes_per_expert,
                  unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used, unsigned n_tok,
                  rein_stream_t s);
/* The one-token expert FFN in two launches instead of the four of qwen35.rs:3071-3167 (no
 * single counterpart in the reference; each is byte / bit identical to the launches it
 * replaces).  rein_moe_gate_up_swiglu_q8: moe_gate_up_swiglu_q4k_repacked_f32 followed by
 * quantize_q8_f32 -- xq_out[tok][slot] receives out_dim/32 BlockQ8 blocks of
 * silu(gate . x) * (up . x); out_dim a multiple of 32; formats Q4_K, Q5_K, Q6_K, Q8_0, Q5_1 (for
 * the formats other than Q4_K, which the reference runs as two moe_matvec_* launches, the bytes of
 * those two followed by swiglu_q8_f32).
 * rein_moe_down_combine: moe_matvec_*_f32 (or its *_down form) followed by moe_combine_f32 --
 * out[tok][i] = sum_j weights[tok][j] * down_exps_s[ids[tok][j]] * (W[ids[tok][j]] . xq[tok][j])[i]
 * in slot order.  Formats Q4_K, Q5_K, Q6_K, Q8_0, Q5_1. */
int rein_moe_gate_up_swiglu_q8(int fmt, const void *gate_slab, const void *up_slab, const int32_t *ids,
                               const void *xq, void *xq_out, unsigned in_dim, unsigned out_dim,
                               unsigned bytes_per_expert, unsigned xq_tok_stride, unsigned xq_slot_stride,
                               unsigned n_used, unsigned n_tok, rein_stream_t s);
int rein_moe_down_combine(int fmt, const void *slab, const int32_t *ids, const float *weights,
                          const float *down_exps_s, const void *xq, float *out, unsigned in_dim,
                          unsigned out_dim, unsigned bytes_per_expert, unsigned xq_tok_stride,
                          unsigned xq_slot_stride, unsigned n_used, unsigned n_tok, rein_stream_t s);
/* launch_moe_gate_up_swiglu (qwen35.rs:3141-3167; kernels/moe_gate_up_swiglu_q4k_repacked.cpp):
 * y = silu(Wgate . xq) * (Wup . xq) in one pass over both slabs.  fmt must be Q4_K. */
int rein_moe_gate_up_swiglu(int fmt, const void *gate_slab, const void *up_slab, const int32_t *ids,
                            const void *xq, float *y, unsigned in_dim, unsigned out_dim,
                            unsigned bytes_per_expert, unsigned xq_tok_stride,
                            unsigned xq_slot_stride, unsigned n_used, unsigned n_tok, rein_stream_t s);
/* swiglu_mul_f32 (kernels/swiglu.cpp:10-21) */
int rein_swiglu_mul(const float *gate, const float *up, float *out, unsigned n, rein_stream_t s);
/* moe_combine_f32 (kernels/moe_combine.cpp:15-38) */
int rein_moe_combine(const float *experts, const int32_t *ids, const float *weights,
                     const float *down_exps_s, float *out, unsigned n_tok, unsigned hidden,
                     unsigned n_used, rein_stream_t s);
/* tokens per grouped-GEMM tile the launcher assumes for `tile_off` (the
 * reference's MOE_GEMM_BN, qwen35.rs:127) */
unsigned rein_moe_gemm_bn(void);

/* Workspace sizes for rein_moe_ffn, in bytes, for n_tok tokens. */
typedef struct {
    unsigned n_tok, hidden, n_expert, n_used, expert_ff;
    int gate_up_fmt;    /* gate_exps / up_exps format (reference: Q4_K) */
    int down_fmt;       /* down_exps format (reference: Q5_K or Q6_K)  */
} rein_moe_shape;
size_t rein_moe_workspace_bytes(const rein_moe_shape *shape);
/* The routed-expert part of step_moe_ffn_batched (qwen35.rs:2788-2870), given
 * router logits: top-k -> quantize -> sort -> gather -> grouped gate / up GEMM ->
 * SwiGLU -> quantize -> grouped down GEMM -> scatter -> weighted combine.
 * gate_exps / up_exps: n_expert slabs [hidden -> expert_ff]; down_exps:
 * [expert_ff -> hidden]; down_exps_s [n_expert] fp32 (the reference passes
 * ones).  `workspace` holds rein_moe_workspace_bytes; out [n_tok][hidden].
 * No host synchronisation, no allocation.  With at most 1.6 routing entries per expert on average
 * (5 n_tok n_used <= 8 n_expert) the same result comes from the decode
 * kernels instead (top-k -> quantize -> rein_moe_gate_up_swiglu_q8 -> rein_moe_down_combine, the
 * launches of qwen35.rs:3071-3167 fused in pairs): no sort, one expert read per entry; for one
 * and two tokens the gate / up launch also routes and quantizes, so the FFN is two launches.
 * The two forms add a token's eight expert rows, and the terms inside each row, in different
 * orders (slot order in the decode form, expert-sorted tiles in the pipeline): the fp32 bits
 * of a token's output row therefore depend on how many tokens share the call (25 against 26
 * at 128 experts top-8), within the path's 1e-3 / 1e-4 tolerance of either order.  The option
 * REIN_MOE_CHAIN = 0 keeps every call on the pipeline. */
int rein_moe_ffn(const rein_moe_shape *shape, const float *x, const float *logits,
                 const void *gate_exps, const void *up_exps, const void *down_exps,
                 const float *down_exps_s, void *workspace, float *out, rein_stream_t s);

#ifdef __cplusplus
}
#endif
#endif /* REIN_H */
