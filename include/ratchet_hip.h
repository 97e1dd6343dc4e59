/*
 * ratchet_hip.h — C ABI of the MI355X (gfx950) backend for ratchet-core's
 * Matmul operator.
 *
 * The library behind this header (libratchet_hip.so) is what a HIP backend of
 * the reference binds for `LazyOp::Matmul`: the Rust side keeps building the
 * lazy graph, and where the WebGPU backend compiles a WGSL kernel and records
 * a dispatch it calls these entry points instead.  Every entry point cites
 * the reference interface it stands in for (paths relative to the reference
 * checkout).
 *
 * Conventions
 *  - plain C types only; every function returns rt_status and never throws or
 *    aborts across the boundary (the reference panics in guards; here the
 *    same conditions are error codes the Rust wrapper turns into panics or
 *    OperationError as it sees fit);
 *  - device buffers are raw device pointers owned by the caller; an enqueue
 *    borrows them until the stream has been synchronised and never frees,
 *    reallocates or allocates;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *  - a quantized tensor is ONE buffer in the reference's segment layout
 *    (crates/ratchet-core/src/dtype/blocks.rs:61-74): int8 values, padded to
 *    256 bytes, then the per-32 scales, padded to 256 bytes.  A Q4_K tensor is
 *    the raw GGUF 144-byte super-blocks (crates/ratchet-loader/src/k_quants.rs:94-103),
 *    row-major over [rows, K/256].
 */
#ifndef RATCHET_HIP_H
#define RATCHET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RT_MAX_RANK 8

#if defined(RT_BUILDING_LIB)
#define RT_API __attribute__((visibility("default")))
#else
#define RT_API
#endif

/* Replaces: anyhow errors of Matmul::compute_c_shape (ops/matmul.rs:312-342),
 * the panics of Matmul::new (ops/matmul.rs:258-272), OpGuards::check_dtypes
 * (ops/matmul.rs:453-478), GEMMSpec::new (ops/matmul.rs:67-69,90-94),
 * OperationError (op.rs:130-144) and DeviceError (gpu/device.rs:7-23). */
typedef enum rt_status {
    RT_OK = 0,
    RT_ERR_INVALID_ARG = 1,    /* null pointer, rank out of range, unknown enum value          */
    RT_ERR_INVALID_SHAPE = 2,  /* broadcast failure, ka != kb, bias not a vector / wrong length, */
                               /* rank < 2 at execution, operand stacks neither equal nor 1      */
    RT_ERR_DTYPE_MISMATCH = 3, /* (lhs, rhs) pair not allowed, or bias dtype != activation dtype */
    RT_ERR_UNSUPPORTED = 4,    /* transposed quantized operand, K not a multiple of the block;   */
                               /* at enqueue: a shape no kernel takes (more than 65535 stacks or */
                               /* 65535 x 64 rows on the generic kernel's path, or a quantized   */
                               /* operand that is not 16-byte aligned)                           */
    RT_ERR_NO_DEVICE = 5,      /* no HIP device / ordinal out of range                           */
    RT_ERR_HIP = 6,            /* a HIP runtime call failed; see rt_last_hip_error               */
    RT_ERR_OOM = 7             /* hipMalloc failed                                               */
} rt_status;

/* Replaces: enum DType (crates/ratchet-core/src/dtype/mod.rs:10-20), the
 * subset the Matmul guards admit, plus Q4_K (GgmlDType::Q4K,
 * crates/ratchet-loader/src/lib.rs:40) which the reference can name but not
 * load. */
typedef enum rt_dtype {
    RT_F32 = 0,
    RT_F16 = 1,
    RT_Q8_0F = 2, /* int8 blocks of 32 with f32 scales */
    RT_Q8_0H = 3, /* int8 blocks of 32 with f16 scales */
    RT_Q4_K = 4   /* GGUF Q4_K super-blocks of 256     */
} rt_dtype;

/* Replaces: struct Matmul {lhs, rhs, bias, trans_lhs, trans_rhs, trans_out}
 * (ops/matmul.rs:247-255) as seen through the tensors' StorageViews: only
 * dtypes and shapes, no data. */
typedef struct rt_matmul_desc {
    int32_t lhs_dt;                  /* rt_dtype */
    int32_t rhs_dt;                  /* rt_dtype */
    int32_t lhs_rank;
    int32_t rhs_rank;
    int64_t lhs_shape[RT_MAX_RANK];
    int64_t rhs_shape[RT_MAX_RANK];
    int32_t trans_lhs;
    int32_t trans_rhs;
    int32_t trans_out;
    int32_t has_bias;
    int32_t bias_dt;                 /* rt_dtype, read only when has_bias */
    int32_t bias_rank;
    int64_t bias_shape[RT_MAX_RANK];
} rt_matmul_desc;

/* Activations: operators of their own (rt_unary_enqueue) and fusable behind a product
 * (rt_matmul_enqueue_fused).  Replaces: UnaryOp::{Gelu, Silu} (ops/unary.rs:21-37,97-171):
 * gelu = x * (0.5 + 0.5 * safe_tanh(x * (0.035677407 x^2 + 0.7978846))), silu = x * sigmoid(x). */
typedef enum rt_activation {
    RT_ACT_NONE = 0,
    RT_ACT_GELU = 1,
    RT_ACT_SILU = 2
} rt_activation;

/* Replaces: enum GEMVHeuristic (ops/matmul.rs:13-29). */
typedef enum rt_gemv_heuristic {
    RT_HEUR_VERY_TALL = 0,
    RT_HEUR_TALL = 1,
    RT_HEUR_SQUARE = 2,
    RT_HEUR_FAT = 3
} rt_gemv_heuristic;

/* Which gfx950 kernel family an enqueue of this descriptor launches; plays
 * the role of the kernel stem in KernelKey (ops/matmul.rs:485-524). */
typedef enum rt_kernel_kind {
    RT_KERNEL_NONE = 0,      /* empty output, nothing launched                              */
    RT_KERNEL_GEMV_Q8 = 1,   /* streaming Q8_0 weight rows x up to 8 activation vectors     */
    RT_KERNEL_GEMV_Q4K = 2,  /* streaming Q4_K weight rows x up to 16 activation vectors    */
    RT_KERNEL_GEMV_FLOAT = 3,/* streaming f16/f32 weight rows x up to 8 activation vectors  */
    RT_KERNEL_GEMM_F16 = 4,  /* LDS-tiled MFMA GEMM, f16 operands (Q8_0H / Q4_K dequantized) */
    RT_KERNEL_GEMM_F32 = 5   /* LDS-tiled MFMA GEMM, f32 operands (Q8_0F dequantized)        */
} rt_kernel_kind;

/* Replaces: struct GEMMSpec and its accessors (ops/matmul.rs:32-245). */
typedef struct rt_gemm_spec {
    int64_t lhs_shape[2]; /* after folding the leading dims into the stack */
    int64_t rhs_shape[2];
    int64_t out_shape[2];
    int64_t lhs_stack;
    int64_t rhs_stack;
    int64_t out_stack;
    int64_t dim_lhs_outer; /* out_shape[0] */
    int64_t dim_rhs_outer; /* out_shape[1] */
    int64_t dim_inner;
    int32_t is_gemv;       /* the reference's own rule: rhs is a vector and !trans_lhs */
    int32_t heuristic;     /* rt_gemv_heuristic */
    int32_t kernel;        /* rt_kernel_kind this library launches */
    int32_t reserved;
} rt_gemm_spec;

typedef struct rt_ctx rt_ctx;

/* ---- host-only: shape, dtype and spec rules (no HIP call is made) -------- */

/* Replaces: Matmul::compute_view = compute_c_shape + "dtype = rhs dtype" +
 * contiguous strides (ops/matmul.rs:284-361,427-440).  `out_shape` must hold
 * RT_MAX_RANK entries.  Operands of rank 1 get the reference's implicit
 * dimension. */
RT_API rt_status rt_matmul_infer(const rt_matmul_desc *desc, int64_t *out_shape, int32_t *out_rank,
                          int32_t *out_dt);

/* Replaces: the panics of Matmul::new (bias must be a vector, no transposed
 * quantized lhs; ops/matmul.rs:258-272), OpGuards::check_shapes and
 * check_dtypes (ops/matmul.rs:442-478), and the execution-time asserts of
 * GEMMSpec::new (both operands rank >= 2, stacks equal or 1;
 * ops/matmul.rs:67-69,90-94).  Returns the first violated rule as a status. */
RT_API rt_status rt_matmul_validate(const rt_matmul_desc *desc);

/* Replaces: Matmul::compute_spec / GEMMSpec::new (ops/matmul.rs:48-134,
 * 363-373) and the kernel choice of MetaOperation::build_kernel
 * (ops/matmul.rs:632-646). */
RT_API rt_status rt_matmul_spec(const rt_matmul_desc *desc, rt_gemm_spec *spec);

/* Replaces: DType::segments / size arithmetic (dtype/mod.rs:85-95,
 * dtype/blocks.rs:61-74): bytes a tensor of `numel` elements occupies. */
RT_API rt_status rt_tensor_nbytes(int32_t dtype, uint64_t numel, uint64_t *nbytes);

/* Replaces: the second BufferSegment's offset of Q8_0<T>::segments
 * (dtype/blocks.rs:61-74): byte offset of the scale stream. */
RT_API uint64_t rt_q8_0_scale_offset(uint64_t numel);

RT_API const char *rt_status_string(rt_status s);
RT_API const char *rt_kernel_string(int32_t kernel_kind);

/* ---- device context and buffers ------------------------------------------ */

/* Replaces: Device::request_device(DeviceRequest::GPU) / WgpuDevice::new
 * (crates/ratchet-core/src/device.rs:37-56, gpu/device.rs:62-140).
 * Checked mode: when the environment variable RATCHET_CHECKED (the reference's switch for its checked
 * shader builds, gpu/pools/kernel_module_pool.rs:62-67) is set to anything but "0" at this call, every
 * matmul enqueue on the context first looks up the device allocation behind each pointer and fails with
 * RT_ERR_INVALID_ARG when it holds fewer bytes than the descriptor implies.  A query per pointer and
 * call: for debugging, not for serving. */
RT_API rt_status rt_ctx_create(int32_t device_ordinal, rt_ctx **ctx);
RT_API rt_status rt_ctx_destroy(rt_ctx *ctx);

/* Text of the last error this context recorded ("" if none), and the raw
 * hipError_t of the last failed HIP call (0 if none). */
RT_API const char *rt_last_error(const rt_ctx *ctx);
RT_API int32_t rt_last_hip_error(const rt_ctx *ctx);

/* Replaces: GPUBuffer creation and CPUBuffer::to_device / GPUBuffer::to_cpu
 * (crates/ratchet-core/src/storage/gpu_buffer.rs:51-61,155-178).  Upload and
 * download are asynchronous on `stream` when the host memory is pinned. */
RT_API rt_status rt_buf_alloc(rt_ctx *ctx, uint64_t nbytes, void **dptr);
RT_API rt_status rt_buf_free(rt_ctx *ctx, void *dptr);
RT_API rt_status rt_buf_upload(rt_ctx *ctx, void *dst_dev, const void *src_host, uint64_t nbytes, void *stream);
RT_API rt_status rt_buf_download(rt_ctx *ctx, void *dst_host, const void *src_dev, uint64_t nbytes, void *stream);

/* Replaces: device.poll(WaitForSubmissionIndex) at the end of
 * Tensor::resolve (crates/ratchet-core/src/tensor.rs:785). */
RT_API rt_status rt_sync(rt_ctx *ctx, void *stream);

/* ---- the operator --------------------------------------------------------- */

/* Replaces: MetaOperation::compile for LazyOp::Matmul followed by its
 * dispatch (op.rs:304-362, ops/matmul.rs:480-647, executable.rs:25-54), i.e.
 * the arm `LazyOp::Matmul(m) => m.compile(...)` of Tensor::compile
 * (tensor.rs:722) when the device is HIP.  Validates the descriptor (as
 * rt_matmul_validate), picks a kernel (as rt_matmul_spec) and launches it on
 * `stream`.  `bias` may be NULL iff !has_bias.  `out` must hold the shape
 * rt_matmul_infer reports, contiguous, in the activation dtype. */
RT_API rt_status rt_matmul_enqueue(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                            const void *bias, void *out, void *stream);

/* ---- block formats on the device ------------------------------------------ */

/* Replaces: Quantizer::sint8_quantize (crates/ratchet-core/src/quant.rs:26-79):
 * f32 -> Q8_0F segments (scale = max|x|/127 per 32, q = round-half-away(x/scale)).
 * `dst` holds rt_tensor_nbytes(RT_Q8_0F, numel) bytes; padding is zeroed. */
RT_API rt_status rt_quantize_q8_0(rt_ctx *ctx, const void *src_f32, uint64_t numel, void *dst, void *stream);

/* Replaces: Quantizer::sint8_dequantize (quant.rs:81-124) for Q8_0F, the same
 * rule with f16 scales for Q8_0H, and ggml's dequantize_row_q4_K for Q4_K
 * (the reference holds only the block struct, k_quants.rs:94-103).
 * `dst_f32` receives numel floats. */
RT_API rt_status rt_dequantize(rt_ctx *ctx, int32_t dtype, const void *src, uint64_t numel, void *dst_f32,
                        void *stream);

/* Replaces: GGUFInterop::transcode for Q8_0F / Q8_0H
 * (crates/ratchet-loader/src/gguf/dtype.rs:40-110): `blocks` are n_blocks GGUF
 * blocks of 34 bytes {f16 d; int8 qs[32]} in device memory; `dst` receives the
 * segment layout for dst_dtype (RT_Q8_0F widens the scales to f32). */
RT_API rt_status rt_transcode_gguf_q8_0(rt_ctx *ctx, const void *blocks, uint64_t n_blocks, int32_t dst_dtype,
                                 void *dst, void *stream);

/* ------------------------------------------------------------------------
 * GGUF container (the format the weights arrive in).
 * Replaces: Header::read, TensorInfo::{read, size_in_bytes, byte_range} and
 * ratchet_from_gguf (crates/ratchet-loader/src/gguf/gguf.rs:63-142,408-496),
 * GgmlDType (crates/ratchet-loader/src/lib.rs:35-140).
 * The file image stays with the caller (a mapping or a buffer); the parsed
 * header only indexes into it.  Host-side parsing, no device needed.
 * ------------------------------------------------------------------------ */
typedef struct rt_gguf rt_gguf;

/* ggml tensor type ids (lib.rs:62-81) */
typedef enum rt_ggml_dtype {
    RT_GGML_F32 = 0, RT_GGML_F16 = 1, RT_GGML_Q4_0 = 2, RT_GGML_Q4_1 = 3, RT_GGML_Q5_0 = 6, RT_GGML_Q5_1 = 7,
    RT_GGML_Q8_0 = 8, RT_GGML_Q8_1 = 9, RT_GGML_Q2K = 10, RT_GGML_Q3K = 11, RT_GGML_Q4K = 12, RT_GGML_Q5K = 13,
    RT_GGML_Q6K = 14, RT_GGML_Q8K = 15
} rt_ggml_dtype;

/* metadata value types (gguf.rs:183-214, ids gguf.rs:384-403) */
typedef enum rt_gguf_type {
    RT_GGUF_U8 = 0, RT_GGUF_I8 = 1, RT_GGUF_U16 = 2, RT_GGUF_I16 = 3, RT_GGUF_U32 = 4, RT_GGUF_I32 = 5,
    RT_GGUF_F32 = 6, RT_GGUF_BOOL = 7, RT_GGUF_STRING = 8, RT_GGUF_ARRAY = 9, RT_GGUF_U64 = 10, RT_GGUF_I64 = 11,
    RT_GGUF_F64 = 12
} rt_gguf_type;

typedef struct rt_gguf_tensor_info {
    const char *name;            /* NUL-terminated, owned by the rt_gguf */
    int32_t ggml_dtype;          /* rt_ggml_dtype */
    int32_t rank;
    int64_t shape[RT_MAX_RANK];  /* outermost first: the file's dimensions reversed (gguf.rs:450) */
    uint64_t offset;             /* relative to rt_gguf_tensor_data_offset */
    uint64_t size_in_bytes;      /* numel / block_numel * type_size (gguf.rs:93-98) */
} rt_gguf_tensor_info;

typedef struct rt_gguf_value {
    int32_t type;                /* rt_gguf_type */
    int32_t elem_type;           /* arrays: element type */
    uint64_t count;              /* arrays: elements; strings: bytes; scalars: 1 */
    uint64_t u64;                /* unsigned integers and bool */
    int64_t i64;                 /* signed integers */
    double f64;                  /* F32 and F64 */
    const char *str;             /* strings: NUL-terminated copy (trailing NULs of the file stripped, gguf.rs:176-178) */
} rt_gguf_value;

/* Header::read (gguf.rs:408-479): magic "GGUF" (either byte order of the constant), versions 1-3
 * (v1 has 32-bit counts and lengths), metadata, tensor infos, and the tensor data offset rounded up to
 * `general.alignment` (default 32).  Errors: RT_ERR_INVALID_ARG (truncated or malformed image),
 * RT_ERR_UNSUPPORTED (unknown magic / version / value type / tensor type). */
RT_API rt_status rt_gguf_parse(const void *image, uint64_t size, rt_gguf **out);
RT_API void rt_gguf_free(rt_gguf *g);
RT_API const char *rt_gguf_error(const rt_gguf *g); /* of the last failing call on g; "" if none */
RT_API uint32_t rt_gguf_version(const rt_gguf *g);
RT_API uint64_t rt_gguf_tensor_count(const rt_gguf *g);
RT_API uint64_t rt_gguf_metadata_count(const rt_gguf *g);
RT_API uint64_t rt_gguf_tensor_data_offset(const rt_gguf *g);
/* Tensors and keys are indexed in file order; lookups by name follow HashMap semantics: a
 * repeated name resolves to its last occurrence (gguf.rs:433,453). */
RT_API rt_status rt_gguf_tensor_info_at(const rt_gguf *g, uint64_t index, rt_gguf_tensor_info *info);
RT_API rt_status rt_gguf_find_tensor(const rt_gguf *g, const char *name, uint64_t *index);
RT_API rt_status rt_gguf_metadata_key_at(const rt_gguf *g, uint64_t index, const char **key);
RT_API rt_status rt_gguf_metadata_get(const rt_gguf *g, const char *key, rt_gguf_value *value); /* Metadata::get */
RT_API rt_status rt_gguf_metadata_array_get(const rt_gguf *g, const char *key, uint64_t i, rt_gguf_value *value);
/* GgmlDType::{type_size, block_numel} (lib.rs:103-140); 0 for an unknown id */
RT_API uint64_t rt_ggml_type_size(int32_t ggml_dtype);
RT_API uint64_t rt_ggml_block_numel(int32_t ggml_dtype);

/* TensorInfo::read + ratchet_from_gguf (gguf.rs:63-84,118-142): copies tensor `index` of the image to
 * the device and brings it into this library's layout for `dst_dtype`:
 *   F32 -> RT_F32, F16 -> RT_F16 (plain copies); Q8_0 -> RT_Q8_0H or RT_Q8_0F (segment layout, through
 *   the device transcoder; `staging` must hold size_in_bytes); Q4_K -> RT_Q4_K (raw super-blocks; this
 *   library's extension).  Any other pairing is RT_ERR_UNSUPPORTED (the reference bails on it).
 * `dst` must hold rt_tensor_nbytes(dst_dtype, numel).  Copies are asynchronous on `stream`; the image
 * must stay valid until the stream is synchronized. */
RT_API rt_status rt_gguf_load_tensor(rt_ctx *ctx, const rt_gguf *g, const void *image, uint64_t size, uint64_t index,
                                     int32_t dst_dtype, void *staging, void *dst, void *stream);

/* ------------------------------------------------------------------------
 * Operators that wrap the products in the reference's models:
 *   x.gelu() / x.silu() after a Linear (whisper/mlp.rs:18-22, phi3/mlp.rs:31-39, phi2/mlp.rs:13-15),
 *   x.cast(dt) / x.full() / x.half() around the attention matmuls (ops/cast.rs:15-18).
 * ------------------------------------------------------------------------ */

/* rt_matmul_enqueue with the activation applied to (product + bias) in f32 before the single
 * rounding to the output type: out = act(lhs x rhs + bias).  The reference runs the activation
 * as a second operator on the rounded product; fusing removes one write and one read of the
 * output and one rounding.  RT_ACT_NONE is rt_matmul_enqueue. */
RT_API rt_status rt_matmul_enqueue_fused(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                                         const void *bias, void *out, int32_t activation, void *stream);

/* rt_matmul_enqueue_fused with device memory the launch may use to share one product's contraction
 * among workgroups.  A product with few output tiles and a long K (a prefill down-projection,
 * [512 x 10240] . W[2560 x 10240]^T: 64 tiles on 256 compute units) is cut along K; each share's f32
 * sums go to the workspace and a second kernel adds them in a fixed order, then bias, activation and
 * the one rounding, so results do not vary from run to run.  rt_matmul_workspace_bytes gives the size
 * with which that happens (0: the product is not split whatever is passed).  A NULL, misaligned
 * (16 bytes) or smaller workspace is not an error: the launch then runs in one pass, exactly as
 * rt_matmul_enqueue_fused.  The workspace holds nothing between calls; launches on different streams
 * must not share one.  The reference has no counterpart: its workgroups always own whole output
 * tiles (ops/matmul.rs:540-590 sizes the dispatch from the output alone). */
RT_API rt_status rt_matmul_workspace_bytes(rt_ctx *ctx, const rt_matmul_desc *desc, uint64_t *bytes);
RT_API rt_status rt_matmul_enqueue_ws(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                                      const void *bias, void *out, int32_t activation, void *workspace,
                                      uint64_t workspace_bytes, void *stream);

/* rt_matmul_enqueue_ws for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the shares' partial sums go to a static
 * buffer of RT_STATIC_SCRATCH_BYTES that the library holds on each GPU it runs on, from
 * rt_ctx_create until the process ends.  Neither this call nor anything it launches allocates or
 * frees.  Results are those of rt_matmul_enqueue_ws with a workspace of rt_matmul_workspace_bytes,
 * bit for bit (the same kernels run).  A split that would need more than the buffer holds is
 * RT_ERR_UNSUPPORTED (on a device of up to 256 compute units none does); a product that is not split
 * runs as rt_matmul_enqueue_fused and touches no scratch.  All calls on one GPU share the one buffer:
 * calls that can overlap there (different streams, different contexts or threads) race; order them.
 * No counterpart in the reference, whose operators never own scratch memory. */
#define RT_STATIC_SCRATCH_BYTES (20u << 20)
RT_API rt_status rt_matmul_enqueue_static(rt_ctx *ctx, const rt_matmul_desc *desc, const void *lhs, const void *rhs,
                                          const void *bias, void *out, int32_t activation, void *stream);

/* The compile-once half of the operator.  In the reference an operator is compiled once per graph
 * (Matmul::kernel_key names the pipeline, ops/matmul.rs:485-524; Operation::compile builds the
 * CompiledOp with its workgroup count and bindings, op.rs:304-362) and Executable::dispatch_operations
 * (executable.rs:25-54) only records the dispatch on every step.  A plan is that for this library:
 * rt_matmul_plan_create runs the guards, the shape rules and the lowering of `desc` (what every
 * rt_matmul_enqueue* call repeats) once and fixes the fused activation; rt_matmul_plan_enqueue takes only
 * the device pointers (and a workspace as rt_matmul_enqueue_ws does, or NULL, 0), offers the product first
 * to the kernel family that took it last time, and launches.  Results are those of rt_matmul_enqueue_ws with
 * the same arguments, bit for bit (the same kernels run).  A plan belongs to the context it was created
 * with, may be enqueued from several threads, and must be destroyed before that context. */
typedef struct rt_matmul_plan rt_matmul_plan;
RT_API rt_status rt_matmul_plan_create(rt_ctx *ctx, const rt_matmul_desc *desc, int32_t activation, rt_matmul_plan **plan);
RT_API rt_status rt_matmul_plan_enqueue(rt_matmul_plan *plan, const void *lhs, const void *rhs, const void *bias,
                                        void *out, void *workspace, uint64_t workspace_bytes, void *stream);
RT_API rt_status rt_matmul_plan_destroy(rt_matmul_plan *plan);

/* Replaces: Unary (ops/unary.rs:71-260) for Gelu and Silu on F32 / F16 tensors; `dst` may be
 * `src` (the reference runs unary operators in place when it can). */
RT_API rt_status rt_unary_enqueue(rt_ctx *ctx, int32_t activation, int32_t dtype, const void *src, void *dst,
                                  uint64_t numel, void *stream);

/* Replaces: Cast (ops/cast.rs:15-200) between F32 and F16 (round to nearest even when narrowing). */
RT_API rt_status rt_cast_enqueue(rt_ctx *ctx, int32_t src_dtype, int32_t dst_dtype, const void *src, void *dst,
                                 uint64_t numel, void *stream);

/* ------------------------------------------------------------------------
 * Softmax, the step between the two attention matmuls.
 * Replaces: Softmax (crates/ratchet-core/src/ops/softmax.rs:15-260): in place
 * only (:47-49), float tensors (:36-39), rank >= 2 and dim < rank (:28-33).
 * The reference's dispatch addresses rows along the last dimension
 * (calculate_dispatch / write_metadata, :244-281), which is how every caller
 * uses it; another `dim` is RT_ERR_UNSUPPORTED here.
 * ------------------------------------------------------------------------ */
RT_API rt_status rt_softmax_validate(int32_t dtype, int32_t rank, const int64_t *shape, int32_t dim);
/* x[..., :] <- exp(x - max) / sum over the last dimension, in place, on `stream`. */
RT_API rt_status rt_softmax_enqueue(rt_ctx *ctx, int32_t dtype, void *x, int32_t rank, const int64_t *shape,
                                    int32_t dim, void *stream);

/* ------------------------------------------------------------------------
 * Fused attention: out = softmax(scale * q k^T + mask) v, one kernel.
 * Replaces the operator sequence of the reference's attention modules
 *   phi3/attn.rs:142-158, phi2/attn.rs:138-152, whisper/mha.rs:105-124:
 *   q.matmul(k, false, true).mul(scale) [.add(mask)] .softmax(3).cast(dt).matmul(v, false, false)
 * whose [q_len x kv_len] scores go through memory between the operators.
 * Tensors are f16, [batch, heads, len, head_dim] with head_dim contiguous and
 * every other dimension strided (in elements), so that
 *   - k and v may point into a persistent key/value cache of capacity > kv_len
 *     (the reference's Cache operator copies the whole cache into a fresh
 *     contiguous tensor every step, ops/cache.rs:71-96), and
 *   - out may be written as [batch, len, heads, head_dim], the layout the
 *     callers permute to afterwards (phi3/attn.rs:157-158).
 * `mask` is the callers' additive mask, [q_len, kv_len], F32 or F16, or NULL;
 * `causal` applies the same mask without a tensor: key j is visible to query i
 * iff j <= i + (kv_len - q_len).  A row with no visible key is NaN, as in the
 * unfused sequence.  Arithmetic is f32 from the scores to the division by the
 * row sum; the probabilities enter the second product as f16, like the
 * reference's cast.
 * ------------------------------------------------------------------------ */
typedef struct rt_attention_desc {
    int32_t dtype;              /* RT_F16 */
    int32_t batch, heads;
    int32_t q_len, kv_len;
    int32_t head_dim;           /* a multiple of 8, at most 128 */
    int64_t q_strides[3];       /* batch, head, row; in elements */
    int64_t k_strides[3];
    int64_t v_strides[3];
    int64_t o_strides[3];
    float scale;                /* softmax_scale (phi2/attn.rs:74: 1 / sqrt(head_dim)) */
    int32_t causal;             /* 0 / 1 */
    int32_t mask_dtype;         /* RT_F32 or RT_F16; ignored when mask is NULL */
    int64_t mask_row_stride;    /* elements between rows of the mask */
} rt_attention_desc;

/* Host-side checks: RT_ERR_DTYPE_MISMATCH (not F16 / bad mask type), RT_ERR_INVALID_SHAPE
 * (non-positive sizes, head_dim), RT_ERR_UNSUPPORTED (strides that break 16-byte row alignment). */
RT_API rt_status rt_attention_validate(const rt_attention_desc *desc);
/* Bytes of device workspace with which rt_attention_enqueue shares the keys of one query block among
 * several workgroups (0 when the problem fills the device in one pass).  It pays when there are few
 * queries and many keys -- a decode step against a long cache -- where one workgroup per head would
 * leave most compute units idle.  The workspace holds partial (maximum, sum, output) triples in f32
 * between the two kernels of such a launch; its contents before and after are irrelevant.  With it, a
 * launch of one query row against 256 or more keys and no mask tensor runs a streaming kernel of its
 * own (128 keys per workgroup) instead of the tiled one. */
RT_API rt_status rt_attention_workspace_bytes(const rt_attention_desc *desc, uint64_t *bytes);
/* `workspace` may be NULL (or smaller than rt_attention_workspace_bytes): the launch then runs in one
 * pass.  Launches that share a workspace must not overlap. */
RT_API rt_status rt_attention_enqueue(rt_ctx *ctx, const rt_attention_desc *desc, const void *q, const void *k,
                                      const void *v, const void *mask, void *out, void *workspace,
                                      uint64_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Key/value cache write.
 * Replaces: Cache (crates/ratchet-core/src/ops/cache.rs:20-140) as the attention
 * modules use it, `kv.k_cache.cache(key_states, 2, offset)` (phi3/attn.rs:134-137):
 *   cache  [batch, heads, capacity, head_dim], contiguous, persistent
 *   src    [batch, heads, len, head_dim], strided (elements: batch, head, row), so the
 *          new keys may be read where a fused Q/K/V projection left them
 *   rows offset .. offset + len - 1 of the cache <- src
 *   dst    NULL, or the reference's result: a fresh contiguous tensor
 *          [batch, heads, offset + len, head_dim] = cache[.., :offset, :] ++ src.
 * With rt_attention_enqueue reading the cache in place (k_strides, kv_len = offset + len)
 * dst is not needed and a decode step copies len rows instead of offset + len.
 * Guards (cache.rs:112-121): offset <= capacity as the reference asserts, and
 * offset + len <= capacity, which the reference leaves to the caller; F32 / F16.
 * ------------------------------------------------------------------------ */
RT_API rt_status rt_cache_write_enqueue(rt_ctx *ctx, int32_t dtype, void *cache, const void *src, const int64_t *src_strides,
                                        void *dst, int32_t batch, int32_t heads, int32_t capacity, int32_t offset,
                                        int32_t len, int32_t head_dim, void *stream);

/* The two cache writes of an attention module, `kv.k_cache.cache(key_states, 2, offset)` and
 * `kv.v_cache.cache(value_states, 2, offset)` (phi3/attn.rs:134-137, phi2/attn.rs:130-133), as one
 * launch: both caches [batch, heads, capacity, head_dim], both sources with the same `src_strides`
 * (the K and V parts of one fused projection output, or two tensors of one layout).  In-place form
 * only (no dst); guards as rt_cache_write_enqueue.  A decode step's two writes are a few kilobytes
 * each, so their cost is the launch, and this halves it. */
RT_API rt_status rt_cache_write_kv_enqueue(rt_ctx *ctx, int32_t dtype, void *k_cache, const void *k_src, void *v_cache,
                                           const void *v_src, const int64_t *src_strides, int32_t batch, int32_t heads,
                                           int32_t capacity, int32_t offset, int32_t len, int32_t head_dim, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RATCHET_HIP_H */
