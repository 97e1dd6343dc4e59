//! Raw FFI declarations of `libratchet_hip.so`, one to one with `include/ratchet_hip.h`.
//!
//! Not compiled in this repository's build image (no rustc there); `tests/test_abi.py` checks that
//! every symbol the header exports is declared here.  Each entry point's contract, and the
//! reference interface it stands in for, is documented in the header.
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_void};

pub const RT_MAX_RANK: usize = 8;
/// Bytes of the static scratch buffer behind `rt_matmul_enqueue_static`.
pub const RT_STATIC_SCRATCH_BYTES: u64 = 20 << 20;

pub type rt_status = i32;
pub const RT_OK: rt_status = 0;
pub const RT_ERR_INVALID_ARG: rt_status = 1;
pub const RT_ERR_INVALID_SHAPE: rt_status = 2;
pub const RT_ERR_DTYPE_MISMATCH: rt_status = 3;
pub const RT_ERR_UNSUPPORTED: rt_status = 4;
pub const RT_ERR_NO_DEVICE: rt_status = 5;
pub const RT_ERR_HIP: rt_status = 6;
pub const RT_ERR_OOM: rt_status = 7;

pub type rt_dtype = i32;
pub const RT_F32: rt_dtype = 0;
pub const RT_F16: rt_dtype = 1;
pub const RT_Q8_0F: rt_dtype = 2;
pub const RT_Q8_0H: rt_dtype = 3;
pub const RT_Q4_K: rt_dtype = 4;

pub type rt_activation = i32;
pub const RT_ACT_NONE: rt_activation = 0;
pub const RT_ACT_GELU: rt_activation = 1;
pub const RT_ACT_SILU: rt_activation = 2;

pub type rt_kernel_kind = i32;
pub const RT_KERNEL_NONE: rt_kernel_kind = 0;
pub const RT_KERNEL_GEMV_Q8: rt_kernel_kind = 1;
pub const RT_KERNEL_GEMV_Q4K: rt_kernel_kind = 2;
pub const RT_KERNEL_GEMV_FLOAT: rt_kernel_kind = 3;
pub const RT_KERNEL_GEMM_F16: rt_kernel_kind = 4;
pub const RT_KERNEL_GEMM_F32: rt_kernel_kind = 5;

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct rt_matmul_desc {
    pub lhs_dt: i32,
    pub rhs_dt: i32,
    pub lhs_rank: i32,
    pub rhs_rank: i32,
    pub lhs_shape: [i64; RT_MAX_RANK],
    pub rhs_shape: [i64; RT_MAX_RANK],
    pub trans_lhs: i32,
    pub trans_rhs: i32,
    pub trans_out: i32,
    pub has_bias: i32,
    pub bias_dt: i32,
    pub bias_rank: i32,
    pub bias_shape: [i64; RT_MAX_RANK],
}

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct rt_gemm_spec {
    pub lhs_shape: [i64; 2],
    pub rhs_shape: [i64; 2],
    pub out_shape: [i64; 2],
    pub lhs_stack: i64,
    pub rhs_stack: i64,
    pub out_stack: i64,
    pub dim_lhs_outer: i64,
    pub dim_rhs_outer: i64,
    pub dim_inner: i64,
    pub is_gemv: i32,
    pub heuristic: i32,
    pub kernel: i32,
    pub reserved: i32,
}

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct rt_attention_desc {
    pub dtype: i32,
    pub batch: i32,
    pub heads: i32,
    pub q_len: i32,
    pub kv_len: i32,
    pub head_dim: i32,
    pub q_strides: [i64; 3], // batch, head, row; in elements
    pub k_strides: [i64; 3],
    pub v_strides: [i64; 3],
    pub o_strides: [i64; 3],
    pub scale: f32,
    pub causal: i32,
    pub mask_dtype: i32,
    pub mask_row_stride: i64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct rt_gguf_tensor_info {
    pub name: *const c_char, // NUL-terminated, owned by the rt_gguf
    pub ggml_dtype: i32,
    pub rank: i32,
    pub shape: [i64; RT_MAX_RANK], // outermost first
    pub offset: u64,               // relative to rt_gguf_tensor_data_offset
    pub size_in_bytes: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct rt_gguf_value {
    pub type_: i32,      // rt_gguf_type
    pub elem_type: i32,  // arrays: element type
    pub count: u64,      // arrays: elements; strings: bytes; scalars: 1
    pub u64_: u64,       // unsigned integers and bool
    pub i64_: i64,       // signed integers
    pub f64_: f64,       // F32 and F64
    pub str_: *const c_char, // strings: NUL-terminated copy owned by the rt_gguf
}

#[repr(C)]
pub struct rt_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rt_gguf {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rt_matmul_plan {
    _private: [u8; 0],
}

#[link(name = "ratchet_hip")]
extern "C" {
    // host-only: shape, dtype and spec rules
    pub fn rt_matmul_infer(d: *const rt_matmul_desc, out_shape: *mut i64, out_rank: *mut i32, out_dt: *mut i32) -> rt_status;
    pub fn rt_matmul_validate(d: *const rt_matmul_desc) -> rt_status;
    pub fn rt_matmul_spec(d: *const rt_matmul_desc, spec: *mut rt_gemm_spec) -> rt_status;
    pub fn rt_tensor_nbytes(dtype: i32, numel: u64, nbytes: *mut u64) -> rt_status;
    pub fn rt_q8_0_scale_offset(numel: u64) -> u64;
    pub fn rt_status_string(s: rt_status) -> *const c_char;
    pub fn rt_kernel_string(kind: i32) -> *const c_char;
    // device context and buffers
    pub fn rt_ctx_create(ordinal: i32, ctx: *mut *mut rt_ctx) -> rt_status;
    pub fn rt_ctx_destroy(ctx: *mut rt_ctx) -> rt_status;
    pub fn rt_last_error(ctx: *const rt_ctx) -> *const c_char;
    pub fn rt_last_hip_error(ctx: *const rt_ctx) -> i32;
    pub fn rt_buf_alloc(ctx: *mut rt_ctx, nbytes: u64, dptr: *mut *mut c_void) -> rt_status;
    pub fn rt_buf_free(ctx: *mut rt_ctx, dptr: *mut c_void) -> rt_status;
    pub fn rt_buf_upload(ctx: *mut rt_ctx, dst: *mut c_void, src: *const c_void, nbytes: u64, stream: *mut c_void) -> rt_status;
    pub fn rt_buf_download(ctx: *mut rt_ctx, dst: *mut c_void, src: *const c_void, nbytes: u64, stream: *mut c_void) -> rt_status;
    pub fn rt_sync(ctx: *mut rt_ctx, stream: *mut c_void) -> rt_status;
    // the operator
    pub fn rt_matmul_enqueue(ctx: *mut rt_ctx, d: *const rt_matmul_desc, lhs: *const c_void, rhs: *const c_void,
                             bias: *const c_void, out: *mut c_void, stream: *mut c_void) -> rt_status;
    pub fn rt_matmul_enqueue_fused(ctx: *mut rt_ctx, d: *const rt_matmul_desc, lhs: *const c_void, rhs: *const c_void,
                                   bias: *const c_void, out: *mut c_void, activation: i32, stream: *mut c_void) -> rt_status;
    pub fn rt_matmul_workspace_bytes(ctx: *mut rt_ctx, d: *const rt_matmul_desc, bytes: *mut u64) -> rt_status;
    pub fn rt_matmul_enqueue_ws(ctx: *mut rt_ctx, d: *const rt_matmul_desc, lhs: *const c_void, rhs: *const c_void,
                                bias: *const c_void, out: *mut c_void, activation: i32, workspace: *mut c_void,
                                workspace_bytes: u64, stream: *mut c_void) -> rt_status;
    pub fn rt_matmul_enqueue_static(ctx: *mut rt_ctx, d: *const rt_matmul_desc, lhs: *const c_void, rhs: *const c_void,
                                    bias: *const c_void, out: *mut c_void, activation: i32, stream: *mut c_void) -> rt_status;
    // the operator, compiled once: guards, shape rules and lowering at creation; an enqueue takes pointers only
    pub fn rt_matmul_plan_create(ctx: *mut rt_ctx, d: *const rt_matmul_desc, activation: i32, plan: *mut *mut rt_matmul_plan) -> rt_status;
    pub fn rt_matmul_plan_enqueue(plan: *mut rt_matmul_plan, lhs: *const c_void, rhs: *const c_void, bias: *const c_void,
                                  out: *mut c_void, workspace: *mut c_void, workspace_bytes: u64, stream: *mut c_void) -> rt_status;
    pub fn rt_matmul_plan_destroy(plan: *mut rt_matmul_plan) -> rt_status;
    // block formats on the device
    pub fn rt_quantize_q8_0(ctx: *mut rt_ctx, src_f32: *const c_void, numel: u64, dst: *mut c_void, stream: *mut c_void) -> rt_status;
    pub fn rt_dequantize(ctx: *mut rt_ctx, dtype: i32, src: *const c_void, numel: u64, dst_f32: *mut c_void, stream: *mut c_void) -> rt_status;
    pub fn rt_transcode_gguf_q8_0(ctx: *mut rt_ctx, blocks: *const c_void, n_blocks: u64, dst_dtype: i32, dst: *mut c_void,
                                  stream: *mut c_void) -> rt_status;
    // operators around the products
    pub fn rt_unary_enqueue(ctx: *mut rt_ctx, activation: i32, dtype: i32, src: *const c_void, dst: *mut c_void, numel: u64,
                            stream: *mut c_void) -> rt_status;
    pub fn rt_cast_enqueue(ctx: *mut rt_ctx, src_dtype: i32, dst_dtype: i32, src: *const c_void, dst: *mut c_void, numel: u64,
                           stream: *mut c_void) -> rt_status;
    pub fn rt_softmax_validate(dtype: i32, rank: i32, shape: *const i64, dim: i32) -> rt_status;
    pub fn rt_softmax_enqueue(ctx: *mut rt_ctx, dtype: i32, x: *mut c_void, rank: i32, shape: *const i64, dim: i32,
                              stream: *mut c_void) -> rt_status;
    pub fn rt_attention_validate(d: *const rt_attention_desc) -> rt_status;
    pub fn rt_attention_workspace_bytes(d: *const rt_attention_desc, bytes: *mut u64) -> rt_status;
    pub fn rt_attention_enqueue(ctx: *mut rt_ctx, d: *const rt_attention_desc, q: *const c_void, k: *const c_void,
                                v: *const c_void, mask: *const c_void, out: *mut c_void, workspace: *mut c_void,
                                workspace_bytes: u64, stream: *mut c_void) -> rt_status;
    pub fn rt_cache_write_enqueue(ctx: *mut rt_ctx, dtype: i32, cache: *mut c_void, src: *const c_void, src_strides: *const i64,
                                  dst: *mut c_void, batch: i32, heads: i32, capacity: i32, offset: i32, len: i32,
                                  head_dim: i32, stream: *mut c_void) -> rt_status;
    pub fn rt_cache_write_kv_enqueue(ctx: *mut rt_ctx, dtype: i32, k_cache: *mut c_void, k_src: *const c_void,
                                     v_cache: *mut c_void, v_src: *const c_void, src_strides: *const i64, batch: i32,
                                     heads: i32, capacity: i32, offset: i32, len: i32, head_dim: i32,
                                     stream: *mut c_void) -> rt_status;
    // GGUF container (host-side parse; load = upload + layout conversion on `stream`)
    pub fn rt_gguf_parse(image: *const c_void, size: u64, out: *mut *mut rt_gguf) -> rt_status;
    pub fn rt_gguf_free(g: *mut rt_gguf);
    pub fn rt_gguf_error(g: *const rt_gguf) -> *const c_char;
    pub fn rt_gguf_version(g: *const rt_gguf) -> u32;
    pub fn rt_gguf_tensor_count(g: *const rt_gguf) -> u64;
    pub fn rt_gguf_metadata_count(g: *const rt_gguf) -> u64;
    pub fn rt_gguf_tensor_data_offset(g: *const rt_gguf) -> u64;
    pub fn rt_gguf_tensor_info_at(g: *const rt_gguf, index: u64, info: *mut rt_gguf_tensor_info) -> rt_status;
    pub fn rt_gguf_find_tensor(g: *const rt_gguf, name: *const c_char, index: *mut u64) -> rt_status;
    pub fn rt_gguf_metadata_key_at(g: *const rt_gguf, index: u64, key: *mut *const c_char) -> rt_status;
    pub fn rt_gguf_metadata_get(g: *const rt_gguf, key: *const c_char, value: *mut rt_gguf_value) -> rt_status;
    pub fn rt_gguf_metadata_array_get(g: *const rt_gguf, key: *const c_char, i: u64, value: *mut rt_gguf_value) -> rt_status;
    pub fn rt_ggml_type_size(ggml_dtype: i32) -> u64;
    pub fn rt_ggml_block_numel(ggml_dtype: i32) -> u64;
    pub fn rt_gguf_load_tensor(ctx: *mut rt_ctx, g: *const rt_gguf, image: *const c_void, size: u64, index: u64,
                               dst_dtype: i32, staging: *mut c_void, dst: *mut c_void, stream: *mut c_void) -> rt_status;
}
