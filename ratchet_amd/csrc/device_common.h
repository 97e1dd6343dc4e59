// Shared device-side helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <type_traits>

#include <cstdint>

#include "spec.h"

namespace rt {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Development switches (force or forbid a kernel variant).  In the shipped library they are
// compile-time constants, so the library has no mutable global state; a microbenchmark that
// wants to flip one builds its own objects with -DRT_DEV_TUNABLES.
#ifdef RT_DEV_TUNABLES
#define RT_TUNABLE(name, value) int name = value
#else
#define RT_TUNABLE(name, value) static constexpr int name = value
#endif

// Raises a kernel's dynamic LDS limit to the 160 KiB of a gfx950 CU, once per process and
// kernel, safely from any thread.  Use as ensure_lds_limit<&kernel<...>>().
template <auto Kernel> inline hipError_t ensure_lds_limit() {
    static const hipError_t e =
        hipFuncSetAttribute((const void *)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    return e;
}

struct DeviceInfo {
    int ordinal = 0;
    int num_cus = 256;
};

// Sum / maximum over the 64 lanes of a wavefront; every lane receives the result.  Four DPP rotations
// inside the 16-lane rows, then v_permlane16_swap and v_permlane32_swap of the register with itself (they
// put the partner row's / half's value beside the lane's own): six vector instructions and their
// additions, no trip through the LDS crossbar (ds_bpermute, which __shfl_xor is, costs one per step).
template <int CTRL> __device__ __forceinline__ float wave_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <typename OP> __device__ __forceinline__ float wave_reduce(float v, OP op) {
    v = op(v, wave_dpp<0x128>(v)); // row_ror:8
    v = op(v, wave_dpp<0x124>(v)); // row_ror:4
    v = op(v, wave_dpp<0x122>(v)); // row_ror:2
    v = op(v, wave_dpp<0x121>(v)); // row_ror:1
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = op(__builtin_bit_cast(float, (uint32_t)a[0]), __builtin_bit_cast(float, (uint32_t)a[1]));
    const uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return op(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}
__device__ __forceinline__ float wave_sum(float v) {
    return wave_reduce(v, [](float a, float b) { return a + b; });
}
__device__ __forceinline__ float wave_max(float v) {
    return wave_reduce(v, [](float a, float b) { return fmaxf(a, b); });
}

// The row-streaming GEMVs' sums: the caller needs the result in one lane only, which five (six) DPP additions give.
template <int CTRL, int ROWMASK> __device__ __forceinline__ float rowdot_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWMASK, 0xf, true));
}
// Sum over each half-wave, valid in lanes 16..31 and 48..63; with WHOLE the sum over all 64 lanes, valid in lanes 48..63.
template <bool WHOLE> __device__ __forceinline__ float rowdot_sum(float v) {
    v += rowdot_dpp<0x128, 0xf>(v); // row_ror:8
    v += rowdot_dpp<0x124, 0xf>(v); // row_ror:4
    v += rowdot_dpp<0x122, 0xf>(v); // row_ror:2
    v += rowdot_dpp<0x121, 0xf>(v); // row_ror:1: every lane of a row of 16 holds the row's sum
    v += rowdot_dpp<0x142, 0xa>(v); // row_bcast:15: rows 1 and 3 add the row before them
    if (WHOLE) v += rowdot_dpp<0x143, 0xc>(v); // row_bcast:31: rows 2 and 3 add lane 31
    return v;
}

__device__ __forceinline__ float to_f32(half_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(float v) { return v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ half_t from_f32<half_t>(float v) { return (half_t)v; } // RNE

// Activations that can be fused behind a product (and run as operators of their own).
// ops/unary.rs:97-131 states gelu as x * (0.5 + 0.5 * safe_tanh(u)), u = x * (0.035677407 x^2 + 0.7978846),
// and silu as x * sigmoid(x).  Since 0.5 + 0.5 * tanh(u) = sigmoid(2u), both are one sigmoid here:
// sigmoid(z) = 1 / (1 + exp(-z)), evaluated with the hardware exponential and reciprocal (about
// ten instructions, so that an epilogue unrolled over a whole accumulator tile stays small).
// exp(-z) overflows to +inf for very negative z and the reciprocal of +inf is 0, the limit the
// reference's two-branch sigmoid and its safe_tanh reach; unlike 0.5 + 0.5 * tanh(u) the
// sigmoid form does not cancel in the negative tail.
// The factors -log2(e) and -2 log2(e) are folded into the constants so that the exponential is
// one v_exp_f32 (base 2) of a polynomial.
__device__ __forceinline__ float rt_silu(float v) {
    return v * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}
__device__ __forceinline__ float rt_gelu(float v) {
    // -2 log2(e) * (0.035677407 v^2 + 0.7978846)
    const float z = v * (-0.10294324f * (v * v) - 2.3022083f);
    return v * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(z));
}
__device__ __forceinline__ float rt_act(float v, int act) {
    if (act == RT_ACT_GELU) return rt_gelu(v);
    if (act == RT_ACT_SILU) return rt_silu(v);
    return v;
}
template <int ACT> __device__ __forceinline__ float rt_act_k(float v) {
    if constexpr (ACT == RT_ACT_GELU) return rt_gelu(v);
    else if constexpr (ACT == RT_ACT_SILU) return rt_silu(v);
    else return v;
}
// Epilogues are written once as a generic lambda over std::integral_constant<int, activation> and entered
// through this switch: the plain product keeps the code it has without activations, and an epilogue
// unrolled over a whole accumulator tile evaluates its one activation without a branch per element.
template <typename F> __device__ __forceinline__ void rt_with_act(int act, F &&body) {
    if (act == RT_ACT_GELU)
        body(std::integral_constant<int, RT_ACT_GELU>{});
    else if (act == RT_ACT_SILU)
        body(std::integral_constant<int, RT_ACT_SILU>{});
    else
        body(std::integral_constant<int, RT_ACT_NONE>{});
}

// 6-bit scale / min of sub-block j of a Q4_K super-block (ggml get_scale_min_k4).
__device__ __forceinline__ void q4k_scale_min(int j, const uint8_t *s, int &sc, int &mn) {
    if (j < 4) {
        sc = s[j] & 63;
        mn = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

// Launchers (one per kernel family).  All pointers are device pointers.
hipError_t launch_gemv(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                       hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_q8h_mfma(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_q8h_quad(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_q8h_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                  hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_float_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                    hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_q4k_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                  hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_q4k_mfma(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemv_chunked(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                               const DeviceInfo &dev);
hipError_t launch_gemm_q4k(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                           const DeviceInfo &dev);
hipError_t launch_gemm_f32(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                           const DeviceInfo &dev);
hipError_t launch_gemm(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                       hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemm_stream(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                              const DeviceInfo &dev);
uint64_t gemm_nt_workspace_bytes(const Problem &p, const DeviceInfo &dev);
hipError_t launch_gemm_nt(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                          hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_gemm_nn_smalln(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                 hipStream_t stream, const DeviceInfo &dev);
hipError_t launch_unary(int act, int dtype, const void *src, void *dst, uint64_t numel, hipStream_t stream);
hipError_t launch_cast(int src_dtype, int dst_dtype, const void *src, void *dst, uint64_t numel, hipStream_t stream);
hipError_t launch_cache_write(void *cache, const void *src, void *cache2, const void *src2, void *dst, int64_t cache_bs,
                              int64_t cache_hs, int64_t src_bs, int64_t src_hs, int64_t src_rs, int batch, int heads, int offset,
                              int len, int64_t row_bytes, hipStream_t stream);
hipError_t launch_softmax(int dtype, void *x, int64_t rows, int64_t n, hipStream_t stream);
hipError_t launch_attention(const rt_attention_desc &d, const void *q, const void *k, const void *v, const void *mask,
                            void *out, void *workspace, uint64_t workspace_bytes, hipStream_t stream);
uint64_t attention_workspace_bytes(const rt_attention_desc &d);
hipError_t launch_quantize_q8_0(const float *src, uint64_t numel, void *dst, hipStream_t stream);
hipError_t launch_dequantize(int dtype, const void *src, uint64_t numel, float *dst, hipStream_t stream);
hipError_t launch_transcode_gguf_q8_0(const void *blocks, uint64_t n_blocks, int dst_dtype, void *dst,
                                      hipStream_t stream);

} // namespace rt
