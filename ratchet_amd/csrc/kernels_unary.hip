// Elementwise operators that surround the products in the reference's models: the two
// activations (ops/unary.rs:97-171), the f32 <-> f16 cast (ops/cast.rs) and the key/value cache
// write (ops/cache.rs).  HBM-bound:
// one read and one write of the tensor, 16 bytes per lane per access on whole vectors, a
// scalar tail for the last few elements.  Arithmetic is f32 whatever the storage type.
#include "device_common.h"

namespace rt {

// A thread takes UNARY_U vectors of 16 bytes a workgroup-width apart and requests them all before it
// evaluates the first: with one vector per thread the launch is a single trip to memory per wavefront
// with nothing else in flight.  Loads and stores are non-temporal: every byte is touched once.
constexpr int UNARY_U = 4;

template <typename T, int ACT>
__global__ __launch_bounds__(256) void unary_kernel(const T *src, T *dst, uint64_t numel) {
    constexpr int EV = 16 / sizeof(T);
    const uint64_t nvec = numel / EV;
    const uint64_t stride = (uint64_t)gridDim.x * (256 * UNARY_U);
    for (uint64_t v0 = (uint64_t)blockIdx.x * (256 * UNARY_U) + threadIdx.x; v0 < nvec; v0 += stride) {
        uint4_t raw[UNARY_U];
#pragma unroll
        for (int u = 0; u < UNARY_U; u++) {
            const uint64_t v = v0 + 256u * u;
            raw[u] = __builtin_nontemporal_load((const uint4_t *)src + (v < nvec ? v : nvec - 1)); // past the end: a valid vector, not stored
        }
#pragma unroll
        for (int u = 0; u < UNARY_U; u++) {
            const uint64_t v = v0 + 256u * u;
            uint4_t res;
            if constexpr (sizeof(T) == 2) {
                half8_t h = __builtin_bit_cast(half8_t, raw[u]);
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = (half_t)rt_act((float)h[e], ACT);
                res = __builtin_bit_cast(uint4_t, h);
            } else {
                float4_t f = __builtin_bit_cast(float4_t, raw[u]);
#pragma unroll
                for (int e = 0; e < 4; e++) f[e] = rt_act(f[e], ACT);
                res = __builtin_bit_cast(uint4_t, f);
            }
            if (v < nvec) __builtin_nontemporal_store(res, (uint4_t *)dst + v);
        }
    }
    // the elements past the last whole vector
    const uint64_t tail0 = nvec * EV;
    const uint64_t i = tail0 + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < numel) dst[i] = from_f32<T>(rt_act(to_f32(src[i]), ACT));
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S *src, D *dst, uint64_t numel) {
    // 8 elements per vector: 32 bytes of f32 <-> 16 bytes of f16; UNARY_U vectors per thread, all requested
    // before the first is converted, non-temporal both ways
    const uint64_t nvec = numel / 8;
    const uint64_t stride = (uint64_t)gridDim.x * (256 * UNARY_U);
    for (uint64_t v0 = (uint64_t)blockIdx.x * (256 * UNARY_U) + threadIdx.x; v0 < nvec; v0 += stride) {
        if constexpr (sizeof(S) == 4) {
            float4_t a[UNARY_U], b[UNARY_U];
#pragma unroll
            for (int u = 0; u < UNARY_U; u++) {
                const uint64_t v = v0 + 256u * u < nvec ? v0 + 256u * u : nvec - 1; // past the end: a valid vector, not stored
                a[u] = __builtin_nontemporal_load((const float4_t *)src + 2 * v);
                b[u] = __builtin_nontemporal_load((const float4_t *)src + 2 * v + 1);
            }
#pragma unroll
            for (int u = 0; u < UNARY_U; u++) {
                const uint64_t v = v0 + 256u * u;
                const half8_t h = {(half_t)a[u][0], (half_t)a[u][1], (half_t)a[u][2], (half_t)a[u][3],
                                   (half_t)b[u][0], (half_t)b[u][1], (half_t)b[u][2], (half_t)b[u][3]};
                if (v < nvec) __builtin_nontemporal_store(__builtin_bit_cast(uint4_t, h), (uint4_t *)dst + v);
            }
        } else {
            uint4_t raw[UNARY_U];
#pragma unroll
            for (int u = 0; u < UNARY_U; u++) {
                const uint64_t v = v0 + 256u * u < nvec ? v0 + 256u * u : nvec - 1;
                raw[u] = __builtin_nontemporal_load((const uint4_t *)src + v);
            }
#pragma unroll
            for (int u = 0; u < UNARY_U; u++) {
                const uint64_t v = v0 + 256u * u;
                const half8_t h = __builtin_bit_cast(half8_t, raw[u]);
                if (v < nvec) {
                    __builtin_nontemporal_store(float4_t{(float)h[0], (float)h[1], (float)h[2], (float)h[3]}, (float4_t *)dst + 2 * v);
                    __builtin_nontemporal_store(float4_t{(float)h[4], (float)h[5], (float)h[6], (float)h[7]}, (float4_t *)dst + 2 * v + 1);
                }
            }
        }
    }
    const uint64_t i = nvec * 8 + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < numel) dst[i] = from_f32<D>(to_f32(src[i]));
}

static unsigned grid_for(uint64_t nvec, const unsigned cap = 256u * 32u) {
    const uint64_t blocks = (nvec + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

template <typename T> static hipError_t launch_unary_t(int act, const void *src, void *dst, uint64_t numel, hipStream_t st) {
    const unsigned grid = grid_for((numel / (16 / sizeof(T)) + UNARY_U - 1) / UNARY_U);
    if (act == RT_ACT_GELU)
        hipLaunchKernelGGL((unary_kernel<T, RT_ACT_GELU>), dim3(grid), dim3(256), 0, st, (const T *)src, (T *)dst, numel);
    else
        hipLaunchKernelGGL((unary_kernel<T, RT_ACT_SILU>), dim3(grid), dim3(256), 0, st, (const T *)src, (T *)dst, numel);
    return hipGetLastError();
}

// Buffers must be 16-byte aligned (every allocation of this library and of torch is).
hipError_t launch_unary(int act, int dtype, const void *src, void *dst, uint64_t numel, hipStream_t stream) {
    if (numel == 0) return hipSuccess;
    return dtype == RT_F16 ? launch_unary_t<half_t>(act, src, dst, numel, stream)
                           : launch_unary_t<float>(act, src, dst, numel, stream);
}

hipError_t launch_cast(int src_dtype, int dst_dtype, const void *src, void *dst, uint64_t numel, hipStream_t stream) {
    if (numel == 0) return hipSuccess;
    const unsigned grid = grid_for((numel / 8 + UNARY_U - 1) / UNARY_U);
    if (src_dtype == RT_F32 && dst_dtype == RT_F16)
        hipLaunchKernelGGL((cast_kernel<float, half_t>), dim3(grid), dim3(256), 0, stream, (const float *)src, (half_t *)dst, numel);
    else if (src_dtype == RT_F16 && dst_dtype == RT_F32)
        hipLaunchKernelGGL((cast_kernel<half_t, float>), dim3(grid), dim3(256), 0, stream, (const half_t *)src, (float *)dst, numel);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

// Key/value cache write (ops/cache.rs:69-96 with dim = 2): rows offset .. offset + len - 1 of
// cache [stacks][capacity][row_bytes] <- src [stacks][len][row_bytes] (strided), and, when dst is
// given, the reference's fresh contiguous tensor dst [stacks][offset + len][row_bytes] =
// cache[.., :offset] ++ src.  One thread per 16-byte vector of the longer of the two jobs.
// blockIdx.z == 1 works on the second cache / source pair (a key and a value cache of one geometry
// written by one launch); dst goes with the first pair only.
__global__ __launch_bounds__(256) void cache_write_kernel(uint8_t *cache, const uint8_t *src, uint8_t *cache2, const uint8_t *src2,
                                                          uint8_t *dst, int64_t cache_bs, int64_t cache_hs, int64_t src_bs,
                                                          int64_t src_hs, int64_t src_rs, int heads, int offset, int len,
                                                          int vec_per_row) {
    const int stack = blockIdx.y, b = stack / heads, h = stack - b * heads;
    const int64_t row_bytes = (int64_t)vec_per_row * 16;
    uint8_t *c = (blockIdx.z ? cache2 : cache) + b * cache_bs + h * cache_hs;
    const uint8_t *s = (blockIdx.z ? src2 : src) + b * src_bs + h * src_hs;
    uint8_t *d = dst ? dst + (int64_t)stack * (offset + len) * row_bytes : nullptr;
    const int rows = dst ? offset + len : len;
    const int64_t nvec = (int64_t)rows * vec_per_row;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * blockDim.x) {
        int r = (int)(v / vec_per_row);
        const int col = (int)(v - (int64_t)r * vec_per_row) * 16;
        if (!dst) r += offset; // only the new rows are visited
        if (r < offset) {
            *(uint4_t *)(d + r * row_bytes + col) = *(const uint4_t *)(c + r * row_bytes + col);
        } else {
            const uint4_t val = *(const uint4_t *)(s + (r - offset) * src_rs + col);
            *(uint4_t *)(c + r * row_bytes + col) = val;
            if (dst) *(uint4_t *)(d + r * row_bytes + col) = val;
        }
    }
}

// All strides in bytes; rows are row_bytes contiguous bytes, a multiple of 16.
// cache2 / src2: a second pair of the same geometry and strides written by the same launch, or NULL (then dst may be given).
hipError_t launch_cache_write(void *cache, const void *src, void *cache2, const void *src2, void *dst, int64_t cache_bs,
                              int64_t cache_hs, int64_t src_bs, int64_t src_hs, int64_t src_rs, int batch, int heads, int offset,
                              int len, int64_t row_bytes, hipStream_t stream) {
    if (cache2 && dst) return hipErrorInvalidValue;
    const int64_t stacks = (int64_t)batch * heads;
    const int rows = dst ? offset + len : len;
    if (stacks == 0 || rows == 0 || row_bytes == 0) return hipSuccess;
    if (stacks > 65535 || row_bytes % 16) return hipErrorInvalidValue;
    const int vpr = (int)(row_bytes / 16);
    const int64_t nvec = (int64_t)rows * vpr;
    const unsigned gx = (unsigned)((nvec + 255) / 256 > 4096 ? 4096 : (nvec + 255) / 256);
    hipLaunchKernelGGL(cache_write_kernel, dim3(gx, (unsigned)stacks, cache2 ? 2u : 1u), dim3(256), 0, stream, (uint8_t *)cache,
                       (const uint8_t *)src, (uint8_t *)cache2, (const uint8_t *)src2, (uint8_t *)dst, cache_bs, cache_hs, src_bs,
                       src_hs, src_rs, heads, offset, len, vpr);
    return hipGetLastError();
}

} // namespace rt
