// In-place softmax over the last dimension:  x[r, :] <- exp(x[r, :] - max_r) / sum_r.
// The step between the two attention matmuls (scores -> probabilities).  HBM-bound: one read
// and one write of the tensor.
//
// Fast path: one wavefront per row, the whole row in registers (up to 8 x 16 bytes per lane),
// so the tensor is read exactly once; maximum, exponentials and sum are f32 whatever the
// storage type, reduced across the wavefront with DPP shuffles; the result is rounded once.
// Rows that are longer, or whose length is not a whole number of 16-byte vectors, take the
// workgroup-per-row kernel, which re-reads the row (from L2) for each of its three passes.
//
// Role in the reference: ops/softmax.rs:52-183 (one 128-thread workgroup per row, reductions
// through workgroup memory, arithmetic in the tensor's own type).  Differences, both tighter:
// f16 tensors are reduced in f32, and the running maximum starts from the data rather than
// from a finite floor, so rows made only of very negative values still normalise.
#include <limits>

#include "device_common.h"

namespace rt {


template <typename T> struct SoftmaxVec;
template <> struct SoftmaxVec<float> {
    static constexpr int EV = 4;
    __device__ __forceinline__ static float get(const uint4_t &v, int e) { return __builtin_bit_cast(float4_t, v)[e]; }
    template <typename F> __device__ __forceinline__ static uint4_t make(F f) {
        return __builtin_bit_cast(uint4_t, float4_t{f(0), f(1), f(2), f(3)});
    }
};
template <> struct SoftmaxVec<half_t> {
    static constexpr int EV = 8;
    __device__ __forceinline__ static float get(const uint4_t &v, int e) { return (float)__builtin_bit_cast(half8_t, v)[e]; }
    template <typename F> __device__ __forceinline__ static uint4_t make(F f) {
        return __builtin_bit_cast(uint4_t, half8_t{(half_t)f(0), (half_t)f(1), (half_t)f(2), (half_t)f(3), (half_t)f(4),
                                                   (half_t)f(5), (half_t)f(6), (half_t)f(7)});
    }
};

// VPL: 16-byte vectors per lane; a row has nvec <= 64 * VPL vectors.
template <typename T, int VPL>
__global__ __launch_bounds__(256) void softmax_rows_kernel(T *x, int64_t rows, int nvec) {
    constexpr int EV = SoftmaxVec<T>::EV;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return; // whole wavefronts leave together
    uint4_t *p = (uint4_t *)(x + row * (int64_t)nvec * EV);
    float f[VPL][EV];
    const float ninf = -std::numeric_limits<float>::infinity();
    float m = ninf;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int v = lane + 64 * i;
        uint4_t raw = {0u, 0u, 0u, 0u};
        if (v < nvec) raw = __builtin_nontemporal_load(p + v); // read once, written once: nothing to keep in the caches
#pragma unroll
        for (int e = 0; e < EV; e++) {
            f[i][e] = v < nvec ? SoftmaxVec<T>::get(raw, e) : ninf;
            m = fmaxf(m, f[i][e]);
        }
    }
    m = wave_max(m);
    if (m == ninf) m = 0.f; // a row of -inf: exp(-inf - 0) = 0 everywhere, 0 / 0 = NaN as the formula says
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++)
#pragma unroll
        for (int e = 0; e < EV; e++) {
            f[i][e] = expf(f[i][e] - m);
            s += f[i][e];
        }
    s = wave_sum(s);
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int v = lane + 64 * i;
        if (v < nvec) __builtin_nontemporal_store(SoftmaxVec<T>::make([&](int e) { return f[i][e] / s; }), p + v);
    }
}

// One 256-thread workgroup per row, any length and alignment.
template <typename T>
__global__ __launch_bounds__(256) void softmax_generic_kernel(T *x, int64_t n) {
    __shared__ float red[4];
    T *p = x + (int64_t)blockIdx.x * n;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const float ninf = -std::numeric_limits<float>::infinity();
    float m = ninf;
    for (int64_t i = t; i < n; i += 256) m = fmaxf(m, to_f32(p[i]));
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (m == ninf) m = 0.f;
    __syncthreads();
    float s = 0.f;
    for (int64_t i = t; i < n; i += 256) s += expf(to_f32(p[i]) - m);
    s = wave_sum(s);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    for (int64_t i = t; i < n; i += 256) p[i] = from_f32<T>(expf(to_f32(p[i]) - m) / s);
}

template <typename T> static hipError_t launch_softmax_t(void *x, int64_t rows, int64_t n, hipStream_t st) {
    constexpr int EV = SoftmaxVec<T>::EV;
    if (rows == 0 || n == 0) return hipSuccess;
    const bool vec = n % EV == 0 && n / EV <= 64 * 8 && ((uintptr_t)x & 15u) == 0;
    if (vec) {
        const int nvec = (int)(n / EV);
        const int64_t blocks = (rows + 3) / 4;
        if (blocks > 0x7fffffff) return hipErrorInvalidValue;
        dim3 grid((unsigned)blocks);
        if (nvec <= 64) hipLaunchKernelGGL((softmax_rows_kernel<T, 1>), grid, dim3(256), 0, st, (T *)x, rows, nvec);
        else if (nvec <= 128) hipLaunchKernelGGL((softmax_rows_kernel<T, 2>), grid, dim3(256), 0, st, (T *)x, rows, nvec);
        else if (nvec <= 256) hipLaunchKernelGGL((softmax_rows_kernel<T, 4>), grid, dim3(256), 0, st, (T *)x, rows, nvec);
        else hipLaunchKernelGGL((softmax_rows_kernel<T, 8>), grid, dim3(256), 0, st, (T *)x, rows, nvec);
        return hipGetLastError();
    }
    if (rows > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL((softmax_generic_kernel<T>), dim3((unsigned)rows), dim3(256), 0, st, (T *)x, n);
    return hipGetLastError();
}

hipError_t launch_softmax(int dtype, void *x, int64_t rows, int64_t n, hipStream_t stream) {
    return dtype == RT_F16 ? launch_softmax_t<half_t>(x, rows, n, stream) : launch_softmax_t<float>(x, rows, n, stream);
}

} // namespace rt
