// Measurement probes for bench.py --read-calibration and --issue-calibration: what one launch costs when it does
// nothing, and when it only reads a buffer the size of the headline weight; and what a wavefront's MFMAs, packed
// vector instructions and LDS fragment reads cost alone and mixed.  They give the
// streaming kernels' times their context (how much of a launch is fixed, how fast this chip
// delivers 27.9 MB to a kernel that has nothing else to do).  Built into their own library,
// libratchet_probes.so; the product library does not contain them and nothing else uses them.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>

typedef uint32_t probe_u4 __attribute__((ext_vector_type(4)));

// The timing-only builds of kernels_gemm_nt.hip that this library also holds (probe_gemm_nt_ablation_<mask>, see
// build.py) refer to this function of the product library; the library's own copy keeps it self-contained.
extern "C" uint64_t rt_q8_0_scale_offset(uint64_t numel) { return (numel + 255u) & ~(uint64_t)255u; }

__global__ void probe_empty_kernel(uint32_t *sink) {
    if (sink == nullptr) sink[0] = 1; // never
}

// Every wavefront reads LOADS x 1 KiB of consecutive bytes, 16 per lane and load; all loads are
// issued before the first is consumed.  NT: non-temporal loads.  STORE: one lane of every wavefront
// also stores four bytes of what it read to out[wavefront], the way the GEMV's wavefronts store their
// two f16 results: a kernel that leaves modified lines in the L2s pays for their write-back when it ends.
template <int LOADS, bool NT, bool STORE>
__global__ __launch_bounds__(256) void probe_read_linear_kernel(const probe_u4 *__restrict__ p, uint64_t nvec, uint32_t *sink) {
    const uint64_t wave = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const uint64_t base = wave * (uint64_t)(LOADS * 64) + (threadIdx.x & 63);
    probe_u4 v[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; i++) {
        const uint64_t idx = base + (uint64_t)i * 64 < nvec ? base + (uint64_t)i * 64 : nvec - 1;
        v[i] = NT ? __builtin_nontemporal_load(p + idx) : p[idx];
    }
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < LOADS; i++) acc ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
    if (STORE) {
        asm volatile("" : "+v"(acc)); // every lane's value exists here: the loads cannot move into the branch
        if ((threadIdx.x & 63) == 0) sink[wave] = acc;
    } else if (acc == 0x12345678u) sink[wave & 1023] = acc; // practically never; keeps the loads alive
}

// The matrix-core GEMV's address pattern: a workgroup of K / 256 wavefronts owns 16 rows of a
// row-major [rows x K] byte matrix; per load a lane reads 16 bytes of row lane % 16 at 16 * (lane / 16).
__global__ __launch_bounds__(1024) void probe_read_rows16_kernel(const uint8_t *__restrict__ p, int64_t K, uint32_t *sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *q = p + ((int64_t)blockIdx.x * 16 + (lane & 15)) * K + (int64_t)wave * 256 + 16 * (lane >> 4);
    probe_u4 v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = *(const probe_u4 *)(q + 64 * i);
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) acc ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
    if (acc == 0x12345678u) sink[blockIdx.x & 1023] = acc;
}

// One wavefront per SIMD (256 threads, 256 workgroups) runs `iters` trips of: NM MFMAs (16x16x32 f16, eight
// independent accumulators), NV packed f16 FMAs behind each of eight slots, ND 16-byte-per-lane LDS reads in the
// fragment pattern of the tiled kernels (16 rows 528 bytes apart, four lane groups 128 bytes apart), whose data
// feed the next trip's MFMAs.  The order inside a trip is pinned: with PL = 0 a read goes in front of an MFMA
// (read, MFMA, vector instructions), with PL = 1 right behind it (MFMA, read, vector instructions).
typedef _Float16 probe_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 probe_h8 __attribute__((ext_vector_type(8)));
typedef float probe_f4 __attribute__((ext_vector_type(4)));
template <int NV, int NM, int ND, int PL>
__global__ __launch_bounds__(256) void probe_issue_mix_kernel(const probe_h8 *in, float *out, int iters) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    for (int i = threadIdx.x; i < 16384; i += 256) ((uint32_t *)smem)[i] = 0;
    __syncthreads();
    probe_h8 a = in[threadIdx.x], b = in[threadIdx.x + 256];
    probe_f4 acc[8];
    for (int i = 0; i < 8; i++) acc[i] = probe_f4{0, 0, 0, 0};
    probe_h2 v[8];
    for (int i = 0; i < 8; i++) v[i] = probe_h2{a[i], b[i]};
    const probe_h2 m = {b[0], b[1]}, c = {b[2], b[3]};
    const uint32_t la = (threadIdx.x & 15) * 528 + ((threadIdx.x >> 4) & 3) * 128 + (threadIdx.x >> 6) * 8448;
    probe_h8 x[2][4];
    for (int d = 0; d < 4; d++) x[0][d] = a, x[1][d] = b;
    for (int it = 0; it < iters; it += 2) {
#pragma unroll
        for (int ph = 0; ph < 2; ph++) {
#pragma unroll
            for (int d = 0; d < ND; d++) x[ph ^ 1][d & 3] = __builtin_bit_cast(probe_h8, *(const probe_u4 *)(smem + la + 16 * d + 128 * ph));
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (i < NM) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x[ph][i & 3], b, acc[i], 0, 0, 0);
#pragma unroll
                for (int j = 0; j < NV; j++) v[(i + j) & 7] = __builtin_elementwise_fma(v[(i + j) & 7], m, c);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const bool rd = ND >= 8 || (ND == 4 && (i & 1) == 0) || (ND == 2 && (i & 3) == 0);
                if (PL == 0 && rd) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if (i < NM) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (PL == 1 && rd) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if (NV) __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0;
    for (int i = 0; i < 8; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + (float)v[i][0] + (float)v[i][1];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

extern "C" {

// `in`: 8 KiB of zeros; `out`: 256 KiB.  Returns hipErrorInvalidValue for a mix that is not instantiated.
__attribute__((visibility("default"))) int probe_issue_mix(int nv, int nm, int nd, int behind, int iters, const void *in, void *out, void *stream) {
#define PROBE_MIX(V, M, D, P)                                                                                                       \
    if (nv == V && nm == M && nd == D && behind == P) {                                                                                          \
        static const hipError_t e = hipFuncSetAttribute((const void *)probe_issue_mix_kernel<V, M, D, P>,                              \
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, 65536);                         \
        if (e != hipSuccess) return (int)e;                                                                                         \
        hipLaunchKernelGGL((probe_issue_mix_kernel<V, M, D, P>), dim3(256), dim3(256), 65536, (hipStream_t)stream,                     \
                           (const probe_h8 *)in, (float *)out, iters);                                                             \
        return (int)hipGetLastError();                                                                                              \
    }
    PROBE_MIX(0, 8, 0, 0) PROBE_MIX(3, 0, 0, 0) PROBE_MIX(3, 8, 0, 0) PROBE_MIX(0, 8, 4, 0) PROBE_MIX(3, 0, 4, 0) PROBE_MIX(3, 8, 2, 0)
    PROBE_MIX(3, 8, 4, 0) PROBE_MIX(1, 8, 0, 0) PROBE_MIX(2, 8, 0, 0) PROBE_MIX(4, 8, 0, 0) PROBE_MIX(6, 8, 0, 0)
    PROBE_MIX(3, 8, 4, 1) PROBE_MIX(3, 8, 8, 0) PROBE_MIX(3, 8, 8, 1)
#undef PROBE_MIX
    return (int)hipErrorInvalidValue;
}

__attribute__((visibility("default"))) int probe_empty(void *sink, void *stream) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (uint32_t *)sink);
    return (int)hipGetLastError();
}

// reads nbytes (a multiple of 16) at p; sink: at least 4 KiB of device memory
__attribute__((visibility("default"))) int probe_read_linear(const void *p, uint64_t nbytes, int nontemporal, void *sink,
                                                             void *stream) {
    constexpr int L = 2;
    const uint64_t nvec = nbytes / 16, waves = (nvec + L * 64 - 1) / (L * 64);
    const unsigned blocks = (unsigned)((waves + 3) / 4);
    if (nvec == 0) return 0;
    if (nontemporal)
        hipLaunchKernelGGL((probe_read_linear_kernel<L, true, false>), dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                           (const probe_u4 *)p, nvec, (uint32_t *)sink);
    else
        hipLaunchKernelGGL((probe_read_linear_kernel<L, false, false>), dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                           (const probe_u4 *)p, nvec, (uint32_t *)sink);
    return (int)hipGetLastError();
}

// reads nbytes (a multiple of 16) at p with non-temporal loads, 5 KiB per wavefront (the GEMV's share at
// K = 2560), and stores 4 bytes per wavefront to out (at least 4 * ceil(nbytes / 5120) bytes, rounded
// up to a multiple of 16)
__attribute__((visibility("default"))) int probe_read_linear_store(const void *p, uint64_t nbytes, void *out, void *stream) {
    constexpr int L = 5;
    const uint64_t nvec = nbytes / 16, waves = (nvec + L * 64 - 1) / (L * 64);
    const unsigned blocks = (unsigned)((waves + 3) / 4);
    if (nvec == 0) return 0;
    hipLaunchKernelGGL((probe_read_linear_kernel<L, true, true>), dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       (const probe_u4 *)p, nvec, (uint32_t *)out);
    return (int)hipGetLastError();
}

// reads a [rows x K] byte matrix (rows % 16 == 0, K % 256 == 0, K <= 4096) in the 16-row pattern
__attribute__((visibility("default"))) int probe_read_rows16(const void *p, int64_t rows, int64_t K, void *sink, void *stream) {
    if (rows % 16 || K % 256 || K < 256 || K > 4096) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_read_rows16_kernel, dim3((unsigned)(rows / 16)), dim3((unsigned)(K / 256) * 64), 0,
                       (hipStream_t)stream, (const uint8_t *)p, K, (uint32_t *)sink);
    return (int)hipGetLastError();
}

// What the host spends per enqueue, with no interpreter in the loop: n back-to-back calls of the entry point whose
// address is `fn` (rt_matmul_enqueue_ws or rt_matmul_plan_enqueue of the product library, handed over by the
// caller so that this library does not link against it), timed with the host's steady clock.  The launches pile up
// on the stream; the caller synchronises afterwards.  Returns nanoseconds per call, or -1 if a call failed.
__attribute__((visibility("default"))) double probe_host_ns_enqueue_ws(void *fn, void *ctx, const void *desc, const void *lhs,
                                                                       const void *rhs, const void *bias, void *out,
                                                                       int32_t act, void *stream, int n) {
    typedef int32_t (*F)(void *, const void *, const void *, const void *, const void *, void *, int32_t, void *, uint64_t, void *);
    const F f = (F)fn;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n; i++)
        if (f(ctx, desc, lhs, rhs, bias, out, act, nullptr, 0, stream) != 0) return -1.0;
    return std::chrono::duration<double, std::nano>(std::chrono::steady_clock::now() - t0).count() / n;
}

__attribute__((visibility("default"))) double probe_host_ns_plan_enqueue(void *fn, void *plan, const void *lhs, const void *rhs,
                                                                         const void *bias, void *out, void *stream, int n) {
    typedef int32_t (*F)(void *, const void *, const void *, const void *, void *, void *, uint64_t, void *);
    const F f = (F)fn;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n; i++)
        if (f(plan, lhs, rhs, bias, out, nullptr, 0, stream) != 0) return -1.0;
    return std::chrono::duration<double, std::nano>(std::chrono::steady_clock::now() - t0).count() / n;
}
}
