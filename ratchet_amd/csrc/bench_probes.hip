// Measurement probes for bench.py --read-calibration: what one launch costs when it does
// nothing, and when it only reads a buffer the size of the headline weight.  They give the
// streaming kernels' times their context (how much of a launch is fixed, how fast this chip
// delivers 27.9 MB to a kernel that has nothing else to do).  Built into their own library,
// libratchet_probes.so; the product library does not contain them and nothing else uses them.
#include <hip/hip_runtime.h>

#include <cstdint>

typedef uint32_t probe_u4 __attribute__((ext_vector_type(4)));

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

extern "C" {

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
}
