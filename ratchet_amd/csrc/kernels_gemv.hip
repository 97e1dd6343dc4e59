// Streaming GEMV kernels for gfx950: y[i, j] = sum_k A[i, k] * x[j, k] (+ bias)
// for a tall weight operand A (rows of K, K contiguous) and a handful of
// activation vectors x[j] (j < 8).  The weight stream is read once, straight
// from HBM into registers with 128-bit loads and dequantized in registers;
// there is no LDS staging of weights.  One wavefront owns one row at a time
// and its 64 lanes stride the row in 16-byte chunks, so every load
// instruction of a wavefront covers 1 KiB of contiguous weights.
//
// Roles in the reference: ops/gemv.rs:156-574 (the workgroup and subgroup
// GEMV generators) and, for 2..8 activation rows, the scalar QGEMM of
// ops/gemm.rs:342-492 which the reference uses for those shapes.
#include "device_common.h"

namespace rt {

struct GemvArgs {
    const uint8_t *A;   // weight bytes (int8 stream / Q4_K blocks / f16 / f32)
    const void *scales; // Q8_0 scale stream
    const void *X;
    const void *bias;
    void *out;
    int64_t M, K;
    int64_t a_stack, b_stack;
    int64_t a_bs, a_rs; // stack and row stride of A in elements (float kernels)
    int64_t b_bs, b_js;
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
};

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;

template <typename AT, int NC>
__device__ __forceinline__ void gemv_store(const GemvArgs &g, int64_t s, int64_t row, int lane, const float *acc) {
    // lane j (< NC) writes column j.  acc[] is wave-uniform after the reduction.
    const AT *bias = (const AT *)g.bias;
    AT *out = (AT *)g.out;
#pragma unroll
    for (int j = 0; j < NC; j++) {
        if (lane == j) {
            float v = acc[j];
            if (g.has_bias) v += to_f32(bias[g.bias_on_rows ? row : (int64_t)j]);
            out[s * g.o_bs + row * g.o_is + j * g.o_js] = from_f32<AT>(rt_act(v, g.act));
        }
    }
}

// Loads 16 consecutive activations starting at x[k0] as floats.
template <typename AT> __device__ __forceinline__ void load_x16(const AT *x, float (&xf)[16]);
template <> __device__ __forceinline__ void load_x16<half_t>(const half_t *x, float (&xf)[16]) {
    half8_t a = *(const half8_t *)x, b = *(const half8_t *)(x + 8);
#pragma unroll
    for (int i = 0; i < 8; i++) xf[i] = (float)a[i], xf[8 + i] = (float)b[i];
}
template <> __device__ __forceinline__ void load_x16<float>(const float *x, float (&xf)[16]) {
#pragma unroll
    for (int v = 0; v < 4; v++) {
        float4_t a = *(const float4_t *)(x + 4 * v);
#pragma unroll
        for (int i = 0; i < 4; i++) xf[4 * v + i] = a[i];
    }
}

// ---------------------------------------------------------------------------
// Q8_0 weights.  Chunk = 16 int8 (half a block) + the block's scale.
// ---------------------------------------------------------------------------
template <typename AT, int NC, int U>
__global__ __launch_bounds__(kGemvThreads) void gemv_q8_kernel(GemvArgs g) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t s = blockIdx.y;
    // an operand's stack is either the full stack or 1 (broadcast)
    const int64_t sa = g.a_stack == 1 ? 0 : s, sb = g.b_stack == 1 ? 0 : s;
    const int nchunks = (int)(g.K >> 4);
    const AT *x = (const AT *)g.X + sb * g.b_bs;
    for (int64_t row = (int64_t)blockIdx.x * kGemvWaves + wave; row < g.M; row += (int64_t)gridDim.x * kGemvWaves) {
        const int64_t rowel = (sa * g.M + row) * g.K;
        const uint8_t *q = g.A + rowel;
        const AT *sc = (const AT *)g.scales + (rowel >> 5);
        float acc[NC];
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = 0.f;
        for (int c0 = 0; c0 < nchunks; c0 += kWave * U) {
            uint4_t w[U];
            float d[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int c = c0 + u * kWave + lane;
                const bool ok = c < nchunks;
                w[u] = ok ? *(const uint4_t *)(q + 16 * (int64_t)c) : uint4_t{0, 0, 0, 0};
                d[u] = ok ? to_f32(sc[c >> 1]) : 0.f;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int c = c0 + u * kWave + lane;
                if (c < nchunks) {
                    float wf[16];
#pragma unroll
                    for (int i = 0; i < 16; i++) wf[i] = (float)(int8_t)(w[u][i >> 2] >> (8 * (i & 3)));
#pragma unroll
                    for (int j = 0; j < NC; j++) {
                        float xf[16];
                        load_x16<AT>(x + j * g.b_js + 16 * (int64_t)c, xf);
                        float part = 0.f;
#pragma unroll
                        for (int i = 0; i < 16; i++) part += wf[i] * xf[i];
                        acc[j] += d[u] * part;
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = wave_sum(acc[j]);
        gemv_store<AT, NC>(g, s, row, lane, acc);
    }
}

// ---------------------------------------------------------------------------
// Q4_K weights.  A lane takes 16 bytes of a super-block's qs: 16 low nibbles
// (sub-block 2c) and 16 high nibbles (sub-block 2c+1), plus the 16-byte header
// {d, dmin, scales[12]} of that super-block.
// ---------------------------------------------------------------------------
template <int NC>
__global__ __launch_bounds__(kGemvThreads) void gemv_q4k_kernel(GemvArgs g) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t s = blockIdx.y;
    // an operand's stack is either the full stack or 1 (broadcast)
    const int64_t sa = g.a_stack == 1 ? 0 : s, sb = g.b_stack == 1 ? 0 : s;
    const int nsb = (int)(g.K >> 8);  // super-blocks per row
    const int npieces = nsb * 8;      // 16-byte qs pieces per row
    const half_t *x = (const half_t *)g.X + sb * g.b_bs;
    for (int64_t row = (int64_t)blockIdx.x * kGemvWaves + wave; row < g.M; row += (int64_t)gridDim.x * kGemvWaves) {
        const uint8_t *blk0 = g.A + ((sa * g.M + row) * nsb) * 144;
        float acc[NC];
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = 0.f;
        for (int p0 = 0; p0 < npieces; p0 += kWave) {
            const int p = p0 + lane;
            if (p < npieces) {
                const int sbi = p >> 3, piece = p & 7, c = piece >> 1, h = piece & 1;
                const uint8_t *blk = blk0 + (int64_t)sbi * 144;
                const uint4_t hdr = *(const uint4_t *)blk;
                const uint4_t qv = *(const uint4_t *)(blk + 16 + 16 * piece);
                half2_t dm = __builtin_bit_cast(half2_t, hdr[0]);
                const float d = (float)dm[0], dmin = (float)dm[1];
                uint8_t sbytes[12];
#pragma unroll
                for (int i = 0; i < 12; i++) sbytes[i] = (uint8_t)(hdr[1 + (i >> 2)] >> (8 * (i & 3)));
                int sc0, mn0, sc1, mn1;
                q4k_scale_min(2 * c, sbytes, sc0, mn0);
                q4k_scale_min(2 * c + 1, sbytes, sc1, mn1);
                const float d0 = d * (float)sc0, m0 = dmin * (float)mn0;
                const float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
                const int64_t k_lo = (int64_t)sbi * 256 + 64 * c + 16 * h, k_hi = k_lo + 32;
#pragma unroll
                for (int j = 0; j < NC; j++) {
                    float xl[16], xh[16];
                    load_x16<half_t>(x + j * g.b_js + k_lo, xl);
                    load_x16<half_t>(x + j * g.b_js + k_hi, xh);
                    float part = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const uint32_t byte = (qv[i >> 2] >> (8 * (i & 3))) & 0xFFu;
                        // same evaluation as the dequantizer: w = d*sc*q - dmin*mn
                        const float wl = d0 * (float)(byte & 0xFu) - m0;
                        const float wh = d1 * (float)(byte >> 4) - m1;
                        part += wl * xl[i];
                        part += wh * xh[i];
                    }
                    acc[j] += part;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = wave_sum(acc[j]);
        gemv_store<half_t, NC>(g, s, row, lane, acc);
    }
}

// ---------------------------------------------------------------------------
// f16 / f32 weights.  VEC selects 16-byte loads (aligned, K % 16 == 0 handled
// by a scalar tail) or a fully scalar walk for odd strides.
// ---------------------------------------------------------------------------
template <typename AT, int NC, bool VEC>
__global__ __launch_bounds__(kGemvThreads) void gemv_float_kernel(GemvArgs g) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t s = blockIdx.y;
    // an operand's stack is either the full stack or 1 (broadcast)
    const int64_t sa = g.a_stack == 1 ? 0 : s, sb = g.b_stack == 1 ? 0 : s;
    const AT *x = (const AT *)g.X + sb * g.b_bs;
    const AT *Abase = (const AT *)g.A + sa * g.a_bs;
    constexpr int E = 16 / (int)sizeof(AT); // elements per 16-byte chunk
    for (int64_t row = (int64_t)blockIdx.x * kGemvWaves + wave; row < g.M; row += (int64_t)gridDim.x * kGemvWaves) {
        const AT *a = Abase + row * g.a_rs;
        float acc[NC];
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = 0.f;
        int64_t kdone = 0;
        if (VEC) {
            const int64_t nchunks = g.K / E;
            for (int64_t c = lane; c < nchunks; c += kWave) {
                const uint4_t raw = *(const uint4_t *)(a + c * E);
                float wf[E];
                if constexpr (sizeof(AT) == 2) {
                    half8_t hv = __builtin_bit_cast(half8_t, raw);
#pragma unroll
                    for (int i = 0; i < E; i++) wf[i] = (float)hv[i];
                } else {
                    float4_t fv = __builtin_bit_cast(float4_t, raw);
#pragma unroll
                    for (int i = 0; i < E; i++) wf[i] = fv[i];
                }
#pragma unroll
                for (int j = 0; j < NC; j++) {
                    const uint4_t xr = *(const uint4_t *)(x + j * g.b_js + c * E);
                    float part = 0.f;
                    if constexpr (sizeof(AT) == 2) {
                        half8_t hv = __builtin_bit_cast(half8_t, xr);
#pragma unroll
                        for (int i = 0; i < E; i++) part += wf[i] * (float)hv[i];
                    } else {
                        float4_t fv = __builtin_bit_cast(float4_t, xr);
#pragma unroll
                        for (int i = 0; i < E; i++) part += wf[i] * fv[i];
                    }
                    acc[j] += part;
                }
            }
            kdone = nchunks * E;
        }
        for (int64_t k = kdone + lane; k < g.K; k += kWave) {
            const float w = to_f32(a[k]);
#pragma unroll
            for (int j = 0; j < NC; j++) acc[j] += w * to_f32(x[j * g.b_js + k]);
        }
#pragma unroll
        for (int j = 0; j < NC; j++) acc[j] = wave_sum(acc[j]);
        gemv_store<AT, NC>(g, s, row, lane, acc);
    }
}

// ---------------------------------------------------------------------------
// Launch
// ---------------------------------------------------------------------------
static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <int NC> static void launch_q8(int act_dt, dim3 grid, hipStream_t st, const GemvArgs &g) {
    if (act_dt == RT_F16)
        hipLaunchKernelGGL((gemv_q8_kernel<half_t, NC, 4>), grid, dim3(kGemvThreads), 0, st, g);
    else
        hipLaunchKernelGGL((gemv_q8_kernel<float, NC, 4>), grid, dim3(kGemvThreads), 0, st, g);
}
template <int NC> static void launch_q4k(dim3 grid, hipStream_t st, const GemvArgs &g) {
    hipLaunchKernelGGL((gemv_q4k_kernel<NC>), grid, dim3(kGemvThreads), 0, st, g);
}
template <int NC> static void launch_float(int act_dt, bool vec, dim3 grid, hipStream_t st, const GemvArgs &g) {
    if (act_dt == RT_F16) {
        if (vec) hipLaunchKernelGGL((gemv_float_kernel<half_t, NC, true>), grid, dim3(kGemvThreads), 0, st, g);
        else hipLaunchKernelGGL((gemv_float_kernel<half_t, NC, false>), grid, dim3(kGemvThreads), 0, st, g);
    } else {
        if (vec) hipLaunchKernelGGL((gemv_float_kernel<float, NC, true>), grid, dim3(kGemvThreads), 0, st, g);
        else hipLaunchKernelGGL((gemv_float_kernel<float, NC, false>), grid, dim3(kGemvThreads), 0, st, g);
    }
}

#define RT_DISPATCH_NC(N, CALL)                                                                    \
    switch (N) {                                                                                   \
    case 1: { constexpr int NC = 1; CALL; } break;                                                 \
    case 2: { constexpr int NC = 2; CALL; } break;                                                 \
    case 3: { constexpr int NC = 3; CALL; } break;                                                 \
    case 4: { constexpr int NC = 4; CALL; } break;                                                 \
    case 5: { constexpr int NC = 5; CALL; } break;                                                 \
    case 6: { constexpr int NC = 6; CALL; } break;                                                 \
    case 7: { constexpr int NC = 7; CALL; } break;                                                 \
    case 8: { constexpr int NC = 8; CALL; } break;                                                 \
    default: return hipErrorInvalidValue;                                                          \
    }

// Tunable: non-zero keeps Q8_0H weights on the VALU kernel (for comparisons).
RT_TUNABLE(g_gemv_disable_mfma, 0);

// Returns hipErrorNotSupported when the operands do not meet the alignment the
// streaming kernels assume; the caller then takes the tiled GEMM, which has no
// such requirement.
// A few more activation vectors than one streaming launch takes: one launch per 16 of them.  Each
// launch streams the weights again (after the first mostly from the Infinity Cache), which still beats
// the tiled kernels while the MFMA work is small: measured at 8192 x 3072 Q4_K, 17 / 32 vectors take
// 12 / 14 us (48: 21) against 15 us tiled: the tiled kernels take over from 33.  (10240 x 2560 Q8_0H:
// 18 / 20 us, 48 / 64 vectors 29 / 38.)
hipError_t launch_gemv_chunked(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                               hipStream_t stream, const DeviceInfo &dev) {
    const bool q8 = p.a_dt == RT_Q8_0H, q4 = p.a_dt == RT_Q4_K;
    if ((!q8 && !q4) || p.act_dt != RT_F16 || g_gemv_disable_mfma) return hipErrorNotSupported;
    if (p.N <= 16 || p.N > 32) return hipErrorNotSupported;
    // Q8_0H weights with enough rows that their 64 x 64 tiles give half of the compute units a workgroup are faster on
    // the tiled kernel (10240 x 2560: 15.7 / 16.2 us at 17 / 32 vectors); with fewer rows (2560 x 2560: 40 tiles) the
    // streaming launches stay ahead
    if (q8 && p.K % 256 == 0 && p.stacks == 1 && (p.M + 63) / 64 >= dev.num_cus / 2) return hipErrorNotSupported;
    for (int64_t j0 = 0; j0 < p.N; j0 += 16) {
        Problem c = p;
        c.N = p.N - j0 < 16 ? p.N - j0 : 16;
        c.kernel = q8 ? RT_KERNEL_GEMV_Q8 : RT_KERNEL_GEMV_Q4K;
        const half_t *Bc = (const half_t *)B + j0 * p.b_js;
        half_t *oc = (half_t *)out + j0 * p.o_js;
        const half_t *bc = bias && !p.bias_on_rows ? (const half_t *)bias + j0 : (const half_t *)bias;
        const hipError_t e = q8 ? launch_gemv_q8h_mfma(c, A, Bc, bc, oc, stream, dev) : launch_gemv_q4k_mfma(c, A, Bc, bc, oc, stream, dev);
        // a shape or alignment the kernel declines is declined on the first chunk (the later ones share
        // its strides and alignment); whatever a failed attempt wrote is overwritten by the kernel that runs instead
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_gemv(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                       hipStream_t stream, const DeviceInfo &dev) {
    if (p.kernel == RT_KERNEL_GEMV_Q8 && p.a_dt == RT_Q8_0H && !g_gemv_disable_mfma) {
        // f16 activations, one or two vectors: the row-streaming kernel; three or four: the row-streaming kernel on
        // the 4x4x4 matrix instruction; then the matrix-core kernel; shapes all of them decline fall through
        hipError_t e = launch_gemv_q8h_rowdot(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
        e = launch_gemv_q8h_quad(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
        e = launch_gemv_q8h_mfma(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
    }
    if (p.kernel == RT_KERNEL_GEMV_Q4K) {
        // one vector: the row-streaming kernel; then the matrix-core kernel
        hipError_t e = launch_gemv_q4k_rowdot(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
        e = launch_gemv_q4k_mfma(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
    }
    if (p.kernel == RT_KERNEL_GEMV_FLOAT) { // up to four vectors, rows of whole 16-byte vectors: the row-streaming kernel
        hipError_t e = launch_gemv_float_rowdot(p, A, B, bias, out, stream, dev);
        if (e != hipErrorNotSupported) return e;
        // 5..8 vectors against an f16 weight with enough rows that 64-row tiles give half of the compute units a
        // workgroup: the weight-streaming GEMM, or the tiled kernel's 64 x 64 tiles (10240 x 2560, weights from HBM:
        // 12.7 / 16 us against 19 / 24 / 26 us at 5 / 7 / 8 vectors here); the conditions are the ones under which
        // the tiled kernel takes the product
        if (p.a_dt == RT_F16 && p.act_dt == RT_F16 && p.N >= 5 && p.stacks == 1 && p.K > 256 && p.K % 64 == 0 &&
            (p.M + 63) / 64 >= dev.num_cus / 2 && p.a_ks == 1 && p.b_ks == 1 && aligned16(A) && aligned16(B) &&
            (p.a_rs * 2) % 16 == 0 && (p.b_js * 2) % 16 == 0 && !(p.o_js == 1 && p.o_is != 1))
            // (a row-major output would make the tiled kernel exchange the operands, and with the weight as its
            // activation side it declines: such a product stays here)
            return hipErrorNotSupported;
    }
    if (p.N < 1 || p.N > kGemvMaxCols || p.stacks > 65535) return hipErrorNotSupported;
    const int64_t esz = p.act_dt == RT_F16 ? 2 : 4;
    GemvArgs g{};
    g.A = (const uint8_t *)A;
    g.X = B;
    g.bias = bias;
    g.out = out;
    g.M = p.M, g.K = p.K;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.a_bs = p.a_bs, g.a_rs = p.a_rs;
    g.b_bs = p.b_bs, g.b_js = p.N == 1 ? 0 : p.b_js; // a single vector has no column stride
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;

    const int64_t row_blocks = (p.M + kGemvWaves - 1) / kGemvWaves;
    const int64_t cap = (int64_t)dev.num_cus * 16;
    dim3 grid((unsigned)(row_blocks < cap ? row_blocks : cap), (unsigned)p.stacks);
    // x rows must be 16-byte aligned for the vector loads.
    const bool x_ok = aligned16(B) && (g.b_js * esz) % 16 == 0 && (p.b_bs * esz) % 16 == 0;

    switch (p.kernel) {
    case RT_KERNEL_GEMV_Q8: {
        if (!x_ok || !aligned16(A) || p.K % 32 != 0) return hipErrorNotSupported;
        const uint64_t numel = (uint64_t)p.a_stack * p.M * p.K;
        g.scales = (const uint8_t *)A + rt_q8_0_scale_offset(numel);
        RT_DISPATCH_NC(p.N, launch_q8<NC>(p.act_dt, grid, stream, g));
        break;
    }
    case RT_KERNEL_GEMV_Q4K: {
        if (!x_ok || !aligned16(A) || p.K % 256 != 0) return hipErrorNotSupported;
        RT_DISPATCH_NC(p.N, launch_q4k<NC>(grid, stream, g));
        break;
    }
    case RT_KERNEL_GEMV_FLOAT: {
        const bool vec = x_ok && aligned16(A) && (p.a_rs * esz) % 16 == 0;
        RT_DISPATCH_NC(p.N, launch_float<NC>(p.act_dt, vec, grid, stream, g));
        break;
    }
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace rt
