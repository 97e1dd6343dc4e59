// Streaming Q4_K GEMV on the matrix cores, for 1..16 activation vectors.
//
// A Q4_K super-block covers 256 values of K for one weight row: 144 bytes
// {d f16, dmin f16, scales[12] (8 x 6-bit scale, 8 x 6-bit min), qs[128]}, and a
// weight is  w = d * sc_j * q - dmin * mn_j  for sub-block j of 32.  Per super-block
//
//   y += d * sum_j sum_{k in j} x_k * (sc_j * q_k)  -  dmin * sum_j mn_j * (sum_{k in j} x_k)
//
// Both inner sums run on v_mfma_f32_16x16x32_f16 with exact operands: sc_j * q_k is an
// integer below 1024 (exact in f16), so the eight sub-blocks of a super-block chain
// through one accumulator and d is applied once, in f32; the second term is one more
// MFMA whose K axis holds the eight sub-block sums of x split into f16 high and low
// parts (exact to 2^-22) against the integer mins.  No weight is ever rounded.
//
// The block stream is read once, straight from HBM into registers: a lane issues three
// 16-byte loads per super-block (the header and two pieces of qs) for row n = lane % 16;
// v_permlane32_swap regroups the nibbles so that each MFMA sees exactly one sub-block.
// A workgroup owns 16 rows, each wavefront one super-block column; activations pass
// through a wavefront-private LDS region; the K slices are summed through LDS at the end.
//
// The arithmetic is ggml's dequantize_row_q4_K (the reference holds only the block
// struct, crates/ratchet-loader/src/k_quants.rs:94-103).
#include "device_common.h"

namespace rt {

struct GemvQ4kArgs {
    const uint8_t *blocks; // [rows][K/256] super-blocks of 144 bytes
    const half_t *X;
    const half_t *bias;
    half_t *out;
    int64_t M, K;
    int NC;     // activation vectors (1..16)
    int nsb;    // super-blocks per row
    int rows_wg; // weight rows per workgroup: at most 16 * RG, a multiple of 8
    int64_t a_stack, b_stack;
    int64_t b_bs, b_js;
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
};

constexpr int kQ4kXPad = 8;

__device__ __forceinline__ int q4k_x_koff(int g) { return 16 * (g & 1) + 8 * (g >> 1); }

// 4 bytes holding integers 0..255 -> two half2 holding the same integers (1024 + b, minus 1024).
__device__ __forceinline__ void q4k_bytes_to_half(uint32_t v, half2_t &lo, half2_t &hi) {
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u);
    const half2_t k = {(half_t)1024.0f, (half_t)1024.0f};
    lo = __builtin_bit_cast(half2_t, a) - k;
    hi = __builtin_bit_cast(half2_t, b) - k;
}

// 8 nibble-bytes (two dwords, each byte 0..15) -> 8 halfs holding sc * nibble, exactly:
// fma(1024 + q, sc, -1024 * sc) rounds once and q * sc < 1024 is representable.
__device__ __forceinline__ half8_t q4k_scaled(uint32_t v0, uint32_t v1, half_t sc) {
    const half2_t s2 = {sc, sc};
    const half2_t n2 = {(half_t)(-1024.0f * (float)sc), (half_t)(-1024.0f * (float)sc)};
    half2_t r[4];
    const uint32_t w[2] = {v0, v1};
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const half2_t a = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, w[i], 0x04010400u));
        const half2_t b = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, w[i], 0x04030402u));
        r[2 * i] = __builtin_elementwise_fma(a, s2, n2);
        r[2 * i + 1] = __builtin_elementwise_fma(b, s2, n2);
    }
    return half8_t{r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
}

// FAST is the regular case, which the launcher recognises: one stack, M a multiple of 16, one
// wavefront per super-block column, exactly NCT vectors, all offsets below 2^31.  Its prologue
// is a handful of 32-bit operations; the kernel is bound by instruction issue (several
// wavefronts per SIMD run the same instructions at the same time), so that shows.
// RG: 16-row groups per workgroup (1 or 2).  They share the staged activations; with 9..16 vectors those leave room
// for one workgroup per compute unit, and two row groups then cover 8192 rows in one round of 256 workgroups.
// SBW: super-blocks per wavefront (1, or 2 for K above 4096: wavefront w takes super-blocks w and w + nwaves, all of
// whose loads are issued before the first is consumed).
template <int NCT, bool FAST, int RG, int SBW>
__global__ __launch_bounds__(1024) void gemv_q4k_mfma_kernel(GemvQ4kArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int XROW = 256 + kQ4kXPad; // halfs per staged activation row (one super-block of K)
    const int t = threadIdx.x, lane = t & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6); // wave-uniform: addresses below stay scalar
    const int NC = FAST ? NCT : g.NC;
    half_t *xs = (half_t *)smem + (size_t)wave * NC * (XROW + 16); // [NC][XROW] then [NC][2][8] sub-block sums
    half_t *sxs = xs + (size_t)NC * XROW;
    float *psum = (float *)((half_t *)smem + (size_t)nwaves * NC * (XROW + 16)); // [nwaves][RG][256]

    const int n = lane & 15, grp = lane >> 4;
    const int64_t s = FAST ? 0 : blockIdx.y;
    const int64_t sa = g.a_stack == 1 ? 0 : s, sb = g.b_stack == 1 ? 0 : s;
    // workgroups go round the eight XCDs in turn: every XCD takes one run of consecutive rows, so that a line of the
    // output is written in one XCD's L2 and leaves it whole when the kernel ends
    const uint32_t nwg = gridDim.x;
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const int64_t row0 = (int64_t)wg * (FAST ? 16 * RG : g.rows_wg);
    // 1. this wave's 256 activations per vector and super-block: 32 16-byte vectors per row
    constexpr int XL = (NCT * 32 + 63) / 64;
    const int nvec = NC * 32;
    uint4_t xv_[SBW][XL], hdr__[SBW][RG], qa__[SBW][RG], qb__[SBW][RG];
    uint32_t bias_raw_[RG];
    bool live_[SBW];
#pragma unroll
    for (int pass = 0; pass < SBW; pass++) {
    uint4_t (&xv)[XL] = xv_[pass], (&hdr_)[RG] = hdr__[pass], (&qa_)[RG] = qa__[pass], (&qb_)[RG] = qb__[pass];
    const bool live = FAST || wave + pass * nwaves < g.nsb; // padding waves (nwaves * SBW > nsb) contribute zero
    live_[pass] = live;
    const int sbi = live ? wave + pass * nwaves : 0;
    if constexpr (FAST) {
        const half_t *xg = g.X + sbi * 256;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const uint32_t v = min(i * 64 + lane, NCT * 32 - 1);
            xv[i] = *(const uint4_t *)(xg + ((v >> 5) * (uint32_t)g.b_js + 8u * (v & 31)));
        }
        asm volatile("" ::: "memory");
        // 2. the block stream: a wave-uniform base plus a 32-bit lane offset
        const uint8_t *base = g.blocks + ((uint32_t)row0 * (uint32_t)g.nsb + (uint32_t)sbi) * 144u;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t loff = (uint32_t)(16 * rg + n) * (uint32_t)g.nsb * 144u;
            hdr_[rg] = *(const uint4_t *)(base + loff);
            qa_[rg] = *(const uint4_t *)(base + (loff + 16u * grp) + 16);
            qb_[rg] = *(const uint4_t *)(base + (loff + 16u * grp) + 80);
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t bias_i = g.bias_on_rows ? (uint32_t)row0 + 16 * rg + (t & 15) : (uint32_t)min((t >> 4) & 15, NCT - 1);
            bias_raw_[rg] = *(const uint16_t *)(g.has_bias ? (const void *)(g.bias + bias_i) : (const void *)base);
        }
        asm volatile("" ::: "memory");
    } else {
        const half_t *xg = g.X + sb * g.b_bs + (int64_t)sbi * 256;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int v = min(i * 64 + lane, nvec - 1);
            xv[i] = *(const uint4_t *)(xg + (v >> 5) * g.b_js + 8 * (v & 31));
        }
        asm volatile("" ::: "memory");
        // 2. the block stream: header + two 16-byte pieces of qs for row n
        const uint8_t *blk0 = g.blocks;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            // rows past the workgroup's or the matrix's end duplicate the last one; never stored
            const int64_t row = min(row0 + min(16 * rg + n, g.rows_wg - 1), g.M - 1);
            const uint8_t *blk = g.blocks + ((sa * g.M + row) * g.nsb + sbi) * 144;
            if (rg == 0) blk0 = blk;
            hdr_[rg] = *(const uint4_t *)blk;
            qa_[rg] = *(const uint4_t *)(blk + 16 + 16 * grp);
            qb_[rg] = *(const uint4_t *)(blk + 80 + 16 * grp);
        }
        // The epilogue's bias value, fetched behind everything else so its latency is hidden.  The load is
        // unconditional (without a bias it re-reads the block header and the value is dropped): a branch
        // here makes the compiler wait for every outstanding load right after issuing this one.
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const int64_t bias_i = g.bias_on_rows ? min(row0 + min(16 * rg + (t & 15), g.rows_wg - 1), g.M - 1) : (int64_t)min((t >> 4) & 15, g.NC - 1);
            bias_raw_[rg] = *(const uint16_t *)(g.has_bias ? (const void *)(g.bias + bias_i) : (const void *)blk0);
        }
        asm volatile("" ::: "memory");
    }

    }
#pragma unroll
    for (int pass = 0; pass < SBW; pass++) {
    const uint4_t (&xv)[XL] = xv_[pass], (&hdr_)[RG] = hdr__[pass], (&qa_)[RG] = qa__[pass], (&qb_)[RG] = qb__[pass];
    const bool live = live_[pass];
    // 3. activations -> LDS, and the sums of x over each sub-block of 32 as f16 high + low parts
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int v = i * 64 + lane;
        const half8_t h = __builtin_bit_cast(half8_t, xv[i]);
        const half2_t one2 = {(half_t)1, (half_t)1};
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) sum = __builtin_amdgcn_fdot2(half2_t{h[2 * e], h[2 * e + 1]}, one2, sum, false);
        sum += wave_dpp<0xB1>(sum); // quad_perm [1,0,3,2]: four consecutive lanes hold the four vectors of a sub-block
        sum += wave_dpp<0x4E>(sum); // quad_perm [2,3,0,1]
        if (v < nvec) {
            const int j = v >> 5, kv = v & 31;
            *(uint4_t *)(xs + j * XROW + 8 * kv) = xv[i];
            if ((kv & 3) == 0) {
                const half_t hi = (half_t)sum;
                const half_t lo = (half_t)(sum - (float)hi);
                sxs[j * 16 + (kv >> 2)] = hi;
                sxs[j * 16 + 8 + (kv >> 2)] = lo;
            }
        }
    }
    asm volatile("" ::: "memory"); // the reads below are by the same wavefront; DS operations complete in order

    const int xj = min(n, NC - 1); // lanes beyond NC re-read a valid row; their outputs are dropped
    const half_t *xrow = xs + xj * XROW + q4k_x_koff(grp);
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        const uint4_t hdr = hdr_[rg], qa = qa_[rg], qb = qb_[rg];
        // 4. unpack the 6-bit scales and mins (ggml get_scale_min_k4), four per dword
        const half2_t dm = __builtin_bit_cast(half2_t, hdr[0]);
        const float d = live ? (float)dm[0] : 0.f, dmin = live ? (float)dm[1] : 0.f;
        const uint32_t S0 = hdr[1], S1 = hdr[2], S2 = hdr[3];
        const uint32_t sc03 = S0 & 0x3F3F3F3Fu, mn03 = S1 & 0x3F3F3F3Fu;
        const uint32_t sc47 = (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u);
        const uint32_t mn47 = ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u);
        half2_t sch[4], mnh[4];
        q4k_bytes_to_half(sc03, sch[0], sch[1]);
        q4k_bytes_to_half(sc47, sch[2], sch[3]);
        q4k_bytes_to_half(mn03, mnh[0], mnh[1]);
        q4k_bytes_to_half(mn47, mnh[2], mnh[3]);
        auto scale_of = [&](int j) -> half_t { return sch[j >> 1][j & 1]; };

        // 5. regroup so that every lane holds 8 nibbles of each of the 8 sub-blocks:
        //    part A of a piece = sub-blocks (low, high nibbles), part B = the next two
        float4_t P = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int piece = 0; piece < 2; piece++) {
            const uint4_t q = piece == 0 ? qa : qb;
            auto p0 = __builtin_amdgcn_permlane32_swap(q[0], q[2], false, false);
            auto p1 = __builtin_amdgcn_permlane32_swap(q[1], q[3], false, false);
#pragma unroll
            for (int part = 0; part < 2; part++) {
                const uint32_t v0 = p0[part], v1 = p1[part];
                const int jlo = piece * 4 + part * 2, jhi = jlo + 1; // sub-blocks of the low / high nibbles
                const half8_t blo = q4k_scaled(v0 & 0x0F0F0F0Fu, v1 & 0x0F0F0F0Fu, scale_of(jlo));
                const half8_t bhi = q4k_scaled((v0 >> 4) & 0x0F0F0F0Fu, (v1 >> 4) & 0x0F0F0F0Fu, scale_of(jhi));
                const half8_t alo = __builtin_bit_cast(half8_t, *(const uint4_t *)(xrow + 32 * jlo));
                const half8_t ahi = __builtin_bit_cast(half8_t, *(const uint4_t *)(xrow + 32 * jhi));
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, blo, P, 0, 0, 0);
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bhi, P, 0, 0, 0);
            }
        }
        // 6. the min term: K slots 0..7 = high parts of the 8 sub-block sums, 8..15 = low parts, rest zero
        half8_t bm = {mnh[0][0], mnh[0][1], mnh[1][0], mnh[1][1], mnh[2][0], mnh[2][1], mnh[3][0], mnh[3][1]};
        if (grp >= 2) bm = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        const half8_t am = __builtin_bit_cast(half8_t, *(const uint4_t *)(sxs + xj * 16 + 8 * (grp & 1)));
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
        const float4_t T = __builtin_amdgcn_mfma_f32_16x16x32_f16(am, bm, zero, 0, 0, 0);
        // a lane's result register r is activation vector 4 * grp + r: only those that exist are summed
        constexpr int NR = NCT < 4 ? NCT : 4;
        if (NCT >= 16 || 4 * grp < NCT) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                float &ps = psum[(wave * RG + rg) * 256 + (4 * grp + r) * 16 + n];
                ps = fmaf(-dmin, T[r], d * P[r]) + (pass == 0 ? 0.f : ps);
            }
        }
    }
    if (SBW > 1) asm volatile("" ::: "memory"); // the next pass restages the activations behind this pass's reads (DS operations complete in order)
    }

    // 7. sum the K slices
    __syncthreads();
    if (t < 16 * NCT) {
        const int j = t >> 4;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            float v = 0.f;
            for (int w2 = 0; w2 < nwaves; w2++) v += psum[(w2 * RG + rg) * 256 + t];
            const int64_t i = row0 + 16 * rg + (t & 15);
            if (FAST || (j < g.NC && i < g.M && 16 * rg + (t & 15) < g.rows_wg))
                g.out[s * g.o_bs + i * g.o_is + j * g.o_js] = (half_t)rt_act(v + (g.has_bias ? (float)__builtin_bit_cast(half2_t, bias_raw_[rg])[0] : 0.f), g.act);
        }
    }
}

template <int NCT, bool FAST, int RG, int SBW = 1>
static hipError_t launch_q4k_kernel(dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvQ4kArgs &g) {
    if (lds > 48 * 1024) {
        const hipError_t e = ensure_lds_limit<&gemv_q4k_mfma_kernel<NCT, FAST, RG, SBW>>();
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemv_q4k_mfma_kernel<NCT, FAST, RG, SBW>), grid, dim3(nwaves * 64), lds, st, g);
    return hipGetLastError();
}

template <int NCT>
static hipError_t launch_q4k_one(int rg, int sbw, dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvQ4kArgs &g) {
    const bool regular = grid.y == 1 && g.a_stack == 1 && g.b_stack == 1 && g.M % (16 * rg) == 0 && g.rows_wg == 16 * rg &&
                         g.NC == NCT && g.nsb == nwaves * sbw && g.M * g.nsb * 144 < (int64_t(1) << 31) &&
                         (int64_t)g.NC * g.b_js < (int64_t(1) << 30);
    if constexpr (NCT <= 8) { // two super-blocks per wavefront: K above 4096
        if (sbw == 2) {
            if (rg != 1) return hipErrorInvalidValue;
            return regular ? launch_q4k_kernel<NCT, true, 1, 2>(grid, nwaves, lds, st, g) : launch_q4k_kernel<NCT, false, 1, 2>(grid, nwaves, lds, st, g);
        }
    }
    if (sbw != 1) return hipErrorNotSupported;
    if constexpr (NCT == 16) { // two row groups are only dealt where 9..16 vectors leave room for one workgroup per compute unit
        if (rg == 2) return regular ? launch_q4k_kernel<NCT, true, 2>(grid, nwaves, lds, st, g) : launch_q4k_kernel<NCT, false, 2>(grid, nwaves, lds, st, g);
    }
    if (rg != 1) return hipErrorInvalidValue;
    if (regular) return launch_q4k_kernel<NCT, true, 1>(grid, nwaves, lds, st, g);
    return launch_q4k_kernel<NCT, false, 1>(grid, nwaves, lds, st, g);
}

// Tunable: non-zero keeps Q4_K weights off this kernel (for comparisons).
RT_TUNABLE(g_gemv_q4k_disable_mfma, 0);
// Tunable: 1 or 2 forces that many 16-row groups per workgroup (0 = by residency, see the launcher).
RT_TUNABLE(g_gemv_q4k_mfma_rg, 0);

// Q4_K weights, f16 activations, 1..16 vectors, K a multiple of 256 and at most 4096 (8192 with up to 8 vectors).
// hipErrorNotSupported means another kernel must run.
hipError_t launch_gemv_q4k_mfma(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemv_q4k_disable_mfma) return hipErrorNotSupported;
    if (p.a_dt != RT_Q4_K || p.act_dt != RT_F16 || p.N < 1 || p.N > 16 || p.K % 256 != 0 || p.K < 256 || p.K > (p.N <= 8 ? 8192 : 4096))
        return hipErrorNotSupported;
    if (p.stacks > 65535 || p.b_ks != 1) return hipErrorNotSupported;
    const int64_t bjs = p.N == 1 ? 0 : p.b_js;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (bjs * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    GemvQ4kArgs g{};
    g.blocks = (const uint8_t *)A, g.X = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    g.M = p.M, g.K = p.K, g.NC = (int)p.N, g.nsb = (int)(p.K / 256);
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.b_bs = p.b_bs, g.b_js = bjs;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    if (p.has_bias && ((uintptr_t)bias & 1u)) return hipErrorNotSupported;
    const int sbw = g.nsb > 16 ? 2 : 1;       // K above 4096: two super-blocks per wavefront
    const int nwaves = g.nsb < 4 ? 4 : (g.nsb + sbw - 1) / sbw; // the final sum uses 256 threads
    // Rows per workgroup: 16, unless the activations' LDS (9..16 vectors) leaves one workgroup per compute unit and
    // the 16-row workgroups would run in rounds; then every compute unit gets one workgroup with its share of the
    // rows, up to 32 (8192 rows, 16 vectors: 512 workgroups in two rounds 9.3 us -> 256 in one 7.7 us).
    const size_t lds_x = (size_t)nwaves * g.NC * (256 + kQ4kXPad + 16) * 2;
    int rg = 1, rows_wg = 16;
    if (g.NC > 8 && p.stacks == 1 && 2 * (lds_x + (size_t)nwaves * 1024) > 160 * 1024 && (p.M + 15) / 16 > dev.num_cus) {
        const int64_t per = ((p.M + dev.num_cus - 1) / dev.num_cus + 7) & ~(int64_t)7;
        if (per <= 32) rows_wg = (int)per, rg = (rows_wg + 15) / 16;
    }
    if (g_gemv_q4k_mfma_rg > 0 && g.NC > 8) rg = g_gemv_q4k_mfma_rg, rows_wg = 16 * rg;
    g.rows_wg = rows_wg;
    const size_t lds = lds_x + (size_t)nwaves * rg * 1024;
    if (lds > 160 * 1024) return hipErrorNotSupported;
    const int64_t groups = (p.M + rows_wg - 1) / rows_wg;
    if (groups > 0x7fffffff) return hipErrorNotSupported;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    if (g.NC <= 1) return launch_q4k_one<1>(rg, sbw, grid, nwaves, lds, stream, g);
    if (g.NC <= 2) return launch_q4k_one<2>(rg, sbw, grid, nwaves, lds, stream, g);
    if (g.NC <= 4) return launch_q4k_one<4>(rg, sbw, grid, nwaves, lds, stream, g);
    if (g.NC <= 8) return launch_q4k_one<8>(rg, sbw, grid, nwaves, lds, stream, g);
    return launch_q4k_one<16>(rg, sbw, grid, nwaves, lds, stream, g);
}

} // namespace rt
