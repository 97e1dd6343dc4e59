// Row-streaming Q4_K GEMV for one activation vector (the decode step).
//
// A Q4_K super-block covers 256 values of K for one weight row: 144 bytes = nine 16-byte vectors,
// the header {d f16, dmin f16, scales[12] (8 x 6-bit scale, 8 x 6-bit min)} and eight pieces of
// qs[128]; a weight is  w = d * sc_j * q - dmin * mn_j  for sub-block j of 32.  Byte i of piece p
// holds, in its low nibble, the weight at 64 * (p / 2) + 16 * (p % 2) + i of the super-block and in
// its high nibble the one 32 further on.
//
// A wavefront owns one row and reads it as what it is in memory, a run of 9 * K / 256 vectors:
// lane l takes vector 64 * step + l, so every load instruction fetches 1 KiB of consecutive bytes,
// each 128-byte line once, non-temporal, and all of a row's loads are issued before the first
// is consumed.  One lane in nine holds a header: those lanes pass theirs through a
// wavefront-private LDS slot to the eight lanes that hold the block's pieces (LDS operations of one
// wavefront complete in order; no barrier).  A piece's lane turns its nibbles into sc * q exactly
// (fma(1024 + q, sc, -1024 * sc) in f16: q * sc < 1024), multiplies them with the 32 activations at
// the same K positions with v_dot2_f32_f16, and applies d and dmin * mn * (sum of those activations)
// in f32.  The activations and their sums over runs of 16 are staged once per workgroup in LDS.
// The 64 partial sums of a row meet in six DPP additions; nothing is summed across wavefronts.
//
// This form needs about 210 vector instructions per row of 3072 (40 per 32 weights for nibbles -> f16 -> dot
// products, the rest scale decoding and bookkeeping) and is bound by them: at 8192 x 3072 it takes 5.7 us where
// the matrix-core kernel (kernels_gemv_q4k_mfma.hip: 16 rows per workgroup, a super-block column per wavefront)
// takes 5.4, at 8192 x 4096 7.2 against 6.4.  It therefore serves the K above 4096 that kernel does not
// take: 3072 x 8192 in 6.7 us (2.1 TB/s) where the one-load-at-a-time kernel of kernels_gemv.hip took 12.8.
//
// The arithmetic is ggml's dequantize_row_q4_K (the reference holds only the block struct,
// crates/ratchet-loader/src/k_quants.rs:94-103); role in the reference: ops/gemv.rs:333-558.
#include "device_common.h"

namespace rt {

struct GemvQ4kRowdotArgs {
    const uint8_t *blocks;  // [rows][K / 256] super-blocks of 144 bytes
    const half_t *X;
    const half_t *bias;     // never null: without a bias the activations, with the bias stride 0, and the value is dropped
    half_t *out;
    uint32_t M;             // weight rows
    uint32_t nsb;           // super-blocks per row
    uint32_t bias_rs;       // 1: a bias per weight row, 0: one for the vector
    int64_t o_is;
    int64_t a_ss, x_ss, o_ss; // per stack: bytes of blocks, activation elements, output elements
    int has_bias, act;
};

// four bytes b0..b3 -> (b0, b1), (b2, b3) as the f16 bit patterns 0x00bb: the subnormals b * 2^-24, which v_dot2_f32_f16
// multiplies like any other f16 (checked on the device); the 2^24 goes into the f32 scale
__device__ __forceinline__ void q4kr_bytes(uint32_t v, half2_t &lo, half2_t &hi) {
    lo = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, v, 0x04010400u));
    hi = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, v, 0x04030402u));
}

// STEPS: 64-vector steps per row; WAVES: wavefronts per workgroup; R: rows per wavefront, which share the lane's
// activations, block and piece numbers (the lane sits at the same place in each of its rows).
template <int STEPS, int WAVES, int R>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_rowdot_kernel(GemvQ4kRowdotArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int THREADS = WAVES * 64, ROWS = WAVES * R;
    const int t = threadIdx.x, lane = t & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t nsb = g.nsb, nvec = 9u * nsb, K = 256u * nsb;
    half_t *xs = (half_t *)smem;                          // [K] activations
    float *sx = (float *)(smem + 2 * (size_t)K);          // [K / 16] their sums over runs of 16
    uint4_t *hdr = (uint4_t *)(smem + 2 * (size_t)K + K / 4) + wave * (R * nsb); // [WAVES][R][nsb] block headers
    // consecutive rows per XCD: an output line is written in one L2
    const uint32_t nwg = gridDim.x;
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t row0 = wg * ROWS + wave * R;            // this wavefront's first row
    const uint8_t *abase = g.blocks;
    const half_t *xg = g.X;
    half_t *obase = g.out;
    if (blockIdx.y != 0) {
        asm volatile("" ::: "memory"); // keeps this a branch: one product pays nothing for the terms of a stack
        const int64_t s = blockIdx.y;
        abase += s * g.a_ss, xg += s * g.x_ss, obase += s * g.o_ss;
    }

    // 1. the activations: K / 8 vectors of eight, staged by the whole workgroup
    constexpr int XV = (STEPS * 64 * 32 / 9 + THREADS - 1) / THREADS; // K / 8 = 32 * nsb vectors, nsb <= 64 * STEPS / 9
    const uint32_t nxv = K / 8;
    uint4_t xv[XV];
#pragma unroll
    for (int i = 0; i < XV; i++) xv[i] = *(const uint4_t *)(xg + 8 * min((uint32_t)(i * THREADS + t), nxv - 1));
    asm volatile("" ::: "memory"); // keep the loads in this order
    // 2. the rows (those past the end repeat the last one; never stored): only the last step can be short, its
    //    spare lanes re-read the row's end
    const uint32_t il = min((uint32_t)(64 * (STEPS - 1) + lane), nvec - 1);
    uint4_t w[R][STEPS];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint8_t *rp = abase + (uint64_t)min(row0 + r, g.M - 1) * (144u * nsb);
#pragma unroll
        for (int st = 0; st < STEPS - 1; st++) w[r][st] = __builtin_nontemporal_load((const uint4_t *)(rp + 16 * (64 * st + lane)));
        w[r][STEPS - 1] = __builtin_nontemporal_load((const uint4_t *)(rp + 16 * il));
    }
    asm volatile("" ::: "memory");
    // 3. the epilogue's bias, unconditional (a branch here would wait for every load above)
    half_t braw[R];
#pragma unroll
    for (int r = 0; r < R; r++) braw[r] = g.bias[(size_t)(min(row0 + r, g.M - 1) * g.bias_rs)];
    asm volatile("" ::: "memory");
    half_t *op = obase + (int64_t)row0 * g.o_is;
    int64_t ois = g.o_is;
    asm volatile("" : "+v"(op), "+s"(ois));
    // 4. activations and their sums over 16 -> LDS; the barrier waits for the LDS writes, not for the rows
#pragma unroll
    for (int i = 0; i < XV; i++) {
        const uint32_t v = i * THREADS + t;
        const half8_t h = __builtin_bit_cast(half8_t, xv[i]);
        const half2_t one2 = {(half_t)1, (half_t)1};
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) sum = __builtin_amdgcn_fdot2(half2_t{h[2 * e], h[2 * e + 1]}, one2, sum, false);
        sum += wave_dpp<0xB1>(sum); // quad_perm [1,0,3,2]: the neighbour's eight
        if (v < nxv) {
            *(uint4_t *)(xs + 8 * v) = xv[i];
            if ((v & 1) == 0) sx[v >> 1] = sum;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // 5. which block and piece this lane's vector of every step is; its activations, held while the rows are on their way
    uint32_t blk[STEPS], sh[STEPS];
    bool live[STEPS], upper[STEPS], ishdr[STEPS];
    uint4_t xa[STEPS][2], xb[STEPS][2];
    float sxa[STEPS], sxb[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        const uint32_t i = st == STEPS - 1 ? il : 64u * st + lane;
        const bool inrow = st < STEPS - 1 || (uint32_t)(64 * (STEPS - 1) + lane) < nvec;
        blk[st] = i / 9u;
        const uint32_t v = i - 9u * blk[st];
        ishdr[st] = inrow && v == 0;
        live[st] = inrow && v != 0;
        const uint32_t piece = v == 0 ? 0u : v - 1, j = piece >> 1;
        sh[st] = 16u * (j & 1), upper[st] = j >= 2; // where the two sub-blocks' 6-bit fields sit in the scale words
        const uint32_t ka = 256u * blk[st] + 64u * j + 16u * (piece & 1);
        xa[st][0] = *(const uint4_t *)(xs + ka), xa[st][1] = *(const uint4_t *)(xs + ka + 8);
        xb[st][0] = *(const uint4_t *)(xs + ka + 32), xb[st][1] = *(const uint4_t *)(xs + ka + 40);
        sxa[st] = sx[ka >> 4], sxb[st] = sx[(ka >> 4) + 2];
    }
    __builtin_amdgcn_sched_barrier(0);
    // 6. headers to the lanes of their blocks
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int st = 0; st < STEPS; st++)
            if (ishdr[st]) hdr[r * nsb + blk[st]] = w[r][st];
    __builtin_amdgcn_wave_barrier();
    // 7. the pieces
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            const uint4_t hd = hdr[r * nsb + blk[st]];
            // ggml get_scale_min_k4 for sub-blocks 2 * (piece / 2) and + 1: the two share a 16-bit run of each scale word
            const half2_t dm = __builtin_bit_cast(half2_t, hd[0]);
            const uint32_t w1 = (hd[1] >> sh[st]) & 0xffffu, w2 = (hd[2] >> sh[st]) & 0xffffu, w3 = (hd[3] >> sh[st]) & 0xffffu;
            const uint32_t sc2 = upper[st] ? ((w3 & 0x0F0Fu) | ((w1 >> 2) & 0x3030u)) : (w1 & 0x3F3Fu);
            const uint32_t mn2 = upper[st] ? (((w3 >> 4) & 0x0F0Fu) | ((w2 >> 2) & 0x3030u)) : (w2 & 0x3F3Fu);
            float pa = 0.f, pb = 0.f; // 2^-24 * sum q x over the low nibbles, 2^-20 * the same over the high nibbles
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t q = w[r][st][d];
                half2_t l0, l1, h0, h1;
                q4kr_bytes(q & 0x0F0F0F0Fu, l0, l1);
                q4kr_bytes(q & 0xF0F0F0F0u, h0, h1);
                const uint32_t x0 = xa[st][d >> 1][2 * (d & 1)], x1 = xa[st][d >> 1][2 * (d & 1) + 1];
                const uint32_t y0 = xb[st][d >> 1][2 * (d & 1)], y1 = xb[st][d >> 1][2 * (d & 1) + 1];
                pa = __builtin_amdgcn_fdot2(l0, __builtin_bit_cast(half2_t, x0), pa, false);
                pa = __builtin_amdgcn_fdot2(l1, __builtin_bit_cast(half2_t, x1), pa, false);
                pb = __builtin_amdgcn_fdot2(h0, __builtin_bit_cast(half2_t, y0), pb, false);
                pb = __builtin_amdgcn_fdot2(h1, __builtin_bit_cast(half2_t, y1), pb, false);
            }
            // every product below is exact for a one-hot activation vector, and the last operation rounds once:
            // the result is then the dequantized weight, bit for bit
            const float d24 = (float)dm[0] * 16777216.0f, dmin = (float)dm[1];
            const float sa = (float)(sc2 & 0xffu), sb16 = (float)(sc2 >> 8) * 0.0625f;
            const float ma = (float)(mn2 & 0xffu), mb = (float)(mn2 >> 8);
            float c = d24 * fmaf(sb16, pb, sa * pa);
            c = fmaf(-dmin, fmaf(mb, sxb[st], ma * sxa[st]), c);
            acc[r] += live[st] ? c : 0.f;
        }
    }
    // 8. each row's lanes meet; one lane writes
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float v = rowdot_sum<true>(acc[r]);
        if (lane == 63 && row0 + r < g.M) {
            const float b = g.has_bias ? (float)braw[r] : 0.f;
            op[r * ois] = (half_t)rt_act(v + b, g.act);
        }
    }
}

// Tunables: 1 = never take this kernel, 2 = also where the matrix-core kernel would run; rows per wavefront and
// wavefronts per workgroup (0 = by the size of the grid).
RT_TUNABLE(g_gemv_q4k_rowdot_disable, 0);
RT_TUNABLE(g_gemv_q4k_rowdot_rows, 0);
RT_TUNABLE(g_gemv_q4k_rowdot_waves, 0);

template <int STEPS, int WAVES, int R>
static hipError_t launch_q4k_rowdot_w(dim3 grid, size_t lds, hipStream_t st, const GemvQ4kRowdotArgs &g) {
    hipLaunchKernelGGL((gemv_q4k_rowdot_kernel<STEPS, WAVES, R>), grid, dim3(WAVES * 64), lds, st, g);
    return hipGetLastError();
}

template <int STEPS>
static hipError_t launch_q4k_rowdot_s(int waves, int rows, dim3 grid, size_t lds, hipStream_t st, const GemvQ4kRowdotArgs &g) {
    if (waves == 4) {
        if (rows == 4) return launch_q4k_rowdot_w<STEPS, 4, 4>(grid, lds, st, g);
        if (rows == 2) return launch_q4k_rowdot_w<STEPS, 4, 2>(grid, lds, st, g);
        return launch_q4k_rowdot_w<STEPS, 4, 1>(grid, lds, st, g);
    }
    if (rows == 4) return launch_q4k_rowdot_w<STEPS, 2, 4>(grid, lds, st, g);
    if (rows == 2) return launch_q4k_rowdot_w<STEPS, 2, 2>(grid, lds, st, g);
    return launch_q4k_rowdot_w<STEPS, 2, 1>(grid, lds, st, g);
}

// Q4_K weights, one f16 activation vector, K a multiple of 256 up to 10752 (six steps of 64 vectors per row).
// hipErrorNotSupported: the shape or alignment does not fit and another kernel must run.
hipError_t launch_gemv_q4k_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                  hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemv_q4k_rowdot_disable == 1 || (g_gemv_q4k_rowdot_disable == 0 && p.K <= 4096)) return hipErrorNotSupported;
    if (p.a_dt != RT_Q4_K || p.act_dt != RT_F16 || p.N != 1 || p.K < 256 || p.K % 256 != 0) return hipErrorNotSupported;
    if (p.stacks > 65535 || p.b_ks != 1 || p.M < 1 || p.M > 0x7fffffff) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    const uint32_t nsb = (uint32_t)(p.K / 256), nvec = 9u * nsb;
    const int steps = (int)((nvec + 63) / 64);
    if (steps > 6) return hipErrorNotSupported;
    // rows per wavefront and wavefronts per workgroup: the most that still give the grid three workgroups per compute unit
    int waves = 4, rows = 4;
    while (rows > 1 && (p.M + waves * rows - 1) / (waves * rows) * p.stacks < 3 * (int64_t)dev.num_cus) rows >>= 1;
    if (rows == 1 && (p.M + waves - 1) / waves * p.stacks < 3 * (int64_t)dev.num_cus) waves = 2;
    if (g_gemv_q4k_rowdot_rows > 0) rows = g_gemv_q4k_rowdot_rows;
    if (g_gemv_q4k_rowdot_waves > 0) waves = g_gemv_q4k_rowdot_waves;
    const int64_t groups = (p.M + waves * rows - 1) / (waves * rows);
    if (groups > 0x7fffffff) return hipErrorNotSupported;

    GemvQ4kRowdotArgs g{};
    g.blocks = (const uint8_t *)A, g.X = (const half_t *)B, g.out = (half_t *)out;
    g.bias = p.has_bias ? (const half_t *)bias : (const half_t *)B;
    g.bias_rs = p.has_bias && p.bias_on_rows ? 1u : 0u;
    g.M = (uint32_t)p.M, g.nsb = nsb;
    g.o_is = p.o_is;
    g.a_ss = p.a_stack == 1 ? 0 : p.M * (int64_t)nsb * 144, g.x_ss = p.b_stack == 1 ? 0 : p.b_bs, g.o_ss = p.o_bs;
    g.has_bias = p.has_bias, g.act = p.act;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    const size_t lds = (size_t)p.K * 2 + (size_t)p.K / 4 + (size_t)waves * rows * nsb * 16;
    switch (steps) {
    case 1: return launch_q4k_rowdot_s<1>(waves, rows, grid, lds, stream, g);
    case 2: return launch_q4k_rowdot_s<2>(waves, rows, grid, lds, stream, g);
    case 3: return launch_q4k_rowdot_s<3>(waves, rows, grid, lds, stream, g);
    case 4: return launch_q4k_rowdot_s<4>(waves, rows, grid, lds, stream, g);
    case 5: return launch_q4k_rowdot_s<5>(waves, rows, grid, lds, stream, g);
    default: return launch_q4k_rowdot_s<6>(waves, rows, grid, lds, stream, g);
    }
}

} // namespace rt
