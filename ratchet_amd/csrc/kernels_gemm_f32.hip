// f32 GEMM on the matrix cores for operands with a contiguous axis:
//   C[s, i, j] = sum_k A[s, i, k] * B[s, k, j] (+ bias),  f32 in, f32 accumulate, f32 out,
// A K-contiguous; B either N-contiguous (`lhs.matmul(rhs)`, the Whisper encoder's
// [1500 x 384] . [384 x 1536]) or K-contiguous (Linear's W.gemm(x, b, false, true, true) with f32
// weights).  v_mfma_f32_16x16x4_f32 takes one f32 per lane and operand, so neither tile needs a
// transpose: A sits in LDS as [row][k] and B as it lies in memory, [k][col] or [col][k].
//
// 128 x 128, 96 x 96 or 32 x 96 outputs per 256-thread workgroup (2 x 2 wavefronts of 4 x 4, 3 x 3 or
// 1 x 3 MFMA tiles).  An f32 MFMA is slow (32 cycles for 2048 flop), so LDS and memory traffic are light and
// the launcher picks the tile by how much the fixed costs weigh (see launch_gemm_f32).  K tile 32,
// two LDS stages, one bare barrier per tile; tile t+1 waits in registers while tile t is multiplied
// and tile t+2 is in flight.  With K a whole number of tiles the loop has no bound to check; other K
// (a multiple of 4: attention scores over a head dimension of 80) run the KTAIL variant, whose loads
// clamp their K offset and whose LDS stores write zeros past K -- selects, not branches, so the loop
// stays straight-line code either way.
//
// LDS rows are padded so that every fragment read is conflict-free on 64 banks:
//   [row][k] tiles, stride 36: lane (r = l % 16, q = l / 16) reads word 36 r + 4 kk + q; 36 r mod 64
//     runs through the 16 multiples of 4, and q fills the gaps;
//   [k][col] tile, stride BN + 16 (= 48 mod 64): word (4 kk + q) (BN + 16) + c, the four q rows
//     start 16 banks apart.
//
// Roles in the reference: ops/gemm.rs:305-657 with f32 operands (test_sgemm, ops/matmul.rs:757-829;
// the Whisper encoder's MLP and attention projections, whisper/mlp.rs:18-22).
#include "device_common.h"

namespace rt {

struct GemmF32Args {
    const float *A, *B, *bias;
    float *out;
    int64_t M, N, K;
    int64_t a_stack, b_stack;
    int64_t a_bs, a_rs;
    int64_t b_bs, b_ks, b_js; // one of b_ks, b_js is 1
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
    int nt_out; // row-major output whose rows are whole 128-byte lines: written with non-temporal stores
};

constexpr int F32_BK = 32;
constexpr int F32_LDA = F32_BK + 4;

// B_KCONT: B's K axis is the contiguous one (its tile is [col][k], like A's); otherwise its
// column axis is (tile [k][col]).
// OJ: the output's column axis is the contiguous one (row-major C).  The MFMA's operands are then
// exchanged, which transposes what a lane holds: four consecutive columns of one row instead of four
// consecutive rows of one column, so the epilogue writes 16 bytes per lane either way.
template <int BM, int BN, bool B_KCONT, bool KTAIL, bool OJ>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmF32Args g) {
    constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
    static_assert(WM % 16 == 0 && WN % 16 == 0, "a wavefront's share must split into 16 x 16 MFMA tiles");
    constexpr int LDB = B_KCONT ? F32_LDA : BN + 16;
    constexpr int A_FLOATS = BM * F32_LDA, B_FLOATS = B_KCONT ? BN * F32_LDA : F32_BK * LDB;
    constexpr int STAGE = A_FLOATS + B_FLOATS;
    constexpr int A_VECS = BM * (F32_BK / 4), B_VECS = BN * (F32_BK / 4); // 16-byte vectors per tile
    constexpr int A_PT = (A_VECS + 255) / 256, B_PT = (B_VECS + 255) / 256;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    float *smem = (float *)smem_raw; // [2][STAGE]

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int fr = lane & 15, fq = lane >> 4;
    const int64_t s = blockIdx.y;
    // Workgroup ids go round the 8 XCDs; remapped, each XCD takes a contiguous run of tiles (whole
    // rows of tiles), so its L2 holds that run's few A row blocks and B once.
    int64_t wg = blockIdx.x;
    const int64_t tiles_j = (g.N + BN - 1) / BN, ntiles = gridDim.x;
    if (ntiles % 8 == 0) wg = (wg & 7) * (ntiles >> 3) + (wg >> 3);
    const int64_t ti = wg / tiles_j, tj = wg - ti * tiles_j;
    const int64_t i0 = ti * BM, j0 = tj * BN;
    const float *A = g.A + (g.a_stack == 1 ? 0 : s) * g.a_bs;
    const float *B = g.B + (g.b_stack == 1 ? 0 : s) * g.b_bs;

    // Per-thread sources of the vectors it moves (rows past the end repeat the last valid one:
    // their products land in outputs that are never stored).
    const float *pa[A_PT], *pb[B_PT];
    int la[A_PT], lb[B_PT]; // LDS word offsets
    int ka[A_PT], kb[B_PT]; // K offset of the vector inside a tile (KTAIL)
#pragma unroll
    for (int e = 0; e < A_PT; e++) {
        const int v = min(e * 256 + t, A_VECS - 1);
        const int row = v / (F32_BK / 4), c4 = v % (F32_BK / 4);
        pa[e] = A + min(i0 + row, g.M - 1) * g.a_rs + (KTAIL ? 0 : 4 * c4);
        la[e] = row * F32_LDA + 4 * c4;
        ka[e] = 4 * c4;
    }
#pragma unroll
    for (int e = 0; e < B_PT; e++) {
        const int v = min(e * 256 + t, B_VECS - 1);
        if constexpr (B_KCONT) {
            const int col = v / (F32_BK / 4), c4 = v % (F32_BK / 4);
            pb[e] = B + min(j0 + col, g.N - 1) * g.b_js + (KTAIL ? 0 : 4 * c4);
            lb[e] = A_FLOATS + col * LDB + 4 * c4;
            kb[e] = 4 * c4;
        } else {
            const int k = v / (BN / 4), c4 = v % (BN / 4);
            pb[e] = B + (KTAIL ? 0 : (int64_t)k * g.b_ks) + min(j0 + 4 * c4, g.N - 4); // N % 4 == 0: a vector is wholly in or out
            lb[e] = A_FLOATS + k * LDB + 4 * c4;
            kb[e] = k;
        }
    }
    struct Regs {
        float4_t a[A_PT], b[B_PT];
    };
    // K is a whole number of tiles (the launcher checks): no load needs a bound, so the loop body is
    // straight-line code and the compiler's wait counts stay exact (a conditional load makes it wait
    // for every outstanding load at the next register it overwrites).
    // KTAIL (K % 4 == 0, any number of tiles): a vector past K re-reads the last valid one (still no bound on
    // the load) and is replaced by zeros on its way into LDS.
    auto load_tile = [&](int64_t k0, Regs &r) {
#pragma unroll
        for (int e = 0; e < A_PT; e++) r.a[e] = *(const float4_t *)(pa[e] + (KTAIL ? min(k0 + ka[e], g.K - 4) : k0));
#pragma unroll
        for (int e = 0; e < B_PT; e++) {
            if constexpr (!KTAIL) r.b[e] = *(const float4_t *)(pb[e] + (B_KCONT ? k0 : k0 * g.b_ks));
            else if constexpr (B_KCONT) r.b[e] = *(const float4_t *)(pb[e] + min(k0 + kb[e], g.K - 4));
            else r.b[e] = *(const float4_t *)(pb[e] + min(k0 + kb[e], g.K - 1) * g.b_ks);
        }
    };
    auto store_tile = [&](int stage, int64_t k0, const Regs &r) {
        float *st = smem + stage * STAGE;
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < A_PT; e++)
            if (A_VECS % 256 == 0 || e * 256 + t < A_VECS) *(float4_t *)(st + la[e]) = (!KTAIL || k0 + ka[e] < g.K) ? r.a[e] : zero;
#pragma unroll
        for (int e = 0; e < B_PT; e++)
            if (B_VECS % 256 == 0 || e * 256 + t < B_VECS) *(float4_t *)(st + lb[e]) = (!KTAIL || k0 + kb[e] < g.K) ? r.b[e] : zero;
    };

    float4_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Tile kt is multiplied from LDS stage kt & 1 while tile kt + 1 waits in registers (stored to
    // the other stage after the MFMAs) and tile kt + 2 is on its way from memory: a load has two
    // tiles' worth of MFMAs (about 2 us) to arrive, a first-touch HBM latency.
    // Past the last tile the loads repeat it and the stores refill a stage nobody reads again: no branch.
    const int64_t nk = (g.K + F32_BK - 1) / F32_BK;
    Regs r0, r1;
    load_tile(0, r0);
    load_tile(min<int64_t>(1, nk - 1) * F32_BK, r1);
    store_tile(0, 0, r0);
    __syncthreads();
    auto k_tile = [&](int64_t kt, Regs &incoming, const Regs &waiting) {
        const int cur = (int)(kt & 1);
        load_tile(min(kt + 2, nk - 1) * F32_BK, incoming);
        const float *as = smem + cur * STAGE + (wi * WM + fr) * F32_LDA + fq;
        const float *bs = smem + cur * STAGE + A_FLOATS + (B_KCONT ? (wj * WN + fr) * LDB + fq : fq * LDB + wj * WN + fr);
        // Operand reads run one K step ahead of the MFMAs that use them, in registers of their own:
        // left to itself the compiler reuses the fragment registers and each read is issued one MFMA
        // before its first use, with the LDS latency in the open.
        float fa[2][TM], fb[2][TN];
        auto read_step = [&](int kk, int set) {
#pragma unroll
            for (int a = 0; a < TM; a++) fa[set][a] = as[a * 16 * F32_LDA + 4 * kk];
#pragma unroll
            for (int b = 0; b < TN; b++) fb[set][b] = B_KCONT ? bs[b * 16 * LDB + 4 * kk] : bs[4 * kk * LDB + b * 16];
        };
        const int klen = KTAIL ? (int)min<int64_t>(F32_BK, g.K - kt * F32_BK) : F32_BK; // the last tile may be short
        read_step(0, 0);
#pragma unroll
        for (int kk = 0; kk < F32_BK / 4; kk++) {
            if (kk + 1 < F32_BK / 4) read_step(kk + 1, (kk + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (!KTAIL || 4 * kk < klen) { // uniform: the zeros past K are not multiplied
#pragma unroll
                for (int a = 0; a < TM; a++)
#pragma unroll
                    for (int b = 0; b < TN; b++)
                        acc[a][b] = OJ ? __builtin_amdgcn_mfma_f32_16x16x4f32(fb[kk & 1][b], fa[kk & 1][a], acc[a][b], 0, 0, 0)
                                       : __builtin_amdgcn_mfma_f32_16x16x4f32(fa[kk & 1][a], fb[kk & 1][b], acc[a][b], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        store_tile(cur ^ 1, min(kt + 1, nk - 1) * F32_BK, waiting);
        // The other stage is complete; this one may be overwritten in the next iteration.  A bare
        // barrier behind a wait for the LDS operations only: __syncthreads() would also wait for the
        // global loads that were just issued for tile kt + 2.
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    for (int64_t kt = 0; kt < nk; kt += 2) {
        k_tile(kt, r0, r1); // r0's tile is in LDS: it takes tile kt + 2; r1 holds tile kt + 1
        if (kt + 1 < nk) k_tile(kt + 1, r1, r0);
    }

    float *out = g.out + s * g.o_bs;
    const int64_t iw = i0 + wi * WM, jw = j0 + wj * WN; // this wavefront's corner
    if constexpr (OJ) {
        // acc[a][b][r] is C[iw + 16 a + fr][jw + 16 b + 4 fq + r]: 16 bytes per lane along a row, 64 contiguous bytes per row
        // and instruction.  Non-temporal (the output is written once) where those 64 bytes are half of a line the next
        // instruction completes; with rows that do not start on a line (Whisper's scores, 1500 columns: 6000 bytes) the
        // pieces straddle lines and streaming them costs more than caching them (48 against 31 us at 6 x [1500 x 64] . [64 x 1500])
        rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const int64_t i = iw + 16 * a + fr;
                if (i >= g.M) continue;
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    const int64_t j = jw + 16 * b + 4 * fq;
                    if (j >= g.N) continue; // N % 4 == 0: a group of four is inside or outside as a whole
                    float4_t v = acc[a][b];
                    if (g.has_bias) {
                        if (g.bias_on_rows) {
                            const float bi = g.bias[i];
                            v += float4_t{bi, bi, bi, bi};
                        } else {
                            v += *(const float4_t *)(g.bias + j);
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) v[r] = rt_act_k<decltype(has_act)::value>(v[r]);
                    if (g.nt_out) __builtin_nontemporal_store(v, (float4_t *)(out + i * g.o_is + j));
                    else *(float4_t *)(out + i * g.o_is + j) = v;
                }
            }
        });
        return;
    }
    // acc[a][b][r] is C[iw + 16 a + 4 fq + r][jw + 16 b + fr]
    auto value = [&](auto has_act, int a, int b, int r) {
        float x = acc[a][b][r];
        if (g.has_bias) x += g.bias[g.bias_on_rows ? min(iw + 16 * a + 4 * fq + r, g.M - 1) : min(jw + 16 * b + fr, g.N - 1)];
        x = rt_act_k<decltype(has_act)::value>(x);
        return x;
    };
    // Straight from the accumulators: 16 bytes per lane along the rows (o_is == 1), or scalar stores.
    // Staging the sub-tile through LDS for 128-bit stores over whole runs measured 1 us slower at the Whisper shape.
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int b = 0; b < TN; b++) {
                const int64_t j = jw + 16 * b + fr, ib = iw + 16 * a + 4 * fq;
                if (j >= g.N) continue;
                float *o = out + ib * g.o_is + j * g.o_js;
                if (g.o_is == 1 && ib + 4 <= g.M && (((uintptr_t)o) & 15u) == 0) {
                    *(float4_t *)o = float4_t{value(has_act, a, b, 0), value(has_act, a, b, 1), value(has_act, a, b, 2), value(has_act, a, b, 3)};
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (ib + r < g.M) o[r * g.o_is] = value(has_act, a, b, r);
                }
            }
    });
}

template <int BM, int BN, bool B_KCONT, bool KTAIL, bool OJ>
static hipError_t launch_f32_oj(const GemmF32Args &g, int64_t stacks, hipStream_t st) {
    constexpr int LDB = B_KCONT ? F32_LDA : BN + 16;
    constexpr size_t lds = (size_t)2 * (BM * F32_LDA + (B_KCONT ? BN * F32_LDA : F32_BK * LDB)) * sizeof(float);
    if (const hipError_t e = ensure_lds_limit<&gemm_f32_kernel<BM, BN, B_KCONT, KTAIL, OJ>>(); e != hipSuccess) return e;
    const int64_t tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    if (tiles > 0x7fffffff) return hipErrorNotSupported;
    hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, B_KCONT, KTAIL, OJ>), dim3((unsigned)tiles, (unsigned)stacks), dim3(256), lds, st, g);
    return hipGetLastError();
}

template <int BM, int BN, bool B_KCONT, bool KTAIL>
static hipError_t launch_f32_kt(const GemmF32Args &g, int64_t stacks, hipStream_t st) {
    // row-major output with 16-byte aligned rows and N % 4 == 0 (bias along the columns read as vectors)
    const bool oj = g.o_js == 1 && g.N % 4 == 0 && g.o_is % 4 == 0 && g.o_bs % 4 == 0 && (!g.has_bias || g.bias_on_rows || ((uintptr_t)g.bias & 15u) == 0);
    return oj ? launch_f32_oj<BM, BN, B_KCONT, KTAIL, true>(g, stacks, st) : launch_f32_oj<BM, BN, B_KCONT, KTAIL, false>(g, stacks, st);
}

template <int BM, int BN, bool B_KCONT>
static hipError_t launch_f32(const GemmF32Args &g, int64_t stacks, hipStream_t st) {
    return g.K % F32_BK == 0 ? launch_f32_kt<BM, BN, B_KCONT, false>(g, stacks, st) : launch_f32_kt<BM, BN, B_KCONT, true>(g, stacks, st);
}

RT_TUNABLE(g_gemm_f32_bm, 0);      // 32 or 96 forces that tile height (0 = by shape)
RT_TUNABLE(g_gemm_f32_disable, 0); // non-zero sends f32 problems to the generic kernel (for comparisons)

// f32 x f32 with A K-contiguous and B contiguous along K or along its columns, 16-byte aligned
// rows.  hipErrorNotSupported: another kernel must take the problem.
hipError_t launch_gemm_f32(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                           const DeviceInfo &dev) {
    if (g_gemm_f32_disable || p.a_dt != RT_F32 || p.act_dt != RT_F32) return hipErrorNotSupported;
    if (p.a_ks != 1 || (p.b_ks != 1 && p.b_js != 1) || p.K < 4 || p.K % 4 != 0) return hipErrorNotSupported;
    if (p.M < 48 || p.N < 48 || p.stacks > 65535) return hipErrorNotSupported; // small outputs: the generic 64 x 64 tiles
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)out) & 15u) return hipErrorNotSupported;
    if (p.a_rs % 4 || p.a_bs % 4 || p.b_bs % 4) return hipErrorNotSupported;
    const bool b_kcont = p.b_ks == 1;
    if (b_kcont ? (p.b_js % 4 != 0) : (p.b_ks % 4 != 0 || p.N % 4 != 0)) return hipErrorNotSupported;

    GemmF32Args g{};
    g.A = (const float *)A, g.B = (const float *)B, g.bias = (const float *)bias, g.out = (float *)out;
    g.M = p.M, g.N = p.N, g.K = p.K;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.a_bs = p.a_bs, g.a_rs = p.a_rs;
    g.b_bs = p.b_bs, g.b_ks = p.b_ks, g.b_js = p.b_js;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    g.nt_out = p.o_js == 1 && (p.o_is * 4) % 128 == 0 && (p.o_bs * 4) % 128 == 0 && ((uintptr_t)out & 127u) == 0;
    // 32-row tiles put about three workgroups on a compute unit, whose prologues and epilogues then
    // overlap with each other's MFMAs: better while the fixed costs weigh (26.3 against 28.2 us at
    // K = 384); 96-row tiles read less LDS per MFMA and win from K of about 1000 on (78 against 81 us at 1536).
    const int64_t tiles96 = ((p.M + 95) / 96) * ((p.N + 95) / 96) * p.stacks;
    int bm = (p.K <= 768 || tiles96 < dev.num_cus) ? 32 : 96;
    // Short contractions (attention scores spelled [.., M, K] . [.., K, N], K = 80): nearly all the time goes
    // into fetching operands and writing the output, so the largest tile wins while it still gives every
    // compute unit two workgroups (25.4 against 30.6 us at 32 x [512 x 80] . [80 x 512]).
    const int64_t tiles128 = ((p.M + 127) / 128) * ((p.N + 127) / 128) * p.stacks;
    if (p.K <= 128 && tiles128 >= 2 * (int64_t)dev.num_cus) bm = 128;
    if (g_gemm_f32_bm == 32 || g_gemm_f32_bm == 96 || g_gemm_f32_bm == 128) bm = g_gemm_f32_bm;
    if (bm == 128) return b_kcont ? launch_f32<128, 128, true>(g, p.stacks, stream) : launch_f32<128, 128, false>(g, p.stacks, stream);
    // up to 64 columns (P . V over a head dimension of 64): 64-column tiles, not two thirds of 96
    if (bm == 32 && p.N <= 64) return b_kcont ? launch_f32<32, 64, true>(g, p.stacks, stream) : launch_f32<32, 64, false>(g, p.stacks, stream);
    if (bm == 32) return b_kcont ? launch_f32<32, 96, true>(g, p.stacks, stream) : launch_f32<32, 96, false>(g, p.stacks, stream);
    return b_kcont ? launch_f32<96, 96, true>(g, p.stacks, stream) : launch_f32<96, 96, false>(g, p.stacks, stream);
}

} // namespace rt
