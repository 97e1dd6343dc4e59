// MFMA GEMMs for the Linear / QK^T form, where both operands are K-contiguous:
//   C[s, i, j] = sum_k A[s, i, k] * B[s, j, k] (+ bias),  f16 in, f32 accumulate, f16 out.
// A is f16 or a Q8_0H weight; B is f16.  Four kernels, chosen by launch_gemm_nt:
//
//   gemm_nt_dl_kernel      f16 x f16, K % 64 == 0: 160 x 128 tiles, tiles loaded global -> LDS
//                          directly into a ring of stages by two wavefronts that do nothing else,
//                          issue order pinned (the fast path for the Phi-2 prefill shape:
//                          10240 x 512 outputs = 256 workgroups, one per CU)
//   gemm_nt_q8w_kernel     Q8_0H x f16, K % 256 == 0: the same pipeline; four loading wavefronts widen the int8
//                          tile to f16 codes on its way into LDS, each block of 32 is multiplied from zero and
//                          its partial sums are folded into the accumulators with the block's scale in f32
//   gemm_nt_shortk_kernel  f16 x f16, K <= 128 (attention scores): a resident strip of B rows,
//                          A tiles prefetched through registers, output written as it is produced
//   gemm_nt_kernel         everything else this file takes (ragged K, Q8_0H with K % 256 != 0,
//                          short K without a contiguous output axis): register-staged, two LDS stages
//
// Common to all: 2 x 2 multiplying wavefronts, v_mfma_f32_16x16x32_f16 with A rows on the MFMA's
// lane index, XOR-swizzled or odd-stride LDS rows so that fragment reads are conflict-free, an
// epilogue that transposes through LDS and stores 128 bits along the contiguous output axis, and
// (large tiles) workgroup ids remapped so that the 8 XCDs each take a contiguous range of A row
// blocks: all column blocks of one A row block share one L2 copy of its tiles.
//
// gemm_nt_kernel's pipeline per K tile of 64: global loads of tile t+2 into registers, MFMAs on LDS
// stage t, then the registers of tile t+1 -> the other LDS stage, one barrier.  For Q8_0H it widens
// the int8 codes to f16 on the way into LDS (exact), accumulates each block of 32 separately and
// folds it in with its scale in f32, so no weight is ever rounded.
//
// Roles in the reference: ops/gemm.rs:305-657 (GEMM generators), with Linear's
// W.gemm(x, b, false, true, true) (crates/ratchet-nn/src/linear.rs:17-24) and attention's
// Q.matmul(K, false, true) (phi3/attn.rs:142-158) as the callers.
#include "device_common.h"
#include <utility>

namespace rt {

struct GemmNtArgs {
    const void *A;       // f16 [.., M, K] or Q8_0H codes
    const half_t *scales; // Q8_0H scale stream of A
    const half_t *B;     // f16 [.., N, K]
    const half_t *bias;
    half_t *out;
    int64_t M, N, K;
    int64_t a_stack, b_stack;
    int64_t a_bs, a_rs;  // elements
    int64_t b_bs, b_js;
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
    int tiles_i, tiles_j;
    int vec_epilogue; // o_is == 1 and rows of the output 16-byte aligned: LDS-staged 128-bit stores
    // split K (direct-to-LDS kernels): blockIdx.z owns K range [z * k_len, (z + 1) * k_len) and writes its
    // f32 sums to partial [stack][split][N][M]; a second kernel adds them up, then bias, activation, rounding
    int ksplit;
    int64_t k_len;
    float *partial;
};

// Which output tile a workgroup takes.  Workgroup ids go round the 8 XCDs, each with an L2 of its own:
// XCD x takes the contiguous range x * ntiles / 8 .. of the tiles in row-major order (A row block major),
// so all column blocks of one A row block share one L2 copy of it.  When that range is whole A row
// blocks and there are more than four column blocks, the range is walked in panels of four column
// blocks (all of the XCD's row blocks against four column blocks, then the next four): the 32
// workgroups an XCD runs at a time then share 8 + 4 operand blocks instead of 1 + 32, which at
// [4096 x 2560] . [10240 x 2560]^T cut what the L2s fetch from 1.39 GB per launch (19 x the operands).
__device__ __forceinline__ void nt_tile_of(int64_t wg, int tiles_i, int tiles_j, int64_t &ti, int64_t &tj) {
    constexpr int PJ = 4;
    const int64_t ntiles = (int64_t)tiles_i * tiles_j;
    if (ntiles % 8 == 0) wg = (wg & 7) * (ntiles >> 3) + (wg >> 3);
    if (tiles_i % 8 == 0 && tiles_j > PJ) {
        const int64_t rows = tiles_i >> 3, chunk = rows * tiles_j; // per XCD
        const int64_t x = wg / chunk, r = wg - x * chunk;
        const int64_t panels = (tiles_j + PJ - 1) / PJ;
        const int64_t p = min(r / (rows * PJ), panels - 1), q = r - p * rows * PJ;
        const int64_t w = min<int64_t>(PJ, tiles_j - p * PJ); // the last panel may be narrower
        ti = x * rows + q / w, tj = p * PJ + q % w;
        return;
    }
    ti = wg / tiles_j, tj = wg - ti * tiles_j;
}

// Timing-only variants of gemm_nt_dl_kernel for the measurement probes (a bit mask: 1 no tile loads, 2 no MFMAs,
// 4 no fragment reads, 8 no output); the product is built with 0.
#ifndef RT_NT_ABLATION
#define RT_NT_ABLATION 0
#endif

constexpr int NT_BK = 64;
constexpr int NT_LDK = NT_BK;     // halfs per LDS row: 128 B = 8 vectors of 16 B, no padding
constexpr int NT_THREADS = 256;

// LDS tile layout: row r holds its 8 K-vectors at slots c ^ ((r >> 1) & 7).  Two
// consecutive rows cover all 64 banks, so a 16-lane group that writes two whole rows
// (the global-load order) and a 16-lane group that reads one vector from each of 16
// rows (the MFMA fragment order) are both free of bank conflicts.
__device__ __forceinline__ int nt_slot(int r, int c) { return (r * 8 + (c ^ ((r >> 1) & 7))) * 8; } // in halfs

__device__ __forceinline__ void nt_cvt_i8x4(uint32_t v, half2_t &lo, half2_t &hi) {
    v ^= 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u);
    const half2_t bias = {(half_t)1152.0f, (half_t)1152.0f};
    lo = __builtin_bit_cast(half2_t, a) - bias;
    hi = __builtin_bit_cast(half2_t, b) - bias;
}

// Output stage shared by the tiled kernels: accumulators (+ bias, activation) to f16.  In tile
// (a, b) lane l holds A row (l % 16) and B rows 4 * (l / 16) + r.  With vec_epilogue the A-row
// axis is contiguous in the output (o_is == 1): the wavefront's sub-tile is transposed through
// LDS (free once the main loop's last barrier has passed) so that every lane stores 8
// consecutive outputs (128 bits); otherwise bounds-checked scalar stores.
template <int TM, int TN, int WM, int WN>
__device__ __forceinline__ void nt_epilogue(const GemmNtArgs &g, float4_t (&acc)[TM][TN], uint8_t *smem, int64_t s,
                                            int64_t i0, int64_t j0, int wi, int wj, int wave, int lane) {
    const int fr = lane & 15, fg = lane >> 4;
    if (g.ksplit > 1) {
        // this workgroup summed only its share of K: the sums go out as they are, [j][i] with i contiguous
        float *pt = g.partial + ((s * g.ksplit + blockIdx.z) * g.N) * g.M;
#pragma unroll
        for (int a = 0; a < TM; a++) {
            const int64_t i = i0 + wi * WM + a * 16 + fr;
#pragma unroll
            for (int b = 0; b < TN; b++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int64_t j = j0 + wj * WN + b * 16 + 4 * fg + r;
                    if (i < g.M && j < g.N) pt[j * g.M + i] = acc[a][b][r];
                }
        }
        return;
    }
    half_t *out = g.out + s * g.o_bs;
    if (g.vec_epilogue) {
        constexpr int EROW = WM + 8;                       // halfs per staged B-row (+16 B pad)
        half_t *es = (half_t *)smem + wave * (WN * EROW);
        rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const int64_t i = i0 + wi * WM + a * 16 + fr;
                float bi = 0.f;
                if (g.has_bias && g.bias_on_rows && i < g.M) bi = (float)g.bias[i];
#pragma unroll
                for (int b = 0; b < TN; b++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int jl = b * 16 + 4 * fg + r;
                        float v = acc[a][b][r] + bi;
                        if (g.has_bias && !g.bias_on_rows) v += (float)g.bias[min(j0 + wj * WN + jl, g.N - 1)];
                        v = rt_act_k<decltype(has_act)::value>(v);
                        es[jl * EROW + a * 16 + fr] = (half_t)v;
                    }
            }
        });
        asm volatile("" ::: "memory"); // same wavefront reads back below; DS operations complete in order
        constexpr int VPR = WM / 8;    // 128-bit vectors per staged row
        for (int v = lane; v < WN * VPR; v += 64) {
            const int jl = v / VPR, c = v - jl * VPR;
            const int64_t j = j0 + wj * WN + jl, i = i0 + wi * WM + 8 * c;
            if (j < g.N) {
                if (i + 8 <= g.M) {
                    __builtin_nontemporal_store(*(const uint4_t *)(es + jl * EROW + 8 * c), (uint4_t *)(out + j * g.o_js + i)); // written once, not read back here
                } else {
                    for (int e = 0; e < 8; e++)
                        if (i + e < g.M) out[j * g.o_js + i + e] = es[jl * EROW + 8 * c + e];
                }
            }
        }
        return;
    }
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int a = 0; a < TM; a++) {
            const int64_t i = i0 + wi * WM + a * 16 + fr;
            float bi = 0.f;
            if (g.has_bias && g.bias_on_rows && i < g.M) bi = (float)g.bias[i];
#pragma unroll
            for (int b = 0; b < TN; b++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int64_t j = j0 + wj * WN + b * 16 + 4 * fg + r;
                    if (i < g.M && j < g.N) {
                        float v = acc[a][b][r] + bi;
                        if (g.has_bias && !g.bias_on_rows) v += (float)g.bias[j];
                        v = rt_act_k<decltype(has_act)::value>(v);
                        out[i * g.o_is + j * g.o_js] = (half_t)v;
                    }
                }
        }
    });
}

// KFULL: K is a multiple of the K step, so no load or store needs a bound.
template <int BM, int BN, bool Q8, bool KFULL>
__global__ __launch_bounds__(NT_THREADS, (BM * BN <= 128 * 64 ? 3 : 1)) void gemm_nt_kernel(GemmNtArgs g) {
    constexpr int WM = BM / 2, WN = BN / 2;      // wavefront sub-tile
    constexpr int TM = WM / 16, TN = WN / 16;    // MFMA tiles per wavefront
    static_assert(WM % 16 == 0 && WN % 16 == 0, "tile must split into 16x16 MFMA tiles");
    // 16-byte vectors per K tile row, and per thread
    constexpr int A_VPR = Q8 ? NT_BK / 16 : NT_BK / 8;
    constexpr int A_VEC = (BM * A_VPR + NT_THREADS - 1) / NT_THREADS;
    constexpr int B_VPR = NT_BK / 8;
    constexpr int B_VEC = (BN * B_VPR + NT_THREADS - 1) / NT_THREADS;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *As = (half_t *)smem;                         // [2][BM][NT_LDK]
    half_t *Bs = As + 2 * BM * NT_LDK;                   // [2][BN][NT_LDK]
    float *Sd = (float *)(Bs + 2 * BN * NT_LDK);         // [2 stages][2 blocks][BM]   (Q8 only)

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int fr = lane & 15, fg = lane >> 4;            // fragment row / K group

    int64_t ti, tj;
    nt_tile_of(blockIdx.x, g.tiles_i, g.tiles_j, ti, tj); // XCD-aware tile order (see the file comment)
    const int64_t i0 = ti * BM, j0 = tj * BN;
    const int64_t s = blockIdx.y;
    const int64_t a_el = (g.a_stack == 1 ? 0 : s) * g.a_bs, b_el = (g.b_stack == 1 ? 0 : s) * g.b_bs;

    // two register sets: the loads of tile t+2 are in flight while tile t is multiplied
    uint4_t ra0[A_VEC], rb0[B_VEC], ra1[A_VEC], rb1[B_VEC];
    half_t rsc0[2], rsc1[2]; // Q8: this thread's scales for the tile's two blocks (threads < BM)

    // Loads are unconditional (addresses past K are clamped to a valid one) so that no branch
    // separates them from the LDS store that consumes them and the hardware counters can let
    // the other register set's loads stay in flight; store_tiles zeroes what lies past K.
    auto load_tiles = [&](int64_t k0, uint4_t (&ra)[A_VEC], uint4_t (&rb)[B_VEC], half_t (&rsc)[2]) {
#pragma unroll
        for (int e = 0; e < A_VEC; e++) {
            const int v = min(e * NT_THREADS + t, BM * A_VPR - 1);
            const int r = v / A_VPR, c = v - r * A_VPR;
            const int64_t gr = min(i0 + r, g.M - 1); // rows past the end duplicate the last one; never stored
            if constexpr (Q8) {
                const int64_t gk = KFULL ? k0 + 16 * c : min(k0 + 16 * c, g.K - 16);
                ra[e] = *(const uint4_t *)((const uint8_t *)g.A + a_el + gr * g.a_rs + gk);
            } else {
                const int64_t gk = KFULL ? k0 + 8 * c : min(k0 + 8 * c, g.K - 8);
                ra[e] = *(const uint4_t *)((const half_t *)g.A + a_el + gr * g.a_rs + gk);
            }
        }
        if constexpr (Q8) {
            const int64_t gr = min(i0 + min(t, BM - 1), g.M - 1);
            const int64_t row_blk = (a_el + gr * g.a_rs) >> 5, kb = k0 >> 5, last = (g.K >> 5) - 1;
            rsc[0] = g.scales[row_blk + (KFULL ? kb : min(kb, last))];
            rsc[1] = g.scales[row_blk + (KFULL ? kb + 1 : min(kb + 1, last))];
        }
#pragma unroll
        for (int e = 0; e < B_VEC; e++) {
            const int v = min(e * NT_THREADS + t, BN * B_VPR - 1);
            const int r = v / B_VPR, c = v - r * B_VPR;
            const int64_t gr = min(j0 + r, g.N - 1);
            const int64_t gk = KFULL ? k0 + 8 * c : min(k0 + 8 * c, g.K - 8);
            rb[e] = *(const uint4_t *)(g.B + b_el + gr * g.b_js + gk);
        }
    };

    auto store_tiles = [&](int stage, int64_t k0, const uint4_t (&ra)[A_VEC], const uint4_t (&rb)[B_VEC],
                           const half_t (&rsc)[2]) {
        half_t *as = As + stage * BM * NT_LDK, *bs = Bs + stage * BN * NT_LDK;
        const uint4_t zero4 = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < A_VEC; e++) {
            const int v = e * NT_THREADS + t;
            if (v < BM * A_VPR) {
                const int r = v / A_VPR, c = v - r * A_VPR;
                if constexpr (Q8) {
                    const uint4_t raw = (KFULL || k0 + 16 * c < g.K) ? ra[e] : zero4;
                    half2_t h[8];
#pragma unroll
                    for (int d = 0; d < 4; d++) nt_cvt_i8x4(raw[d], h[2 * d], h[2 * d + 1]);
                    uint4_t lo = {__builtin_bit_cast(uint32_t, h[0]), __builtin_bit_cast(uint32_t, h[1]),
                                  __builtin_bit_cast(uint32_t, h[2]), __builtin_bit_cast(uint32_t, h[3])};
                    uint4_t hi = {__builtin_bit_cast(uint32_t, h[4]), __builtin_bit_cast(uint32_t, h[5]),
                                  __builtin_bit_cast(uint32_t, h[6]), __builtin_bit_cast(uint32_t, h[7])};
                    *(uint4_t *)(as + nt_slot(r, 2 * c)) = lo;
                    *(uint4_t *)(as + nt_slot(r, 2 * c + 1)) = hi;
                } else {
                    *(uint4_t *)(as + nt_slot(r, c)) = (KFULL || k0 + 8 * c < g.K) ? ra[e] : zero4;
                }
            }
        }
        if constexpr (Q8) {
            if (t < BM) {
                Sd[(stage * 2 + 0) * BM + t] = (KFULL || k0 < g.K) ? (float)rsc[0] : 0.f;
                Sd[(stage * 2 + 1) * BM + t] = (KFULL || k0 + 32 < g.K) ? (float)rsc[1] : 0.f;
            }
        }
#pragma unroll
        for (int e = 0; e < B_VEC; e++) {
            const int v = e * NT_THREADS + t;
            if (v < BN * B_VPR) {
                const int r = v / B_VPR, c = v - r * B_VPR;
                *(uint4_t *)(bs + nt_slot(r, c)) = (KFULL || k0 + 8 * c < g.K) ? rb[e] : zero4;
            }
        }
    };

    float4_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Fragment addressing: lane (fr, fg) reads row base + 16 * tile + fr, K-vector kk * 4 + fg.  The
    // wavefront's row bases are multiples of 16, so the row's swizzle term depends on fr only.
    const int swz = (fr >> 1) & 7;
    struct Frags {
        half8_t fa[TM], fb[TN];
        float d[Q8 ? TM : 1]; // Q8: scale of this lane's A row, per tile, for the block this K step covers
    };
    auto read_frags = [&](int stage, int kk, Frags &f) {
        const half_t *as = As + stage * BM * NT_LDK + (wi * WM + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
        const half_t *bs = Bs + stage * BN * NT_LDK + (wj * WN + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
#pragma unroll
        for (int a = 0; a < TM; a++) f.fa[a] = __builtin_bit_cast(half8_t, *(const uint4_t *)(as + a * 16 * NT_LDK));
#pragma unroll
        for (int b = 0; b < TN; b++) f.fb[b] = __builtin_bit_cast(half8_t, *(const uint4_t *)(bs + b * 16 * NT_LDK));
        if constexpr (Q8) {
#pragma unroll
            for (int a = 0; a < TM; a++) f.d[a] = Sd[(stage * 2 + kk) * BM + wi * WM + a * 16 + fr];
        }
    };
    auto mma_step = [&](const Frags &f) {
        if constexpr (Q8) {
            // one Q8_0 block: fresh partial sums, then acc += scale * partial (scale per lane = per A row)
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
                    const float4_t p = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.fb[b], f.fa[a], zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[a][b][r] = fmaf(f.d[a], p[r], acc[a][b][r]);
                }
        } else {
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.fb[b], f.fa[a], acc[a][b], 0, 0, 0);
        }
    };

    // Software pipeline: tile t is multiplied from LDS stage t % 2 while tile t+1 sits in one
    // register set (written to the other stage after the MFMAs) and tile t+2 is being loaded
    // into the other register set.  Loads past the last tile re-read it (their data is unused),
    // which keeps the loop body free of branches around memory operations.  Within a tile the
    // second K step's fragments are requested before the first step's MFMAs are issued.
    const int64_t nk = (g.K + NT_BK - 1) / NT_BK;
    auto kclamp = [&](int64_t kt) { return min(kt, nk - 1) * NT_BK; };
    auto compute = [&](int stage) {
        Frags f0, f1;
        read_frags(stage, 0, f0);
        read_frags(stage, 1, f1);
        mma_step(f0);
        mma_step(f1);
    };
    if (nk > 0) {
        load_tiles(0, ra0, rb0, rsc0);
        load_tiles(kclamp(1), ra1, rb1, rsc1);
        store_tiles(0, 0, ra0, rb0, rsc0);
    }
    __syncthreads();
    for (int64_t kt = 0; kt < nk; kt += 2) {
        // even tile: set 1 holds tile kt+1, set 0 is free for tile kt+2
        load_tiles(kclamp(kt + 2), ra0, rb0, rsc0);
        compute(0);
        store_tiles(1, (kt + 1) * NT_BK, ra1, rb1, rsc1);
        __syncthreads();
        if (kt + 1 >= nk) break;
        // odd tile: set 0 holds tile kt+2, set 1 is free for tile kt+3
        load_tiles(kclamp(kt + 3), ra1, rb1, rsc1);
        compute(1);
        store_tiles(0, (kt + 2) * NT_BK, ra0, rb0, rsc0);
        __syncthreads();
    }
    __syncthreads(); // every wavefront is done with the tile stages: the epilogue reuses them

    nt_epilogue<TM, TN, WM, WN>(g, acc, smem, s, i0, j0, wi, wj, wave, lane);
}

// ---------------------------------------------------------------------------
// f16 x f16 variant with direct-to-LDS loads (global_load_lds_dwordx4): tiles go
// from global memory straight into a three-stage LDS ring without passing through
// registers.  A wavefront's load instruction writes 1 KiB of LDS contiguously
// (lane l at base + 16 l), i.e. 8 whole rows of the swizzled tile; the swizzle is
// applied on the global side by choosing which K-vector each lane fetches.
// Requires K % 64 == 0; full tiles are not required (rows are clamped).
//
// The loads are issued by wavefronts of their own.  A wavefront issues in order, one per SIMD
// here: when the memory pipeline pushes back on a load, the MFMAs behind it wait too, and with
// every wavefront loading its share the fill (16.5 us alone at the [512 x 2560] . [10240 x 2560]^T
// shape) and the MFMAs (12.8 us alone) nearly added up.  So wavefronts 0..3 only read fragments
// and multiply; LW further wavefronts only issue the ring's loads (chunks dealt round-robin) and
// meet the others at the one barrier per K tile: a stalled load stalls nobody else (40 -> 33 us).
//
// Iteration t, loading wavefronts: issue tile t + STAGES - 1 into the stage that was read for
// the last time before the barrier of iteration t - 1, wait until tile t + 1 has landed, barrier.
// Multiplying wavefronts: the first K step's MFMAs with the second step's fragment reads between
// them, barrier (every read has returned, tile t + 1 is visible), the second step's MFMAs with
// the reads of tile t + 1's first-step fragments between them.
// ---------------------------------------------------------------------------
template <int BM, int BN, int STAGES, int LW>
__global__ __launch_bounds__(NT_THREADS + 64 * LW) void gemm_nt_dl_kernel(GemmNtArgs g) {
    constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
    constexpr int CH = (BM + BN) / 8;  // 8-row chunks of one K tile: the A rows, then the B rows
    constexpr int LCH = CH / LW;       // per loading wavefront
    static_assert(BM % 16 == 0 && BN % 8 == 0 && CH % LW == 0, "chunks must deal out evenly");
    static_assert((STAGES - 2) * LCH < 64, "the wait counter has six bits");
    constexpr int STAGE_HALFS = (BM + BN) * NT_LDK;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *ring = (half_t *)smem; // [STAGES][BM + BN][64]

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);

    int64_t ti, tj;
    nt_tile_of(blockIdx.x, g.tiles_i, g.tiles_j, ti, tj); // XCD-aware tile order (see the file comment)
    const int64_t i0 = ti * BM, j0 = tj * BN;
    const int64_t s = blockIdx.y;
    const int64_t kbase = (int64_t)blockIdx.z * g.k_len;
    const int64_t a_el = (g.a_stack == 1 ? 0 : s) * g.a_bs + kbase, b_el = (g.b_stack == 1 ? 0 : s) * g.b_bs + kbase;
    const int64_t nk = g.k_len / NT_BK; // nk >= 1

    if (wave >= 4) {
        // ---- loading wavefront: lane l fills LDS row chunk * 8 + l / 8, slot l % 8, which must
        // hold K-vector (l % 8) ^ ((row >> 1) & 7); BM is a multiple of 16, so the swizzle of a B
        // row is the same counted from the top of the stage as from the top of the B tile
        const int lw = wave - 4;
        const half_t *gp[LCH];
#pragma unroll
        for (int c = 0; c < LCH; c++) {
            const int row = (lw + c * LW) * 8 + (lane >> 3);
            const int kv = (lane & 7) ^ ((row >> 1) & 7);
            gp[c] = row < BM ? (const half_t *)g.A + a_el + min(i0 + row, g.M - 1) * g.a_rs + 8 * kv
                             : g.B + b_el + min(j0 + (row - BM), g.N - 1) * g.b_js + 8 * kv;
        }
        auto issue_tile = [&](int stage, int64_t k0) {
            half_t *st = ring + stage * STAGE_HALFS;
            if (RT_NT_ABLATION & 1) return; // timing only: no tile loads
#pragma unroll
            for (int c = 0; c < LCH; c++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gp[c] + k0),
                                                 (__attribute__((address_space(3))) void *)(st + (lw + c * LW) * 8 * NT_LDK),
                                                 16, 0, 0);
        };
        // all but the newest STAGES - 2 tiles have landed
        constexpr int kNew = (STAGES - 2) * LCH;
        constexpr int kWaitOlder = 0x0F70 | (kNew & 0xF) | (((kNew >> 4) & 0x3) << 14);
        auto publish = [&]() {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(kWaitOlder);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
#pragma unroll
        for (int st = 0; st < STAGES - 1; st++) issue_tile(st, min<int64_t>(st, nk - 1) * NT_BK);
        publish(); // tile 0
        int wr = STAGES - 1;
        for (int64_t kt = 0; kt < nk; kt++) {
            // stage wr was read for the last time before the barrier that ended iteration kt - 1
            issue_tile(wr, min(kt + STAGES - 1, nk - 1) * NT_BK);
            publish(); // tile kt + 1
            wr = wr + 1 == STAGES ? 0 : wr + 1;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): nothing may land once the epilogue reuses the ring
        __syncthreads();
        return;
    }

    // ---- multiplying wavefronts
    const int wi = wave >> 1, wj = wave & 1;
    const int fr = lane & 15, fg = lane >> 4;
    const int swz = (fr >> 1) & 7;
    struct Frags {
        half8_t fa[TM], fb[TN];
    };
    auto read_one = [&](int stage, int kk, Frags &f, int i) {
        if (RT_NT_ABLATION & 4) return; // timing only: no fragment reads
        const half_t *as = ring + stage * STAGE_HALFS + (wi * WM + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
        const half_t *bs = ring + stage * STAGE_HALFS + BM * NT_LDK + (wj * WN + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
        if (i < TM)
            f.fa[i] = __builtin_bit_cast(half8_t, *(const uint4_t *)(as + i * 16 * NT_LDK));
        else
            f.fb[i - TM] = __builtin_bit_cast(half8_t, *(const uint4_t *)(bs + (i - TM) * 16 * NT_LDK));
    };
    float4_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
    // every fragment read has returned (the stage may be refilled after the barrier); no loads of its own
    auto meet = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    meet(); // tile 0 visible
#if RT_NT_ABLATION & 4
    Frags f0 = {}, f1 = {};
    asm volatile("" : "+v"(f0.fa[0]), "+v"(f1.fa[0]));
#else
    Frags f0, f1;
#endif
#pragma unroll
    for (int i = 0; i < TM + TN; i++) read_one(0, 0, f0, i);
    int cur = 0, nxt = 1;
    // a fragment read behind every second MFMA, or behind every one where the tile has too few of them
    constexpr int RS = TM * TN / 2 >= TM + TN ? 2 : 1;
    static_assert(TM * TN / RS >= TM + TN, "not enough MFMAs to spread the reads over");
    for (int64_t kt = 0; kt < nk; kt++) {
#pragma unroll
        for (int m = 0; m < TM * TN; m++) {
            if (!(RT_NT_ABLATION & 2)) acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f0.fb[m % TN], f0.fa[m / TN], acc[m / TN][m % TN], 0, 0, 0);
            if (m % RS == RS - 1) {
                if (m / RS < TM + TN) read_one(cur, 1, f1, m / RS);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        meet(); // tile kt + 1 visible
#pragma unroll
        for (int m = 0; m < TM * TN; m++) {
            if (!(RT_NT_ABLATION & 2)) acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f1.fb[m % TN], f1.fa[m / TN], acc[m / TN][m % TN], 0, 0, 0);
            if (m % RS == RS - 1) {
                if (m / RS < TM + TN) read_one(nxt, 0, f0, m / RS);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        cur = nxt;
        nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __syncthreads();
    if (RT_NT_ABLATION & 8) { // timing only: no output (one store per lane keeps the accumulators alive)
        float v = 0.f;
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int b = 0; b < TN; b++) v += acc[a][b][0] + acc[a][b][1] + acc[a][b][2] + acc[a][b][3];
        if (RT_NT_ABLATION & 4) v += (float)f0.fa[0][0] + (float)f1.fb[0][0];
        if (v == 12345.678f) g.out[t] = (half_t)v;
        return;
    }
    nt_epilogue<TM, TN, WM, WN>(g, acc, smem, s, i0, j0, wi, wj, wave, lane);
}

// ---------------------------------------------------------------------------
// Q8_0H x f16.  Four loading wavefronts, one per SIMD, fetch the int8 tile into registers (a lane: 16 codes of
// one row), widen it to f16 (exact) and store f16 code tiles into the ring in the f16 kernel's swizzled layout;
// the activation tile goes global -> LDS directly.  The four multiplying wavefronts run the f16 kernel's
// fragment reads and, per block of 32, one MFMA from zero whose four sums per lane are folded into the
// accumulators with the block's f16 scale two MFMAs later (v_fma_mix: the f16 scale is an operand as it is).
// No weight is rounded.  Two earlier forms: the operand q * d itself, exactly, as the sum of two f16
// (hi = rn(q * d), lo = fma(q, d, -hi)) with two MFMAs per tile into the running accumulator, 64.5 us at
// [512 x 2560] . [10240 x 2560]^T; int8 tiles in LDS, widened by the multiplying wavefronts when they read their
// fragments (50 of their 153 vector instructions per K step), 43.2 us; this one 41.6: what is left is the
// fold, four fused multiply-adds per MFMA, which the multiplying wavefronts cannot hand to anyone.
// Rounding q * d to f16 (the reference's own shader does, ops/gemm.rs:547-548) would remove the fold, and was
// measured: the outputs near zero then miss the 2e-2 tolerance (0.115).  The hi / lo form was built once more on this
// pipeline (the loading wavefronts computing both tiles, two weight stages of hi and lo and four activation stages,
// the multiplying wavefronts issuing MFMAs only): 57.1 us against this kernel's 44.3 in the same harness.  The lo tile
// is subnormal f16 as a rule, which the matrix cores take at full speed (scaled into the normal range it ran the
// same); the form doubles the weight fragments read from LDS and the stores of the loading wavefronts.
//
// Ring of four stages of (BM + BN) x 64 halves.  Loading wavefront, iteration j: request the codes of tile
// j + 3 (registers, set (j + 3) % 4) and its activation rows (LDS-DMA into stage (j + 3) % 4, last read
// before the barrier that ended iteration j - 1); wait for the codes of tile j + 1, requested two
// iterations ago (everything older has landed with them, the activation rows of tile j + 1 included);
// widen and store them into stage (j + 1) % 4; barrier.  Requires K % 256 == 0 (scales in groups of 8).
// ---------------------------------------------------------------------------
template <int BM, int BN, int LW>
__global__ __launch_bounds__(NT_THREADS + 64 * LW) void gemm_nt_q8w_kernel(GemmNtArgs g) {
    constexpr int STAGES = 4, AHEAD = 2;
    constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
    constexpr int STAGE_HALFS = (BM + BN) * NT_LDK;
    constexpr int NREAD = TM + TN;
    static_assert(BM % 16 == 0 && BN % (8 * LW) == 0, "tile rows must fill whole chunks");
    static_assert(TM * TN >= NREAD, "not enough MFMAs to spread the reads over");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *ring = (half_t *)smem; // [STAGES][BM + BN][64]
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);

    int64_t ti, tj;
    nt_tile_of(blockIdx.x, g.tiles_i, g.tiles_j, ti, tj); // XCD-aware tile order (see the file comment)
    const int64_t i0 = ti * BM, j0 = tj * BN;
    const int64_t s = blockIdx.y;
    const int64_t kbase = (int64_t)blockIdx.z * g.k_len; // this workgroup's share of K (all of it without a split)
    const int64_t a_el = (g.a_stack == 1 ? 0 : s) * g.a_bs + kbase, b_el = (g.b_stack == 1 ? 0 : s) * g.b_bs + kbase;
    const int64_t nk = g.k_len / NT_BK; // a multiple of 4

    if (wave >= 4) {
        const int lw = wave - 4;
        constexpr int ACH = BM / 16;            // 16-row pieces of the code tile (one load instruction each)
        constexpr int NA = (ACH + LW - 1) / LW; // per loading wavefront
        constexpr int LCHB = BN / 8 / LW;       // 8-row chunks of the activation tile per loading wavefront
        static_assert(AHEAD * (LCHB + NA) < 64, "the wait counter has six bits");
        const uint8_t *ga[NA];
        int adst[NA]; // this lane's row within the code tile
        bool alive[NA];
        const int piece = lane & 3;
#pragma unroll
        for (int c = 0; c < NA; c++) {
            const int ch = lw + c * LW;
            alive[c] = ch < ACH; // wave-uniform
            const int row = min(ch, ACH - 1) * 16 + (lane >> 2);
            ga[c] = (const uint8_t *)g.A + a_el + min(i0 + row, g.M - 1) * g.a_rs + 16 * piece;
            adst[c] = row;
        }
        const half_t *gb[LCHB];
#pragma unroll
        for (int c = 0; c < LCHB; c++) {
            const int row = (lw + c * LW) * 8 + (lane >> 3);
            const int kv = (lane & 7) ^ ((row >> 1) & 7);
            gb[c] = g.B + b_el + min(j0 + row, g.N - 1) * g.b_js + 8 * kv;
        }
        uint4_t ra[STAGES][NA];
        auto request = [&](int slot, int64_t tile) __attribute__((always_inline)) {
            const int64_t k0 = min(tile, nk - 1) * NT_BK; // past the last tile: re-read it, never used
            half_t *st = ring + slot * STAGE_HALFS + BM * NT_LDK;
#pragma unroll
            for (int c = 0; c < LCHB; c++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gb[c] + k0),
                                                 (__attribute__((address_space(3))) void *)(st + (lw + c * LW) * 8 * NT_LDK), 16, 0, 0);
            __builtin_amdgcn_sched_barrier(0); // the wait in widen_store counts the loads in this order
#pragma unroll
            for (int c = 0; c < NA; c++) ra[slot][c] = *(const uint4_t *)(ga[c] + k0);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto widen_store = [&](int slot) __attribute__((always_inline)) {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0x0F70 | ((AHEAD * (LCHB + NA)) & 0xF) | ((((AHEAD * (LCHB + NA)) >> 4) & 0x3) << 14));
            half_t *st = ring + slot * STAGE_HALFS;
#pragma unroll
            for (int c = 0; c < NA; c++) {
                if (alive[c]) {
                    half2_t h[8];
#pragma unroll
                    for (int d = 0; d < 4; d++) nt_cvt_i8x4(ra[slot][c][d], h[2 * d], h[2 * d + 1]);
                    const uint4_t lo = {__builtin_bit_cast(uint32_t, h[0]), __builtin_bit_cast(uint32_t, h[1]),
                                        __builtin_bit_cast(uint32_t, h[2]), __builtin_bit_cast(uint32_t, h[3])};
                    const uint4_t hi = {__builtin_bit_cast(uint32_t, h[4]), __builtin_bit_cast(uint32_t, h[5]),
                                        __builtin_bit_cast(uint32_t, h[6]), __builtin_bit_cast(uint32_t, h[7])};
                    // the four lanes of a row store four of its eight slots, and two neighbouring rows have the same
                    // swizzle: odd rows store their odd slots first, so that eight consecutive lanes cover eight
                    // different 16-byte bank groups
                    const int flip = adst[c] & 1;
                    *(uint4_t *)(st + nt_slot(adst[c], 2 * piece + flip)) = flip ? hi : lo;
                    *(uint4_t *)(st + nt_slot(adst[c], 2 * piece + 1 - flip)) = flip ? lo : hi;
                }
            }
        };
        auto publish = [&]() __attribute__((always_inline)) {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the widened tile is in LDS
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        request(0, 0);
        request(1, 1);
        request(2, 2);
        widen_store(0);
        publish(); // tile 0
        for (int64_t kg = 0; kg < nk; kg += 4) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                request((u + 3) & 3, kg + u + 3); // into the stage that was read for the last time before the barrier of iteration kg + u - 1
                widen_store((u + 1) & 3);         // tile kg + u + 1
                publish();
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): nothing may land once the epilogue reuses the ring
        __syncthreads();
        return;
    }

    // ---- multiplying wavefronts: the f16 kernel's fragments, the Q8 fold
    const int wi = wave >> 1, wj = wave & 1;
    const int fr = lane & 15, fg = lane >> 4;
    const int swz = (fr >> 1) & 7;
    // this lane's scale rows: 16 bytes = the 8 blocks of four K tiles
    const half_t *sp[TM];
#pragma unroll
    for (int a = 0; a < TM; a++) {
        const int64_t gr = min(i0 + wi * WM + a * 16 + fr, g.M - 1);
        sp[a] = g.scales + ((a_el + gr * g.a_rs) >> 5);
    }
    struct Frags {
        half8_t a[TM], b[TN];
    };
    auto read_one = [&](int stage, int kk, Frags &f, int i) {
        const half_t *as = ring + stage * STAGE_HALFS + (wi * WM + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
        const half_t *bs = ring + stage * STAGE_HALFS + BM * NT_LDK + (wj * WN + fr) * NT_LDK + (((kk * 4 + fg) ^ swz) << 3);
        if (i < TM)
            f.a[i] = __builtin_bit_cast(half8_t, *(const uint4_t *)(as + i * 16 * NT_LDK));
        else
            f.b[i - TM] = __builtin_bit_cast(half8_t, *(const uint4_t *)(bs + (i - TM) * 16 * NT_LDK));
    };
    uint4_t sc_cur[TM], sc_nxt[TM];
#pragma unroll
    for (int a = 0; a < TM; a++) sc_cur[a] = *(const uint4_t *)sp[a];
    auto next_tile = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this tile's fragment reads have returned
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    next_tile(); // tile 0

    Frags r0, r1;
#pragma unroll
    for (int i = 0; i < NREAD; i++) read_one(0, 0, r0, i);
    int cur = 0, nxt = 1;
    auto scale_of = [&](int a, int blk) -> half_t { return __builtin_bit_cast(half8_t, sc_cur[a])[blk]; };
    float accs[TM][TN][4]; // the accumulators as scalars: each is written by a vector instruction of its own
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
#pragma unroll
            for (int r = 0; r < 4; r++) accs[a][b][r] = 0.f;
    // One K step (a block of 32): TM * TN MFMAs on the fragments in `rc` from zero, each folded into the
    // accumulators two MFMAs later with the scale of block `blk`; between them the fragment reads of the
    // following K step into `rn`.
    auto k_step = [&](const Frags &rc, Frags &rn, int blk, int rstage, int rkk) {
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
        float4_t P[3]; // partial sums of three tiles in flight: a tile is folded two MFMAs after its own
        int slot = 0;
#pragma unroll
        for (int idx = 0; idx < TM * TN + 2; idx++) {
            const int a = idx / TN, b = idx % TN;
            if (idx < TM * TN) {
                P[idx % 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(rc.b[b], rc.a[a], zero, 0, 0, 0);
                asm volatile("" : "+v"(P[idx % 3])); // instruction selection lets results nobody orders float: this MFMA is issued here
                if (slot < NREAD) read_one(rstage, rkk, rn, slot++); // the fragments of the following K step
            }
            if (idx >= 2) {
                const int fa = (idx - 2) / TN, fb = (idx - 2) % TN;
                const float d = (float)scale_of(fa, blk);
#pragma unroll
                for (int r = 0; r < 4; r++) accs[fa][fb][r] = fmaf(d, P[(idx - 2) % 3][r], accs[fa][fb][r]);
                // ... and the sums are folded here, not gathered at the end of the loop body with every partial sum kept alive
                asm volatile("" : "+v"(accs[fa][fb][0]), "+v"(accs[fa][fb][1]), "+v"(accs[fa][fb][2]), "+v"(accs[fa][fb][3]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int64_t kg = 0; kg < nk; kg += 4) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (u == 0) {
                // scales of the next group of four tiles, a group ahead of their use
                const int64_t gn = min(kg + 4, nk - 4) >> 2;
#pragma unroll
                for (int a = 0; a < TM; a++) sc_nxt[a] = *(const uint4_t *)(sp[a] + 8 * gn);
            }
            k_step(r0, r1, 2 * u, cur, 1);
            next_tile();
            k_step(r1, r0, 2 * u + 1, nxt, 0);
            cur = nxt;
            nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
        }
#pragma unroll
        for (int a = 0; a < TM; a++) sc_cur[a] = sc_nxt[a];
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    float4_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) acc[a][b] = float4_t{accs[a][b][0], accs[a][b][1], accs[a][b][2], accs[a][b][3]};
    nt_epilogue<TM, TN, WM, WN>(g, acc, smem, s, i0, j0, wi, wj, wave, lane);
}

// Second pass of a split-K launch: out = round(act(sum over the splits + bias)).  One thread per four
// consecutive i (the partial sums' contiguous axis); M need not be a multiple of four.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmNtArgs g) {
    const int64_t s = blockIdx.y;
    const int64_t mq = (g.M + 3) >> 2, total = mq * g.N;
    const float *pt = g.partial + s * g.ksplit * g.N * g.M;
    const int64_t sstride = g.N * g.M;
    half_t *out = g.out + s * g.o_bs;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t j = idx / mq, i = (idx - j * mq) << 2;
        const int n = (int)min<int64_t>(4, g.M - i);
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        const float *src = pt + j * g.M + i;
        if ((g.M & 3) == 0) {
            for (int sp = 0; sp < g.ksplit; sp++) {
                const float4_t t = *(const float4_t *)(src + sp * sstride);
                v[0] += t[0], v[1] += t[1], v[2] += t[2], v[3] += t[3];
            }
        } else {
            for (int sp = 0; sp < g.ksplit; sp++)
                for (int e = 0; e < n; e++) v[e] += src[sp * sstride + e];
        }
        half_t r[4];
        for (int e = 0; e < 4; e++) {
            float t = v[e];
            if (g.has_bias && e < n) t += (float)g.bias[g.bias_on_rows ? i + e : j];
            r[e] = (half_t)rt_act(t, g.act);
        }
        half_t *dst = out + i * g.o_is + j * g.o_js;
        if (n == 4 && g.vec_epilogue) {
            *(uint2_t *)dst = __builtin_bit_cast(uint2_t, half4_t{r[0], r[1], r[2], r[3]});
        } else {
            for (int e = 0; e < n; e++) dst[e * g.o_is] = r[e];
        }
    }
}

static hipError_t launch_splitk_reduce(const GemmNtArgs &g, int64_t stacks, hipStream_t st) {
    const int64_t total = ((g.M + 3) >> 2) * g.N;
    const unsigned gx = (unsigned)((total + 255) / 256 > 8192 ? 8192 : (total + 255) / 256);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(gx, (unsigned)stacks), dim3(256), 0, st, g);
    return hipGetLastError();
}

template <int BM, int BN, int LW>
static hipError_t launch_nt_q8w(const GemmNtArgs &g, int64_t stacks, hipStream_t st) {
    const size_t lds = (size_t)4 * (BM + BN) * NT_LDK * 2;
    if (const hipError_t e = ensure_lds_limit<&gemm_nt_q8w_kernel<BM, BN, LW>>(); e != hipSuccess) return e;
    dim3 grid((unsigned)((int64_t)g.tiles_i * g.tiles_j), (unsigned)stacks, (unsigned)g.ksplit);
    hipLaunchKernelGGL((gemm_nt_q8w_kernel<BM, BN, LW>), grid, dim3(NT_THREADS + 64 * LW), lds, st, g);
    if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    return g.ksplit > 1 ? launch_splitk_reduce(g, stacks, st) : hipSuccess;
}

// ---------------------------------------------------------------------------
// Short contractions (K <= 128: attention scores).  Such a product is a stream: the time
// goes into reading the operands once and writing the output.  A workgroup keeps a strip of
// 64 B rows (all of K) resident in LDS and walks the A row tiles of 128; the tile for step
// t+1 is prefetched into registers while step t is multiplied, and each wavefront stages and
// writes its own part of the output, so the stores of one step overlap the loads and MFMAs
// of the next.  K is padded with zeros to a multiple of 32 inside LDS only.
// ---------------------------------------------------------------------------
template <int KP>
__global__ __launch_bounds__(NT_THREADS, 2) void gemm_nt_shortk_kernel(GemmNtArgs g) {
    constexpr int BM = 128, BN = 64, WM = 64, WN = 32, TM = 4, TN = 2;
    constexpr int LDK = KP + 8;  // halfs per LDS row: an odd number of 16-byte slots, conflict-free fragment reads
    constexpr int KPV = KP / 8;  // 16-byte vectors per padded row
    constexpr int A_VEC = BM * KPV / NT_THREADS, B_VEC = BN * KPV / NT_THREADS;
    static_assert(KP % 32 == 0 && (BM * KPV) % NT_THREADS == 0 && (BN * KPV) % NT_THREADS == 0, "tile / thread split");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *Bs = (half_t *)smem;            // [BN][LDK]
    half_t *As = Bs + BN * LDK;             // [BM][LDK]
    uint8_t *Es = (uint8_t *)(As + BM * LDK); // per-wavefront output staging

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int fr = lane & 15, fg = lane >> 4;
    // Workgroups go to the eight XCDs round-robin by their linear number.  Taken as it comes, the strips of one stack
    // land on all eight and every L2 fetches that stack's operands (3 x the operand bytes at 32 x [512 x 80] . [512 x 80]^T);
    // when the grid divides by eight, XCD x takes the x-th eighth of the (stack, strip, part) items instead.
    uint32_t bx = blockIdx.x, by = blockIdx.y;
    if (const uint64_t total64 = (uint64_t)gridDim.x * gridDim.y; total64 < (1u << 31) && (total64 & 7u) == 0) {
        const uint32_t total = (uint32_t)total64;
        const uint32_t lin = blockIdx.x + gridDim.x * blockIdx.y, w = (lin & 7u) * (total >> 3) + (lin >> 3);
        by = w / gridDim.x, bx = w - by * gridDim.x;
    }
    // bx = strip * parts + part: the workgroups of a strip take its A tiles round-robin
    const int parts = g.tiles_i, part = (int)(bx % parts);
    const int64_t j0 = (int64_t)(bx / parts) * BN;
    const int64_t s = by;
    const int64_t a_el = (g.a_stack == 1 ? 0 : s) * g.a_bs, b_el = (g.b_stack == 1 ? 0 : s) * g.b_bs;
    const int kvecs = (int)(g.K >> 3);
    const uint4_t zero4 = {0u, 0u, 0u, 0u};

    // the B strip: global -> registers -> LDS, vectors past K zeroed
    {
        uint4_t rb[B_VEC];
#pragma unroll
        for (int e = 0; e < B_VEC; e++) {
            const int v = e * NT_THREADS + t, r = v / KPV, c = v - r * KPV;
            const int64_t gr = min(j0 + r, g.N - 1);
            rb[e] = *(const uint4_t *)(g.B + b_el + gr * g.b_js + 8 * min(c, kvecs - 1));
        }
#pragma unroll
        for (int e = 0; e < B_VEC; e++) {
            const int v = e * NT_THREADS + t, r = v / KPV, c = v - r * KPV;
            *(uint4_t *)(Bs + r * LDK + 8 * c) = c < kvecs ? rb[e] : zero4;
        }
    }
    uint4_t ra[A_VEC];
    auto load_a = [&](int64_t i0) {
#pragma unroll
        for (int e = 0; e < A_VEC; e++) {
            const int v = e * NT_THREADS + t, r = v / KPV, c = v - r * KPV;
            const int64_t gr = min(i0 + r, g.M - 1); // rows past the end duplicate the last one; never stored
            ra[e] = *(const uint4_t *)((const half_t *)g.A + a_el + gr * g.a_rs + 8 * min(c, kvecs - 1));
        }
    };
    auto store_a = [&]() {
#pragma unroll
        for (int e = 0; e < A_VEC; e++) {
            const int v = e * NT_THREADS + t, r = v / KPV, c = v - r * KPV;
            *(uint4_t *)(As + r * LDK + 8 * c) = c < kvecs ? ra[e] : zero4;
        }
    };
    const int64_t ntile = (g.M + BM - 1) / BM;
    load_a((int64_t)part * BM);
    for (int64_t it = part; it < ntile; it += parts) {
        store_a();
        __syncthreads();
        if (it + parts < ntile) load_a((it + parts) * BM); // in flight under the MFMAs and the output stage
        float4_t acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int b = 0; b < TN; b++) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KP / 32; kk++) {
            half8_t fa[TM], fb[TN];
#pragma unroll
            for (int a = 0; a < TM; a++)
                fa[a] = __builtin_bit_cast(half8_t, *(const uint4_t *)(As + (wi * WM + a * 16 + fr) * LDK + kk * 32 + 8 * fg));
#pragma unroll
            for (int b = 0; b < TN; b++)
                fb[b] = __builtin_bit_cast(half8_t, *(const uint4_t *)(Bs + (wj * WN + b * 16 + fr) * LDK + kk * 32 + 8 * fg));
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[b], fa[a], acc[a][b], 0, 0, 0);
        }
        __syncthreads(); // every wavefront is done with As before the next tile overwrites it
        nt_epilogue<TM, TN, WM, WN>(g, acc, Es, s, it * BM, j0, wi, wj, wave, lane);
    }
}

// g.tiles_i carries the number of workgroups that share a strip.
template <int KP> static hipError_t launch_nt_shortk(const GemmNtArgs &g, int64_t stacks, hipStream_t st) {
    const size_t lds = (size_t)(64 + 128) * (KP + 8) * 2 + (size_t)4 * 32 * (64 + 8) * 2;
    if (const hipError_t e = ensure_lds_limit<&gemm_nt_shortk_kernel<KP>>(); e != hipSuccess) return e;
    dim3 grid((unsigned)((g.N + 63) / 64 * g.tiles_i), (unsigned)stacks);
    hipLaunchKernelGGL((gemm_nt_shortk_kernel<KP>), grid, dim3(NT_THREADS), lds, st, g);
    return hipGetLastError();
}

template <int BM, int BN, int STAGES, int LW>
static hipError_t launch_nt_dl(const GemmNtArgs &g, int64_t stacks, hipStream_t st) {
    const size_t lds = (size_t)STAGES * (BM + BN) * NT_LDK * 2;
    if (const hipError_t e = ensure_lds_limit<&gemm_nt_dl_kernel<BM, BN, STAGES, LW>>(); e != hipSuccess) return e;
    dim3 grid((unsigned)((int64_t)g.tiles_i * g.tiles_j), (unsigned)stacks, (unsigned)g.ksplit);
    hipLaunchKernelGGL((gemm_nt_dl_kernel<BM, BN, STAGES, LW>), grid, dim3(NT_THREADS + 64 * LW), lds, st, g);
    if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    return g.ksplit > 1 ? launch_splitk_reduce(g, stacks, st) : hipSuccess;
}

// Tunables: non-zero keeps f16 problems on the register-staged kernel; LDS ring depth
// (3 or 4, 0 = 3) of the direct-to-LDS kernel (for comparisons).
RT_TUNABLE(g_gemm_nt_no_direct, 0);
RT_TUNABLE(g_gemm_nt_stages, 0);
RT_TUNABLE(g_gemm_nt_narrow, 0); // 1: never the 64- and 96-row tiles for few activation rows (for comparisons)
RT_TUNABLE(g_gemm_nt_shortk_parts, 0); // workgroups per strip of the short-K kernel (0 = automatic)

template <int BM, int BN, bool Q8, bool KFULL>
static hipError_t launch_nt(const GemmNtArgs &g, int64_t stacks, hipStream_t st) {
    const size_t lds = (size_t)2 * (BM + BN) * NT_LDK * 2 + (Q8 ? (size_t)4 * BM * 4 : 0);
    if (const hipError_t e = ensure_lds_limit<&gemm_nt_kernel<BM, BN, Q8, KFULL>>(); e != hipSuccess) return e;
    dim3 grid((unsigned)((int64_t)g.tiles_i * g.tiles_j), (unsigned)stacks);
    hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, Q8, KFULL>), grid, dim3(NT_THREADS), lds, st, g);
    return hipGetLastError();
}

// Tunable: 0 = automatic, 1 = never take this kernel (for comparisons).
RT_TUNABLE(g_gemm_nt_disable, 0);

// f16 or Q8_0H A with K-contiguous rows, f16 B with K-contiguous rows.
// hipErrorNotSupported: the problem does not fit; the generic tiled GEMM runs instead.
// Workgroups that share one output tile's K.  A product with few output tiles and a long K (the
// Phi-2 down-projection: 64 tiles of 160 x 128, K = 10240) leaves most compute units idle; with a
// workspace its K is cut into equal shares of a whole number of 256-wide units, at least 1024 each.
// Applies to the shapes the direct-to-LDS kernels take (after the operand exchange for row-major outputs).
static int gemm_nt_ksplit(const Problem &p, const DeviceInfo &dev) {
    if (p.act_dt != RT_F16 || (p.a_dt != RT_F16 && p.a_dt != RT_Q8_0H) || p.K % 256 != 0 || p.K <= 256) return 1;
    const int64_t tiles = ((p.M + 159) / 160) * ((p.N + 127) / 128) * p.stacks;
    if (tiles <= 0 || tiles * 2 > dev.num_cus) return 1;
    const int64_t units = p.K / 256;
    int best = 1;
    for (int ks = 2; ks <= 8 && tiles * ks <= dev.num_cus; ks++)
        if (units % ks == 0 && units / ks >= 4) best = ks;
    return best;
}

// exchanges the operands' roles when that makes the output's contiguous axis the kernel's i axis
static bool nt_orient(Problem &p) {
    if (p.a_dt == RT_F16 && p.act_dt == RT_F16 && p.o_js == 1 && p.o_is != 1) {
        std::swap(p.M, p.N);
        std::swap(p.a_stack, p.b_stack);
        std::swap(p.a_bs, p.b_bs);
        std::swap(p.a_rs, p.b_js);
        std::swap(p.a_ks, p.b_ks);
        std::swap(p.o_is, p.o_js);
        p.bias_on_rows = !p.bias_on_rows;
        return true;
    }
    return false;
}

// bytes of workspace with which launch_gemm_nt splits this problem's K (0: it does not)
uint64_t gemm_nt_workspace_bytes(const Problem &p0, const DeviceInfo &dev) {
    Problem p = p0;
    nt_orient(p);
    if (p.a_ks != 1 || p.b_ks != 1 || p.M < 160 || p.N < 5) return 0;
    const int ks = gemm_nt_ksplit(p, dev);
    return ks > 1 ? (uint64_t)p.stacks * ks * p.M * p.N * sizeof(float) : 0;
}

hipError_t launch_gemm_nt(const Problem &p0, const void *A, const void *B, const void *bias, void *out,
                          hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemm_nt_disable) return hipErrorNotSupported;
    Problem p = p0;
    // Row-major output: compute the transposed product (operands exchanged), so that the
    // kernel's contiguous output axis, the one its 128-bit epilogue writes along, is this
    // problem's column axis.
    if (nt_orient(p)) std::swap(A, B);
    if (p.act_dt != RT_F16 || (p.a_dt != RT_F16 && p.a_dt != RT_Q8_0H)) return hipErrorNotSupported;
    if (p.a_ks != 1 || p.b_ks != 1 || p.K % 8 != 0 || p.K < 8) return hipErrorNotSupported;
    if (p.stacks > 65535 || p.M < 1 || p.N < 1) return hipErrorNotSupported;
    const bool q8 = p.a_dt == RT_Q8_0H;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_js * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    if (q8 ? (p.K % 32 != 0) : ((p.a_rs * 2) % 16 != 0 || (p.a_bs * 2) % 16 != 0)) return hipErrorNotSupported;
    // small problems do not fill the tiles; the generic kernel handles them (at 10240 x 2560 f16 weights it takes
    // 19.7 us for 8 activation rows and 33 us for 16..48, the 64-row tiles here 17.4 us for any count up to 64)
    if (p.M < 160 || p.N < 5) return hipErrorNotSupported;

    GemmNtArgs g{};
    g.A = A, g.B = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    if (q8) g.scales = (const half_t *)((const uint8_t *)A + rt_q8_0_scale_offset((uint64_t)p.a_stack * p.M * p.K));
    g.M = p.M, g.N = p.N, g.K = p.K;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.a_bs = p.a_bs, g.a_rs = p.a_rs;
    g.b_bs = p.b_bs, g.b_js = p.b_js;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    g.vec_epilogue = p.o_is == 1 && p.o_js % 8 == 0 && p.o_bs % 8 == 0 && ((uintptr_t)out & 15u) == 0;
    g.ksplit = 1, g.k_len = p.K, g.partial = nullptr;
    const bool kfull = p.K % NT_BK == 0;
    if (!q8 && p.K <= 128 && g.vec_epilogue && !g_gemm_nt_no_direct && (p.N + 63) / 64 <= 0x7fffffff) {
        // resident-strip kernel; vec_epilogue means the output's i axis is contiguous.  Strips are
        // split over several workgroups until the grid has a few workgroups per compute unit.
        const int64_t strips = (p.N + 63) / 64 * p.stacks, atiles = (p.M + 127) / 128;
        int parts = 1;
        while (parts < atiles && strips * parts < 2 * (int64_t)dev.num_cus) parts *= 2;
        if (g_gemm_nt_shortk_parts > 0) parts = g_gemm_nt_shortk_parts;
        g.tiles_i = (int)(parts < atiles ? parts : atiles);
        if (p.K <= 32) return launch_nt_shortk<32>(g, p.stacks, stream);
        if (p.K <= 64) return launch_nt_shortk<64>(g, p.stacks, stream);
        if (p.K <= 96) return launch_nt_shortk<96>(g, p.stacks, stream);
        return launch_nt_shortk<128>(g, p.stacks, stream);
    }
    if (!q8 && p.K <= 256) {
        // Short contractions (attention scores): the time goes into writing the output, not into
        // the K loop.  128 x 64 tiles need a third of the registers and LDS, so several
        // workgroups share a compute unit and one's epilogue overlaps another's loads.
        constexpr int SBM = 128, SBN = 64; // 128 outputs along the contiguous axis: whole cache lines per wavefront row
        const int64_t ti = (p.M + SBM - 1) / SBM, tj = (p.N + SBN - 1) / SBN;
        if (ti * tj > 0x7fffffff) return hipErrorNotSupported;
        g.tiles_i = (int)ti, g.tiles_j = (int)tj;
        return kfull ? launch_nt<SBM, SBN, false, true>(g, p.stacks, stream)
                     : launch_nt<SBM, SBN, false, false>(g, p.stacks, stream);
    }
    constexpr int BM = 160, BN = 128;
    const int64_t ti = (p.M + BM - 1) / BM, tj = (p.N + BN - 1) / BN;
    if (ti * tj > 0x7fffffff) return hipErrorNotSupported;
    g.tiles_i = (int)ti, g.tiles_j = (int)tj;
    // few activation rows: 160-row tiles leave most compute units idle and a workgroup takes as long for one
    // column of tiles as for four; 64-row tiles, while all of them still run at once, put 2.5 times the workgroups to work
    // (10240 x 2560 f16 weights: 65..128 rows 24.6-25.4 -> 17.2-18.1 us); 96-row tiles where those no longer fit.
    const int64_t ti64 = (p.M + 63) / 64, ti96 = (p.M + 95) / 96;
    const bool few = g_gemm_nt_narrow != 1 && ti * tj * p.stacks * 2 <= dev.num_cus;
    const int bm = few && ti64 * tj * p.stacks <= dev.num_cus ? 64 : few && ti96 * tj * p.stacks <= dev.num_cus ? 96 : BM;
    const bool dl_f16 = !q8 && kfull && !g_gemm_nt_no_direct;
    const bool dl_q8 = q8 && p.K % 256 == 0 && !g_gemm_nt_no_direct && ((uintptr_t)g.scales & 15u) == 0 && (p.a_bs % 512) == 0;
    if (dl_f16 || dl_q8) {
        const int ks = gemm_nt_ksplit(p, dev);
        if (ks > 1 && p.workspace && !((uintptr_t)p.workspace & 15u) &&
            p.workspace_bytes >= (uint64_t)p.stacks * ks * p.M * p.N * sizeof(float))
            g.ksplit = ks, g.k_len = p.K / ks, g.partial = (float *)p.workspace;
    }
    if ((dl_f16 || dl_q8) && bm != BM && g.ksplit == 1) {
        g.tiles_i = (int)(bm == 64 ? ti64 : ti96);
        // the narrow tiles take as deep a ring as the LDS holds: a stage has only 8 or 12 KB of weights, and what a compute
        // unit has in flight is what it can pull (10240 x 2560 f16 weights, 40 / 64 activation rows, three stages -> six:
        // 22.7 / 23.6 -> 20.0 / 22.1 us with the weights in HBM, 16.3 / 16.8 -> 14.8 / 15.7 from the Infinity Cache)
        if (dl_f16 && bm == 64 && p.N <= 64) {
            // up to 64 activation rows: half the activation tile, a stage of 16 KB and nine of them (40 / 64 rows:
            // 20.0 / 22.1 -> 18.3 / 20.5 us with the weights in HBM, 14.8 / 15.7 -> 12.6 / 13.6 from the Infinity Cache)
            g.tiles_j = 1;
            return launch_nt_dl<64, 64, 9, 2>(g, p.stacks, stream);
        }
        if (dl_f16) return bm == 64 ? launch_nt_dl<64, BN, 6, 2>(g, p.stacks, stream) : launch_nt_dl<96, BN, 5, 2>(g, p.stacks, stream);
        if (bm == 64 && p.N <= 64) {
            // up to 64 activation rows: half the activation tile is half the MFMAs and folds of a workgroup
            g.tiles_j = 1;
            return launch_nt_q8w<64, 64, 4>(g, p.stacks, stream);
        }
        return bm == 64 ? launch_nt_q8w<64, BN, 4>(g, p.stacks, stream) : launch_nt_q8w<96, BN, 4>(g, p.stacks, stream);
    }
    if (dl_f16) {
        // two loading wavefronts: one and four measured the same within run-to-run spread
        return g_gemm_nt_stages == 4 ? launch_nt_dl<BM, BN, 4, 2>(g, p.stacks, stream)
                                     : launch_nt_dl<BM, BN, 3, 2>(g, p.stacks, stream);
    }
    if (dl_q8)
        return launch_nt_q8w<BM, BN, 4>(g, p.stacks, stream);
    if (q8) return kfull ? launch_nt<BM, BN, true, true>(g, p.stacks, stream) : launch_nt<BM, BN, true, false>(g, p.stacks, stream);
    return kfull ? launch_nt<BM, BN, false, true>(g, p.stacks, stream) : launch_nt<BM, BN, false, false>(g, p.stacks, stream);
}

} // namespace rt

#if RT_NT_ABLATION
// Entry point of a timing-only build of this file (see RT_NT_ABLATION): the Linear form W[n x k] . X[m x k]^T + bias
// with f16 weights, output [m x n].  The measurement probes library holds one such build per variant.
extern "C" __attribute__((visibility("default"))) int RT_NT_ABL_ENTRY(const void *W, const void *X, const void *bias, void *out,
                                                                      int64_t n, int64_t m, int64_t k, void *stream) {
    rt::Problem p;
    p.a_dt = RT_F16, p.act_dt = RT_F16, p.M = n, p.N = m, p.K = k;
    p.a_rs = k, p.a_ks = 1, p.b_ks = 1, p.b_js = k, p.o_is = 1, p.o_js = n, p.has_bias = true, p.bias_on_rows = true;
    p.kernel = RT_KERNEL_GEMM_F16;
    return (int)rt::launch_gemm_nt(p, W, X, bias, out, (hipStream_t)stream, rt::DeviceInfo{});
}
#endif
