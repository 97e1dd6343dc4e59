// LDS-tiled MFMA GEMM for gfx950:  C[s, i, j] = sum_k A[s, i, k] * B[s, k, j] (+ bias)
// with arbitrary element strides on both operands and on the output, so the
// operator's trans_lhs / trans_rhs / trans_out flags and the stack broadcast
// are pure addressing.  The product always accumulates in f32 on the matrix
// cores (v_mfma_f32_32x32x16_f16 for f16 operands, v_mfma_f32_32x32x2_f32 for
// f32).
//
// A may also be a quantized weight (Q8_0 segments, Q4_K super-blocks).  Its
// integer codes are written to LDS unscaled (an int8 or a nibble is exact in
// f16), one K tile is exactly one quantization block, and the block's scale is
// applied in f32 to the tile's partial sums:
//   Q8_0:  acc += d * sum_k q x
//   Q4_K:  acc += (d*sc) * sum_k q x  -  (dmin*mn) * sum_k x
// so no weight is ever rounded to f16.  For these modes the MFMA operands are
// exchanged so that a lane owns one weight row and needs one scale per tile.
//
// Tile: 128 x 128 outputs per 256-thread workgroup (4 wavefronts as 2 x 2, each
// 64 x 64 = 2 x 2 MFMA tiles), K step 32; problems whose 128 x 128 tiling would
// leave compute units idle take 64 x 64 tiles (one MFMA tile per wavefront).  Both operand tiles sit in LDS with K
// contiguous so every MFMA fragment is one vector read.  Global loads for
// tile t+1 are issued before the MFMAs of tile t and written to LDS after them.
//
// Roles in the reference: ops/gemm.rs:305-657 (scalar, vec4 and Q8_0 GEMM
// generators).
#include "device_common.h"

namespace rt {

constexpr int BK = 32;
constexpr int kGemmThreads = 256;

enum LoadMode { LM_GEN = 0, LM_VECK = 1, LM_VECR = 2, LM_Q8 = 3, LM_Q4K = 4 };

struct GemmArgs {
    const void *A;
    const void *scales; // Q8_0 scale stream of A
    const void *B;
    const void *bias;
    void *out;
    int64_t M, N, K;
    int64_t a_stack, b_stack;
    int64_t a_bs, a_rs, a_ks;
    int64_t b_bs, b_ks, b_js;
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
};

template <typename T> struct Tile;
template <> struct Tile<half_t> {
    static constexpr int PAD = 8, VEC = 8, KSTEP = 16;
    using Frag = half8_t;
    using Vec = half8_t;
};
template <> struct Tile<float> {
    static constexpr int PAD = 4, VEC = 4, KSTEP = 2;
    using Frag = float;
    using Vec = float4_t;
};

// Registers a thread holds for one operand tile between the global load and
// the LDS store.
template <typename T, int MODE, int E> struct TileRegs {
    T v[E];
};
template <typename T, int E> struct TileRegs<T, LM_Q8, E> {
    uint4_t q;
    T d; // the block's scale as stored (f16 for Q8_0H, f32 for Q8_0F): widened when stored to LDS
};
template <typename T, int E> struct TileRegs<T, LM_Q4K, E> {
    uint4_t q, hdr; // raw nibbles and the super-block's header: decoded when stored, not when loaded,
    int j;          // so that nothing waits for the load where it is issued; j = sub-block within the super-block
};

// Operand tile loader for a tile of ROWS rows (64 or 128).  `rows` is the operand's
// outer extent (M for A, N for B), `r0` the tile's first row, `rs`/`ks` the element
// strides of (row, k).
template <typename T, int MODE, int ROWS> struct Loader {
    static constexpr int E = ROWS * BK / kGemmThreads; // elements per thread
    using R = TileRegs<T, MODE, E>;
    static constexpr int VEC = Tile<T>::VEC;
    static constexpr int LDK = BK + Tile<T>::PAD;

    // KFULL: K is a whole number of tiles, so the vector loaders need no bound along K.
    template <bool KFULL = false>
    __device__ __forceinline__ static void load(R &r, const void *base_v, const void *scales_v, int64_t stack_el,
                                                int64_t rows, int64_t r0, int64_t K, int64_t k0, int64_t rs,
                                                int64_t ks, int t) {
        if constexpr (MODE == LM_GEN) {
            const T *base = (const T *)base_v + stack_el;
            // Walk the tile so that consecutive threads touch consecutive
            // addresses of whichever axis is contiguous in memory.
            const bool k_fast = ks <= rs;
#pragma unroll
            for (int e = 0; e < E; e++) {
                const int idx = e * kGemmThreads + t;
                const int rr = k_fast ? idx / BK : idx % ROWS;
                const int kk = k_fast ? idx % BK : idx / ROWS;
                const int64_t gr = r0 + rr, gk = k0 + kk;
                T v = (T)0;
                if (gr < rows && gk < K) v = base[gr * rs + gk * ks];
                r.v[e] = v;
            }
        } else if constexpr (MODE == LM_VECK) {
            const T *base = (const T *)base_v + stack_el;
            constexpr int VPR = BK / VEC; // vectors per row
#pragma unroll
            for (int e = 0; e < E / VEC; e++) {
                const int v = e * kGemmThreads + t;
                const int rr = v / VPR, kv = v % VPR;
                int64_t gr = r0 + rr;
                if (gr >= rows) gr = rows - 1; // duplicate row; its outputs are never stored
                const int64_t gk = k0 + kv * VEC;
                typename Tile<T>::Vec x = {};
                if (KFULL || gk < K) x = *(const typename Tile<T>::Vec *)(base + gr * rs + gk);
#pragma unroll
                for (int i = 0; i < VEC; i++) r.v[e * VEC + i] = x[i];
            }
        } else if constexpr (MODE == LM_VECR) {
            const T *base = (const T *)base_v + stack_el;
            constexpr int VPK = ROWS / VEC; // vectors per k
#pragma unroll
            for (int e = 0; e < E / VEC; e++) {
                const int v = e * kGemmThreads + t;
                const int kk = v / VPK, rv = v % VPK;
                int64_t gr = r0 + rv * VEC;
                if (gr >= rows) gr = rows - VEC; // rows % VEC == 0: a vector is wholly in or out; out -> any valid one
                const int64_t gk = k0 + kk;
                typename Tile<T>::Vec x = {};
                if (KFULL || gk < K) x = *(const typename Tile<T>::Vec *)(base + gk * ks + gr);
#pragma unroll
                for (int i = 0; i < VEC; i++) r.v[e * VEC + i] = x[i];
            }
        } else if constexpr (MODE == LM_Q8) {
            // 32 int8 per row per k tile: two threads per row, 16 bytes each.
            const int rr = (t >> 1) % ROWS, hf = t & 1; // ROWS = 64: the upper half of the block repeats the lower
            int64_t gr = r0 + rr;
            if (gr >= rows) gr = rows - 1;
            const int64_t el = stack_el + gr * rs + k0; // flat element index of the block start
            r.q = *(const uint4_t *)((const uint8_t *)base_v + el + 16 * hf);
            r.d = ((const T *)scales_v)[el >> 5];
        } else { // LM_Q4K: one sub-block of 32 weights per row per k tile
            const int rr = (t >> 1) % ROWS, hf = t & 1;
            int64_t gr = r0 + rr;
            if (gr >= rows) gr = rows - 1;
            const int64_t sb = (stack_el + gr * rs + k0) >> 8; // super-block index
            const int j = (int)((k0 & 255) >> 5);              // sub-block within it
            const uint8_t *blk = (const uint8_t *)base_v + sb * 144;
            r.hdr = *(const uint4_t *)blk;
            r.q = *(const uint4_t *)(blk + 16 + 32 * (j >> 1) + 16 * hf);
            r.j = j;
        }
    }

    // `sd` / `sm` receive the tile's per-row scale (and Q4_K min) for the quantized modes.
    __device__ __forceinline__ static void store(const R &r, T (*S)[LDK], float *sd, float *sm, int64_t rs,
                                                 int64_t ks, int t) {
        if constexpr (MODE == LM_GEN) {
            const bool k_fast = ks <= rs;
#pragma unroll
            for (int e = 0; e < E; e++) {
                const int idx = e * kGemmThreads + t;
                const int rr = k_fast ? idx / BK : idx % ROWS;
                const int kk = k_fast ? idx % BK : idx / ROWS;
                S[rr][kk] = r.v[e];
            }
        } else if constexpr (MODE == LM_VECK) {
            constexpr int VPR = BK / VEC;
#pragma unroll
            for (int e = 0; e < E / VEC; e++) {
                const int v = e * kGemmThreads + t;
                const int rr = v / VPR, kv = v % VPR;
                typename Tile<T>::Vec x;
#pragma unroll
                for (int i = 0; i < VEC; i++) x[i] = r.v[e * VEC + i];
                *(typename Tile<T>::Vec *)&S[rr][kv * VEC] = x;
            }
        } else if constexpr (MODE == LM_VECR) {
            constexpr int VPK = ROWS / VEC;
#pragma unroll
            for (int e = 0; e < E / VEC; e++) {
                const int v = e * kGemmThreads + t;
                const int kk = v / VPK, rv = v % VPK;
#pragma unroll
                for (int i = 0; i < VEC; i++) S[rv * VEC + i][kk] = r.v[e * VEC + i];
            }
        } else if constexpr (MODE == LM_Q8) {
            const int rr = (t >> 1) % ROWS, hf = t & 1;
            T w[16];
#pragma unroll
            for (int i = 0; i < 16; i++) w[i] = (T)(int)(int8_t)(r.q[i >> 2] >> (8 * (i & 3))); // exact
#pragma unroll
            for (int v = 0; v < 16 / VEC; v++) {
                typename Tile<T>::Vec x;
#pragma unroll
                for (int i = 0; i < VEC; i++) x[i] = w[v * VEC + i];
                *(typename Tile<T>::Vec *)&S[rr][16 * hf + v * VEC] = x;
            }
            if (hf == 0) sd[rr] = (float)r.d;
        } else {
            const int rr = (t >> 1) % ROWS, hf = t & 1;
            const uint4_t hdr = r.hdr;
            const int j = r.j;
            const half2_t dm = __builtin_bit_cast(half2_t, hdr[0]);
            // scale bytes live in hdr[1..3]; select without indexing memory
            auto sbyte = [&](int i) -> uint32_t { return (hdr[1 + (i >> 2)] >> (8 * (i & 3))) & 0xFFu; };
            uint32_t sc, mn;
            if (j < 4) {
                sc = sbyte(j) & 63u;
                mn = sbyte(j + 4) & 63u;
            } else {
                sc = (sbyte(j + 4) & 0xFu) | ((sbyte(j - 4) >> 6) << 4);
                mn = (sbyte(j + 4) >> 4) | ((sbyte(j) >> 6) << 4);
            }
            const float d = (float)dm[0] * (float)sc, m = (float)dm[1] * (float)mn;
            // the nibble the tile needs in the low 4 bits of every byte
            const uint4_t q = (j & 1) ? uint4_t{r.q[0] >> 4, r.q[1] >> 4, r.q[2] >> 4, r.q[3] >> 4} : r.q;
            T w[16];
#pragma unroll
            for (int i = 0; i < 16; i++) w[i] = (T)(int)((q[i >> 2] >> (8 * (i & 3))) & 0xFu); // exact
#pragma unroll
            for (int v = 0; v < 16 / VEC; v++) {
                typename Tile<T>::Vec x;
#pragma unroll
                for (int i = 0; i < VEC; i++) x[i] = w[v * VEC + i];
                *(typename Tile<T>::Vec *)&S[rr][16 * hf + v * VEC] = x;
            }
            if (hf == 0) sd[rr] = d, sm[rr] = m;
        }
    }
};

template <typename T>
__device__ __forceinline__ float16_t mma(typename Tile<T>::Frag a, typename Tile<T>::Frag b, float16_t c) {
    if constexpr (sizeof(T) == 2)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <typename T, int AMODE, int BMODE, int BM, int BN>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmArgs g) {
    constexpr int LDK = BK + Tile<T>::PAD;
    constexpr int WM = BM / 2, WN = BN / 2; // a wavefront's share of the tile
    constexpr int TA = WM / 32, TB = WN / 32; // in 32 x 32 MFMA tiles
    constexpr bool QUANT = AMODE == LM_Q8 || AMODE == LM_Q4K;
    // quantized weights: two LDS stages (the next tile is stored while this one is multiplied)
    constexpr int NST = QUANT ? 2 : 1;
    __shared__ __attribute__((aligned(16))) T As[NST][BM][LDK];
    __shared__ __attribute__((aligned(16))) T Bs[NST][BN][LDK];
    __shared__ float Sd[NST][QUANT ? BM : 1]; // per-row scale of the K tile
    __shared__ float Sm[NST][AMODE == LM_Q4K ? BM : 1];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wi = wave >> 1, wj = wave & 1; // wave position in the 2 x 2 grid
    const int64_t s = blockIdx.z;
    const int64_t i0 = (int64_t)blockIdx.y * BM, j0 = (int64_t)blockIdx.x * BN;
    // an operand's stack is either the full stack or 1 (broadcast)
    const int64_t a_el = (g.a_stack == 1 ? 0 : s) * g.a_bs, b_el = (g.b_stack == 1 ? 0 : s) * g.b_bs;

    using LA = Loader<T, AMODE, BM>;
    using LB = Loader<T, BMODE, BN>;
    float16_t acc[TA][TB];
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < TB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    typename Tile<T>::Frag ones;
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < 8; i++) ones[i] = (half_t)1;
    } else {
        ones = 1.f;
    }

    // MFMAs of the K tile that sits in LDS
    auto compute_tile = [&](int st) {
        constexpr int KSTEP = Tile<T>::KSTEP;
        float16_t part[TA][TB], xsum[TB];
        if constexpr (QUANT) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
#pragma unroll
                for (int b = 0; b < TB; b++) {
                    xsum[b][r] = 0.f;
#pragma unroll
                    for (int a = 0; a < TA; a++) part[a][b][r] = 0.f;
                }
            }
        }
#pragma unroll
        for (int kk = 0; kk < BK / KSTEP; kk++) {
            typename Tile<T>::Frag fa[TA], fb[TB];
            if constexpr (sizeof(T) == 2) {
                const int ko = kk * 16 + 8 * (lane >> 5);
#pragma unroll
                for (int a = 0; a < TA; a++) fa[a] = *(const half8_t *)&As[st][wi * WM + a * 32 + (lane & 31)][ko];
#pragma unroll
                for (int b = 0; b < TB; b++) fb[b] = *(const half8_t *)&Bs[st][wj * WN + b * 32 + (lane & 31)][ko];
            } else {
                const int ko = kk * 2 + (lane >> 5);
#pragma unroll
                for (int a = 0; a < TA; a++) fa[a] = As[st][wi * WM + a * 32 + (lane & 31)][ko];
#pragma unroll
                for (int b = 0; b < TB; b++) fb[b] = Bs[st][wj * WN + b * 32 + (lane & 31)][ko];
            }
            if constexpr (QUANT) {
                // operands exchanged: the lane index follows A's row (one scale per lane),
                // the register index follows B's column
#pragma unroll
                for (int a = 0; a < TA; a++)
#pragma unroll
                    for (int b = 0; b < TB; b++) part[a][b] = mma<T>(fb[b], fa[a], part[a][b]);
                if constexpr (AMODE == LM_Q4K) {
                    // sum_k x[j, k] for the columns this lane's registers follow
#pragma unroll
                    for (int b = 0; b < TB; b++) xsum[b] = mma<T>(fb[b], ones, xsum[b]);
                }
            } else {
#pragma unroll
                for (int a = 0; a < TA; a++)
#pragma unroll
                    for (int b = 0; b < TB; b++) acc[a][b] = mma<T>(fa[a], fb[b], acc[a][b]);
            }
        }
        if constexpr (QUANT) {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                const float d = Sd[st][wi * WM + a * 32 + (lane & 31)];
                float m = 0.f;
                if constexpr (AMODE == LM_Q4K) m = Sm[st][wi * WM + a * 32 + (lane & 31)];
#pragma unroll
                for (int b = 0; b < TB; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        acc[a][b][r] = fmaf(d, part[a][b][r], acc[a][b][r]);
                        if constexpr (AMODE == LM_Q4K) acc[a][b][r] = fmaf(-m, xsum[b][r], acc[a][b][r]);
                    }
            }
        }
    };

    const int64_t ntiles = (g.K + BK - 1) / BK;
    if constexpr (QUANT) {
        // Quantized weights: a K tile is one block of 32 and its MFMAs are few, so a load issued one
        // tile ahead would be waited for almost at once.  Four tiles (two for 128-row tiles, whose
        // accumulators leave fewer registers: a third wavefront-per-SIMD slot lost costs more than the
        // shorter ring) are kept in flight in a ring of register sets; the loads have no bounds (K is a whole number of blocks; past the last tile
        // the last one is loaded again and never stored), so the loop is straight-line code and the
        // compiler's wait counts are exact; and the barriers wait for the LDS operations only, not
        // for the loads that are meant to stay in flight across them.
        constexpr int PF = BM >= 128 ? 2 : 4;
        typename LA::R qa[PF];
        typename LB::R qb[PF];
        auto load_tile = [&](int64_t kt, typename LA::R &a, typename LB::R &b) {
            const int64_t k0 = min(kt, ntiles - 1) * BK;
            LA::template load<true>(a, g.A, g.scales, a_el, g.M, i0, g.K, k0, g.a_rs, g.a_ks, t);
            LB::template load<true>(b, g.B, nullptr, b_el, g.N, j0, g.K, k0, g.b_js, g.b_ks, t);
        };
        auto lds_barrier = [&]() {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        // Tile kt is multiplied from stage kt & 1; `a` / `b` hold tile kt + 1 (loaded PF - 1 iterations
        // ago), which goes to the other stage after the MFMAs, and then take tile kt + 1 + PF.  One
        // barrier per tile: behind it stage (kt + 1) & 1 is complete and stage kt & 1 is free.
        auto k_tile = [&](int64_t kt, typename LA::R &a, typename LB::R &b) {
            const int st = (int)(kt & 1);
            compute_tile(st);
            LA::store(a, As[st ^ 1], Sd[st ^ 1], Sm[st ^ 1], g.a_rs, g.a_ks, t);
            LB::store(b, Bs[st ^ 1], nullptr, nullptr, g.b_js, g.b_ks, t);
            load_tile(kt + 1 + PF, a, b);
            lds_barrier();
        };
        if (ntiles > 0) {
            // tile 0 goes through register set PF - 1 into stage 0; sets 0 .. PF - 1 then hold tiles 1 .. PF
            load_tile(0, qa[PF - 1], qb[PF - 1]);
#pragma unroll
            for (int p2 = 0; p2 < PF - 1; p2++) load_tile(p2 + 1, qa[p2], qb[p2]);
            LA::store(qa[PF - 1], As[0], Sd[0], Sm[0], g.a_rs, g.a_ks, t);
            LB::store(qb[PF - 1], Bs[0], nullptr, nullptr, g.b_js, g.b_ks, t);
            load_tile(PF, qa[PF - 1], qb[PF - 1]);
            lds_barrier();
            for (int64_t kt = 0;;) {
                k_tile(kt, qa[0], qb[0]);
                if (++kt == ntiles) break;
                k_tile(kt, qa[1], qb[1]);
                if (++kt == ntiles) break;
                if constexpr (PF == 4) {
                    k_tile(kt, qa[2], qb[2]);
                    if (++kt == ntiles) break;
                    k_tile(kt, qa[3], qb[3]);
                    if (++kt == ntiles) break;
                }
            }
        }
    } else {
        typename LA::R ra;
        typename LB::R rb;
        if (ntiles > 0) {
            LA::load(ra, g.A, g.scales, a_el, g.M, i0, g.K, 0, g.a_rs, g.a_ks, t);
            LB::load(rb, g.B, nullptr, b_el, g.N, j0, g.K, 0, g.b_js, g.b_ks, t);
        }
        for (int64_t kt = 0; kt < ntiles; kt++) {
            LA::store(ra, As[0], Sd[0], Sm[0], g.a_rs, g.a_ks, t);
            LB::store(rb, Bs[0], nullptr, nullptr, g.b_js, g.b_ks, t);
            __syncthreads();
            if (kt + 1 < ntiles) {
                LA::load(ra, g.A, g.scales, a_el, g.M, i0, g.K, (kt + 1) * BK, g.a_rs, g.a_ks, t);
                LB::load(rb, g.B, nullptr, b_el, g.N, j0, g.K, (kt + 1) * BK, g.b_js, g.b_ks, t);
            }
            compute_tile(0);
            __syncthreads();
        }
    }

    // Epilogue.  In a 32x32 MFMA result, lane l holds the second operand's index
    // (l % 32) and, in register r, the first operand's index
    // 8*(r/4) + 4*(l/32) + (r%4).
    const T *bias = (const T *)g.bias;
    T *out = (T *)g.out + s * g.o_bs;
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int a = 0; a < TA; a++)
#pragma unroll
            for (int b = 0; b < TB; b++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int by_lane = lane & 31, by_reg = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    const int64_t i = i0 + wi * WM + a * 32 + (QUANT ? by_lane : by_reg);
                    const int64_t j = j0 + wj * WN + b * 32 + (QUANT ? by_reg : by_lane);
                    if (i < g.M && j < g.N) {
                        float v = acc[a][b][r];
                        if (g.has_bias) v += to_f32(bias[g.bias_on_rows ? i : j]);
                        v = rt_act_k<decltype(has_act)::value>(v);
                        out[i * g.o_is + j * g.o_js] = from_f32<T>(v);
                    }
                }
            }
    });
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T, int AMODE, int TS>
static void launch_b(int bmode, dim3 grid, hipStream_t st, const GemmArgs &g) {
    switch (bmode) {
    case LM_VECK: hipLaunchKernelGGL((gemm_kernel<T, AMODE, LM_VECK, TS, TS>), grid, dim3(kGemmThreads), 0, st, g); break;
    case LM_VECR: hipLaunchKernelGGL((gemm_kernel<T, AMODE, LM_VECR, TS, TS>), grid, dim3(kGemmThreads), 0, st, g); break;
    default: hipLaunchKernelGGL((gemm_kernel<T, AMODE, LM_GEN, TS, TS>), grid, dim3(kGemmThreads), 0, st, g); break;
    }
}

template <typename T, int TS>
static void launch_a(int amode, int bmode, dim3 grid, hipStream_t st, const GemmArgs &g) {
    switch (amode) {
    case LM_VECK: launch_b<T, LM_VECK, TS>(bmode, grid, st, g); break;
    case LM_VECR: launch_b<T, LM_VECR, TS>(bmode, grid, st, g); break;
    case LM_Q8: launch_b<T, LM_Q8, TS>(bmode, grid, st, g); break;
    case LM_Q4K:
        if constexpr (sizeof(T) == 2) launch_b<T, LM_Q4K, TS>(bmode, grid, st, g);
        break;
    default: launch_b<T, LM_GEN, TS>(bmode, grid, st, g); break;
    }
}

// Picks the vector loader an operand qualifies for: K-contiguous rows
// (LM_VECK), row-contiguous K slices (LM_VECR), else the bounds-checked scalar
// walk.  Vector loads need a 16-byte aligned base, strides that keep every
// vector aligned, and a contiguous extent that is a whole number of vectors.
static int float_mode(const void *p, int64_t esz, int64_t rows, int64_t K, int64_t rs, int64_t ks, int64_t bs) {
    const int64_t vec = 16 / esz;
    if (!aligned16(p) || (bs * esz) % 16 != 0) return LM_GEN;
    if (ks == 1 && (rs * esz) % 16 == 0 && K % vec == 0) return LM_VECK;
    if (rs == 1 && (ks * esz) % 16 == 0 && rows % vec == 0) return LM_VECR;
    return LM_GEN;
}

// Tunable: 0 = automatic, 64 or 128 = force that tile size (for comparisons).
RT_TUNABLE(g_gemm_tile, 0);

hipError_t launch_gemm(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                       hipStream_t stream, const DeviceInfo &dev) {
    if (p.stacks > 65535) return hipErrorNotSupported;
    // 128 x 128 tiles unless they would leave the chip under two workgroups per compute unit
    int ts = 128;
    const int64_t big = ((p.M + 127) / 128) * ((p.N + 127) / 128) * p.stacks;
    if (big < 2 * (int64_t)dev.num_cus) ts = 64;
    if (g_gemm_tile == 64 || g_gemm_tile == 128) ts = g_gemm_tile;
    const int64_t gy = (p.M + ts - 1) / ts, gx = (p.N + ts - 1) / ts;
    if (gy > 65535) return hipErrorNotSupported;
    GemmArgs g{};
    g.A = A, g.B = B, g.bias = bias, g.out = out;
    g.M = p.M, g.N = p.N, g.K = p.K;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.a_bs = p.a_bs, g.a_rs = p.a_rs, g.a_ks = p.a_ks;
    g.b_bs = p.b_bs, g.b_ks = p.b_ks, g.b_js = p.b_js;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    const int64_t esz = p.act_dt == RT_F16 ? 2 : 4;

    int amode;
    if (p.a_dt == RT_Q8_0F || p.a_dt == RT_Q8_0H) {
        if (!aligned16(A)) return hipErrorNotSupported;
        amode = LM_Q8;
        g.scales = (const uint8_t *)A + rt_q8_0_scale_offset((uint64_t)p.a_stack * p.M * p.K);
    } else if (p.a_dt == RT_Q4_K) {
        if (!aligned16(A)) return hipErrorNotSupported;
        amode = LM_Q4K;
    } else {
        amode = float_mode(A, esz, p.M, p.K, p.a_rs, p.a_ks, p.a_bs);
    }
    const int bmode = float_mode(B, esz, p.N, p.K, p.b_js, p.b_ks, p.b_bs);

    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)p.stacks);
    if (p.act_dt == RT_F16) {
        if (ts == 64) launch_a<half_t, 64>(amode, bmode, grid, stream, g);
        else launch_a<half_t, 128>(amode, bmode, grid, stream, g);
    } else {
        if (ts == 64) launch_a<float, 64>(amode, bmode, grid, stream, g);
        else launch_a<float, 128>(amode, bmode, grid, stream, g);
    }
    return hipGetLastError();
}

} // namespace rt
