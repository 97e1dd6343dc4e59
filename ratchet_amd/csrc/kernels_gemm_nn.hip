// f16 product with an untransposed, narrow right operand:  C[s, i, n] = sum_k A[s, i, k] * B[s, k, n]
// (+ bias), A rows K-contiguous, B rows N-contiguous, N <= 128, C row-major.  This is the
// attention P.V form (P [seq x seq], V [seq x head_dim]): a stream over A, read exactly once.
//
// A workgroup of eight wavefronts owns 64 rows of A and all of N.  A is used once and read in whole
// lines: wavefronts 0..3 take the even K tiles of 64 and 4..7 the odd ones, a wavefront's two loads
// per tile are its 16 rows x 128 bytes (eight lanes per row), which it passes through a 2 KiB LDS region
// of its own (swizzled rows; LDS operations of one wavefront complete in order, no barrier) to come
// back as the MFMA operands of the tile's two K steps.  B is shared by the workgroup and goes through
// LDS as it lies in memory, [k][n]: ds_read_b64_tr_b16 hands each lane the four consecutive k of one
// column that an MFMA operand wants (within 16 lanes, lane s addresses columns 4 (s % 4) .. + 3 of row
// s / 4 and lane i receives column i of the four rows), so nothing is transposed by hand.  B tiles go
// to LDS in pairs (four stages, one barrier per pair); four pairs are in flight in registers: at the sizes
// this kernel sees (a few tens of MB) the whole problem has to be requested at once to keep HBM busy.
// The two wavefront groups' partial sums meet in LDS at the end; the result is staged in LDS and written
// with 128-bit stores.
//
// EXACT: M and K are multiples of 64, N of 16 and a workgroup's operands span less than 2 GiB: no
// clamps or zero fills, and every load is a wave-uniform base plus a 32-bit lane offset fixed for
// the whole kernel.
//
// Measured on the attention shape (32 x [512 x 512] . [512 x 80], 22 MB): 9.6 us.  The form before
// loaded A straight into MFMA operand layout, 16 rows x 64 bytes per instruction (half a line per row):
// 10.2 us; a read-only probe over the 16.8 MB of A takes 5.2 us in that pattern and 3.9 us in this one.
// Of the rest, the arithmetic alone (LDS stores and barriers, transposing reads, MFMAs, epilogue), without
// the loads, takes 4.1 us.
//
// Role in the reference: ops/gemm.rs:305-657 with trans_rhs = false (phi2 / whisper attention,
// `matmul(V, false, false)`).
#include "device_common.h"

namespace rt {

struct GemmNnArgs {
    const half_t *A, *B, *bias;
    half_t *out;
    int64_t M, N, K;
    int64_t a_stack, b_stack;
    int64_t a_bs, a_rs; // elements
    int64_t b_bs, b_ks;
    int64_t o_bs, o_is;
    int has_bias, bias_on_rows, act;
};

constexpr int NN_BK = 64;

constexpr int NNT_BM = 64, NNT_THREADS = 512;

template <int TN, bool EXACT>
__global__ __launch_bounds__(NNT_THREADS) void gemm_nn_tr_kernel(GemmNnArgs g) {
    constexpr int NP = 16 * TN;
    constexpr int BR = NP + 8;
    constexpr int B_VECS = NN_BK * (NP / 8);
    constexpr int B_VEC = (B_VECS + NNT_THREADS - 1) / NNT_THREADS;
    constexpr int STAGE = NN_BK * BR;
    constexpr int EROW = NP + 8;
    constexpr int RED_FLOATS = 4 * TN * 4 * 64;
    constexpr int PAIRS = 4; // pairs of K tiles in flight in registers

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *S0 = (half_t *)smem;                     // [4][64][BR]; afterwards the partial sums and the output staging
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    half_t *T = S0 + 4 * STAGE + wave * (16 * 64);   // this wavefront's 16 rows x 64 halves of A
    const int rw = wave & 3, grp = wave >> 2;        // 16 rows of A, and which tile of every pair
    const int fr = lane & 15, fg = lane >> 4;
    const int ar = lane >> 3, ap = lane & 7;         // loading: row (and row + 8) of the 16, 16-byte piece of the tile's 128
    const uint32_t mb = (uint32_t)((g.M + NNT_BM - 1) / NNT_BM), nstacks = gridDim.x / mb;
    uint32_t blk = blockIdx.x % mb, stk = blockIdx.x / mb;
    if (nstacks % 8 == 0) {
        const uint32_t idx = blockIdx.x >> 3;
        stk = (blockIdx.x & 7) + 8 * (idx / mb), blk = idx % mb;
    }
    const int64_t i0 = (int64_t)blk * NNT_BM;
    const int64_t s = stk;
    const half_t *A = g.A + (g.a_stack == 1 ? 0 : s) * g.a_bs;
    const half_t *B = g.B + (g.b_stack == 1 ? 0 : s) * g.b_bs;
    const int nvec = EXACT ? NP / 8 : (int)(g.N >> 3);
    const uint4_t zero4 = {0u, 0u, 0u, 0u};

    const half_t *ap0 = A + min(i0 + rw * 16 + ar, g.M - 1) * g.a_rs + 8 * ap;      // rows past the end duplicate the last one
    const half_t *ap1 = A + min(i0 + rw * 16 + ar + 8, g.M - 1) * g.a_rs + 8 * ap;
    int bk[B_VEC], bc[B_VEC];
#pragma unroll
    for (int i = 0; i < B_VEC; i++) {
        const int v = min(t + NNT_THREADS * i, NN_BK * nvec - 1);
        bk[i] = v / nvec, bc[i] = v - bk[i] * nvec;
    }
    const uint32_t aoff0 = 2u * (uint32_t)((rw * 16 + ar) * (int)g.a_rs + 8 * ap), aoff1 = aoff0 + 2u * 8u * (uint32_t)g.a_rs;
    uint32_t boff[B_VEC];
#pragma unroll
    for (int i = 0; i < B_VEC; i++) boff[i] = 2u * (uint32_t)(bk[i] * (int)g.b_ks + 8 * bc[i]);
    const char *abase = (const char *)(A + i0 * g.a_rs);
    const int64_t b_tile_bytes = 2 * NN_BK * g.b_ks;
    auto b_mine = [&](int i) { return NNT_THREADS * (i + 1) <= B_VECS || t + NNT_THREADS * i < (EXACT ? B_VECS : NN_BK * nvec); };

    const int nk = (int)((g.K + NN_BK - 1) / NN_BK), nkp = (nk + 1) / 2;
    uint4_t ra_[PAIRS][2], rb_[PAIRS][2][B_VEC];
    // pair q = tiles 2 q and 2 q + 1: both tiles' share of B, and this wavefront group's tile of A (past K: a valid
    // vector, replaced by zeros)
    auto load_pair = [&](int q, uint4_t (&ra)[2], uint4_t (&rb)[2][B_VEC]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int64_t k0 = (int64_t)min(2 * q + h, nk - 1) * NN_BK;
            if constexpr (EXACT) {
                const char *bt = (const char *)B + (k0 / NN_BK) * b_tile_bytes; // uniform
#pragma unroll
                for (int i = 0; i < B_VEC; i++) rb[h][i] = *(const uint4_t *)(bt + boff[i]);
            } else {
#pragma unroll
                for (int i = 0; i < B_VEC; i++) rb[h][i] = *(const uint4_t *)(B + min(k0 + bk[i], g.K - 1) * g.b_ks + 8 * bc[i]);
            }
        }
        const int64_t k0 = (int64_t)min(2 * q + grp, nk - 1) * NN_BK;
        if constexpr (EXACT) {
            const char *at = abase + 2 * k0;
            ra[0] = *(const uint4_t *)(at + aoff0), ra[1] = *(const uint4_t *)(at + aoff1);
        } else {
            const int64_t kc = max(min(k0, g.K - 8 - 8 * ap), (int64_t)(-8 * ap)); // the vector read lies inside the row whatever K is
            const uint4_t v0 = *(const uint4_t *)(ap0 + kc), v1 = *(const uint4_t *)(ap1 + kc);
            const bool in = k0 + 8 * ap < g.K;
            ra[0] = in ? v0 : zero4, ra[1] = in ? v1 : zero4;
        }
    };
    auto store_pair = [&](int q, const uint4_t (&rb)[2][B_VEC]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            half_t *st = S0 + (2 * (q & 1) + h) * STAGE;
            const int64_t k0 = (int64_t)(2 * q + h) * NN_BK;
            const bool full = EXACT || k0 + NN_BK <= g.K; // uniform: only the last tile can be ragged; a tile past K is all zeros
#pragma unroll
            for (int i = 0; i < B_VEC; i++)
                if (b_mine(i)) *(uint4_t *)(st + bk[i] * BR + 8 * bc[i]) = (full || k0 + bk[i] < g.K) ? rb[h][i] : zero4;
        }
    };

    float4_t acc[TN];
#pragma unroll
    for (int b = 0; b < TN; b++) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const half_t *)S0;
    const uint32_t b_off = lds0 + 2u * (uint32_t)((8 * fg + (fr >> 2)) * BR + 4 * (fr & 3));
    auto tslot = [](int r, int c) { return (r * 8 + (c ^ ((r >> 1) & 7))) * 8; }; // halves: rows of 128 bytes, 16-byte slots swizzled by row pair
    auto compute = [&](int q, const uint4_t (&ra)[2]) __attribute__((always_inline)) {
        *(uint4_t *)(T + tslot(ar, ap)) = ra[0];
        *(uint4_t *)(T + tslot(ar + 8, ap)) = ra[1];
        asm volatile("" ::: "memory");
        const uint32_t sb = b_off + 2u * (uint32_t)((2 * (q & 1) + grp) * STAGE);
        // both K steps' operands are requested before the first MFMA: one trip through the LDS latency per tile
        half8_t fa[2];
        uint64_t lo[2][TN], hi[2][TN];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            fa[ks] = __builtin_bit_cast(half8_t, *(const uint4_t *)(T + tslot(fr, 4 * ks + fg)));
#pragma unroll
            for (int b = 0; b < TN; b++)
                asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                             : "=&v"(lo[ks][b]), "=&v"(hi[ks][b])
                             : "v"(sb + 2u * (uint32_t)(32 * ks * BR)), "n"(2 * 16 * b), "n"(2 * (16 * b + 4 * BR))
                             : "memory");
        }
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int b = 0; b < TN; b++) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[ks][b]), "+v"(hi[ks][b])::"memory");
        typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int b = 0; b < TN; b++)
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[ks], __builtin_bit_cast(half8_t, u64x2_t{lo[ks][b], hi[ks][b]}), acc[b], 0, 0, 0);
    };
    // (unconditional: a branch here would leave the compiler unable to count the loads in flight)
#pragma unroll
    for (int d = 0; d < PAIRS - 1; d++) {
        load_pair(min(d, nkp - 1), ra_[d], rb_[d]);
        __builtin_amdgcn_sched_barrier(0); // in this order: the first pair's data is waited for first
    }
    auto trip = [&](int q0) {
#pragma unroll
        for (int u = 0; u < PAIRS; u++) {
            const int q = q0 + u;
            if (q < nkp) { // uniform
                if (q + PAIRS - 1 < nkp) load_pair(q + PAIRS - 1, ra_[(u + PAIRS - 1) % PAIRS], rb_[(u + PAIRS - 1) % PAIRS]);
                store_pair(q, rb_[u]);
                // everybody's stores of this pair are done; everybody has finished with the other stage pair's last tiles
                __syncthreads();
                if (2 * q + grp < nk) compute(q, ra_[u]); // uniform per wavefront
            }
        }
    };
    trip(0); // outside the loop: at a loop header the compiler would wait for every load in flight
    for (int q0 = PAIRS; q0 < nkp; q0 += PAIRS) trip(q0);
    __syncthreads(); // the stages become the partial sums and the output staging

    float4_t *red = (float4_t *)smem + rw * TN * 64;
    if (grp == 1) {
#pragma unroll
        for (int b = 0; b < TN; b++) red[b * 64 + lane] = acc[b];
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int b = 0; b < TN; b++) acc[b] += red[b * 64 + lane];

    half_t *es = (half_t *)(smem + 4 * RED_FLOATS) + rw * 16 * EROW;
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int b = 0; b < TN; b++) {
            const int n = 16 * b + fr;
            float bn = 0.f;
            if (g.has_bias && !g.bias_on_rows) bn = (float)g.bias[min(n, (int)g.N - 1)];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int il = 4 * fg + r;
                float v = acc[b][r] + bn;
                if (g.has_bias && g.bias_on_rows) v += (float)g.bias[min(i0 + rw * 16 + il, g.M - 1)];
                v = rt_act_k<decltype(has_act)::value>(v);
                es[il * EROW + n] = (half_t)v;
            }
        }
    });
    asm volatile("" ::: "memory"); // read back by the same wavefront; DS operations complete in order
    half_t *out = g.out + s * g.o_bs;
    for (int v = lane; v < 16 * nvec; v += 64) {
        const int il = v / nvec, c = v - il * nvec;
        const int64_t i = i0 + rw * 16 + il;
        if (i < g.M) __builtin_nontemporal_store(*(const uint4_t *)(es + il * EROW + 8 * c), (uint4_t *)(out + i * g.o_is + 8 * c));
    }
}

template <int TN> static hipError_t launch_nn_tr(const GemmNnArgs &g, int64_t stacks, hipStream_t st) {
    constexpr int NP = 16 * TN;
    const size_t lds = std::max<size_t>((size_t)4 * NN_BK * (NP + 8) * 2 + 8 * 16 * 64 * 2, (size_t)4 * 4 * TN * 4 * 64 + (size_t)4 * 16 * (NP + 8) * 2);
    dim3 grid((unsigned)((g.M + NNT_BM - 1) / NNT_BM * stacks));
    const bool exact = g.M % NNT_BM == 0 && g.K % NN_BK == 0 && g.N == NP && g.a_rs < (1 << 23) && g.K * g.b_ks < (1 << 29);
    if (lds > 48 * 1024) {
        const hipError_t e = exact ? ensure_lds_limit<&gemm_nn_tr_kernel<TN, true>>() : ensure_lds_limit<&gemm_nn_tr_kernel<TN, false>>();
        if (e != hipSuccess) return e;
    }
    if (exact) hipLaunchKernelGGL((gemm_nn_tr_kernel<TN, true>), grid, dim3(NNT_THREADS), lds, st, g);
    else hipLaunchKernelGGL((gemm_nn_tr_kernel<TN, false>), grid, dim3(NNT_THREADS), lds, st, g);
    return hipGetLastError();
}

// Tunable: non-zero keeps these shapes on the generic kernel (for comparisons).
RT_TUNABLE(g_gemm_nn_disable, 0);

// hipErrorNotSupported: the problem does not fit; the generic tiled GEMM runs instead.
hipError_t launch_gemm_nn_smalln(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                 hipStream_t stream, const DeviceInfo &) {
    if (g_gemm_nn_disable) return hipErrorNotSupported;
    if (p.a_dt != RT_F16 || p.act_dt != RT_F16) return hipErrorNotSupported;
    if (p.a_ks != 1 || p.b_js != 1 || p.o_js != 1) return hipErrorNotSupported;
    if (p.N < 8 || p.N > 128 || p.N % 8 != 0 || p.K < 8 || p.K % 8 != 0 || p.M < 64) return hipErrorNotSupported;
    if (p.stacks > 65535 || (p.M + NNT_BM - 1) / NNT_BM * p.stacks > 0x7fffffff) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || ((uintptr_t)out & 15u)) return hipErrorNotSupported;
    if (p.a_rs % 8 || p.a_bs % 8 || p.b_ks % 8 || p.b_bs % 8 || p.o_is % 8 || p.o_bs % 8) return hipErrorNotSupported;
    GemmNnArgs g{};
    g.A = (const half_t *)A, g.B = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    g.M = p.M, g.N = p.N, g.K = p.K;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.a_bs = p.a_bs, g.a_rs = p.a_rs;
    g.b_bs = p.b_bs, g.b_ks = p.b_ks;
    g.o_bs = p.o_bs, g.o_is = p.o_is;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    const int tn = (int)((p.N + 15) / 16);
    switch (tn) {
    case 1: return launch_nn_tr<1>(g, p.stacks, stream);
    case 2: return launch_nn_tr<2>(g, p.stacks, stream);
    case 3: return launch_nn_tr<3>(g, p.stacks, stream);
    case 4: return launch_nn_tr<4>(g, p.stacks, stream);
    case 5: return launch_nn_tr<5>(g, p.stacks, stream);
    case 6: return launch_nn_tr<6>(g, p.stacks, stream);
    case 7: return launch_nn_tr<7>(g, p.stacks, stream);
    default: return launch_nn_tr<8>(g, p.stacks, stream);
    }
}

} // namespace rt
