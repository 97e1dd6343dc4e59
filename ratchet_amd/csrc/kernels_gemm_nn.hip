// f16 product with an untransposed, narrow right operand:  C[s, i, n] = sum_k A[s, i, k] * B[s, k, n]
// (+ bias), A rows K-contiguous, B rows N-contiguous, N <= 128, C row-major.  This is the
// attention P.V form (P [seq x seq], V [seq x head_dim]): a stream over A, read exactly once.
//
// A workgroup of eight wavefronts owns 64 rows of A and all of N.  A is used once, so it never
// touches LDS: lane (fr, fg) loads the 16 bytes A[row fr][32 kh + 8 fg ..] that are its operand
// of a K step.  B is shared by the workgroup and goes through LDS as it lies in memory, [k][n]:
// ds_read_b64_tr_b16 hands each lane the four consecutive k of one column that an MFMA operand
// wants (within 16 lanes, lane s addresses columns 4 (s % 4) .. + 3 of row s / 4 and lane i
// receives column i of the four rows), so nothing is transposed by hand.  Per K tile of 64 the
// wavefronts 0..3 multiply their 16 rows by the tile's first 32 rows of B and the wavefronts 4..7
// by the other 32 (v_mfma_f32_16x16x32_f16); the two partial sums meet in LDS at the end.  Two LDS
// stages, one barrier per tile; the loads of the next seven tiles are in flight in registers: at
// the sizes this kernel sees (a few tens of MB) the whole problem has to be requested at once to
// keep HBM busy.  The result is staged in LDS and written with 128-bit stores.
//
// EXACT: M and K are multiples of 64, N of 16 and a workgroup's operands span less than 2 GiB: no
// clamps or zero fills, and every load is a wave-uniform base plus a 32-bit lane offset fixed for
// the whole kernel.
//
// Measured on the attention shape (32 x [512 x 512] . [512 x 80], 22 MB): loads alone 8.5 us, of
// which A alone 7.6 (6.8 if a wavefront read whole rows instead of 16 rows x 64 bytes), LDS stores
// and barriers + 0.3, transposing reads and MFMAs + 1.4; the arithmetic alone, without the loads, 4.1.
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

constexpr int NNT_BM = 64, NNT_DEPTH = 8, NNT_THREADS = 512;

template <int TN, bool EXACT>
__global__ __launch_bounds__(NNT_THREADS) void gemm_nn_tr_kernel(GemmNnArgs g) {
    constexpr int NP = 16 * TN;                        // padded N
    constexpr int BR = NP + 8;                         // halfs per row of the B tile
    constexpr int B_VECS = NN_BK * (NP / 8);           // 16-byte vectors of a full B tile
    constexpr int B_VEC = (B_VECS + NNT_THREADS - 1) / NNT_THREADS; // per thread
    constexpr int STAGE = NN_BK * BR;
    constexpr int EROW = NP + 8;
    constexpr int RED_FLOATS = 4 * TN * 4 * 64;        // the second wavefront group's accumulators
    static_assert(NN_BK == 64, "two K steps per tile, one per wavefront group");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    half_t *S0 = (half_t *)smem; // [2][64][BR]; afterwards the partial sums [4][TN][4][64] f32 and the output staging

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int rw = wave & 3, kh = wave >> 2; // 16 rows of A, and which K step of every tile
    const int fr = lane & 15, fg = lane >> 4;
    // Workgroups go to the eight XCDs round robin by their linear index, and each XCD has its own L2:
    // the row blocks of one stack share its B, so they are given indices that land on one XCD.
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

    // this lane's row of A (rows past the end duplicate the last one), its K offset inside a tile, and
    // its vectors of the B tile: vector v = t + 512 i is (row v / nvec, column 8 (v % nvec))
    const int arow = rw * 16 + fr, ak = 32 * kh + 8 * fg;
    const half_t *ap = A + min(i0 + arow, g.M - 1) * g.a_rs + ak;
    int bk[B_VEC], bc[B_VEC];
#pragma unroll
    for (int i = 0; i < B_VEC; i++) {
        const int v = min(t + NNT_THREADS * i, NN_BK * nvec - 1);
        bk[i] = v / nvec, bc[i] = v - bk[i] * nvec;
    }
    // EXACT: byte offsets from the tile's first byte
    const uint32_t aoff = 2u * (uint32_t)(arow * (int)g.a_rs + ak);
    uint32_t boff[B_VEC];
#pragma unroll
    for (int i = 0; i < B_VEC; i++) boff[i] = 2u * (uint32_t)(bk[i] * (int)g.b_ks + 8 * bc[i]);
    const char *abase = (const char *)(A + i0 * g.a_rs);
    const int64_t b_tile_bytes = 2 * NN_BK * g.b_ks;
    auto b_mine = [&](int i) { return NNT_THREADS * (i + 1) <= B_VECS || t + NNT_THREADS * i < (EXACT ? B_VECS : NN_BK * nvec); };

    constexpr int D = NNT_DEPTH;
    uint4_t ra_[D], rb_[D][B_VEC];
    auto load_tiles = [&](int64_t k0, uint4_t &ra, uint4_t (&rb)[B_VEC]) {
        if constexpr (EXACT) {
            const char *at = abase + 2 * k0, *bt = (const char *)B + (k0 / NN_BK) * b_tile_bytes; // uniform
#pragma unroll
            for (int i = 0; i < B_VEC; i++) rb[i] = *(const uint4_t *)(bt + boff[i]); // (threads without a vector re-read the last one)
            ra = *(const uint4_t *)(at + aoff);
        } else {
#pragma unroll
            for (int i = 0; i < B_VEC; i++) rb[i] = *(const uint4_t *)(B + min(k0 + bk[i], g.K - 1) * g.b_ks + 8 * bc[i]);
            const uint4_t v = *(const uint4_t *)(ap + min(k0, g.K - 8 - ak)); // past K: a valid vector, replaced by zeros
            ra = k0 + ak < g.K ? v : zero4;
        }
    };
    // registers -> LDS: B rows as they are (rows past K zeroed: the padded part of the last K tile adds nothing)
    auto store_tile = [&](half_t *st, int64_t k0, const uint4_t (&rb)[B_VEC]) {
        const bool full = EXACT || k0 + NN_BK <= g.K; // uniform: only the last tile can be ragged
#pragma unroll
        for (int i = 0; i < B_VEC; i++)
            if (b_mine(i)) *(uint4_t *)(st + bk[i] * BR + 8 * bc[i]) = (full || k0 + bk[i] < g.K) ? rb[i] : zero4;
    };

    float4_t acc[TN];
#pragma unroll
    for (int b = 0; b < TN; b++) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};
    // byte address in LDS of the first row / columns this lane addresses for B
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const half_t *)S0;
    const uint32_t b_off = lds0 + 2u * (uint32_t)((32 * kh + 8 * fg + (fr >> 2)) * BR + 4 * (fr & 3));

    const int nk = (int)((g.K + NN_BK - 1) / NN_BK);
    auto tile_k0 = [&](int kt) { return (int64_t)kt * NN_BK; };
    // (unconditional: a branch here would leave the compiler unable to count the loads in flight, and it
    // would then wait for all of them before the first tile; short problems load their last tile again)
#pragma unroll
    for (int d = 0; d < D - 1; d++) {
        load_tiles(tile_k0(min(d, nk - 1)), ra_[d], rb_[d]);
        __builtin_amdgcn_sched_barrier(0); // in this order: the first tile's data is waited for first
    }
    auto trip = [&](int kt0) {
#pragma unroll
        for (int u = 0; u < D; u++) {
            const int kt = kt0 + u;
            if (kt < nk) { // uniform
                if (kt + D - 1 < nk) load_tiles(tile_k0(kt + D - 1), ra_[(u + D - 1) % D], rb_[(u + D - 1) % D]);
                store_tile(S0 + (u & 1) * STAGE, tile_k0(kt), rb_[u]); // D is even: tile kt lives in stage kt % 2
                // everybody's stores of this tile are done; everybody has finished with the other stage's last tile
                __syncthreads();
                const uint32_t sb = b_off + 2u * (uint32_t)((u & 1) * STAGE);
                uint64_t lo[TN], hi[TN];
#pragma unroll
                for (int b = 0; b < TN; b++)
                    asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                                 : "=&v"(lo[b]), "=&v"(hi[b])
                                 : "v"(sb), "n"(2 * 16 * b), "n"(2 * (16 * b + 4 * BR))
                                 : "memory");
#pragma unroll
                for (int b = 0; b < TN; b++) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[b]), "+v"(hi[b])::"memory");
                typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));
                const half8_t fa = __builtin_bit_cast(half8_t, ra_[u]);
#pragma unroll
                for (int b = 0; b < TN; b++)
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, __builtin_bit_cast(half8_t, u64x2_t{lo[b], hi[b]}), acc[b], 0, 0, 0);
            }
        }
    };
    // The first D tiles stand outside the loop: at a loop header the compiler's count of loads in flight
    // is the cautious merge of both ways in, and it would wait for all of them before the first tile.
    trip(0);
    for (int kt0 = D; kt0 < nk; kt0 += D) trip(kt0);
    __syncthreads(); // the stages become the partial sums and the output staging

    // the second group hands its sums to the first
    float4_t *red = (float4_t *)smem + rw * TN * 64;
    if (kh == 1) {
#pragma unroll
        for (int b = 0; b < TN; b++) red[b * 64 + lane] = acc[b];
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int b = 0; b < TN; b++) acc[b] += red[b * 64 + lane];

    // acc[b][r] is row 4 * fg + r of the wavefront's 16, column 16 * b + fr
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
    const size_t lds = std::max<size_t>((size_t)2 * NN_BK * (NP + 8) * 2, (size_t)4 * 4 * TN * 4 * 64 + (size_t)4 * 16 * (NP + 8) * 2);
    dim3 grid((unsigned)((g.M + NNT_BM - 1) / NNT_BM * stacks));
    const bool exact = g.M % NNT_BM == 0 && g.K % NN_BK == 0 && g.N == NP && g.a_rs < (1 << 23) && g.K * g.b_ks < (1 << 29);
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
