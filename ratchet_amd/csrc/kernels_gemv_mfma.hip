// Streaming Q8_0H GEMV on the matrix cores, for 1..16 activation vectors.
//
//   y[j, n] = sum_b d[n, b] * ( sum_{k in block b} q[n, k] * x[j, k] )  (+ bias[n])
//
// The weight stream (int8 codes + f16 block scales, the reference's segment
// layout) is read exactly once from HBM with one 128-bit load per lane and
// never touches LDS.  The codes are widened to f16 in registers (an int8 is
// exact in f16) and each block of 32 goes through one v_mfma_f32_16x16x32_f16
// against the activations; the block's scale multiplies the f32 partial sums,
// so no weight is ever rounded.  The few activation vectors pass through LDS
// only to be re-read in MFMA fragment order.
//
// Work split: a workgroup owns 16, 32 or 64 weight rows; each of its wavefronts
// owns a contiguous slice of K (one or more units of 256) and issues all of
// that slice's loads before the first MFMA, so close to the whole matrix is in
// flight at once; the slices are summed through LDS at the end.
//
// The kernel is bound by instruction issue, not by the matrix cores or (yet) by HBM: several
// wavefronts per SIMD run the same few hundred instructions at the same time, and every one
// removed shows in the launch time.  Hence the regular-case variant (FAST) with a prologue of
// 32-bit offsets and no clamps, the order of the loads (activations first: they come from the
// L2 and their detour through LDS is over before the first weights arrive; issuing the first
// weight load ahead of them measured 3 % slower), and one unit of K per wavefront (two
// measured 2 % slower).
//
// Lane layout of one step (64 values of K for 16 rows): lane l reads 16 bytes
// of row n = l % 16 at K offset 16 * (l / 16).  Lanes 0..31 thus hold block
// 2s of their row and lanes 32..63 block 2s+1.  One v_permlane32_swap per
// dword pair regroups them so that the first MFMA sees only block 2s and the
// second only block 2s+1; within a block the order of K is irrelevant as long
// as the activation fragment uses the same order, which x_koff() provides.
// The regular-case variant loads the same 16 rows x 64 bytes in address order instead (lane l: row l / 4, piece
// l % 4, so that a quad of lanes reads 64 consecutive bytes and the L1 handles one access per quad, not four) and
// brings a step to the layout above through a 1 KB LDS slot, the wavefront's slab of the final sums' region
// (swizzled ds_write_b128, ds_read_b128): 10240 x 2560 at 8 vectors 9.6 -> 9.0 us.
#include "device_common.h"

namespace rt {

struct GemvMfmaArgs {
    const uint8_t *qs;     // int8 codes, row-major [rows, K]
    const half_t *scales;  // f16 scales, row-major [rows, K/32]
    const half_t *X;
    const half_t *bias;
    half_t *out;
    int64_t M, K;          // weight rows, contraction (K % 256 == 0)
    int NC;                // activation vectors (1..16)
    int nunits;            // K / 256
    int rows_wg;           // weight rows per workgroup: at most 16 * RG, a multiple of 8
    int64_t a_stack, b_stack;
    int64_t b_bs, b_js;
    int64_t o_bs, o_is, o_js;
    int has_bias, bias_on_rows, act;
    int lin;               // the regular case loads its weights in address order
};

// K offset (within a 64-wide step) of the 8 values lane group g feeds to the
// first MFMA of the step; the second MFMA uses the same offsets + 32.
__device__ __forceinline__ int x_koff(int g) { return 16 * (g & 1) + 8 * (g >> 1); }

// 4 packed int8 -> two half2 holding the same integers, exactly:
// (q ^ 0x80) is q + 128 as an unsigned byte; 0x6400 | byte is the f16 1024 + byte;
// subtracting 1152 leaves q.
__device__ __forceinline__ void cvt_i8x4_f16x4(uint32_t v, half2_t &lo, half2_t &hi) {
    v ^= 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u);
    const half2_t bias = {(half_t)1152.0f, (half_t)1152.0f};
    lo = __builtin_bit_cast(half2_t, a) - bias;
    hi = __builtin_bit_cast(half2_t, b) - bias;
}

__device__ __forceinline__ half8_t cvt_i8x8_f16x8(uint32_t v0, uint32_t v1) {
    half2_t a, b, c, d;
    cvt_i8x4_f16x4(v0, a, b);
    cvt_i8x4_f16x4(v1, c, d);
    return half8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

RT_TUNABLE(g_gemv_mfma_lin, 1); // 0: the regular case loads its weights in operand order (for comparisons)

constexpr int kUnitK = 256; // K covered by one unit: 4 steps of 64, 8 scale blocks
constexpr int kXPad = 8;    // halfs of padding per staged row (keeps 16-lane LDS reads conflict-free)

// A workgroup owns 16*RG weight rows; wavefront w owns units [w*UPW, (w+1)*UPW)
// of K for all of them.  Everything up to the final cross-wave sum is private to
// the wavefront, so no barrier sits between the loads and the MFMAs:
//   - its slice of the activations goes global -> registers -> its own LDS region
//     and comes back as MFMA fragments (DS operations of one wavefront complete in
//     order);
//   - each lane loads the 8 scales of its row and unit directly (the four lane
//     groups of a row read the same 16 bytes, one transaction);
//   - loads are issued in the order they are needed: activations, weights, scales.
// NCT is the compile-time ceiling of the number of activation vectors (it sizes the
// staging registers).
// FAST is the regular case, which the launcher recognises: one stack, every one of the
// workgroup's rows and every one of its wavefronts' units exists, and all offsets below 2^31.  Its prologue is a handful of 32-bit operations (no clamps, no stack
// arithmetic), which matters because every wavefront runs it before its first load is issued
// and several wavefronts per SIMD run it at the same time.
template <int UPW, int RG, int NCT, bool FAST>
__global__ __launch_bounds__(1024) void gemv_q8h_mfma_kernel(GemvMfmaArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int XROW = UPW * kUnitK + kXPad; // halfs per staged activation row (this wave's K slice)
    const int t = threadIdx.x, lane = t & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6); // wave-uniform: addresses below stay scalar
    const int NC = g.NC;
    half_t *xs = (half_t *)smem + (size_t)wave * NC * XROW;          // [NC][XROW], private to this wave
    float *psum = (float *)((half_t *)smem + (size_t)nwaves * NC * XROW); // [nwaves][RG][256]

    const int n = lane & 15, grp = lane >> 4;
    const int64_t s = FAST ? 0 : blockIdx.y;
    // an operand's stack is either the full stack or 1 (broadcast)
    const int64_t sa = g.a_stack == 1 ? 0 : s, sb = g.b_stack == 1 ? 0 : s;
    const int64_t row0 = (int64_t)blockIdx.x * (FAST ? 16 * RG : g.rows_wg);
    const int u0 = wave * UPW;                            // first unit of this wave
    const int nu = FAST ? UPW : min(UPW, g.nunits - u0);  // units this wave really has (<= 0 for a padding wave)
    const int u0c = nu > 0 ? u0 : 0;                      // a padding wave reads unit 0 and discards the result

    constexpr int VPR = UPW * kUnitK / 8;      // 16-byte vectors per activation row of this wave's slice
    constexpr int XL = (NCT * VPR + 63) / 64;
    const int nvec = NC * VPR;
    uint4_t xv[XL];
    uint4_t w[RG][UPW][4], dsc[RG][UPW];
    uint32_t bias_raw[RG];
    const uint32_t kq = (uint32_t)(g.K >> 5);

    if constexpr (FAST) {
        // Offsets fit 32 bits (the launcher checks).
        // 1. this wave's slice of the activation vectors
        const half_t *xg = g.X + u0 * kUnitK;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const uint32_t v = min(i * 64 + lane, NCT * VPR - 1); // lanes past the end re-read the last vector
            const uint32_t j = min(v / VPR, (uint32_t)NC - 1u), kv = v % VPR; // fewer than NCT vectors: the last one again, never staged
            xv[i] = *(const uint4_t *)(xg + (j * (uint32_t)g.b_js + 8u * kv));
        }
        asm volatile("" ::: "memory"); // keep the loads in this order
        // 2. the weight stream: a wave-uniform 64-bit base plus a 32-bit lane offset
        const uint8_t *qbase = g.qs + ((uint32_t)row0 * (uint32_t)g.K + (uint32_t)(u0 * kUnitK));
        // address order (RT_MFMA_LIN): a quad of lanes reads 64 consecutive bytes of row lane / 4; the step passes
        // through an LDS slot on its way to operand order.  Operand order: row lane % 16, piece lane / 16.
        const uint32_t loff = g.lin ? (uint32_t)(lane >> 2) * (uint32_t)g.K + 16u * (lane & 3) : (uint32_t)n * (uint32_t)g.K + 16u * grp;
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int u = 0; u < UPW; u++)
#pragma unroll
                for (int st = 0; st < 4; st++)
                    w[rg][u][st] = *(const uint4_t *)(qbase + (loff + (uint32_t)(16 * rg) * (uint32_t)g.K) + u * kUnitK + st * 64);
        asm volatile("" ::: "memory");
        // 3. the scales of this lane's rows, then the epilogue's bias value (unconditional: without a
        //    bias it reads a scale and the value is dropped)
        const half_t *sbase = g.scales + ((uint32_t)row0 * kq + (uint32_t)(u0 * 8));
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int u = 0; u < UPW; u++) dsc[rg][u] = *(const uint4_t *)(sbase + ((uint32_t)(16 * rg + n) * kq + u * 8));
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t bi = g.bias_on_rows ? (uint32_t)row0 + 16 * rg + (t & 15) : (uint32_t)min((t >> 4) & 15, NC - 1);
            const half_t *bp = g.has_bias ? g.bias + bi : sbase;
            bias_raw[rg] = *(const uint16_t *)bp;
        }
        asm volatile("" ::: "memory");
    } else {
        // 1. this wave's slice of the activation vectors: 16-byte vectors, NC rows of UPW*32 vectors
        const half_t *xg = g.X + sb * g.b_bs + (int64_t)u0c * kUnitK;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int v = min(i * 64 + lane, nvec - 1); // lanes past the end re-read the last vector
            const int j = v / VPR, kv = v - j * VPR;    // VPR is a power of two
            // a unit past the end of K (ragged last wave) re-reads the wave's first unit; it is never used
            const int kvc = (kv / (kUnitK / 8) < nu) ? kv : kv % (kUnitK / 8);
            xv[i] = *(const uint4_t *)(xg + j * g.b_js + 8 * kvc);
        }
        asm volatile("" ::: "memory"); // keep the loads in this order

        // 2. the weight stream: 4 x 16 bytes per unit per row group per lane
        // (a wave-uniform 64-bit base plus a 32-bit lane offset: K <= 16384, so 64 rows stay below 2^20)
        const uint8_t *qbase = g.qs + (sa * g.M + row0) * g.K + (int64_t)u0c * kUnitK;
        const half_t *sbase = g.scales + (sa * g.M + row0) * (int64_t)kq + (int64_t)u0c * 8;
        const int last = (int)min((int64_t)(g.rows_wg - 1), g.M - 1 - row0); // rows past the workgroup's or the matrix's end duplicate the last one; never stored
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t rowl = (uint32_t)min(16 * rg + n, last);
            const uint8_t *q = qbase + (rowl * (uint32_t)g.K + 16u * grp);
#pragma unroll
            for (int u = 0; u < UPW; u++) {
                const int uc = u < nu ? u : 0;
#pragma unroll
                for (int st = 0; st < 4; st++) w[rg][u][st] = *(const uint4_t *)(q + uc * kUnitK + st * 64);
            }
        }
        asm volatile("" ::: "memory");
        // 3. the scales of this lane's rows for the wave's units (8 f16 = 16 bytes per row and unit)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t rowl = (uint32_t)min(16 * rg + n, last);
            const half_t *sc = sbase + rowl * kq;
#pragma unroll
            for (int u = 0; u < UPW; u++) dsc[rg][u] = *(const uint4_t *)(sc + (u < nu ? u : 0) * 8);
        }
        // The epilogue's bias value, fetched behind everything else so its latency is hidden.  The load is
        // unconditional (without a bias it reads a scale and the value is dropped): a branch here makes the
        // compiler wait for every outstanding load right after issuing this one.
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const int64_t bi = g.bias_on_rows ? min(row0 + min(16 * rg + (t & 15), g.rows_wg - 1), g.M - 1) : (int64_t)min((t >> 4) & 15, g.NC - 1);
            const half_t *bp = g.has_bias ? g.bias + bi : sbase;
            bias_raw[rg] = *(const uint16_t *)bp;
        }
        asm volatile("" ::: "memory");
    }

    // 4. activations -> this wave's LDS region (the reads below are by the same wavefront)
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int v = i * 64 + lane;
        if (v < nvec) {
            const int j = v / VPR, kv = v % VPR;
            *(uint4_t *)(xs + j * XROW + 8 * kv) = xv[i];
        }
    }
    asm volatile("" ::: "memory");

    // 5. MFMAs: one per block of 32; the block's scale multiplies the f32 partial sums
    // a lane's MFMA result register r is activation vector 4*grp + r: with fewer than 4 vectors
    // only registers r < NCT of lane group 0 carry results
    constexpr int NR = NCT < 4 ? NCT : 4;
    const int xj = min(n, NC - 1); // lanes beyond NC re-read a valid row; their outputs are dropped
    const half_t *xrow = xs + xj * XROW + x_koff(grp);
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < UPW; u++) {
            if (u < nu) { // wave-uniform
                const half8_t dh = __builtin_bit_cast(half8_t, dsc[rg][u]);
#pragma unroll
                for (int st = 0; st < 4; st++) {
                    uint4_t wq = w[rg][u][st];
                    if (FAST && g.lin) {
                        // load order -> operand order through this wavefront's slab of the sums' region (unused until
                        // the MFMAs are done; one wavefront's DS operations complete in order)
                        uint8_t *slot = (uint8_t *)(psum + (wave * RG + rg) * 256);
                        const int lr = lane >> 2, lc = lane & 3;
                        *(uint4_t *)(slot + lr * 64 + 16 * (lc ^ ((lr >> 2) & 3))) = wq;
                        wq = *(const uint4_t *)(slot + n * 64 + 16 * (grp ^ ((n >> 2) & 3)));
                    }
                    // regroup: afterwards p?[0] is this lane's share of block 2*st and p?[1] of block 2*st+1
                    auto p0 = __builtin_amdgcn_permlane32_swap(wq[0], wq[2], false, false);
                    auto p1 = __builtin_amdgcn_permlane32_swap(wq[1], wq[3], false, false);
                    const half8_t b0 = cvt_i8x8_f16x8(p0[0], p1[0]);
                    const half8_t b1 = cvt_i8x8_f16x8(p0[1], p1[1]);
                    const half8_t a0 = __builtin_bit_cast(half8_t, *(const uint4_t *)(xrow + u * kUnitK + st * 64));
                    const half8_t a1 = __builtin_bit_cast(half8_t, *(const uint4_t *)(xrow + u * kUnitK + st * 64 + 32));
                    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
                    const float4_t P0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, zero, 0, 0, 0);
                    const float4_t P1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, zero, 0, 0, 0);
                    const float s0 = (float)dh[2 * st], s1 = (float)dh[2 * st + 1];
#pragma unroll
                    for (int r = 0; r < NR; r++) acc[r] = fmaf(s0, P0[r], acc[r]);
#pragma unroll
                    for (int r = 0; r < NR; r++) acc[r] = fmaf(s1, P1[r], acc[r]);
                }
            }
        }
        // acc[r] belongs to activation vector 4*grp + r and weight row 16*rg + n
        if (NCT >= 16 || 4 * grp < NCT) {
#pragma unroll
            for (int r = 0; r < NR; r++) psum[(wave * RG + rg) * 256 + (4 * grp + r) * 16 + n] = acc[r];
        }
    }

    // 6. sum the K slices
    __syncthreads();
    if (t < 16 * NCT) {
        const int j = t >> 4;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            float v = 0.f;
            for (int w2 = 0; w2 < nwaves; w2++) v += psum[(w2 * RG + rg) * 256 + t];
            const int64_t i = row0 + 16 * rg + (t & 15);
            if (FAST ? j < g.NC : (j < g.NC && i < g.M && 16 * rg + (t & 15) < g.rows_wg)) g.out[s * g.o_bs + i * g.o_is + j * g.o_js] = (half_t)rt_act(v + (g.has_bias ? (float)__builtin_bit_cast(half2_t, bias_raw[rg])[0] : 0.f), g.act);
        }
    }
}

// Tunables: units of 256 K-values per wavefront (1, 2, 4) and 16-row groups
// per workgroup (1, 2, 4); 0 lets the launcher decide.
RT_TUNABLE(g_gemv_mfma_upw, 0);
RT_TUNABLE(g_gemv_mfma_rg, 0);

template <int UPW, int RG, int NCT, bool FAST>
static hipError_t launch_kernel(dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvMfmaArgs &g) {
    if (lds > 48 * 1024) {
        const hipError_t e = ensure_lds_limit<&gemv_q8h_mfma_kernel<UPW, RG, NCT, FAST>>();
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemv_q8h_mfma_kernel<UPW, RG, NCT, FAST>), grid, dim3(nwaves * 64), lds, st, g);
    return hipGetLastError();
}

// The regular case (see the kernel): only compiled for one row group per workgroup, which is
// what the launcher uses unless told otherwise.
template <int UPW, int RG, int NCT>
static hipError_t launch_one(dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvMfmaArgs &g) {
    if constexpr (RG == 1) {
        const bool regular = grid.y == 1 && g.a_stack == 1 && g.b_stack == 1 && g.M % 16 == 0 &&
                             g.nunits == nwaves * UPW && g.M * g.K < (int64_t(1) << 31) &&
                             (int64_t)g.NC * g.b_js < (int64_t(1) << 30);
        if (regular) return launch_kernel<UPW, RG, NCT, true>(grid, nwaves, lds, st, g);
    }
    return launch_kernel<UPW, RG, NCT, false>(grid, nwaves, lds, st, g);
}

template <int UPW, int RG>
static hipError_t launch_nc(dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvMfmaArgs &g) {
    if (g.NC <= 1) return launch_one<UPW, RG, 1>(grid, nwaves, lds, st, g);
    if (g.NC <= 2) return launch_one<UPW, RG, 2>(grid, nwaves, lds, st, g);
    if (g.NC <= 4) return launch_one<UPW, RG, 4>(grid, nwaves, lds, st, g);
    if (g.NC <= 8) return launch_one<UPW, RG, 8>(grid, nwaves, lds, st, g);
    return launch_one<UPW, RG, 16>(grid, nwaves, lds, st, g);
}

template <int UPW>
static hipError_t launch_rg(int rg, dim3 grid, int nwaves, size_t lds, hipStream_t st, const GemvMfmaArgs &g) {
    switch (rg) {
    case 1: return launch_nc<UPW, 1>(grid, nwaves, lds, st, g);
    case 2: return launch_nc<UPW, 2>(grid, nwaves, lds, st, g);
    case 3:
        if constexpr (UPW == 1) return launch_nc<UPW, 3>(grid, nwaves, lds, st, g);
        return hipErrorInvalidValue;
    case 4: return launch_nc<UPW, 4>(grid, nwaves, lds, st, g);
    default: return hipErrorInvalidValue;
    }
}

// Q8_0H weights, f16 activations, 1..16 vectors, K a multiple of 256.
// hipErrorNotSupported means the shape or alignment does not fit this kernel
// and another one must run.
hipError_t launch_gemv_q8h_mfma(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev) {
    if (p.a_dt != RT_Q8_0H || p.act_dt != RT_F16 || p.N < 1 || p.N > 16 || p.K % kUnitK != 0 || p.K < kUnitK)
        return hipErrorNotSupported;
    if (p.stacks > 65535 || p.K > 16384) return hipErrorNotSupported;
    const int64_t bjs = p.N == 1 ? 0 : p.b_js;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (bjs * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    if (p.b_ks != 1) return hipErrorNotSupported;

    GemvMfmaArgs g{};
    const uint64_t numel = (uint64_t)p.a_stack * p.M * p.K;
    g.qs = (const uint8_t *)A;
    g.scales = (const half_t *)((const uint8_t *)A + rt_q8_0_scale_offset(numel));
    g.X = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    g.M = p.M, g.K = p.K, g.NC = (int)p.N;
    g.nunits = (int)(p.K / kUnitK);
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.b_bs = p.b_bs, g.b_js = bjs;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act, g.lin = g_gemv_mfma_lin;

    // Units per wavefront: as few as keeps the workgroup within 16 wavefronts.
    int upw = g_gemv_mfma_upw;
    if (upw == 0) upw = g.nunits <= 16 ? 1 : (g.nunits <= 32 ? 2 : 4);
    while (upw < 4 && (g.nunits + upw - 1) / upw > 16) upw *= 2;
    int nwaves = (g.nunits + upw - 1) / upw;
    if (nwaves > 16) return hipErrorNotSupported; // K > 16384
    if (nwaves < 4) nwaves = 4;                   // the final sum uses 256 threads
    // Rows per workgroup.  16 (one MFMA row group) while all workgroups are resident at once: more groups per
    // workgroup mean more loads per wavefront and a longer tail after the last one returns.  With many vectors the
    // activations' LDS leaves room for two workgroups per compute unit, or one, and the grid then runs in rounds
    // (10240 rows, 16 vectors: 640 workgroups, one per compute unit = 3 rounds, 13.2 us).  There every compute unit
    // gets one workgroup with its share of the rows, ceil(rows / num_cus) rounded up to 8, in up to four row groups
    // the last of which may be half empty (40 rows per workgroup: 10.5 us; 9 / 12 vectors 11.0 / 11.4 -> 10.3 / 10.4;
    // two workgroups of 24 rows per compute unit measured slower than either, 12.3 us at 9 vectors).
    int rg = g_gemv_mfma_rg, rows_wg = 0;
    if (rg == 0) {
        rg = 1;
        const size_t lds_x = (size_t)nwaves * g.NC * (upw * kUnitK + kXPad) * 2;
        auto fit = [&](int r) { // workgroups of r row groups that fit a compute unit
            const int by_lds = (int)((160 * 1024) / (lds_x + (size_t)nwaves * r * 1024)), by_waves = 32 / nwaves;
            return by_lds < by_waves ? by_lds : by_waves;
        };
        if (upw == 1 && p.stacks == 1 && (p.M + 15) / 16 > (int64_t)dev.num_cus * fit(1)) {
            const int64_t per = ((p.M + dev.num_cus - 1) / dev.num_cus + 7) & ~(int64_t)7;
            if (per <= 64 && fit((int)(per + 15) / 16) >= 1) rows_wg = (int)per, rg = (rows_wg + 15) / 16;
        }
    }
    if (upw * rg > 4) rg = 4 / upw > 0 ? 4 / upw : 1; // at most 16 weight loads in flight per lane
    if (rows_wg == 0 || rows_wg > 16 * rg) rows_wg = 16 * rg;
    g.rows_wg = rows_wg;
    const size_t lds = (size_t)nwaves * g.NC * (upw * kUnitK + kXPad) * 2 + (size_t)nwaves * rg * 1024;
    if (lds > 160 * 1024) return hipErrorNotSupported;
    const int64_t groups = (p.M + rows_wg - 1) / rows_wg;
    if (groups > 0x7fffffff) return hipErrorNotSupported;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    switch (upw) {
    case 1: return launch_rg<1>(rg, grid, nwaves, lds, stream, g);
    case 2: return launch_rg<2>(rg, grid, nwaves, lds, stream, g);
    case 4: return launch_rg<4>(rg, grid, nwaves, lds, stream, g);
    default: return hipErrorInvalidValue;
    }
}

} // namespace rt
