// Row-streaming Q8_0H GEMV for 3 or 4 activation vectors on the 4x4x4 matrix instruction.
//
//   y[j, n] = sum_b d[n, b] * ( sum_{k in block b} q[n, k] * x[j, k] )  (+ bias)
//
// v_mfma_f32_4x4x4_16b_f16 is sixteen independent 4x4x4 products, one per group of four lanes.
// In group b the four lanes hold the same four K positions of four different weight rows (operand A)
// and of four different activation vectors (operand B), so 16 bytes of a row feed four of these
// instructions.  One load instruction of a wavefront covers 256 consecutive bytes of each of four rows
// (sixteen lanes per row: eight whole 128-byte lines, each read exactly once, which is what lets the
// loads be non-temporal), and one ds_bpermute per register then hands lane 16 i + b's bytes to lane
// 4 b + i, the place operand A wants them: the crossbar moves registers, the codes are never stored in
// LDS.  Loading in operand order directly (four rows interleaved 16 bytes at a time) costs 0.6 us of
// 5.7 on a read-only probe of the Phi-2 up-projection; the bpermutes cost 0.2-0.3.  A wavefront owns
// four rows over the whole of K and issues every load of them before the first is used.
//
// A lane's 16 codes are half a Q8_0 block: the four instructions of a step chain through one
// accumulator that starts at zero, and the block's f16 scale multiplies that f32 sum (the scale of row i
// sits in lane i of the group and is handed to the other three by a quad-permute DPP operand), so no
// weight is ever rounded.  The scales of a workgroup's 16 rows are one run of bytes: one 16-byte load
// per thread, issued ahead of the weights, and through LDS to the lanes that use them (a 2-byte load per
// lane and step instead measured 1.3 us slower at the Phi-2 shape).  The sixteen groups' sums meet at
// the end in two DPP rotations and two permlane swaps per result register.
//
// The activations are staged once per workgroup in LDS in the order the lanes read them (a wavefront's
// read of one operand is 1 KiB of consecutive bytes) and then held in registers.  Their loads are the
// first thing every wavefront issues, and a barrier without a wait puts all of them into the compute
// unit's memory pipeline ahead of any weight load (0.2 us).
//
// Measured at 10240 x 2560 against the matrix-core kernel of kernels_gemv_mfma.hip, same timing: 3 / 4
// vectors 7.7 / 7.85 against 8.2 / 8.3 us.  With a second set of four vectors (twice the products, folds
// and activation registers) 5..8 vectors took 9.2-9.7 us, no better than that kernel, so it keeps them;
// what is left above the 5.7 us of the bare reads is the scale stream (0.8 us: its 6 % of the bytes and
// a second dependency of every product) and the arithmetic of the wavefronts whose bytes arrive last.
//
// Roles in the reference: ops/gemv.rs:333-558 (subgroup GEMV; the reference sends 2..8 vectors to its
// tiled GEMM, ops/matmul.rs:221-223), kernel_builder.rs:222-240 (unpack), dtype/blocks.rs:61-74.
#include "device_common.h"

namespace rt {

struct GemvQuadArgs {
    const uint8_t *qs;
    const half_t *scales;
    const half_t *X;
    const half_t *bias;     // never null: without a bias the scales, with both bias strides 0, and the value is dropped
    half_t *out;
    uint32_t M;             // weight rows
    uint32_t NC;            // activation vectors (1..4)
    uint32_t bias_rs;       // 1: a bias per weight row, 0: per vector
    int64_t b_js;           // elements between the activation vectors
    int64_t o_is, o_js;
    int64_t q_ss, s_ss, x_ss, o_ss; // per stack: bytes of codes, scales, activation elements, output elements
    int has_bias, act;
};

// (q ^ 0x80) is q + 128 as an unsigned byte; 0x6400 | byte is the f16 1024 + byte; minus 1152 leaves q
__device__ __forceinline__ half4_t quad_cvt_i8x4(uint32_t v) {
    v ^= 0x80808080u;
    const half2_t off = {(half_t)1152.0f, (half_t)1152.0f};
    const half2_t lo = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - off;
    const half2_t hi = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - off;
    return half4_t{lo[0], lo[1], hi[0], hi[1]};
}

template <int I> __device__ __forceinline__ float quad_bcast(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), I * 0x55, 0xf, 0xf, true));
}

// Sum over the sixteen lane groups (lanes with the same lane % 4); every lane receives it.
__device__ __forceinline__ float quad_groups_sum(float v) {
    v += wave_dpp<0x124>(v); // row_ror:4
    v += wave_dpp<0x128>(v); // row_ror:8
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
    const uint32_t x = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __builtin_bit_cast(float, (uint32_t)b[0]) + __builtin_bit_cast(float, (uint32_t)b[1]);
}

constexpr int kQuadWaves = 4, kQuadRows = 4 * kQuadWaves; // wavefronts and weight rows per workgroup

// K = 256 * STEPS.  Lane 4 b + i of a wavefront multiplies row i of the wavefront's four rows at K positions
// 256 s + 16 b .. + 15 of every step s with vector i's values there.
template <int STEPS>
__global__ __launch_bounds__(kQuadWaves * 64) void gemv_q8h_quad_kernel(GemvQuadArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int K = 256 * STEPS, KQ = K / 32, THREADS = kQuadWaves * 64, ROWS = kQuadRows;
    constexpr int XBYTES = 4 * 2 * K; // the staged activations
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int i = lane & 3, b = lane >> 2;
    const uint32_t nwg = gridDim.x;
    // every XCD takes one run of consecutive rows (workgroups go round the eight XCDs in turn)
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t row0 = wg * ROWS;
    const uint32_t last = g.M - 1 - row0; // rows past the end repeat the last one; never stored
    const uint8_t *qbase = g.qs + (uint64_t)row0 * K;
    const half_t *sbase = g.scales + (uint64_t)row0 * KQ;
    const half_t *xg = g.X;
    half_t *obase = g.out;
    if (blockIdx.y != 0) {
        asm volatile("" ::: "memory"); // keeps this a branch
        const int64_t s = blockIdx.y;
        qbase += s * g.q_ss, sbase += s * g.s_ss, xg += s * g.x_ss, obase += s * g.o_ss;
    }

    // 1. the activations: the workgroup stages all of K per vector
    const uint32_t nxv = g.NC * (K / 8);
    constexpr int XV = (4 * K / 8 + THREADS - 1) / THREADS;
    uint4_t xv[XV];
#pragma unroll
    for (int n = 0; n < XV; n++) {
        const uint32_t v = min((uint32_t)(n * THREADS + t), nxv - 1); // threads past the end re-read the last vector
        const uint32_t j = v / (K / 8), kv = v % (K / 8);
        xv[n] = *(const uint4_t *)(xg + (j * g.b_js + 8 * kv));
    }
    asm volatile("" ::: "memory"); // keep the loads in this order
    // every wavefront's activation loads enter the compute unit's memory pipeline ahead of any weight load
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // 2. the scales of the workgroup's rows are one run of ROWS * KQ f16: 16 bytes per thread, whole lines
    constexpr int SV = (ROWS * KQ / 8 + THREADS - 1) / THREADS;
    const uint32_t nsv = (min((uint32_t)(ROWS - 1), last) + 1) * (KQ / 8); // 16-byte pieces that exist
    uint4_t sv[SV];
#pragma unroll
    for (int n = 0; n < SV; n++) sv[n] = *(const uint4_t *)(sbase + 8 * min((uint32_t)(n * THREADS + t), nsv - 1));
    asm volatile("" ::: "memory");
    // 3. the weight stream: lane 16 r + c reads 16 bytes of row r of the wavefront's four at K offset 16 c of every step
    const uint32_t rl = min((uint32_t)(wave * 4 + (lane >> 4)), last);
    const uint8_t *qp = qbase + (rl * (uint32_t)K + (uint32_t)(16 * (lane & 15)));
    uint4_t w[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) w[st] = __builtin_nontemporal_load((const uint4_t *)(qp + 256 * st));
    asm volatile("" ::: "memory");
    // the lane that stores row ii of vector j is lane (b = ii, i = j) (lanes with b >= 4 idle); its bias value,
    // unconditional and raw (a branch here would wait for every load above)
    const uint32_t brow = row0 + min((uint32_t)(wave * 4 + (b & 3)), last);
    const uint32_t bj = min((uint32_t)i, g.NC - 1);
    const uint16_t bias_raw = *(const uint16_t *)(g.bias + (brow * g.bias_rs + bj * (1u - g.bias_rs)));
    asm volatile("" ::: "memory");
    // 4. activations -> LDS in operand order: slot (2 s + h) * 64 + 4 b + j holds the eight values
    //    K = 256 s + 16 b + 8 h .. + 7 of vector j (the slots of a group of 64 are swizzled so that sixteen
    //    consecutive writers hit sixteen different bank groups); the barrier waits for these writes, not for the weights
#pragma unroll
    for (int n = 0; n < XV; n++) {
        const uint32_t v = n * THREADS + t;
        if (v < nxv) {
            const uint32_t j = v / (K / 8), kv = v % (K / 8);
            const uint32_t s = kv >> 5, bb = (kv >> 1) & 15, h = kv & 1;
            const uint32_t slot = ((s * 2 + h) * 64) + ((4 * bb + j) ^ (2 * h + ((bb >> 2) & 1)));
            *(uint4_t *)(smem + 16 * slot) = xv[n];
        }
    }
    // the scales -> LDS as they lie in memory, [ROWS][KQ]
    uint8_t *sl = smem + XBYTES;
#pragma unroll
    for (int n = 0; n < SV; n++)
        if (n * THREADS + t < ROWS * KQ / 8) *(uint4_t *)(sl + 16 * (n * THREADS + t)) = sv[n];
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // the scale of this lane's half block (row i, block 8 st + b / 2) at every step
    uint16_t dsc[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) dsc[st] = *(const uint16_t *)(sl + 2 * ((wave * 4 + i) * KQ + st * 8 + (b >> 1)));
    // this lane's operand B of every step: few enough to sit in registers while the weights are in flight
    const uint32_t xo[2] = {16u * (lane ^ ((lane >> 4) & 1)), 16u * (lane ^ (2 + ((lane >> 4) & 1)))};
    uint4_t xr[STEPS][2];
#pragma unroll
    for (int st = 0; st < STEPS; st++)
#pragma unroll
        for (int h = 0; h < 2; h++) xr[st][h] = *(const uint4_t *)(smem + xo[h] + 16 * 64 * (st * 2 + h));
    __builtin_amdgcn_sched_barrier(0);

    // 5. four chained 4x4x4 products per step, one block scale per step; lane 4 b + i takes its codes from lane 16 i + b
    const int src_lane4 = 4 * (16 * i + b);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    uint32_t wn[4];
#pragma unroll
    for (int d = 0; d < 4; d++) wn[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane4, (int)(uint32_t)w[0][d]);
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        uint32_t wp[4];
#pragma unroll
        for (int d = 0; d < 4; d++) wp[d] = wn[d];
        // the next step's codes cross the lanes while this step is multiplied
        if (st + 1 < STEPS) {
#pragma unroll
            for (int d = 0; d < 4; d++) wn[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane4, (int)(uint32_t)w[st + 1][d]);
        }
        __builtin_amdgcn_sched_barrier(0);
        float4_t p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t x0 = xr[st][d >> 1][2 * (d & 1)], x1 = xr[st][d >> 1][2 * (d & 1) + 1];
            const uint2_t xx = {x0, x1};
            p = __builtin_amdgcn_mfma_f32_4x4x4f16(quad_cvt_i8x4(wp[d]), __builtin_bit_cast(half4_t, xx), p, 0, 0, 0);
        }
        const float sc = (float)__builtin_bit_cast(half_t, dsc[st]);
        acc[0] = fmaf(quad_bcast<0>(sc), p[0], acc[0]);
        acc[1] = fmaf(quad_bcast<1>(sc), p[1], acc[1]);
        acc[2] = fmaf(quad_bcast<2>(sc), p[2], acc[2]);
        acc[3] = fmaf(quad_bcast<3>(sc), p[3], acc[3]);
    }

    // 6. the sixteen groups meet; lane (b = ii, i = j) keeps row ii of vector j and stores it
    const float r0 = quad_groups_sum(acc[0]), r1 = quad_groups_sum(acc[1]);
    const float r2 = quad_groups_sum(acc[2]), r3 = quad_groups_sum(acc[3]);
    const float res = (b & 2) ? ((b & 1) ? r3 : r2) : ((b & 1) ? r1 : r0);
    const uint32_t rw = wave * 4 + b;
    if (b < 4 && rw <= last && (uint32_t)i < g.NC) {
        const float bv = g.has_bias ? (float)__builtin_bit_cast(half_t, bias_raw) : 0.f;
        obase[(int64_t)(row0 + rw) * g.o_is + (int64_t)i * g.o_js] = (half_t)rt_act(res + bv, g.act);
    }
}

// Tunable: 1 = never take this kernel (for comparisons).
RT_TUNABLE(g_gemv_quad_disable, 0);

template <int STEPS> static hipError_t launch_quad_k(dim3 grid, hipStream_t st, const GemvQuadArgs &g) {
    constexpr size_t lds = (size_t)4 * 2 * 256 * STEPS + (size_t)kQuadRows * 8 * STEPS * 2;
    hipLaunchKernelGGL((gemv_q8h_quad_kernel<STEPS>), grid, dim3(kQuadWaves * 64), lds, st, g);
    return hipGetLastError();
}

// Q8_0H weights, 3 or 4 f16 activation vectors, K a multiple of 256 up to 4096, enough rows that the grid of 16-row
// workgroups covers the compute units.  hipErrorNotSupported: the shape or alignment does not fit and another kernel must run.
hipError_t launch_gemv_q8h_quad(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemv_quad_disable) return hipErrorNotSupported;
    if (p.a_dt != RT_Q8_0H || p.act_dt != RT_F16 || p.N < 3 || p.N > 4 || p.K < 256 || p.K % 256 != 0 || p.K > 4096)
        return hipErrorNotSupported;
    if (p.stacks > 65535 || p.b_ks != 1 || p.M < 1 || p.M > 0x7fffffff) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_js * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    const int64_t groups = (p.M + kQuadRows - 1) / kQuadRows;
    if (groups * p.stacks < dev.num_cus) return hipErrorNotSupported;

    GemvQuadArgs g{};
    const uint64_t numel = (uint64_t)p.a_stack * p.M * p.K;
    g.qs = (const uint8_t *)A;
    g.scales = (const half_t *)((const uint8_t *)A + rt_q8_0_scale_offset(numel));
    g.X = (const half_t *)B, g.out = (half_t *)out;
    g.bias = p.has_bias ? (const half_t *)bias : g.scales;
    g.bias_rs = p.has_bias && p.bias_on_rows ? 1u : 0u;
    g.M = (uint32_t)p.M, g.NC = (uint32_t)p.N;
    g.b_js = p.b_js;
    g.o_is = p.o_is, g.o_js = p.o_js;
    g.q_ss = p.a_stack == 1 ? 0 : p.M * p.K, g.s_ss = p.a_stack == 1 ? 0 : p.M * (p.K / 32);
    g.x_ss = p.b_stack == 1 ? 0 : p.b_bs, g.o_ss = p.o_bs;
    g.has_bias = p.has_bias, g.act = p.act;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    switch (p.K / 256) {
    case 1: return launch_quad_k<1>(grid, stream, g);
    case 2: return launch_quad_k<2>(grid, stream, g);
    case 3: return launch_quad_k<3>(grid, stream, g);
    case 4: return launch_quad_k<4>(grid, stream, g);
    case 5: return launch_quad_k<5>(grid, stream, g);
    case 6: return launch_quad_k<6>(grid, stream, g);
    case 7: return launch_quad_k<7>(grid, stream, g);
    case 8: return launch_quad_k<8>(grid, stream, g);
    case 9: return launch_quad_k<9>(grid, stream, g);
    case 10: return launch_quad_k<10>(grid, stream, g);
    case 11: return launch_quad_k<11>(grid, stream, g);
    case 12: return launch_quad_k<12>(grid, stream, g);
    case 13: return launch_quad_k<13>(grid, stream, g);
    case 14: return launch_quad_k<14>(grid, stream, g);
    case 15: return launch_quad_k<15>(grid, stream, g);
    case 16: return launch_quad_k<16>(grid, stream, g);
    default: return hipErrorNotSupported;
    }
}

} // namespace rt
