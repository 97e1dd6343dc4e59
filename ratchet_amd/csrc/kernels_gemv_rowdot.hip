// Row-streaming Q8_0H GEMV for one or two activation vectors (the decode step).
//
//   y[j, n] = sum_b d[n, b] * ( sum_{k in block b} q[n, k] * x[j, k] )  (+ bias)
//
// The weight matrix is read as what it is in memory, one long run of bytes: a wavefront
// (for short rows a half-wave) owns one weight row and every load instruction fetches 1 KiB
// (512) consecutive bytes of it, 16 per lane, so a wavefront touches whole 128-byte lines and
// touches each exactly once.  That is what lets the loads be non-temporal (the stream is not
// kept in the caches it passes through) and it is worth 0.8 us of 7.6 at the Phi-2 shape
// against the matrix-core kernel, whose operand layout (16 rows x 64 bytes per instruction)
// reads every line in two halves from two instructions.  Measured with that kernel's own
// arithmetic on a linear address pattern: 7.56 -> 7.06 us, non-temporal 6.78 us; the
// same non-temporal loads on the 16-row pattern: 9.05 us.
//
// A lane multiplies its 16 codes with the 16 activations at the same K positions:
// the codes are widened to f16 exactly, v_dot2_f32_f16 accumulates the products in
// f32 and the half-block's sum is scaled by the block's f16 scale in f32, so no weight is
// rounded.  The partial sums of a row meet in six (five) DPP additions; nothing is
// summed across wavefronts and the kernel ends without a barrier.  The activations
// are staged once per workgroup in LDS (their loads are issued first and the one
// barrier waits for them only), then held in registers.
//
// What a launch of this kernel costs beyond reading the bytes, measured at the Phi-2
// up-projection by taking parts away: the store of the results 0.35 us (any store: a
// kernel that leaves modified lines in the eight L2s pays for their write-back when it
// ends), the scales 0.45 (0.3 of it their 6 % of the bytes), staging the activations 0.2,
// the arithmetic 0.2, the bias 0.05.
//
// With more vectors the dot products repeat per vector while a matrix instruction takes
// 16 vectors at once: this kernel wins for one and two vectors (6.4 / 7.2 us against
// 7.6 / 7.8 us) and loses from three (9.0 against 8.6 us), where the matrix-core
// kernel stays in charge.
//
// Roles in the reference: ops/gemv.rs:333-558 (subgroup GEMV), kernel_builder.rs:222-240
// (unpack), dtype/blocks.rs:61-74 (segment layout).
#include "device_common.h"

namespace rt {

// What a wavefront needs before its first load comes first; everything a stack of products adds is a stride the
// launcher has already multiplied out (0 where the operand is shared by the stack).
struct GemvRowdotArgs {
    const uint8_t *qs;
    const half_t *scales;
    const half_t *X;
    const half_t *bias;     // never null: without a bias the scales, with both bias strides 0, and the value is dropped
    half_t *out;
    uint32_t M;             // weight rows
    uint32_t bias_rs;       // 1: a bias per weight row, 0: per vector
    int64_t b_js;           // elements between the activation vectors
    int64_t o_is, o_js;
    int64_t q_ss, s_ss, x_ss, o_ss; // per stack: bytes of codes, scales, activation elements, output elements
    int has_bias, act;
};

// WAVES: wavefronts per workgroup (4, 2 or 1), chosen by the launcher so that small grids still have a few workgroups
// per compute unit: with four wavefronts the Phi-2 down-projection (2560 rows, a wavefront per row) is 640 workgroups,
// two and a half per compute unit -- half of the chip with a third more work than the other -- and a 2560-row
// projection at K = 2560 is 320, one and a quarter.

// (q ^ 0x80) is q + 128 as an unsigned byte; 0x6400 | byte is the f16 1024 + byte; minus 1152 leaves q
__device__ __forceinline__ void rowdot_cvt_i8x4(uint32_t v, half2_t &lo, half2_t &hi) {
    v ^= 0x80808080u;
    const half2_t off = {(half_t)1152.0f, (half_t)1152.0f};
    lo = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - off;
    hi = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - off;
}

// How a wavefront's lanes are laid over the rows and K (LAY):
//   LAY == 1: K = 512 * STEPS; a wavefront owns two rows, one per half-wave, 512 bytes of each per step.
//   LAY == 2: K = 1024 * STEPS; a wavefront owns one row and reads 1 KiB of it per step.
//   LAY == 3: K = 1024 * STEPS - 512; as 2, but the last step is 512 bytes and lanes 32..63 sit it out.
// NCT activation vectors (1 or 2).  Offsets inside a workgroup's rows are 32-bit; the workgroup's base is 64-bit
// and wave-uniform.
template <int STEPS, int LAY, int NCT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_q8h_rowdot_kernel(GemvRowdotArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr bool LINEAR = LAY >= 2, HALF = LAY == 3;
    constexpr int K = LINEAR ? 1024 * STEPS - (HALF ? 512 : 0) : 512 * STEPS;
    constexpr int KQ = K / 32;
    constexpr int KSTEP = LINEAR ? 1024 : 512;
    constexpr int THREADS = WAVES * 64;
    constexpr int ROWS = LINEAR ? WAVES : WAVES * 2; // rows per workgroup
    half_t *xs = (half_t *)smem;                      // [NCT][K]
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int c = lane & 31, hr = lane >> 5;
    // Workgroups go round the eight XCDs in turn.  Give every XCD one run of consecutive rows, so that a 128-byte line
    // of the output (64 rows, eight workgroups) is written in one XCD's L2 and leaves it as one whole line when the kernel
    // ends, not as eight partial ones (6.44 -> 6.32 us at the Phi-2 up-projection).
    const uint32_t nwg = gridDim.x;
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t row0 = wg * ROWS;
    const int rw = LINEAR ? wave : 2 * wave + hr;                     // this lane's row within the workgroup
    const uint32_t last = min((uint32_t)(ROWS - 1), g.M - 1 - row0);    // rows past the end repeat the last one; never stored
    const uint32_t rc = min((uint32_t)rw, last);
    // this lane's offset into its row's K: k0 + KSTEP * st, but klast at the short last step of LAY 3
    const uint32_t k0 = LINEAR ? 16u * lane : 16u * c;
    const uint32_t klast = HALF ? 1024u * (STEPS - 1) + 16u * c : k0 + (uint32_t)(KSTEP * (STEPS - 1));
    // The bases of this workgroup's rows.  A wavefront's first load cannot leave before the scalar arithmetic in front
    // of it is done, so the terms of a stack of products (grid.y > 1) are only computed where there is one.
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
    constexpr int XV = (NCT * K / 8 + THREADS - 1) / THREADS;
    uint4_t xv[XV];
#pragma unroll
    for (int i = 0; i < XV; i++) {
        const uint32_t v = min((uint32_t)(i * THREADS + t), (uint32_t)(NCT * K / 8 - 1)); // threads past the end re-read the last vector
        const uint32_t j = v / (K / 8), kv = v % (K / 8);
        xv[i] = *(const uint4_t *)(xg + (j * g.b_js + 8 * kv));
    }
    asm volatile("" ::: "memory"); // keep the loads in this order
    // 2. the weight stream: 16 bytes per lane and step, 512 consecutive bytes per half-wave
    const uint8_t *qp = qbase + (rc * (uint32_t)K + k0);
    uint4_t w[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS - 1; st++) w[st] = __builtin_nontemporal_load((const uint4_t *)(qp + KSTEP * st));
    w[STEPS - 1] = __builtin_nontemporal_load((const uint4_t *)(qbase + (rc * (uint32_t)K + klast)));
    asm volatile("" ::: "memory");
    // 3. the scale of this lane's half block at every step, then the epilogue's bias (unconditional: without
    //    a bias it reads a scale and the value is dropped; a branch here would wait for every load above)
    const half_t *sp = sbase + (rc * (uint32_t)KQ + (k0 >> 5));
    uint16_t dsc[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS - 1; st++) dsc[st] = *(const uint16_t *)(sp + (KSTEP / 32) * st);
    dsc[STEPS - 1] = *(const uint16_t *)(sbase + (rc * (uint32_t)KQ + (klast >> 5)));
    uint16_t bias_raw[NCT];
#pragma unroll
    for (int j = 0; j < NCT; j++) {
        bias_raw[j] = *(const uint16_t *)(g.bias + ((row0 + rc) * g.bias_rs + j * (1u - g.bias_rs)));
    }
    asm volatile("" ::: "memory");
    // where this lane's row goes: computed here, while the loads are on their way, not after the last of them has arrived
    half_t *op = obase + (int64_t)(row0 + rw) * g.o_is;
    int64_t ojs = g.o_js;
    asm volatile("" : "+v"(op), "+s"(ojs));
    // 4. activations -> LDS; the barrier waits for the LDS writes, not for the weights
#pragma unroll
    for (int i = 0; i < XV; i++) {
        const uint32_t v = i * THREADS + t;
        if (v < NCT * K / 8) *(uint4_t *)(xs + 8 * v) = xv[i];
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // Nothing that touches a weight may move above this line or between the LDS reads below: the compiler likes to start
    // widening the first weight vector ahead of the barrier, and then the barrier and the reads of the activations wait for
    // that vector to arrive from memory instead of happening while it is on its way (0.06 us of 6.3 at the Phi-2 shape).
    __builtin_amdgcn_sched_barrier(0);
    // this lane's 16 activations per step; few enough to sit in registers while the weights are in flight
    constexpr bool HOIST = NCT * STEPS <= 6;
    uint4_t xa[HOIST ? NCT : 1][HOIST ? STEPS : 1], xb[HOIST ? NCT : 1][HOIST ? STEPS : 1];
    if (HOIST) {
#pragma unroll
        for (int j = 0; j < NCT; j++)
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                const half_t *xp = st == STEPS - 1 ? xs + klast : xs + k0 + KSTEP * st;
                xa[j][st] = *(const uint4_t *)(xp + j * K);
                xb[j][st] = *(const uint4_t *)(xp + j * K + 8);
            }
        __builtin_amdgcn_sched_barrier(0);
    }
    // 5. dot products, one block scale per step
    float acc[NCT];
#pragma unroll
    for (int j = 0; j < NCT; j++) acc[j] = 0.f;
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        half2_t wh[8];
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t ww = w[st][d];
            rowdot_cvt_i8x4(ww, wh[2 * d], wh[2 * d + 1]);
        }
        float sc = (float)__builtin_bit_cast(half_t, dsc[st]);
        if (HALF && st == STEPS - 1 && hr) sc = 0.f; // the short last step: lanes 32..63 re-read the first half
#pragma unroll
        for (int j = 0; j < NCT; j++) {
            uint4_t ya, yb;
            if (HOIST) ya = xa[j][st], yb = xb[j][st];
            else {
                const half_t *xp = st == STEPS - 1 ? xs + klast : xs + k0 + KSTEP * st;
                ya = *(const uint4_t *)(xp + j * K), yb = *(const uint4_t *)(xp + j * K + 8);
            }
            float p = 0.f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t xw = ya[d];
                p = __builtin_amdgcn_fdot2(wh[d], __builtin_bit_cast(half2_t, xw), p, false);
            }
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t xw = yb[d];
                p = __builtin_amdgcn_fdot2(wh[4 + d], __builtin_bit_cast(half2_t, xw), p, false);
            }
            acc[j] = fmaf(sc, p, acc[j]);
        }
    }
    // 6. the row's lanes meet; one lane per row writes
    const bool writer = LINEAR ? lane == 48 : c == 16;
#pragma unroll
    for (int j = 0; j < NCT; j++) {
        const float v = rowdot_sum<LINEAR>(acc[j]);
        if (writer && (uint32_t)rw <= last) {
            const float b = g.has_bias ? (float)__builtin_bit_cast(half_t, bias_raw[j]) : 0.f;
            op[j * ojs] = (half_t)rt_act(v + b, g.act);
        }
    }
}

// Tunable: 1 = never take this kernel (for comparisons).
RT_TUNABLE(g_gemv_rowdot_disable, 0);
// Tunable: 4, 2 or 1 forces that many wavefronts per workgroup (0 = by the size of the grid).
RT_TUNABLE(g_gemv_rowdot_waves, 0);

template <int STEPS, int LAY, int NCT, int WAVES>
static hipError_t launch_rowdot_w(dim3 grid, hipStream_t st, const GemvRowdotArgs &g) {
    constexpr size_t lds = (size_t)NCT * 2 * (LAY >= 2 ? 1024 * STEPS - (LAY == 3 ? 512 : 0) : 512 * STEPS);
    hipLaunchKernelGGL((gemv_q8h_rowdot_kernel<STEPS, LAY, NCT, WAVES>), grid, dim3(WAVES * 64), lds, st, g);
    return hipGetLastError();
}

// The step counts each layout is built for are the ones launch_gemv_q8h_rowdot can choose.
template <int STEPS, int LAY, int NCT>
static hipError_t launch_rowdot(int waves, dim3 grid, hipStream_t st, const GemvRowdotArgs &g) {
    constexpr int lo = LAY == 1 ? 1 : LAY == 2 ? 4 : 5;
    constexpr int hi = LAY == 1 ? 7 : 10;
    if constexpr (STEPS >= lo && STEPS <= hi) {
        if (waves == 4) return launch_rowdot_w<STEPS, LAY, NCT, 4>(grid, st, g);
        if (waves == 2) return launch_rowdot_w<STEPS, LAY, NCT, 2>(grid, st, g);
        if constexpr (LAY == 1) return launch_rowdot_w<STEPS, LAY, NCT, 1>(grid, st, g);
    }
    return hipErrorNotSupported;
}

template <int LAY, int NCT>
static hipError_t launch_rowdot_steps(int steps, int waves, dim3 grid, hipStream_t st, const GemvRowdotArgs &g) {
    switch (steps) {
    case 1: return launch_rowdot<1, LAY, NCT>(waves, grid, st, g);
    case 2: return launch_rowdot<2, LAY, NCT>(waves, grid, st, g);
    case 3: return launch_rowdot<3, LAY, NCT>(waves, grid, st, g);
    case 4: return launch_rowdot<4, LAY, NCT>(waves, grid, st, g);
    case 5: return launch_rowdot<5, LAY, NCT>(waves, grid, st, g);
    case 6: return launch_rowdot<6, LAY, NCT>(waves, grid, st, g);
    case 7: return launch_rowdot<7, LAY, NCT>(waves, grid, st, g);
    case 8: return launch_rowdot<8, LAY, NCT>(waves, grid, st, g);
    case 9: return launch_rowdot<9, LAY, NCT>(waves, grid, st, g);
    case 10: return launch_rowdot<10, LAY, NCT>(waves, grid, st, g);
    default: return hipErrorNotSupported;
    }
}

// Q8_0H weights, one or two f16 activation vectors, K a multiple of 512 up to 10240.
// hipErrorNotSupported: the shape or alignment does not fit and another kernel must run.
hipError_t launch_gemv_q8h_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                  hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemv_rowdot_disable) return hipErrorNotSupported;
    if (p.a_dt != RT_Q8_0H || p.act_dt != RT_F16 || p.N < 1 || p.N > 2 || p.K < 512 || p.K % 512 != 0)
        return hipErrorNotSupported;
    if (p.stacks > 65535 || p.b_ks != 1 || p.M < 1 || p.M > 0x7fffffff) return hipErrorNotSupported;
    const int64_t bjs = p.N == 1 ? 0 : p.b_js;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (bjs * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    if (p.K > 10240) return hipErrorNotSupported;
    // The layout.  Short rows: a half-wave per row, so that every lane has work at every step.  From K = 4096 a
    // wavefront per row with 1 KiB per step: half as many steps, scale loads and activation registers per lane, twice
    // as many wavefronts.  Measured, half-wave against wavefront per row, one vector: 16384 x 512 3.5 / 4.6 us;
    // 8192 x 1024 3.5 / 3.5; 4096 x 1536 3.2 / 3.2; 10240 x 2560 6.24 / 6.23 (and 4.9 / 5.2 with the weights in the
    // Infinity Cache); 4096 x 4096 5.2 / 4.9; 11008 x 4096 10.0 / 9.2; 5120 x 5120 6.9 / 6.4.  Two vectors:
    // 10240 x 2560 7.0 / 7.9; 4096 x 4096 5.9 / 5.8; 11008 x 4096 12.1 / 10.9; 5120 x 5120 8.9 / 7.5.
    int lay = 1, steps = (int)(p.K / 512);
    if (p.K >= 4096) lay = p.K % 1024 ? 3 : 2, steps = (int)((p.K + 512) / 1024);
    const int rpw = lay == 1 ? 2 : 1; // rows per wavefront
    // wavefronts per workgroup: for one vector, the most that still give the grid three workgroups per compute unit
    // (but at least two rows per workgroup).  With two vectors the activations a workgroup stages double and four
    // wavefronts stay best everywhere.
    int waves = 4;
    if (p.N == 1)
        while (waves * rpw > 2 && (p.M + waves * rpw - 1) / (waves * rpw) * p.stacks < 3 * (int64_t)dev.num_cus) waves >>= 1;
    if (g_gemv_rowdot_waves > 0) waves = g_gemv_rowdot_waves;
    const int rows = waves * rpw;
    const int64_t groups = (p.M + rows - 1) / rows;
    if (groups > 0x7fffffff) return hipErrorNotSupported;

    GemvRowdotArgs g{};
    const uint64_t numel = (uint64_t)p.a_stack * p.M * p.K;
    g.qs = (const uint8_t *)A;
    g.scales = (const half_t *)((const uint8_t *)A + rt_q8_0_scale_offset(numel));
    g.X = (const half_t *)B, g.out = (half_t *)out;
    g.bias = p.has_bias ? (const half_t *)bias : g.scales;
    g.bias_rs = p.has_bias && p.bias_on_rows ? 1u : 0u;
    g.M = (uint32_t)p.M;
    g.b_js = bjs;
    g.o_is = p.o_is, g.o_js = p.o_js;
    g.q_ss = p.a_stack == 1 ? 0 : p.M * p.K, g.s_ss = p.a_stack == 1 ? 0 : p.M * (p.K / 32);
    g.x_ss = p.b_stack == 1 ? 0 : p.b_bs, g.o_ss = p.o_bs;
    g.has_bias = p.has_bias, g.act = p.act;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    switch (lay) {
    case 1: return p.N == 1 ? launch_rowdot_steps<1, 1>(steps, waves, grid, stream, g) : launch_rowdot_steps<1, 2>(steps, waves, grid, stream, g);
    case 2: return p.N == 1 ? launch_rowdot_steps<2, 1>(steps, waves, grid, stream, g) : launch_rowdot_steps<2, 2>(steps, waves, grid, stream, g);
    default: return p.N == 1 ? launch_rowdot_steps<3, 1>(steps, waves, grid, stream, g) : launch_rowdot_steps<3, 2>(steps, waves, grid, stream, g);
    }
}

} // namespace rt
