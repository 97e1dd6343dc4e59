// Row-streaming GEMV for f16 and f32 weights, one activation vector (the decode step of an
// unquantized checkpoint) or a few.
//
//   y[n] = sum_k W[n, k] * x[k]  (+ bias)
//
// The layout of the Q8_0H row-streaming kernel with a whole wavefront per row: every load
// instruction of a wavefront fetches 1 KiB of consecutive bytes of its row, 16 per lane, each
// 128-byte line exactly once, non-temporal; all of a row's loads (at most ten: rows up to 10 KiB)
// are issued before the first is consumed.  The activations are staged once per workgroup in LDS
// (their loads are issued first and the one barrier waits for them only), then held in
// registers while the weights are on their way.  f16 products go through v_dot2_f32_f16 (exact
// products, f32 accumulation), f32 through fused multiply-adds; the 64 partial sums of a row meet in
// six DPP additions and nothing is summed across wavefronts.  Workgroups take the XCDs in turn, so
// every XCD is given one run of consecutive rows and an output line leaves one L2 whole.
//
// Measured at 10240 x 2560: f16 13.1 -> 9.1 us (0.72 of the HBM peak), f32 23.1 -> 16.6 us (0.79) against the one-load-at-a-time
// kernel in kernels_gemv.hip, which keeps every other shape (more vectors, unaligned rows).  Rows longer than
// 10 KiB (up to 64) take the looping form of the same stream, gemv_float_rowlong_kernel.
//
// Roles in the reference: ops/gemv.rs:156-331 (workgroup GEMV), ops/gemv.rs:333-558 (subgroup GEMV).
#include "device_common.h"

namespace rt {

struct GemvRowFloatArgs {
    const uint8_t *A;
    const uint8_t *X;
    const uint8_t *bias;    // never null: without a bias the activations, with the bias stride 0, and the value is dropped
    uint8_t *out;
    uint32_t M;             // weight rows
    uint32_t nvec;          // 16-byte vectors per row
    uint32_t bias_rs;       // 1: a bias per weight row, 0: one per activation vector
    uint32_t bias_js;       // 1: a bias per activation vector, 0: one per weight row (or none)
    uint32_t NC;            // activation vectors (1 .. the kernel's NCT)
    int64_t a_rs;           // bytes between rows
    int64_t x_js;           // bytes between activation vectors
    int64_t o_is, o_js;     // elements between the outputs of consecutive rows / vectors
    int64_t a_ss, x_ss, o_ss; // per stack: bytes of weights, bytes of activations, output elements
    int has_bias, act;
};

// NCT: activation vectors the kernel is built for (1, 2, 4); with fewer (g.NC) the spare ones repeat the last and are
// not stored.  The weights are read once for all of them; every vector adds its staged copy, its registers and its
// dot products.
template <typename AT, int STEPS, int WAVES, int NCT>
__global__ __launch_bounds__(WAVES * 64) void gemv_float_rowdot_kernel(GemvRowFloatArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int THREADS = WAVES * 64;
    uint4_t *xs = (uint4_t *)smem; // [NCT][nvec]
    const int t = threadIdx.x, lane = t & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t nwg = gridDim.x;
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t row0 = wg * WAVES;
    const uint32_t last = min((uint32_t)(WAVES - 1), g.M - 1 - row0); // rows past the end repeat the last one; never stored
    const uint32_t rc = min(wave, last);
    const uint8_t *abase = g.A + (uint64_t)(row0 + rc) * g.a_rs;
    const uint8_t *xg = g.X;
    AT *obase = (AT *)g.out;
    if (blockIdx.y != 0) {
        asm volatile("" ::: "memory"); // keeps this a branch: one product pays nothing for the terms of a stack
        const int64_t s = blockIdx.y;
        abase += s * g.a_ss, xg += s * g.x_ss, obase += s * g.o_ss;
    }
    const uint32_t nvec = g.nvec;

    // 1. the activations: the workgroup stages the whole vectors
    constexpr int XV = (64 * STEPS + THREADS - 1) / THREADS;
    uint4_t xv[NCT][XV];
#pragma unroll
    for (int j = 0; j < NCT; j++) {
        const uint8_t *xj = NCT == 1 ? xg : xg + (int64_t)min((uint32_t)j, g.NC - 1) * g.x_js;
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const uint32_t v = min((uint32_t)(i * THREADS + t), nvec - 1); // threads past the end re-read the last vector
            xv[j][i] = *(const uint4_t *)(xj + 16 * v);
        }
    }
    asm volatile("" ::: "memory"); // keep the loads in this order
    // 2. the row: 16 bytes per lane and step; only the last step can be short, its spare lanes re-read the row's end
    const uint32_t vl = min((uint32_t)(64 * (STEPS - 1) + lane), nvec - 1);
    uint4_t w[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS - 1; st++) w[st] = __builtin_nontemporal_load((const uint4_t *)(abase + 16 * (64 * st + lane)));
    w[STEPS - 1] = __builtin_nontemporal_load((const uint4_t *)(abase + 16 * vl));
    asm volatile("" ::: "memory");
    // 3. the epilogue's bias, unconditional (a branch here would wait for every load above)
    AT braw[NCT];
#pragma unroll
    for (int j = 0; j < NCT; j++)
        braw[j] = *(const AT *)(g.bias + sizeof(AT) * (size_t)((row0 + rc) * g.bias_rs + min((uint32_t)j, g.NC - 1) * g.bias_js));
    asm volatile("" ::: "memory");
    // where this row goes: computed while the loads are on their way
    AT *op = obase + (int64_t)(row0 + wave) * g.o_is;
    asm volatile("" : "+v"(op));
    // 4. activations -> LDS; the barrier waits for the LDS writes, not for the weights
#pragma unroll
    for (int j = 0; j < NCT; j++)
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const uint32_t v = i * THREADS + t;
            if (v < nvec) xs[j * nvec + v] = xv[j][i];
        }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0); // nothing that touches a weight moves above the barrier or between the LDS reads
    uint4_t xr[NCT][STEPS];
#pragma unroll
    for (int j = 0; j < NCT; j++) {
#pragma unroll
        for (int st = 0; st < STEPS - 1; st++) xr[j][st] = xs[j * nvec + 64 * st + lane];
        xr[j][STEPS - 1] = xs[j * nvec + vl];
    }
    __builtin_amdgcn_sched_barrier(0);
    // 5. dot products
    float acc[NCT];
#pragma unroll
    for (int j = 0; j < NCT; j++) acc[j] = 0.f;
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        const bool spare = st == STEPS - 1 && (uint32_t)(64 * (STEPS - 1) + lane) >= nvec; // a spare lane of the short step
#pragma unroll
        for (int j = 0; j < NCT; j++) {
            float p = 0.f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t ww = w[st][d], xw = xr[j][st][d];
                if constexpr (sizeof(AT) == 2) p = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ww), __builtin_bit_cast(half2_t, xw), p, false);
                else p = fmaf(__builtin_bit_cast(float, ww), __builtin_bit_cast(float, xw), p);
            }
            acc[j] += spare ? 0.f : p;
        }
    }
    // 6. the row's lanes meet; one lane writes
    float v[NCT];
#pragma unroll
    for (int j = 0; j < NCT; j++) v[j] = rowdot_sum<true>(acc[j]);
    if (lane == 63 && wave <= last) {
#pragma unroll
        for (int j = 0; j < NCT; j++) {
            const float b = g.has_bias ? to_f32(braw[j]) : 0.f;
            if (NCT == 1 || (uint32_t)j < g.NC) op[j * g.o_js] = from_f32<AT>(rt_act(v[j] + b, g.act));
        }
    }
}


// Rows longer than 10 KiB: the same wavefront-per-row stream in passes of 8 KiB, the next pass's loads in flight while
// this one is multiplied (two register sets).  Loads past the end of the row re-read its last vector and their
// products are dropped, so the loop has no branch around a load.  The activations stay in LDS (up to 64 KiB).
constexpr int kRowLongSteps = 8;

template <typename AT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_float_rowlong_kernel(GemvRowFloatArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int THREADS = WAVES * 64, PS = kRowLongSteps;
    uint4_t *xs = (uint4_t *)smem; // [nvec]
    const int t = threadIdx.x, lane = t & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t nwg = gridDim.x;
    const uint32_t wg = (nwg & 7) == 0 ? (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t row0 = wg * WAVES;
    const uint32_t last = min((uint32_t)(WAVES - 1), g.M - 1 - row0);
    const uint32_t rc = min(wave, last);
    const uint8_t *abase = g.A + (uint64_t)(row0 + rc) * g.a_rs;
    const uint8_t *xg = g.X;
    AT *obase = (AT *)g.out;
    if (blockIdx.y != 0) {
        asm volatile("" ::: "memory");
        const int64_t s = blockIdx.y;
        abase += s * g.a_ss, xg += s * g.x_ss, obase += s * g.o_ss;
    }
    const uint32_t nvec = g.nvec;
    const uint32_t npass = (nvec + 64 * PS - 1) / (64 * PS);

    uint4_t w0[PS], w1[PS];
    auto issue = [&](uint4_t (&w)[PS], uint32_t pass) __attribute__((always_inline)) {
#pragma unroll
        for (int st = 0; st < PS; st++) {
            const uint32_t i = min(64u * (pass * PS + st) + lane, nvec - 1);
            w[st] = __builtin_nontemporal_load((const uint4_t *)(abase + 16 * (size_t)i));
        }
    };
    // the activations first (they come from the L2), then the first pass of the row
    for (uint32_t v0 = 0; v0 < nvec; v0 += 4 * THREADS) {
        uint4_t xv[4];
#pragma unroll
        for (int i = 0; i < 4; i++) xv[i] = *(const uint4_t *)(xg + 16 * (size_t)min(v0 + i * THREADS + t, nvec - 1));
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (v0 + i * THREADS + t < nvec) xs[v0 + i * THREADS + t] = xv[i];
    }
    issue(w0, 0);
    const AT braw = *(const AT *)(g.bias + sizeof(AT) * (size_t)((row0 + rc) * g.bias_rs));
    AT *op = obase + (int64_t)(row0 + wave) * g.o_is;
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the barrier waits for the LDS writes, not for the row
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    float acc = 0.f;
    auto multiply = [&](const uint4_t (&w)[PS], uint32_t pass) __attribute__((always_inline)) {
#pragma unroll
        for (int st = 0; st < PS; st++) {
            const uint32_t i = 64u * (pass * PS + st) + lane;
            const uint4_t xv = xs[min(i, nvec - 1)];
            float p = 0.f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t ww = w[st][d], xw = xv[d];
                if constexpr (sizeof(AT) == 2) p = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ww), __builtin_bit_cast(half2_t, xw), p, false);
                else p = fmaf(__builtin_bit_cast(float, ww), __builtin_bit_cast(float, xw), p);
            }
            acc += i < nvec ? p : 0.f;
        }
    };
    for (uint32_t pass = 0; pass < npass; pass += 2) {
        issue(w1, pass + 1); // past the last pass: re-reads the row's end, dropped
        __builtin_amdgcn_sched_barrier(0);
        multiply(w0, pass);
        __builtin_amdgcn_sched_barrier(0);
        issue(w0, pass + 2);
        __builtin_amdgcn_sched_barrier(0);
        multiply(w1, pass + 1); // contributes nothing past the last pass
        __builtin_amdgcn_sched_barrier(0);
    }
    const float v = rowdot_sum<true>(acc);
    if (lane == 63 && wave <= last) {
        const float b = g.has_bias ? to_f32(braw) : 0.f;
        *op = from_f32<AT>(rt_act(v + b, g.act));
    }
}

// Tunable: 1 = never take these kernels (for comparisons).
RT_TUNABLE(g_gemv_rowfloat_disable, 0);
// Tunable: wavefronts (= rows) per workgroup, 0 = by the size of the grid.
RT_TUNABLE(g_gemv_rowfloat_waves, 0);

template <typename AT, int STEPS, int WAVES, int NCT>
static hipError_t launch_rowfloat_w(dim3 grid, size_t lds, hipStream_t st, const GemvRowFloatArgs &g) {
    hipLaunchKernelGGL((gemv_float_rowdot_kernel<AT, STEPS, WAVES, NCT>), grid, dim3(WAVES * 64), lds, st, g);
    return hipGetLastError();
}

// nct: 1, 2 or 4 vectors; more than one only with four wavefronts per workgroup, four only for f16 rows of up to 5 KiB
template <typename AT, int STEPS>
static hipError_t launch_rowfloat(int waves, int nct, dim3 grid, size_t lds, hipStream_t st, const GemvRowFloatArgs &g) {
    if (nct == 2) return launch_rowfloat_w<AT, STEPS, 4, 2>(grid, lds, st, g);
    if constexpr (sizeof(AT) == 2 && STEPS <= 5) {
        if (nct == 4) return launch_rowfloat_w<AT, STEPS, 4, 4>(grid, lds, st, g);
    }
    if (nct != 1) return hipErrorNotSupported;
    if (waves == 4) return launch_rowfloat_w<AT, STEPS, 4, 1>(grid, lds, st, g);
#ifdef RT_DEV_TUNABLES
    if (waves == 8) return launch_rowfloat_w<AT, STEPS, 8, 1>(grid, lds, st, g);
    if (waves == 5) return launch_rowfloat_w<AT, STEPS, 5, 1>(grid, lds, st, g);
    if (waves == 10) return launch_rowfloat_w<AT, STEPS, 10, 1>(grid, lds, st, g);
#endif
    return launch_rowfloat_w<AT, STEPS, 2, 1>(grid, lds, st, g);
}

template <typename AT>
static hipError_t launch_rowfloat_steps(int steps, int waves, int nct, dim3 grid, size_t lds, hipStream_t st, const GemvRowFloatArgs &g) {
    switch (steps) {
    case 1: return launch_rowfloat<AT, 1>(waves, nct, grid, lds, st, g);
    case 2: return launch_rowfloat<AT, 2>(waves, nct, grid, lds, st, g);
    case 3: return launch_rowfloat<AT, 3>(waves, nct, grid, lds, st, g);
    case 4: return launch_rowfloat<AT, 4>(waves, nct, grid, lds, st, g);
    case 5: return launch_rowfloat<AT, 5>(waves, nct, grid, lds, st, g);
    case 6: return launch_rowfloat<AT, 6>(waves, nct, grid, lds, st, g);
    case 7: return launch_rowfloat<AT, 7>(waves, nct, grid, lds, st, g);
    case 8: return launch_rowfloat<AT, 8>(waves, nct, grid, lds, st, g);
    case 9: return launch_rowfloat<AT, 9>(waves, nct, grid, lds, st, g);
    case 10: return launch_rowfloat<AT, 10>(waves, nct, grid, lds, st, g);
    default: return hipErrorNotSupported;
    }
}

template <typename AT, int WAVES>
static hipError_t launch_rowlong_w(dim3 grid, size_t lds, hipStream_t st, const GemvRowFloatArgs &g) {
    if (lds > 48 * 1024) {
        const hipError_t e = ensure_lds_limit<&gemv_float_rowlong_kernel<AT, WAVES>>();
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemv_float_rowlong_kernel<AT, WAVES>), grid, dim3(WAVES * 64), lds, st, g);
    return hipGetLastError();
}

static hipError_t launch_rowlong(bool f16, int waves, dim3 grid, size_t lds, hipStream_t st, const GemvRowFloatArgs &g) {
#ifdef RT_DEV_TUNABLES
    if (f16 && waves == 8) return launch_rowlong_w<half_t, 8>(grid, lds, st, g);
    if (f16 && waves == 5) return launch_rowlong_w<half_t, 5>(grid, lds, st, g);
    if (f16 && waves == 10) return launch_rowlong_w<half_t, 10>(grid, lds, st, g);
#endif
    if (f16) return waves == 4 ? launch_rowlong_w<half_t, 4>(grid, lds, st, g) : launch_rowlong_w<half_t, 2>(grid, lds, st, g);
    return waves == 4 ? launch_rowlong_w<float, 4>(grid, lds, st, g) : launch_rowlong_w<float, 2>(grid, lds, st, g);
}

// f16 or f32 weights with rows of whole 16-byte vectors, at most 64 KiB long, one activation vector of the same type;
// rows of up to 10 KiB also two vectors, f16 rows of up to 5 KiB up to four (10240 x 2560 f16: 2 / 4 vectors 11.0 / 14
// us on the one-load-at-a-time kernel).
// hipErrorNotSupported: the shape or alignment does not fit and another kernel must run.
hipError_t launch_gemv_float_rowdot(const Problem &p, const void *A, const void *B, const void *bias, void *out,
                                    hipStream_t stream, const DeviceInfo &dev) {
    if (g_gemv_rowfloat_disable) return hipErrorNotSupported;
    if (p.kernel != RT_KERNEL_GEMV_FLOAT || (p.act_dt != RT_F16 && p.act_dt != RT_F32) || p.N < 1 || p.N > 4) return hipErrorNotSupported;
    if (p.stacks > 65535 || p.a_ks != 1 || p.b_ks != 1 || p.M < 1 || p.M > 0x7fffffff) return hipErrorNotSupported;
    const int64_t esz = p.act_dt == RT_F16 ? 2 : 4;
    const int64_t row_bytes = p.K * esz;
    if (row_bytes < 16 || row_bytes % 16 != 0 || row_bytes > 64 * 1024) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.a_rs * esz) % 16 || (p.a_bs * esz) % 16 || (p.b_bs * esz) % 16)
        return hipErrorNotSupported;
    const uint32_t nvec = (uint32_t)(row_bytes / 16);
    const int steps = (int)((nvec + 63) / 64);
    const int nct = p.N == 1 ? 1 : p.N == 2 ? 2 : 4;
    if (nct > 1 && (steps > 10 || (p.b_js * esz) % 16 != 0)) return hipErrorNotSupported;
    if (nct == 4 && (p.act_dt != RT_F16 || steps > 5)) return hipErrorNotSupported;
    // four rows per workgroup; two where that leaves the grid under three workgroups per compute unit
    int waves = 4;
    if ((p.M + 3) / 4 * p.stacks < 3 * (int64_t)dev.num_cus) waves = 2;
    if (g_gemv_rowfloat_waves > 0) waves = g_gemv_rowfloat_waves;
    if (nct > 1) waves = 4;
    const int64_t groups = (p.M + waves - 1) / waves;
    if (groups > 0x7fffffff) return hipErrorNotSupported;

    GemvRowFloatArgs g{};
    g.A = (const uint8_t *)A, g.X = (const uint8_t *)B, g.out = (uint8_t *)out;
    g.bias = p.has_bias ? (const uint8_t *)bias : (const uint8_t *)B;
    g.bias_rs = p.has_bias && p.bias_on_rows ? 1u : 0u;
    g.bias_js = p.has_bias && !p.bias_on_rows ? 1u : 0u;
    g.NC = (uint32_t)p.N;
    g.x_js = p.N == 1 ? 0 : p.b_js * esz;
    g.o_js = p.o_js;
    g.M = (uint32_t)p.M, g.nvec = nvec;
    g.a_rs = p.a_rs * esz;
    g.o_is = p.o_is;
    g.a_ss = p.a_stack == 1 ? 0 : p.a_bs * esz, g.x_ss = p.b_stack == 1 ? 0 : p.b_bs * esz, g.o_ss = p.o_bs;
    g.has_bias = p.has_bias, g.act = p.act;
    dim3 grid((unsigned)groups, (unsigned)p.stacks);
    const size_t lds = (size_t)nct * nvec * 16;
    if (steps > 10) return launch_rowlong(p.act_dt == RT_F16, waves, grid, lds, stream, g);
    return p.act_dt == RT_F16 ? launch_rowfloat_steps<half_t>(steps, waves, nct, grid, lds, stream, g)
                              : launch_rowfloat_steps<float>(steps, waves, nct, grid, lds, stream, g);
}

} // namespace rt
