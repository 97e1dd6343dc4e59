// Weight-streaming GEMM for short prompts: f16 or Q8_0H weights x a few dozen K-contiguous f16 activation rows.
//
//   y[j, i] = sum_k W[i, k] x[j, k]  (+ bias)          f16 weights
//   y[j, i] = sum_b d[i, b] ( sum_{k in block b} q[i, k] x[j, k] )  (+ bias)   Q8_0H weights
//
// With this few activation rows the product is one pass over the weight.  A workgroup owns the weight rows of
// one compute unit's share (rows / compute units, rounded up to 8: up to TA tiles of 16) against ALL activation
// rows (TB tiles of 16), and its four wavefronts split K in quarters: no workgroup barrier in the loop, the four
// partial sums meet in LDS once at the end.  Wavefront w walks its quarter in steps of 64 K-values:
//   * weights: plain 16-byte loads in address order (a quad of lanes reads 64 consecutive bytes; 8 rows x 128
//     bytes or 16 rows x 64 bytes per instruction), DW steps ahead, held in registers: the registers are the
//     prefetch buffer for the HBM stream.  A step's registers pass through a 6 KB LDS slot of the wavefront
//     (swizzled ds_write_b128, then ds_read_b128 in MFMA operand order; one wavefront's DS operations complete
//     in order, so nothing synchronises).  Loading them in operand order instead (lane l: row l % 16, piece
//     l / 16) is correct and 2-8 us slower: neighbouring lanes then touch different lines, and the L1 handles
//     an instruction a quad of lanes at a time;
//   * activations: LDS-DMA (global_load_lds) into a ring of DX stages private to the wavefront, slot s of a row
//     holding piece s ^ ((row >> 1) & 7) so that the operand-order reads spread over the banks.  Vector-memory
//     instructions of a wavefront return in order, so "the activations of this step have landed" is one
//     s_waitcnt vmcnt(n) with n the number of instructions issued behind them; the weights of the step are
//     older still.
// What it costs (timing-only variants at 10240 x 2560, weights from HBM): the parts add up rather than overlap.
// At 128 activation rows the MFMAs, fragment reads and the weight slot take 8 us, the activations' fill 6.6
// (every workgroup pulls all of X from L2: 168 MB), the weight stream 8.6, the epilogue 4.4: 27.6 us, no better
// than the tiled kernel; at 16 rows 13.0 us against 16.1.  With one wavefront per SIMD a wavefront's waits,
// LDS round trips and MFMAs take turns.  The launcher therefore only takes the row counts where it is ahead.
//
// Q8_0H: a lane's 16 bytes are 16 codes; lanes 0..31 hold block 2s of their row and lanes 32..63 block
// 2s + 1, and one v_permlane32_swap per dword pair regroups them so that each of the two MFMAs of a step
// sees one block (the order of K inside a block is free as long as the activation fragment agrees).  A
// block's f32 sums are multiplied by its scale in f32: no weight is rounded.
//
// The caller convention is Linear's W.gemm(x, b, false, true, true) (crates/ratchet-nn/src/linear.rs:17-24);
// the reference's kernel for it is the tiled shader of ops/gemm.rs:305-657.
#include "device_common.h"

namespace rt {

struct GemmStreamArgs {
    const uint8_t *W;      // f16 [rows][K] or int8 codes [rows][K]
    const half_t *scales;  // Q8_0H: f16 [rows][K / 32]
    const half_t *X;       // [N][b_js], K contiguous
    const half_t *bias;
    half_t *out;
    int64_t M, N, K;       // weight rows, activation rows, contraction (K % 256 == 0)
    int rows_wg;           // weight rows per workgroup: a multiple of 8, at most 16 TA
    int64_t b_js, o_is, o_js;
    int has_bias, bias_on_rows, act, vec_out, rot;
};

// 4 packed int8 -> the same integers as f16, exactly: 0x6400 | (q + 128) is 1024 + q + 128
__device__ __forceinline__ half8_t stream_cvt_i8x8(uint32_t v0, uint32_t v1) {
    const half2_t k = {(half_t)1152.0f, (half_t)1152.0f};
    v0 ^= 0x80808080u, v1 ^= 0x80808080u;
    const half2_t a = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v0, 0x04010400u)) - k;
    const half2_t b = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v0, 0x04030402u)) - k;
    const half2_t c = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v1, 0x04010400u)) - k;
    const half2_t d = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v1, 0x04030402u)) - k;
    return half8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

constexpr int GS_WAVES = 4;
// LDS of one wavefront: DX stages of its activation steps ([16 TB rows][128 bytes]), then the slot its weight
// step passes through on the way from load order to MFMA operand order
template <int TA, int TB, bool Q8, int DX> constexpr int gs_wave_lds() { return DX * 16 * TB * 128 + TA * 16 * (Q8 ? 64 : 128); }
template <int TA, int TB, bool Q8, int DX> constexpr size_t gs_lds_bytes() {
    constexpr size_t ring = (size_t)GS_WAVES * gs_wave_lds<TA, TB, Q8, DX>();
    // afterwards: a wavefront's partial sums in its own region, the f16 output tile [16 TB][16 TA + 8] behind all of them
    constexpr size_t red = (size_t)GS_WAVES * TA * TB * 1024 + (size_t)16 * TB * (16 * TA + 8) * 2;
    static_assert(TA * TB * 1024 <= gs_wave_lds<TA, TB, Q8, DX>() || true, "");
    return ring > red ? ring : red;
}
constexpr int gs_vmcnt(int n) { return 0x0F70 | (n & 0xF) | (((n >> 4) & 0x3) << 14); }

// TA / TB: tiles of 16 weight rows / activation rows; Q8: Q8_0H weights; DW / DX: steps a weight / activation load runs ahead
template <int TA, int TB, bool Q8, int DW, int DX>
__global__ __launch_bounds__(64 * GS_WAVES) void gemm_stream_kernel(GemmStreamArgs g) {
    static_assert(DW % DX == 0, "the activation ring divides the weight ring");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int fr = lane & 15, fg = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.x * g.rows_wg;
    const int last = (int)min((int64_t)g.rows_wg, g.M - row0) - 1; // rows past the share's end repeat its last row; never stored
    const uint32_t K = (uint32_t)g.K, kq = K >> 2;                 // this wavefront's K range: [wave kq, + kq)
    const int nsteps = (int)(kq >> 6);
    constexpr int WLD = Q8 ? TA : 2 * TA;  // 16-byte loads per weight step: 16 rows x 64 bytes or 8 rows x 128 bytes each
    constexpr int XLD = 2 * TB;            // LDS-DMA instructions per activation step: 8 rows x 128 bytes each
    constexpr int XSTAGE = 16 * TB * 128;
    constexpr int NW = WLD + (Q8 ? TA : 0); // vector-memory instructions per step that are not the activations'
    uint8_t *xring = smem + wave * gs_wave_lds<TA, TB, Q8, DX>();
    uint8_t *wslot = xring + DX * XSTAGE;

    struct WBuf {
        uint4_t v[WLD];
        uint32_t sc[Q8 ? TA : 1];
    };
    // 32-bit lane offsets from wave-uniform bases (the launcher checks the ranges).
    // Weights, load order: instruction i takes rows 8 i + lane / 8 (16 i + lane / 4) and the 16-byte piece lane % 8
    // (lane % 4) of the step's 128 (64) bytes of each: whole lines, neighbouring lanes on neighbouring addresses.
    uint32_t woff[WLD], wst[WLD], soff[Q8 ? TA : 1], xsrc[XLD];
#pragma unroll
    for (int i = 0; i < WLD; i++) {
        const int rl = Q8 ? 16 * i + (lane >> 2) : 8 * i + (lane >> 3), c = Q8 ? lane & 3 : lane & 7;
        woff[i] = (uint32_t)min(rl, last) * K * (Q8 ? 1u : 2u) + 16u * c;
        // its place in the slot: piece c of row rl at slot c ^ swizzle(rl), so that the operand-order reads
        // (16 rows, one piece each) spread over the banks
        wst[i] = Q8 ? (uint32_t)(rl * 64 + 16 * (c ^ ((rl >> 2) & 3))) : (uint32_t)(rl * 128 + 16 * (c ^ ((rl >> 1) & 7)));
    }
    if constexpr (Q8) {
#pragma unroll
        for (int a = 0; a < TA; a++) soff[a] = (uint32_t)min(16 * a + fr, last) * (K >> 5) * 2u;
    }
    // Activations: LDS-DMA instruction i fills rows 8 i + lane / 8 of a stage, lane l's 16 bytes landing at 16 l:
    // slot lane % 8 of the row holds piece (lane % 8) ^ ((row >> 1) & 7)
#pragma unroll
    for (int i = 0; i < XLD; i++) {
        const int row = 8 * i + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[i] = ((uint32_t)min((int64_t)row, g.N - 1) * (uint32_t)g.b_js + 8u * c) * 2u;
    }
    // operand-order reads: lane (fr, fg) wants piece 4 v + pc of row 16 tile + fr; Q8_0H: lane group fg feeds the
    // first MFMA of a step with K offsets 16 (fg & 1) + 8 (fg >> 1), the second with + 32
    const int pc = Q8 ? 2 * (fg & 1) + (fg >> 1) : fg;
    const uint32_t xrd0 = (uint32_t)(fr * 128 + 16 * (pc ^ ((fr >> 1) & 7))), xrd1 = (uint32_t)(fr * 128 + 16 * ((4 + pc) ^ ((fr >> 1) & 7)));
    const uint32_t wrd0 = Q8 ? (uint32_t)(fr * 64 + 16 * (fg ^ ((fr >> 2) & 3))) : xrd0, wrd1 = xrd1;

    const uint8_t *wbase = g.W + (row0 * g.K + (int64_t)wave * kq) * (Q8 ? 1 : 2);
    const uint8_t *sbase = (const uint8_t *)(g.scales + (Q8 ? row0 * (g.K >> 5) + (int64_t)wave * (kq >> 5) : 0));
    const uint8_t *xbase = (const uint8_t *)(g.X + (int64_t)wave * kq);

    auto load_w = [&](int s, WBuf &w) {
        const uint8_t *ws = wbase + (int64_t)s * (Q8 ? 64 : 128);
#pragma unroll
        for (int i = 0; i < WLD; i++) w.v[i] = *(const uint4_t *)(ws + woff[i]);
        if constexpr (Q8) {
            const uint8_t *ss = sbase + (int64_t)s * 4;
#pragma unroll
            for (int a = 0; a < TA; a++) w.sc[a] = *(const uint32_t *)(ss + soff[a]);
        }
    };
    auto dma_x = [&](int s, int stage) {
        const uint8_t *xs = xbase + (int64_t)s * 128;
#pragma unroll
        for (int i = 0; i < XLD; i++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xs + xsrc[i]),
                                             (__attribute__((address_space(3))) void *)(xring + stage * XSTAGE + i * 1024), 16, 0, 0);
    };
    // one step's loads, the activations' last: the wait below counts on that order
    auto issue = [&](int sw, WBuf &w, int sx, int stage) {
        __builtin_amdgcn_sched_barrier(0);
        load_w(sw, w);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        dma_x(sx, stage);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };

    // the epilogue's bias values, ahead of every other load: fetched at the end they would cost a trip to memory
    // with nothing to hide it (without a bias the load reads a weight and the value is dropped; no branch)
    uint16_t bias_raw[TA];
#pragma unroll
    for (int a = 0; a < TA; a++) {
        const uint16_t *bp = (g.has_bias && g.bias_on_rows) ? (const uint16_t *)g.bias + min(row0 + 16 * a + fr, g.M - 1) : (const uint16_t *)g.W;
        bias_raw[a] = *bp;
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    float4_t acc[TA][TB];
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < TB; b++) acc[a][b] = zero;

    // X of this step has landed when at most `younger` vector-memory instructions are outstanding (they return in
    // order); the step's weights are older still.  The wait comes first: with it in front of them the compiler
    // knows the weight registers have arrived and adds no wait of its own (which, with LDS-DMA in flight, is vmcnt(0)).
    auto compute = [&](auto younger, const WBuf &w, int stage) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(gs_vmcnt(decltype(younger)::value));
        asm volatile("" ::: "memory");
        // weights: load order -> slot -> operand order (one wavefront's DS operations complete in order)
#pragma unroll
        for (int i = 0; i < WLD; i++) *(uint4_t *)(wslot + wst[i]) = w.v[i];
        asm volatile("" ::: "memory");
        const uint8_t *xs = xring + stage * XSTAGE;
        auto xread = [&](int b, half8_t (&x)[2]) {
            x[0] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + b * 2048 + xrd0));
            x[1] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + b * 2048 + xrd1));
        };
        half8_t wf[TA][2];
        float d0[Q8 ? TA : 1], d1[Q8 ? TA : 1];
        if constexpr (Q8) {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                const uint4_t q = *(const uint4_t *)(wslot + a * 1024 + wrd0);
                const auto p0 = __builtin_amdgcn_permlane32_swap(q[0], q[2], false, false);
                const auto p1 = __builtin_amdgcn_permlane32_swap(q[1], q[3], false, false);
                wf[a][0] = stream_cvt_i8x8(p0[0], p1[0]);
                wf[a][1] = stream_cvt_i8x8(p0[1], p1[1]);
                const half2_t d2 = __builtin_bit_cast(half2_t, w.sc[a]);
                d0[a] = (float)d2[0], d1[a] = (float)d2[1];
            }
        } else {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                wf[a][0] = __builtin_bit_cast(half8_t, *(const uint4_t *)(wslot + a * 2048 + wrd0));
                wf[a][1] = __builtin_bit_cast(half8_t, *(const uint4_t *)(wslot + a * 2048 + wrd1));
            }
        }
        // fragment reads one tile of activation rows ahead of their MFMAs
        half8_t xf[2][2];
        xread(0, xf[0]);
        __builtin_amdgcn_sched_group_barrier(0x100, Q8 ? TA + 2 : 2 * TA + 2, 0);
#pragma unroll
        for (int b = 0; b < TB; b++) {
            if (b + 1 < TB) xread(b + 1, xf[(b + 1) & 1]);
            const half8_t x0 = xf[b & 1][0], x1 = xf[b & 1][1];
            if constexpr (Q8) {
#pragma unroll
                for (int a = 0; a < TA; a++) {
                    const float4_t P0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(x0, wf[a][0], zero, 0, 0, 0);
                    const float4_t P1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(x1, wf[a][1], zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[a][b][r] = fmaf(d1[a], P1[r], fmaf(d0[a], P0[r], acc[a][b][r]));
                }
            } else {
#pragma unroll
                for (int a = 0; a < TA; a++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x0, wf[a][0], acc[a][b], 0, 0, 0);
#pragma unroll
                for (int a = 0; a < TA; a++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x1, wf[a][1], acc[a][b], 0, 0, 0);
                if (b + 1 < TB) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2 * TA, 0);
            }
        }
        // the fragment reads have returned (their MFMAs are issued) before this step's slot and stage are written again
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        asm volatile("" ::: "memory");
    };

    WBuf wb[DW];
    const int lasts = nsteps - 1;
    // the loads of the first steps in the order the loop keeps: a step's weights, then its activations
#pragma unroll
    for (int u = 0; u < DW; u++) {
        if (u < DX) issue(min(u, lasts), wb[u], min(u, lasts), u);
        else {
            __builtin_amdgcn_sched_barrier(0);
            load_w(min(u, lasts), wb[u]);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // In the loop the activations of step s were issued DX steps before it, followed by DX - 1 whole steps of loads;
    // in the first trip by at least as many.
    constexpr int kYounger = (DX - 1) * (NW + XLD) < 63 ? (DX - 1) * (NW + XLD) : 63;
    int s0 = 0;
    for (; s0 + DW <= nsteps; s0 += DW) {
#pragma unroll
        for (int u = 0; u < DW; u++) {
            compute(std::integral_constant<int, kYounger>{}, wb[u], u % DX);
            issue(min(s0 + u + DW, lasts), wb[u], min(s0 + u + DX, lasts), u % DX); // past the end: the last step again, never multiplied
        }
    }
#pragma unroll
    for (int u = 0; u < DW - 1; u++) {
        if (s0 + u < nsteps) { // wave-uniform; the buffers hold steps s0 .. (clamped)
            compute(std::integral_constant<int, (DX - 1) * XLD>{}, wb[u], u % DX); // only activations are issued from here on
            __builtin_amdgcn_sched_barrier(0);
            dma_x(min(s0 + u + DX, lasts), u % DX);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __builtin_amdgcn_s_waitcnt(gs_vmcnt(0)); // nothing lands in LDS after this
    __syncthreads();                          // every wavefront is done with its ring: the regions change hands

    // ---- the four K ranges meet: every wavefront leaves its sums, then takes every fourth tile
    float4_t *red = (float4_t *)smem;                                       // [wave][TA * TB][64]
    half_t *Os = (half_t *)(smem + (size_t)GS_WAVES * TA * TB * 1024);      // [16 TB][16 TA + 8]
    constexpr int OLD = 16 * TA + 8;
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < TB; b++) red[(wave * TA * TB + a * TB + b) * 64 + lane] = acc[a][b];
    __syncthreads();
    half_t *out = g.out;
    const bool vec_out = g.vec_out != 0;
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int idx = 0; idx < TA * TB; idx++) {
            if ((idx & 3) != wave) continue; // wave-uniform
            const int a = idx / TB, b = idx % TB;
            float4_t v = red[idx * 64 + lane];
#pragma unroll
            for (int w2 = 1; w2 < GS_WAVES; w2++) {
                const float4_t o = red[(w2 * TA * TB + idx) * 64 + lane];
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] += o[r];
            }
            // v[r]: weight row row0 + 16 a + fr, activation row 16 b + 4 fg + r
            const int il = 16 * a + fr;
            const int64_t i = row0 + il;
            const bool row_ok = il <= last;
            const float bi = (g.has_bias && g.bias_on_rows) ? (float)__builtin_bit_cast(half_t, bias_raw[a]) : 0.f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int jl = 16 * b + 4 * fg + r;
                float y = v[r] + bi;
                if (g.has_bias && !g.bias_on_rows) y += (float)g.bias[min((int64_t)jl, g.N - 1)];
                const half_t h = (half_t)rt_act_k<decltype(has_act)::value>(y);
                if (vec_out) Os[jl * OLD + il] = h;
                else if (row_ok && jl < g.N) out[i * g.o_is + (int64_t)jl * g.o_js] = h;
            }
        }
    });
    if (!vec_out) return;
    __syncthreads();
    // the tile leaves as 16-byte stores along the weight rows (the share is a multiple of 8 rows)
    const int cpr = (last + 1) >> 3; // 16-byte pieces per activation row
    const int total = cpr * (int)min((int64_t)(16 * TB), g.N);
    for (int idx = t; idx < total; idx += 64 * GS_WAVES) {
        const int row = idx / cpr, c = idx - row * cpr;
        *(uint4_t *)(out + (int64_t)row * g.o_js + row0 + 8 * c) = *(const uint4_t *)(Os + row * OLD + 8 * c);
    }
}

RT_TUNABLE(g_gemm_stream_disable, 0); // non-zero keeps short prompts on the tiled kernels (for comparisons)
RT_TUNABLE(g_gemm_stream_max_n, 0);   // activation rows up to which the kernel takes a product (0: the measured crossovers)
RT_TUNABLE(g_gemm_stream_rows, 0);    // weight rows per workgroup (0: the launcher decides)
RT_TUNABLE(g_gemm_stream_rot, 1);     // workgroups start at different steps of K

template <int TA, int TB, bool Q8, int DW, int DX>
static hipError_t gs_launch(const GemmStreamArgs &g, unsigned nwg, hipStream_t stream) {
    constexpr size_t lds = gs_lds_bytes<TA, TB, Q8, DX>();
    static_assert(lds <= 160 * 1024, "one workgroup's rings fit a compute unit's LDS");
    if (lds > 48 * 1024) {
        if (const hipError_t e = ensure_lds_limit<&gemm_stream_kernel<TA, TB, Q8, DW, DX>>(); e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemm_stream_kernel<TA, TB, Q8, DW, DX>), dim3(nwg), dim3(64 * GS_WAVES), lds, stream, g);
    return hipGetLastError();
}

template <int TA, int TB, bool Q8> static hipError_t gs_depth(const GemmStreamArgs &g, unsigned nwg, hipStream_t stream) {
    // LDS: a wavefront's activation ring is DX stages of 2 KB x TB; registers: a weight step is 8 TA (5 TA for Q8_0H).
    // Weight loads 8 steps ahead measured 1 us slower than 4 at every row count (10240 x 2560).
    constexpr int DX = TB >= 5 ? 2 : 4;
    return gs_launch<TA, TB, Q8, 4, DX>(g, nwg, stream);
}

template <int TA, bool Q8> static hipError_t gs_tb(int tb, const GemmStreamArgs &g, unsigned nwg, hipStream_t stream) {
    switch (tb) {
    case 1: return gs_depth<TA, 1, Q8>(g, nwg, stream);
    case 2: return gs_depth<TA, 2, Q8>(g, nwg, stream);
    case 3: return gs_depth<TA, 3, Q8>(g, nwg, stream);
    case 4: return gs_depth<TA, 4, Q8>(g, nwg, stream);
    case 5:
    case 6: return gs_depth<TA, 6, Q8>(g, nwg, stream);
    case 7:
    case 8: return gs_depth<TA, 8, Q8>(g, nwg, stream);
    }
    return hipErrorNotSupported;
}

// f16 or Q8_0H weights (rows of K), K-contiguous f16 activations, one stack.
// Measured at 10240 x 2560 with the weights from HBM (this kernel / the tiled one, us): f16 weights 8 rows 12.7 / 15.4,
// 16: 13.1 / 16.1, 32: 15.1 / 17.7, 48: 17.7 / 19.3, 64: 19.8 / 20.5, 128: 27.6 / 27.3; Q8_0H 16: 12.9 / 15.8,
// 32: 15.3 / 16.3, 48: 17.6 / 17.0, 64: 20.0 / 17.5.  Up to 16 rows Q8_0H products are the streaming GEMV's.
// hipErrorNotSupported: another kernel must take the problem.
hipError_t launch_gemm_stream(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                              const DeviceInfo &dev) {
    const bool q8 = p.a_dt == RT_Q8_0H, f16 = p.a_dt == RT_F16;
    if (g_gemm_stream_disable || (!q8 && !f16) || p.act_dt != RT_F16) return hipErrorNotSupported;
    const int64_t max_n = g_gemm_stream_max_n ? g_gemm_stream_max_n : (q8 ? 32 : 64);
    if (p.stacks != 1 || p.N < 1 || p.N > max_n || p.N > 128 || p.K % 256 != 0 || p.K < 256 || p.b_ks != 1) return hipErrorNotSupported;
    if (f16 && (p.a_ks != 1 || p.a_rs != p.K)) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_js * 2) % 16) return hipErrorNotSupported;
    // every compute unit gets one workgroup with its share of the rows, up to 48; more rows: whole rounds of such shares
    const int64_t rounds = (p.M + 48 * (int64_t)dev.num_cus - 1) / (48 * (int64_t)dev.num_cus);
    const int64_t per = (p.M + rounds * dev.num_cus - 1) / (rounds * dev.num_cus);
    const int rows_wg = g_gemm_stream_rows ? g_gemm_stream_rows : (int)((per + 7) / 8 * 8);
    const int ta = (rows_wg + 15) / 16;
    const int64_t nwg = (p.M + rows_wg - 1) / rows_wg;
    // a weight with so few rows that a quarter of the compute units would stay idle is the tiled kernels' (they cut K)
    if (nwg * 4 < (int64_t)dev.num_cus * 3 || ta > 3) return hipErrorNotSupported;
    // a share's offsets are 32-bit: 48 rows of K, 128 activation rows of b_js
    if ((int64_t)rows_wg * p.K * 2 >= (int64_t(1) << 31) || p.N * p.b_js * 2 >= (int64_t(1) << 31)) return hipErrorNotSupported;
    GemmStreamArgs g{};
    g.W = (const uint8_t *)A;
    g.scales = q8 ? (const half_t *)((const uint8_t *)A + rt_q8_0_scale_offset((uint64_t)(p.M * p.K))) : nullptr;
    g.X = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    g.M = p.M, g.N = p.N, g.K = p.K, g.rows_wg = rows_wg;
    g.b_js = p.b_js, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act, g.rot = g_gemm_stream_rot;
    g.vec_out = p.M % 8 == 0 && p.o_is == 1 && p.o_js % 8 == 0 && ((uintptr_t)out & 15u) == 0;
    const int tb = (int)((p.N + 15) / 16);
    auto by_ta = [&](auto q8c) -> hipError_t {
        constexpr bool Q = decltype(q8c)::value;
        switch (ta) {
        case 1: return gs_tb<1, Q>(tb, g, (unsigned)nwg, stream);
        case 2: return gs_tb<2, Q>(tb, g, (unsigned)nwg, stream);
        case 3: return gs_tb<3, Q>(tb, g, (unsigned)nwg, stream);
        }
        return hipErrorNotSupported;
    };
    return q8 ? by_ta(std::true_type{}) : by_ta(std::false_type{});
}

} // namespace rt
