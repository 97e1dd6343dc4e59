// Weight-streaming GEMM for short prompts: f16 or Q8_0H weights x a few dozen K-contiguous f16 activation rows.
//
//   y[j, i] = sum_k W[i, k] x[j, k]  (+ bias)          f16 weights
//   y[j, i] = sum_b d[i, b] ( sum_{k in block b} q[i, k] x[j, k] )  (+ bias)   Q8_0H weights
//
// With this few activation rows the product is one pass over the weight.  A workgroup owns the weight rows of
// one compute unit's share (rows / compute units, rounded up to 8: up to TA tiles of 16) against ALL activation
// rows (TB tiles of 16), and K is split in quarters inside it; the four partial sums meet in LDS once at the end.
// Twelve wavefronts split the work three ways, in steps of 64 values of K (128 bytes, a whole line, per row):
//   * wavefront w (0..3) only reads MFMA fragments from LDS and multiplies quarter w of K;
//   * wavefront 4 + w streams that quarter's weights from HBM into its registers with plain 16-byte loads in
//     address order (a quad of lanes reads 64 consecutive bytes), DW steps ahead -- the registers are the
//     prefetch buffer of the HBM stream -- and writes a step at a time into one of two LDS slots in swizzled row
//     order (piece c of a row at slot c ^ ((row >> 1) & 7), so that the operand-order reads spread over the banks);
//   * wavefront 8 + w issues the LDS-DMA (global_load_lds) of that quarter's activations into a ring of SX
//     stages, swizzled the same way on the global side.
// One workgroup barrier per step.  Before barrier h the activation loader has seen stage (h + 1) % SX land, the
// weight loader has written slot (h + 1) % 2, the multiplying wavefront has read slot h % 2 and stage h % SX for
// the last time.  From five tiles of activation rows (f16 weights) K is split in halves instead and the two
// multiplying wavefronts of a half take half of the activation tiles each: see the kernel's NK.
//
// Why three roles.  A wavefront issues in order: one that cannot issue its next load (the compute unit's vector
// memory pipeline pushes back when its queue is full) cannot issue its MFMAs either.  With every wavefront loading
// and multiplying in turn (the first form of this kernel: 13.1 / 15.3 / 19.8 / 27.4 us at 16 / 32 / 64 / 128 rows
// of 10240 x 2560 f16 weights from HBM, against 12.5 / 14.4 / 17.3 us for this one) timestamps show a step as
// 1400 cycles of MFMAs and LDS reads followed by 2300 cycles in which 22 load instructions are issued, all four
// wavefronts in phase, the pipeline idle while they multiply.  Weights and activations come from different
// wavefronts because a wavefront's vector-memory instructions return in order: activations (L2 hits) issued
// behind weight loads (HBM misses) by the same wavefront do not count as landed before those.
// What bounds it now: the rate at which a compute unit's memory pipeline takes LDS-DMA (a step's eight instructions
// of an activation loader take about 1800 cycles to issue at 64 rows: 25 B/clk per compute unit with the weights,
// where the tiled GEMM's fill reaches 32), the 4.6 us before the first MFMA (HBM latency through cold TLBs, every
// compute unit asking at once) and 2 us of epilogue.
// Steps of 32 values of K (64 bytes per row) were measured: every line is then asked for twice, a step apart, and
// has left the L1 in between (17.1 against 12.5 us at 16 rows).  Loading the operands straight into registers in
// MFMA operand order (lane l: row l % 16, piece l / 16) is 2-8 us slower: neighbouring lanes then touch different
// lines, and the L1 handles an instruction a quad of lanes at a time.
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
    int has_bias, bias_on_rows, act, vec_out;
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

constexpr int gs_vmcnt(int n) { return 0x0F70 | (n & 0xF) | (((n >> 4) & 0x3) << 14); }

// The K ranges meet.  Called by the four multiplying wavefronts (threads 0..255) once nothing of theirs is on its way
// into LDS; three workgroup barriers (two when the output is not vectorised), which any other wavefront of the
// workgroup must match with gs_epilogue_barriers().
template <int TA, int TB, int NK>
__device__ __forceinline__ void gs_epilogue(const GemmStreamArgs &g, float4_t (&acc)[TA][TB / (4 / NK)], uint8_t *smem, int kpart, int bgrp,
                                            int lane, int t, int64_t row0, int last, const uint16_t (&bias_raw)[TA]) {
    constexpr int TBW = TB / (4 / NK); // activation tiles of one multiplying wavefront
    const int fr = lane & 15, fg = lane >> 4;
    __syncthreads(); // every wavefront is done with its ring: the regions change hands
    // every wavefront leaves its sums; the NK wavefronts that hold parts of the same tiles then take every NK-th of them
    float4_t *red = (float4_t *)smem;                             // [K part][TA * TB][64]
    half_t *Os = (half_t *)(smem + (size_t)NK * TA * TB * 1024);  // [16 TB][16 TA + 8]
    constexpr int OLD = 16 * TA + 8;
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < TBW; b++) red[(kpart * TA * TB + a * TB + bgrp * TBW + b) * 64 + lane] = acc[a][b];
    __syncthreads();
    half_t *out = g.out;
    const bool vec_out = g.vec_out != 0;
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int idx = 0; idx < TA * TBW; idx++) {
            if ((idx & (NK - 1)) != kpart) continue; // wave-uniform
            const int a = idx / TBW, b = bgrp * TBW + idx % TBW;
            float4_t v = red[(a * TB + b) * 64 + lane];
#pragma unroll
            for (int w2 = 1; w2 < NK; w2++) {
                const float4_t o = red[(w2 * TA * TB + a * TB + b) * 64 + lane];
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
    for (int idx = t; idx < total; idx += 256) {
        const int row = idx / cpr, c = idx - row * cpr;
        *(uint4_t *)(out + (int64_t)row * g.o_js + row0 + 8 * c) = *(const uint4_t *)(Os + row * OLD + 8 * c);
    }
}
__device__ __forceinline__ void gs_epilogue_barriers(const GemmStreamArgs &g) {
    __syncthreads();
    __syncthreads();
    if (g.vec_out) __syncthreads();
}

// a weight slot: a step of the wavefront's rows in swizzled row order (Q8_0H: 64 bytes of codes per row, then the
// rows' two block scales, a dword per row)
template <int TA, bool Q8> constexpr int gs3_wslot() { return Q8 ? TA * 16 * 64 + 256 : TA * 16 * 128; }
template <int TA, int TB, int SX, bool Q8> constexpr int gs3_pair_lds() { return SX * 16 * TB * 128 + 2 * gs3_wslot<TA, Q8>(); }
template <int TA, int TB, int SX, bool Q8, int NK> constexpr size_t gs3_lds_bytes() {
    constexpr size_t ring = (size_t)NK * gs3_pair_lds<TA, TB, SX, Q8>();
    constexpr size_t red = (size_t)NK * TA * TB * 1024 + (size_t)16 * TB * (16 * TA + 8) * 2;
    return ring > red ? ring : red;
}

// TA / TB: tiles of 16 weight rows / activation rows; SX: activation stages; DW: steps the weight loads run ahead; Q8: Q8_0H weights.
// NK: parts of K (4 or 2).  With K in halves the two multiplying wavefronts of a half take half of the activation tiles
// each (both read every weight fragment), each half has two weight and two activation loaders that deal its load
// instructions between them, there are half as many rings to hold and half as many partial sums to add: the form for
// six and eight tiles of activation rows, whose stages are too large for four rings.
template <int TA, int TB, int SX, int DW, bool Q8, int NK>
__global__ __launch_bounds__(768) void gemm_stream_kernel(GemmStreamArgs g) {
    static_assert(NK == 4 || (NK == 2 && !Q8 && TB % 2 == 0), "K in quarters, or in halves for f16 weights and an even tile count");
    constexpr int NB = 4 / NK, TBW = TB / NB, NLS = 4 / NK; // wavefronts per K part: multiplying, and loading of either kind
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int wv = __builtin_amdgcn_readfirstlane(t >> 6);
    const int role = wv >> 2; // 0 multiplies, 1 loads weights, 2 loads activations
    const int wave = (wv & 3) / NB, sub = (wv & 3) % NB; // the K part; the wavefront's number among its kind in that part
    const int fr = lane & 15, fg = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.x * g.rows_wg;
    const int last = (int)min((int64_t)g.rows_wg, g.M - row0) - 1; // rows past the share's end repeat its last row; never stored
    const uint32_t K = (uint32_t)g.K, kq = K / NK;
    const int nh = (int)(kq >> 6); // steps of 64 values of K
    constexpr int XSTAGE = 16 * TB * 128, WSLOT = gs3_wslot<TA, Q8>();
    constexpr int XLD = 2 * TB / NLS, WLD = (Q8 ? TA : 2 * TA) / NLS; // load instructions per step and loading wavefront
    uint8_t *xring = smem + wave * gs3_pair_lds<TA, TB, SX, Q8>();
    uint8_t *wslots = xring + SX * XSTAGE;

    if (role == 2) {
        // ---- activations: LDS-DMA instruction i fills rows 8 i + lane / 8 of a stage, lane l's 16 bytes landing at 16 l
        uint32_t xsrc[XLD];
#pragma unroll
        for (int i = 0; i < XLD; i++) {
            const int row = 8 * (i * NLS + sub) + (lane >> 3);
            const int c = (lane & 7) ^ ((row >> 1) & 7);
            xsrc[i] = ((uint32_t)min((int64_t)row, g.N - 1) * (uint32_t)g.b_js + 8u * c) * 2u;
        }
        const uint8_t *xbase = (const uint8_t *)(g.X + (int64_t)wave * kq);
        auto dma_x = [&](int h, int stage) {
            const uint8_t *xs = xbase + (int64_t)h * 128;
#pragma unroll
            for (int i = 0; i < XLD; i++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xs + xsrc[i]),
                                                 (__attribute__((address_space(3))) void *)(xring + stage * XSTAGE + (i * NLS + sub) * 1024), 16, 0, 0);
        };
        const int lasth = nh - 1;
#pragma unroll
        for (int u = 0; u < SX - 1; u++) dma_x(min(u, lasth), u); // steps 0 .. SX - 2
        // every step issues XLD instructions: "step h + 1 has landed" = all but the newest (SX - 2) x XLD have returned
        constexpr int kNewer = (SX - 2) * XLD;
        static_assert(kNewer < 64, "the wait counter has six bits");
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(gs_vmcnt(kNewer)); // step 0 has landed
        __builtin_amdgcn_s_barrier();                 // barrier -1
        int fill = SX - 1;
        for (int h = 0; h < nh; h++) {
            // stage (h - 1) % SX was read for the last time before the barrier just passed
            dma_x(min(h + SX - 1, lasth), fill); // past the end: the last step again, into a stage nobody reads
            fill = fill + 1 == SX ? 0 : fill + 1;
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(gs_vmcnt(kNewer));
            __builtin_amdgcn_s_barrier(); // barrier h: step h + 1 has landed
            asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_s_waitcnt(gs_vmcnt(0)); // nothing lands once the regions change hands
        gs_epilogue_barriers(g);
        return;
    }
    if (role == 1) {
        // ---- weights: instruction i takes rows 8 i + lane / 8 and the 16-byte piece lane % 8 of the step's 128 bytes of each
        // (Q8_0H: rows 16 i + lane / 4, piece lane % 4 of the step's 64 bytes of codes; and lane l the dword of
        // the step's two block scales of row l, for the first 16 TA lanes)
        uint32_t woff[WLD], wst[WLD];
#pragma unroll
        for (int i = 0; i < WLD; i++) {
            const int rl = Q8 ? 16 * (i * NLS + sub) + (lane >> 2) : 8 * (i * NLS + sub) + (lane >> 3), c = Q8 ? lane & 3 : lane & 7;
            woff[i] = Q8 ? (uint32_t)min(rl, last) * K + 16u * c : (uint32_t)min(rl, last) * K * 2u + 16u * c;
            wst[i] = Q8 ? (uint32_t)(rl * 64 + 16 * (c ^ ((rl >> 2) & 3))) : (uint32_t)(rl * 128 + 16 * (c ^ ((rl >> 1) & 7)));
        }
        const uint32_t soff = (uint32_t)min(min(lane, 16 * TA - 1), last) * (K >> 5) * 2u;
        const uint8_t *wbase = g.W + (row0 * g.K + (int64_t)wave * kq) * (Q8 ? 1 : 2);
        const uint8_t *sbase = (const uint8_t *)(g.scales + (Q8 ? row0 * (g.K >> 5) + (int64_t)wave * (kq >> 5) : 0));
        struct WBuf {
            uint4_t v[WLD];
            uint32_t sc;
        };
        auto load_w = [&](int h, WBuf &w) {
            const uint8_t *ws = wbase + (int64_t)h * (Q8 ? 64 : 128);
#pragma unroll
            for (int i = 0; i < WLD; i++) w.v[i] = __builtin_nontemporal_load((const uint4_t *)(ws + woff[i]));
            if constexpr (Q8) w.sc = *(const uint32_t *)(sbase + (int64_t)h * 4 + soff);
        };
        auto put = [&](const WBuf &w, int slot) {
#pragma unroll
            for (int i = 0; i < WLD; i++) *(uint4_t *)(wslots + slot * WSLOT + wst[i]) = w.v[i];
            if constexpr (Q8) *(uint32_t *)(wslots + slot * WSLOT + TA * 1024 + 4 * lane) = w.sc;
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the slot is written before the barrier that publishes it
            asm volatile("" ::: "memory");
        };
        WBuf wb[DW];
        const int lasth = nh - 1;
#pragma unroll
        for (int u = 0; u < DW; u++) load_w(min(u, lasth), wb[u]);
        __builtin_amdgcn_sched_barrier(0);
        put(wb[0], 0);
        __builtin_amdgcn_s_barrier(); // barrier -1: slot 0 holds step 0
        // between barriers h - 1 and h: slot (h + 1) % 2 gets step h + 1 (wb[(h + 1) % DW]); wb[h % DW], written out a
        // step ago, takes the loads of step h + DW
        static_assert(DW % 2 == 0, "the slot of a step is its parity");
        int h0 = 0;
        for (; h0 + DW <= nh; h0 += DW) {
#pragma unroll
            for (int u = 0; u < DW; u++) {
                __builtin_amdgcn_sched_barrier(0);
                load_w(min(h0 + u + DW, lasth), wb[u]);
                __builtin_amdgcn_sched_barrier(0);
                    put(wb[(u + 1) % DW], (u + 1) & 1);
                __builtin_amdgcn_s_barrier();
            }
        }
#pragma unroll
        for (int u = 0; u < DW - 1; u++) {
            if (h0 + u < nh) { // wave-uniform
                put(wb[(u + 1) % DW], (h0 + u + 1) & 1);
                __builtin_amdgcn_s_barrier();
            }
        }
        gs_epilogue_barriers(g);
        return;
    }

    // ---- multiplying wavefront `wave`
    uint16_t bias_raw[TA];
#pragma unroll
    for (int a = 0; a < TA; a++) {
        const uint16_t *bp = (g.has_bias && g.bias_on_rows) ? (const uint16_t *)g.bias + min(row0 + 16 * a + fr, g.M - 1) : (const uint16_t *)g.W;
        bias_raw[a] = *bp;
    }
    float4_t acc[TA][TBW];
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < TBW; b++) acc[a][b] = zero;
    // operand-order reads: lane (fr, fg) wants pieces pc and 4 + pc of row 16 tile + fr (Q8_0H: lane group fg feeds the
    // first MFMA of a step with K offsets 16 (fg & 1) + 8 (fg >> 1), the second with + 32; its 16 codes are piece fg)
    const int pc = Q8 ? 2 * (fg & 1) + (fg >> 1) : fg;
    const uint32_t rd0 = (uint32_t)(fr * 128 + 16 * (pc ^ ((fr >> 1) & 7))), rd1 = (uint32_t)(fr * 128 + 16 * ((4 + pc) ^ ((fr >> 1) & 7)));
    const uint32_t wq = (uint32_t)(fr * 64 + 16 * (fg ^ ((fr >> 2) & 3)));
    __builtin_amdgcn_s_barrier(); // barrier -1
    int stage = 0;
    for (int h = 0; h < nh; h++) {
        asm volatile("" ::: "memory");
        const uint8_t *ws = wslots + (h & 1) * WSLOT, *xs = xring + stage * XSTAGE + sub * (TBW * 2048);
        half8_t wf[TA][2];
        float d0[Q8 ? TA : 1], d1[Q8 ? TA : 1];
        if constexpr (Q8) {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                const uint4_t q = *(const uint4_t *)(ws + a * 1024 + wq);
                const half2_t d2 = __builtin_bit_cast(half2_t, *(const uint32_t *)(ws + TA * 1024 + 4 * (16 * a + fr)));
                const auto p0 = __builtin_amdgcn_permlane32_swap(q[0], q[2], false, false);
                const auto p1 = __builtin_amdgcn_permlane32_swap(q[1], q[3], false, false);
                wf[a][0] = stream_cvt_i8x8(p0[0], p1[0]);
                wf[a][1] = stream_cvt_i8x8(p0[1], p1[1]);
                d0[a] = (float)d2[0], d1[a] = (float)d2[1];
            }
        } else {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                wf[a][0] = __builtin_bit_cast(half8_t, *(const uint4_t *)(ws + a * 2048 + rd0));
                wf[a][1] = __builtin_bit_cast(half8_t, *(const uint4_t *)(ws + a * 2048 + rd1));
            }
        }
        half8_t xf[2][2];
        xf[0][0] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + rd0));
        xf[0][1] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + rd1));
#pragma unroll
        for (int b = 0; b < TBW; b++) {
            if (b + 1 < TBW) {
                xf[(b + 1) & 1][0] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + (b + 1) * 2048 + rd0));
                xf[(b + 1) & 1][1] = __builtin_bit_cast(half8_t, *(const uint4_t *)(xs + (b + 1) * 2048 + rd1));
            }
            if constexpr (Q8) {
#pragma unroll
                for (int a = 0; a < TA; a++) {
                    const float4_t P0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[b & 1][0], wf[a][0], zero, 0, 0, 0);
                    const float4_t P1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[b & 1][1], wf[a][1], zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[a][b][r] = fmaf(d1[a], P1[r], fmaf(d0[a], P0[r], acc[a][b][r]));
                }
            } else {
#pragma unroll
                for (int a = 0; a < TA; a++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[b & 1][0], wf[a][0], acc[a][b], 0, 0, 0);
#pragma unroll
                for (int a = 0; a < TA; a++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[b & 1][1], wf[a][1], acc[a][b], 0, 0, 0);
            }
        }
        stage = stage + 1 == SX ? 0 : stage + 1;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this step's fragment reads have returned
        __builtin_amdgcn_s_barrier();       // barrier h
    }
    gs_epilogue<TA, TB, NK>(g, acc, smem, wave, sub, lane, t, row0, last, bias_raw);
}

RT_TUNABLE(g_gemm_stream_disable, 0); // non-zero keeps short prompts on the tiled kernels (for comparisons)
RT_TUNABLE(g_gemm_stream_max_n, 0);   // activation rows up to which the kernel takes a product (0: the measured crossovers)

template <int TA, int TB, bool Q8, int NK> static hipError_t gs_launch(const GemmStreamArgs &g, unsigned nwg, hipStream_t stream) {
    // as many activation stages as fit a K part's share of 160 KB beside its two weight slots, at most 6.  The weight
    // loads run four steps ahead (2 or 6: the same to 2 %).
    constexpr int SXfit = (160 * 1024 / NK - 2 * gs3_wslot<TA, Q8>()) / (16 * TB * 128), SX = SXfit > 6 ? 6 : SXfit;
    static_assert(SX >= 2, "a stage to fill while one is read");
    constexpr size_t lds = gs3_lds_bytes<TA, TB, SX, Q8, NK>();
    static_assert(lds <= 160 * 1024, "one workgroup's rings fit a compute unit's LDS");
    if (lds > 48 * 1024) {
        if (const hipError_t e = ensure_lds_limit<&gemm_stream_kernel<TA, TB, SX, 4, Q8, NK>>(); e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemm_stream_kernel<TA, TB, SX, 4, Q8, NK>), dim3(nwg), dim3(768), lds, stream, g);
    return hipGetLastError();
}

RT_TUNABLE(g_gemm_stream_halves_from, 5); // activation tiles from which f16 weights take K in halves

template <int TA, bool Q8> static hipError_t gs_tb(int tb, const GemmStreamArgs &g, unsigned nwg, hipStream_t stream) {
    if constexpr (!Q8) {
        // f16 weights, five to eight tiles of activation rows: K in halves (10240 x 2560: 80 / 96 rows 19.8 / 20.4 us against
        // 21.2 / 21.4 with K in quarters, 64 rows 18.0 against 17.2; 112 / 128 rows, which do not fit four rings, 22.0 / 22.2)
        if (tb >= g_gemm_stream_halves_from) {
            if (tb <= 6) return gs_launch<TA, 6, Q8, 2>(g, nwg, stream);
            if (tb <= 8) return gs_launch<TA, 8, Q8, 2>(g, nwg, stream);
        }
    }
    switch (tb) {
    case 1: return gs_launch<TA, 1, Q8, 4>(g, nwg, stream);
    case 2: return gs_launch<TA, 2, Q8, 4>(g, nwg, stream);
    case 3: return gs_launch<TA, 3, Q8, 4>(g, nwg, stream);
    case 4: return gs_launch<TA, 4, Q8, 4>(g, nwg, stream);
    case 5:
    case 6: return gs_launch<TA, 6, Q8, 4>(g, nwg, stream);
    }
    return hipErrorNotSupported;
}

// f16 or Q8_0H weights (rows of K), K-contiguous f16 activations, one stack.
// Measured at 10240 x 2560 with the weights from HBM (this kernel / the tiled one, us): f16 weights 16 rows 12.5 / 16.1,
// 32: 14.4 / 17.7, 48: 16.1 / 19.3, 64: 17.3 / 20.5, 96: 20.4 / 25.2, 112: 22.0 / 26.5, 128: 22.2 / 27.2; Q8_0H 16: 11.9 /
// 15.8 (the streaming GEMV: 10.8), 32: 14.1 / 16.4, 48: 16.5 / 17.0, 64: 17.8 / 17.7, 96: 22.6 / 21.3.
// hipErrorNotSupported: another kernel must take the problem.
hipError_t launch_gemm_stream(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                              const DeviceInfo &dev) {
    const bool q8 = p.a_dt == RT_Q8_0H, f16 = p.a_dt == RT_F16;
    if (g_gemm_stream_disable || (!q8 && !f16) || p.act_dt != RT_F16) return hipErrorNotSupported;
    const int64_t max_n = g_gemm_stream_max_n ? g_gemm_stream_max_n : (q8 ? 48 : 128);
    if (p.stacks != 1 || p.N < 1 || p.N > max_n || p.N > (q8 ? 96 : 128) || p.K % 256 != 0 || p.K < 256 || p.b_ks != 1) return hipErrorNotSupported;
    if (f16 && (p.a_ks != 1 || p.a_rs != p.K)) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_js * 2) % 16) return hipErrorNotSupported;
    // every compute unit gets one workgroup with its share of the rows, up to 48; more rows: whole rounds of such shares
    const int64_t rounds = (p.M + 48 * (int64_t)dev.num_cus - 1) / (48 * (int64_t)dev.num_cus);
    const int64_t per = (p.M + rounds * dev.num_cus - 1) / (rounds * dev.num_cus);
    const int rows_wg = (int)((per + 7) / 8 * 8);
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
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
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
