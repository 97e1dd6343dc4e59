// Q4_K weights x f16 activations for many activation rows (prefill), the weights never touching LDS:
// every multiplying wavefront decodes the raw blocks of its own 32 weight rows in registers, straight
// into the MFMA operand, and only the activation tile goes through LDS.
//
//   y[j, i] = sum_sb ( d_i,sb * sum_sub sum_{k in sub} x[j,k] (sc_i,sub q_i,k)  -  dmin_i,sb * sum_sub mn_i,sub S[j,sub] )
//   S[j, sub] = sum_{k in sub} x[j, k]
//
// The order of K inside an MFMA is free as long as both operands agree, so lane group g (lane / 16)
// of a weight fragment owns the 32 bytes g of a super-block's qs: the low nibbles are the values
// 64 g .. + 31 of the super-block (sub-block 2 g), the high nibbles the values 64 g + 32 .. + 63
// (sub-block 2 g + 1).  MFMA step t of a super-block takes from lane group g the values
// 64 g + 8 t .. + 7: bytes 8 (t % 4) .. + 7, low nibbles for t < 4, high for t >= 4.  A thread
// therefore reads a header and two 16-byte pieces per super-block and needs two of the eight scales
// and mins.  sc * q < 1024 is exact in f16 (fma(1024 + q, sc, -1024 sc) rounds once; the high
// nibbles stay in place as 1024 + 16 q against sc / 16), so a super-block chains through one MFMA
// accumulator and d is applied once per super-block in f32.  No weight is rounded.
//
// The sub-block sums of x fall out of the same layout: a lane of an activation fragment holds
// 8 values of sub-block 2 g (t < 4) or 2 g + 1 (t >= 4) of activation row lane % 16, so four dot
// products against ones per step give S for exactly the (row, sub-block pair) that the min-term MFMA
// wants from this lane.  Wavefront w sums the 16 activation rows of fragment w and shares them
// through LDS (f16 high + low parts, exact to 2^-22); the min term of super-block sb is one MFMA per
// output tile, run under super-block sb + 1.
//
// A workgroup owns 128 weight rows x 64 activation rows: four multiplying wavefronts (32 weight rows
// x 64 activation rows each: 64 MFMAs per super-block, 8 for the min term) and four that only issue
// the activation tiles' LDS-DMA loads (one per SIMD, so that no multiplying wavefront shares its SIMD
// with all of them), one super-block ahead in a ring of two stages.  A staged row is 32 K-vectors
// and one of padding: the 16 rows of a fragment read start 4 banks apart and a read address is a
// base + 16 * step, an immediate.  One barrier per super-block.  The output tile leaves through LDS
// as 16-byte stores when the output is contiguous along the weight rows.
//
// What bounds it (measured by leaving parts out): the parts add up.  A wavefront's MFMAs (8 issue
// cycles each when vector instructions follow), its 335 vector instructions per super-block and the
// LDS pipe time of the compute unit's fragment reads (128 KB per super-block at 128 B/clk) each
// cost their full time whatever the order of instructions.  Two multiplying wavefronts per SIMD were
// measured: with 16 x 64 outputs each they double the fragment reads (27.7 against 26.7 us), with
// 32 x 32 each they decode every weight twice (32.3 us).
//
// The arithmetic is ggml's dequantize_row_q4_K (the reference holds only the block struct,
// crates/ratchet-loader/src/k_quants.rs:94-103); the caller convention is Linear's
// W.gemm(x, b, false, true, true) (crates/ratchet-nn/src/linear.rs:17-24).
#include "device_common.h"

namespace rt {

struct GemmQ4kArgs {
    const uint8_t *blocks; // [stack][rows][K/256] super-blocks of 144 bytes
    const half_t *X;
    const half_t *bias;
    half_t *out;
    int64_t M, N; // weight rows, activation rows
    int64_t nsb;  // super-blocks per row
    int64_t a_stack, b_stack;
    int64_t b_bs, b_js;
    int64_t o_bs, o_is, o_js;
    int tiles_j, remap, vec_out;
    int has_bias, bias_on_rows, act;
};

constexpr int QR_BN = 64; // activation rows per workgroup; weight rows: 16 per MFMA tile x TA tiles x MW multiplying wavefronts
// An activation stage holds one super-block of K for 64 rows: 32 K-vectors of 16 bytes per row and one of padding,
// so that the 16 rows of a fragment read start 4 banks apart and a read address is base + 16 * step.
constexpr int QR_ROWB = 33 * 16;       // bytes per staged row
constexpr int QR_XSB = QR_BN * QR_ROWB; // bytes per stage = 33 LDS-DMA instructions of 1 KB
// Activation stages: the tile of the next super-block is on its way while this one is multiplied.  A third stage (two
// tiles in flight) measured the same to 1 % at every grid size tried (alternating runs on one device), so the smaller
// footprint stays: two workgroups fit a compute unit's LDS.
constexpr int QR_XST = 2;
constexpr int QR_LW = 4;               // wavefronts that only issue the LDS-DMA, one per SIMD
constexpr size_t QR_LDS = (size_t)QR_XST * QR_XSB + 2 * QR_BN * 4 * 8;

// TA: MFMA tiles of weight rows per wavefront; MW: multiplying wavefronts (4: each sums the activation fragment of its number)
template <int TA, int MW>
__global__ __launch_bounds__(64 * (MW + QR_LW)) void gemm_q4k_kernel(GemmQ4kArgs g) {
    constexpr int TB = 4;             // MFMA tiles per wavefront: TA of weight rows (second operand), TB of activation rows (first)
    constexpr int BM = 16 * TA * MW;  // weight rows per workgroup
    static_assert(MW == 4, "wavefront w sums the x of activation fragment w: four fragments, four wavefronts");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t *Xs = smem;                             // [QR_XST][64 rows][33 slots of 16 bytes]: K-vector v of row r in slot v
    uint2_t *Sx = (uint2_t *)(Xs + QR_XST * QR_XSB); // [2][64][4]: sums of x of super-block parity p, row, lane group: (high pair, low pair)

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int fr = lane & 15, fg = lane >> 4;
    const int64_t s = blockIdx.y;
    // the workgroups of one weight row block (one per block of activation rows) run on one XCD, whose L2 then
    // holds that block's raw weights for all of them
    uint32_t b = blockIdx.x;
    if (g.remap) b = (b & 7) * (gridDim.x >> 3) + (b >> 3);
    const uint32_t ti = b / (uint32_t)g.tiles_j, tj = b - ti * (uint32_t)g.tiles_j;
    const int64_t i0 = (int64_t)ti * BM, j0 = (int64_t)tj * QR_BN;
    const uint8_t *blocks = g.blocks + (g.a_stack == 1 ? 0 : s) * g.M * g.nsb * 144;
    const half_t *X = g.X + (g.b_stack == 1 ? 0 : s) * g.b_bs;
    const int64_t last = g.nsb - 1;
    const bool vec_out = g.vec_out && i0 + BM <= g.M; // a whole tile of weight rows, stored 16 bytes at a time

    if (wave >= MW) {
        // ---- loading wavefront lw: LDS-DMA instruction i of a stage (i = lw, lw + 4, ...; 33 in all) fills the 1 KB
        // run of slots 64 i .. + 63; slot p is K-vector p % 33 of row p / 33 (the 33rd is padding and repeats the 32nd).
        // Each of the four issues nine: the ninth of wavefronts 1..3 repeats instruction 32.
        constexpr int NI = 9;
        const int lw = wave - MW;
        uint32_t xsrc[NI];
#pragma unroll
        for (int n = 0; n < NI; n++) {
            const uint32_t p = 64u * (uint32_t)min(4 * n + lw, 32) + (uint32_t)lane;
            const uint32_t row = p / 33u, v = min(p - 33u * row, 31u);
            xsrc[n] = (uint32_t)min(j0 + (int64_t)row, g.N - 1) * (uint32_t)g.b_js + 8u * v;
        }
        auto issue_x = [&](int stage, int64_t sb) {
            const half_t *xk = X + sb * 256;
#pragma unroll
            for (int n = 0; n < NI; n++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xk + xsrc[n]),
                                                 (__attribute__((address_space(3))) void *)(Xs + stage * QR_XSB + min(4 * n + lw, 32) * 1024), 16, 0, 0);
        };
        constexpr int kNewer = QR_XST == 3 ? NI : 0; // with three stages the newest tile may still be on its way
        constexpr int kOlder = 0x0F70 | (kNewer & 0xF) | (((kNewer >> 4) & 0x3) << 14);
        auto publish = [&]() {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(kOlder);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        issue_x(0, 0);
        if (QR_XST == 3) issue_x(1, min((int64_t)1, last));
        publish(); // super-block 0
        int fill = QR_XST - 1;
        for (int64_t sb = 0; sb < last; sb++) {
            // stage `fill` held super-block sb - 1, read for the last time before the barrier just passed
            issue_x(fill, min(sb + QR_XST - 1, last)); // past the end: the last one again, into a stage nobody reads
            publish();                                 // super-block sb + 1
            fill = fill == QR_XST - 1 ? 0 : fill + 1;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): nothing lands after the wavefront has ended
        __builtin_amdgcn_s_barrier();       // the multiplying wavefronts' last exchange of sums
        if (vec_out) __builtin_amdgcn_s_barrier(); // and their staged output tile
        return;
    }

    // ---- multiplying wavefront `wave`: weight rows i0 + 32 wave .. + 31.  Rows past the end repeat the last
    // valid one.  Offsets are 32-bit from wave-uniform bases (the launcher checks the ranges).
    struct Raw {
        uint4_t hdr, qa, qb;
    };
    uint32_t woff[TA];
#pragma unroll
    for (int a = 0; a < TA; a++) woff[a] = (uint32_t)min(i0 + wave * (16 * TA) + 16 * a + fr, g.M - 1) * (uint32_t)g.nsb * 144u;
    auto load_raw = [&](int64_t sb, Raw (&r)[TA]) {
        const uint8_t *bsb = blocks + sb * 144; // wave-uniform
#pragma unroll
        for (int a = 0; a < TA; a++) {
            r[a].hdr = *(const uint4_t *)(bsb + woff[a]);
            r[a].qa = *(const uint4_t *)(bsb + (woff[a] + 16u + 32u * (uint32_t)fg));
            r[a].qb = *(const uint4_t *)(bsb + (woff[a] + 32u + 32u * (uint32_t)fg));
        }
    };
    // what a thread keeps of a super-block's header: the scale pairs for its two sub-blocks as FMA operands,
    // and for the min term (a super-block late) d, dmin and the two mins as f16 integers
    struct Scl {
        half2_t s_lo, n_lo, s_hi, n_hi;
    };
    struct Fin {
        float d, dmin;
        uint32_t mn;
    };
    const int sh = 16 * (fg & 1);
    const uint32_t upper = (fg & 2) ? ~0u : 0u; // sub-blocks 4..7: the scales and mins split over two bytes
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    auto header = [&](const Raw &r, Scl &sc, Fin &f) {
        // the 6-bit scales and mins (ggml get_scale_min_k4), four per dword; this thread's are 2 fg, 2 fg + 1
        const uint32_t S0 = r.hdr[1], S1 = r.hdr[2], S2 = r.hdr[3];
        const uint32_t sc47 = (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u), mn47 = ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u);
        const uint32_t scw = (sc47 & upper) | (S0 & 0x3F3F3F3Fu & ~upper); // no branch: a divergent one makes the compiler wait for every load
        const uint32_t mnw = (mn47 & upper) | (S1 & 0x3F3F3F3Fu & ~upper);
        const half2_t s2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, scw >> sh, 0x04010400u)) - k1024;
        const half2_t m2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, mnw >> sh, 0x04010400u)) - k1024;
        const half_t lo = s2[0], hi = s2[1] * (half_t)0.0625f;
        sc.s_lo = half2_t{lo, lo}, sc.s_hi = half2_t{hi, hi};
        sc.n_lo = sc.s_lo * (half_t)-1024.0f, sc.n_hi = sc.s_hi * (half_t)-1024.0f;
        const half2_t dm = __builtin_bit_cast(half2_t, r.hdr[0]);
        f.d = (float)dm[0], f.dmin = (float)dm[1], f.mn = __builtin_bit_cast(uint32_t, m2);
    };
    // weight fragment of step T: 8 values sc * q of this thread's row
    auto wfrag = [&](auto Tc, const Raw &r, const Scl &sc) {
        constexpr int T = decltype(Tc)::value;
        const uint4_t &q = (T & 2) ? r.qb : r.qa;
        const uint32_t mask = T < 4 ? 0x0F0F0F0Fu : 0xF0F0F0F0u;
        const uint32_t v0 = q[2 * (T & 1)] & mask, v1 = q[2 * (T & 1) + 1] & mask;
        const half2_t s2 = T < 4 ? sc.s_lo : sc.s_hi, n2 = T < 4 ? sc.n_lo : sc.n_hi;
        half2_t a = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v0, 0x04010400u));
        half2_t bb = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v0, 0x04030402u));
        half2_t c = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v1, 0x04010400u));
        half2_t d = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v1, 0x04030402u));
        a = __builtin_elementwise_fma(a, s2, n2), bb = __builtin_elementwise_fma(bb, s2, n2);
        c = __builtin_elementwise_fma(c, s2, n2), d = __builtin_elementwise_fma(d, s2, n2);
        return __builtin_bit_cast(half8_t, uint4_t{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, bb),
                                                   __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)});
    };
    // This wavefront's LDS stores (its sums of x) are done; past the barrier the next activation tile is whole,
    // the loading wavefront having waited for its slots, the stage of the tile before is free, and every
    // wavefront's sums of the super-block before are visible.
    auto tile_ready = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    float4_t acc[TA][TB], P[2][TA][TB];
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int bq = 0; bq < TB; bq++) acc[a][bq] = zero, P[1][a][bq] = zero;
    Fin fin[2][TA];
#pragma unroll
    for (int a = 0; a < TA; a++) fin[1][a] = Fin{0.f, 0.f, 0u};
    // activation fragment bq of this wavefront is rows 16 ((bq + wave) % 4) .. + 15 of the tile, so that its
    // fragment 0, the one it sums, is fragment `wave`
    const uint32_t xlane = (uint32_t)(QR_ROWB * fr + 128 * fg);
    uint2_t *sx_mine = Sx + (16 * wave + fr) * 4 + fg;
    sx_mine[QR_BN * 4] = uint2_t{0u, 0u}; // parity 1 is read (against zero mins) under super-block 0
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};

    // The min term of the super-block before (parity Q) and its fold into the accumulators.
    auto read_sums = [&](int Q, uint2_t (&hl)[TB]) {
#pragma unroll
        for (int bq = 0; bq < TB; bq++) hl[bq] = Sx[Q * QR_BN * 4 + (16 * ((bq + wave) & 3) + fr) * 4 + fg];
    };
    auto finish = [&](auto Qc, const uint2_t (&hl)[TB]) {
        constexpr int Q = decltype(Qc)::value;
#pragma unroll
        for (int bq = 0; bq < TB; bq++) {
            const half8_t sf = __builtin_bit_cast(half8_t, uint4_t{hl[bq][0], hl[bq][1], 0u, 0u});
#pragma unroll
            for (int a = 0; a < TA; a++) {
                const half8_t mf = __builtin_bit_cast(half8_t, uint4_t{fin[Q][a].mn, fin[Q][a].mn, 0u, 0u});
                const float4_t T = __builtin_amdgcn_mfma_f32_16x16x32_f16(sf, mf, zero, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; r++) acc[a][bq][r] = fmaf(-fin[Q][a].dmin, T[r], fmaf(fin[Q][a].d, P[Q][a][bq][r], acc[a][bq][r]));
            }
        }
    };

    // One super-block of parity Pc: `cur` holds its raw blocks (loaded a super-block ago), `nxt` is the register
    // set that the super-block before has left.
    int xcur = 0;
    auto step = [&](auto Pc, int64_t sb, const Raw (&cur)[TA], Raw (&nxt)[TA]) {
        constexpr int PP = decltype(Pc)::value;
        tile_ready();
        load_raw(min(sb + 1, last), nxt);
        uint2_t hl[TB];
        read_sums(PP ^ 1, hl);
        __builtin_amdgcn_sched_barrier(0); // the loads stay here, a super-block ahead of their decoding
        Scl sc[TA];
#pragma unroll
        for (int a = 0; a < TA; a++) header(cur[a], sc[a], fin[PP][a]);
        finish(std::integral_constant<int, PP ^ 1>{}, hl);
        uint32_t xb[TB];
#pragma unroll
        for (int bq = 0; bq < TB; bq++) xb[bq] = xlane + (uint32_t)(xcur * QR_XSB + 16 * QR_ROWB * ((bq + wave) & 3));
        float S0 = 0.f, S1 = 0.f;
        auto xread = [&](int T, half8_t (&xf)[TB]) {
#pragma unroll
            for (int bq = 0; bq < TB; bq++) xf[bq] = __builtin_bit_cast(half8_t, *(const uint4_t *)(Xs + xb[bq] + 16 * T));
        };
        half8_t xf[2][TB];
        xread(0, xf[0]);
        // The order inside a super-block is the compiler's.  Pinned orders were measured: fragment reads a step ahead
        // of their MFMAs, one read in front of every second MFMA, one right behind every MFMA (where a bare loop of
        // MFMAs, packed FMAs and fragment reads issues them for 2 ns instead of 10: bench.py --issue-calibration);
        // with two weight tiles per wavefront all were the same or up to 4 % slower, with one tile the last was
        // 6 % faster.
        auto mfma_step = [&](auto Tc) {
            constexpr int T = decltype(Tc)::value;
            if constexpr (T < 7) xread(T + 1, xf[(T + 1) & 1]);
            half8_t wf[TA];
#pragma unroll
            for (int a = 0; a < TA; a++) wf[a] = wfrag(Tc, cur[a], sc[a]);
#pragma unroll
            for (int a = 0; a < TA; a++)
#pragma unroll
                for (int bq = 0; bq < TB; bq++) // a super-block's first MFMA starts from zero: no clearing of P between super-blocks
                    P[PP][a][bq] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[T & 1][bq], wf[a], T == 0 ? zero : P[PP][a][bq], 0, 0, 0);
            const half8_t xs0 = xf[T & 1][0];
            float &S = T < 4 ? S0 : S1;
#pragma unroll
            for (int c = 0; c < 4; c++) S = __builtin_amdgcn_fdot2(half2_t{xs0[2 * c], xs0[2 * c + 1]}, ones, S, false);
        };
        mfma_step(std::integral_constant<int, 0>{});
        mfma_step(std::integral_constant<int, 1>{});
        mfma_step(std::integral_constant<int, 2>{});
        mfma_step(std::integral_constant<int, 3>{});
        mfma_step(std::integral_constant<int, 4>{});
        mfma_step(std::integral_constant<int, 5>{});
        mfma_step(std::integral_constant<int, 6>{});
        mfma_step(std::integral_constant<int, 7>{});
        // high part: the sum truncated to f16 (any f16 near it will do); low part: the exact remainder, rounded
        const half2_t h = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(S0, S1));
        const half2_t l = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(S0 - (float)h[0], S1 - (float)h[1]));
        sx_mine[PP * QR_BN * 4] = uint2_t{__builtin_bit_cast(uint32_t, h), __builtin_bit_cast(uint32_t, l)};
        xcur = xcur == QR_XST - 1 ? 0 : xcur + 1;
    };

    Raw r0[TA], r1[TA];
    load_raw(0, r0);
    // two super-blocks per trip, one straight run of instructions (a branch inside it makes the compiler wait
    // for every load in flight)
    int64_t sb = 0;
    for (; sb + 1 < g.nsb; sb += 2) {
        step(std::integral_constant<int, 0>{}, sb, r0, r1);
        step(std::integral_constant<int, 1>{}, sb + 1, r1, r0);
    }
    uint2_t hl[TB];
    if (sb < g.nsb) {
        step(std::integral_constant<int, 0>{}, sb, r0, r1);
        tile_ready();
        read_sums(0, hl);
        finish(std::integral_constant<int, 0>{}, hl);
    } else {
        tile_ready();
        read_sums(1, hl);
        finish(std::integral_constant<int, 1>{}, hl);
    }

    // acc[a][bq][r]: weight row i0 + 32 wave + 16 a + fr, activation row j0 + 16 ((bq + wave) % 4) + 4 fg + r
    half_t *out = g.out + s * g.o_bs;
    if (vec_out) {
        // Output contiguous along the weight rows: the tile goes through LDS (the activation stages are free: every
        // wavefront's last fragment read and the last LDS-DMA lie before the barrier above) and leaves as 16-byte
        // stores, 256 bytes per activation row.
        constexpr int OLD = BM + 8; // halfs per staged row: rows 272 bytes apart spread the lane groups over the banks
        half_t *Os = (half_t *)smem;
        static_assert((size_t)QR_BN * OLD * 2 <= (size_t)QR_XST * QR_XSB, "the staged output tile fits the activation stages");
        rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
            for (int a = 0; a < TA; a++) {
                const int il = wave * (16 * TA) + 16 * a + fr;
                const float bi = (g.has_bias && g.bias_on_rows) ? (float)g.bias[i0 + il] : 0.f;
#pragma unroll
                for (int bq = 0; bq < TB; bq++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int jl = 16 * ((bq + wave) & 3) + 4 * fg + r;
                        float v = acc[a][bq][r] + bi;
                        if (g.has_bias && !g.bias_on_rows) v += (float)g.bias[min(j0 + jl, g.N - 1)];
                        Os[jl * OLD + il] = (half_t)rt_act_k<decltype(has_act)::value>(v);
                    }
            }
        });
        tile_ready();
#pragma unroll
        for (int k = 0; k < 2 * TA; k++) {
            constexpr int CPR = BM / 8; // 16-byte pieces per row
            const int idx = t + 64 * MW * k, row = idx / CPR, c = idx % CPR;
            if (j0 + row < g.N) *(uint4_t *)(out + (j0 + row) * g.o_js + i0 + 8 * c) = *(const uint4_t *)(Os + row * OLD + 8 * c);
        }
        return;
    }
    rt_with_act(g.act, [&](auto has_act) {
#pragma unroll
        for (int a = 0; a < TA; a++) {
            const int64_t i = i0 + wave * (16 * TA) + 16 * a + fr;
            if (i >= g.M) continue;
#pragma unroll
            for (int bq = 0; bq < TB; bq++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int64_t j = j0 + 16 * ((bq + wave) & 3) + 4 * fg + r;
                    if (j >= g.N) continue;
                    float v = acc[a][bq][r];
                    if (g.has_bias) v += (float)g.bias[g.bias_on_rows ? i : j];
                    v = rt_act_k<decltype(has_act)::value>(v);
                    out[i * g.o_is + j * g.o_js] = (half_t)v;
                }
        }
    });
}

RT_TUNABLE(g_gemm_q4k_cfg, 0); // 14 / 24: always one / two weight tiles per wavefront (for comparisons)
RT_TUNABLE(g_gemm_q4k_disable, 0); // non-zero keeps Q4_K prefill on the generic kernel (for comparisons)

// Q4_K weights x K-contiguous f16 activations, more rows than one streaming launch takes.
// hipErrorNotSupported: another kernel must take the problem.
hipError_t launch_gemm_q4k(const Problem &p, const void *A, const void *B, const void *bias, void *out, hipStream_t stream,
                           const DeviceInfo &dev) {
    if (g_gemm_q4k_disable || p.a_dt != RT_Q4_K || p.act_dt != RT_F16) return hipErrorNotSupported;
    if (p.K % 256 != 0 || p.K < 256 || p.b_ks != 1 || p.M < 64 || p.N < 17 || p.stacks > 65535) return hipErrorNotSupported;
    if (((uintptr_t)A & 15u) || ((uintptr_t)B & 15u) || (p.b_js * 2) % 16 || (p.b_bs * 2) % 16) return hipErrorNotSupported;
    // 32-bit offsets within a stack
    if (p.M * (p.K / 256) * 144 >= (int64_t(1) << 32) || p.N * p.b_js >= (int64_t(1) << 31)) return hipErrorNotSupported;
    GemmQ4kArgs g{};
    g.blocks = (const uint8_t *)A, g.X = (const half_t *)B, g.bias = (const half_t *)bias, g.out = (half_t *)out;
    g.M = p.M, g.N = p.N, g.nsb = p.K / 256;
    g.a_stack = p.a_stack, g.b_stack = p.b_stack;
    g.b_bs = p.b_bs, g.b_js = p.b_js;
    g.o_bs = p.o_bs, g.o_is = p.o_is, g.o_js = p.o_js;
    g.has_bias = p.has_bias, g.bias_on_rows = p.bias_on_rows, g.act = p.act;
    const int64_t tiles_j = (p.N + QR_BN - 1) / QR_BN;
    g.tiles_j = (int)tiles_j;
    g.vec_out = p.o_is == 1 && p.o_js % 8 == 0 && p.o_bs % 8 == 0 && ((uintptr_t)out & 15u) == 0;
    auto go = [&](auto kernel, int bm) -> hipError_t {
        const int64_t tiles_i = (p.M + bm - 1) / bm;
        if (tiles_i * tiles_j > 0x7fffffff) return hipErrorNotSupported;
        g.remap = (tiles_i * tiles_j) % 8 == 0;
        if (const hipError_t e = ensure_lds_limit<decltype(kernel)::value>(); e != hipSuccess) return e;
        hipLaunchKernelGGL(decltype(kernel)::value, dim3((unsigned)(tiles_i * tiles_j), (unsigned)p.stacks), dim3(64 * (4 + QR_LW)), QR_LDS, stream, g);
        return hipGetLastError();
    };
    // Four multiplying wavefronts of 32 weight rows x 64 activation rows each; when the grid of 16-row wavefronts
    // (64 weight rows per workgroup) still fits the compute units in one round, those: half the work per wavefront
    // (8192 x 3072 at 64 / 128 rows: 15.7 / 16.8 us against 22.6 / 23.6; 3072 x 8192 at 256 rows: 35 against 52 us).
    const int64_t wgs_small = ((p.M + 63) / 64) * tiles_j;
    const bool small = g_gemm_q4k_cfg == 14 || (g_gemm_q4k_cfg == 0 && wgs_small <= dev.num_cus);
    if (small) return go(std::integral_constant<void (*)(GemmQ4kArgs), &gemm_q4k_kernel<1, 4>>{}, 64);
    return go(std::integral_constant<void (*)(GemmQ4kArgs), &gemm_q4k_kernel<2, 4>>{}, 128);
}

} // namespace rt
