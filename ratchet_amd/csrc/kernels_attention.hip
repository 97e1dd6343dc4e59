// Fused attention:  O = softmax(scale * Q K^T + mask) V  for f16 tensors [batch, heads, len, head_dim].
//
// The reference runs this as separate operators (phi3/attn.rs:142-158, phi2/attn.rs:138-152,
// whisper/mha.rs:105-124): matmul(Q, K^T), mul(scale), add(mask), softmax, matmul(P, V), with
// the [len x len] scores written to and read from memory four times.  Both products are bound
// by that traffic, so here the scores never leave the compute unit: a workgroup owns 64 query
// rows of one head, streams the keys and values past them in blocks of 64, and keeps a running
// maximum, a running sum and the unnormalised output per row (the online form of the same
// max-subtracted softmax, ops/softmax.rs:120-183).  Each of Q, K, V is read once per query
// block and O written once.
//
// Layout of one step.  Eight wavefronts: wavefront (qt, kh) owns 16 query rows and 32 of the
// block's 64 keys; its Q fragments stay in registers.
//   S = Q K^T:   v_mfma_f32_16x16x32_f16 with the key block (LDS, [key][d]) as first operand and
//                Q as second, so that lane l holds, for query row l % 16, the scores of keys
//                16 b + 4 (l / 16) + r of key tile b (r = result register).
//   softmax:     a row's 32 scores sit in four lanes (8 registers each): the maximum needs two
//                cross-lane steps per block, the sum is kept per lane and reduced once at the end.
//   O += P V:    the lane's eight probabilities are, as they lie, the K-slots 8 (l / 16) .. + 7 of
//                one MFMA over the wavefront's 32 keys in a permuted order.  The V operand needs,
//                per lane, four consecutive keys of one column: ds_read_b64_tr_b16 delivers exactly
//                that from the value block as it lies in memory ([key][d]): within 16 lanes, lane
//                s addresses the four columns 4 (s % 4) .. + 3 of row s / 4 and lane i receives
//                column i of the four rows.  Two such reads per MFMA, no transposed copy of V.
//   The two key halves of a row keep separate running maxima, sums and outputs and are merged
//   once, after the last block.
// Key and value blocks go from global memory straight into a ring of LDS stages
// (global_load_lds_dwordx4: no registers, nothing for the compiler to wait on), rows packed without
// padding and, where a row is 128 or 256 bytes, with their 16-byte chunks XOR-swizzled by the row so
// that fragment reads spread over the banks.  The kernel counts its own loads: every wavefront
// issues the same number per block, waits with an explicit s_waitcnt vmcnt(n) that leaves the newest
// blocks in flight, and a bare s_barrier publishes the block (a __syncthreads() would drain every
// load, and so does the compiler's own accounting once a loop carries loads across iterations:
// with register-staged blocks every step waited out a full trip to memory).
#include "device_common.h"

namespace rt {

struct AttnArgs {
    const half_t *Q, *K, *V;
    const void *mask;   // additive [q_len][kv_len] (f16 or f32), or null
    half_t *O;
    int heads, q_len, kv_len, D;
    int64_t q_bs, q_hs, q_rs;   // element strides: batch, head, row
    int64_t k_bs, k_hs, k_rs;
    int64_t v_bs, v_hs, v_rs;
    int64_t o_bs, o_hs, o_rs;
    int64_t mask_rs;
    int mask_f32;
    int causal;         // key j is visible to query i iff j <= i + (kv_len - q_len)
    float scale_log2e;  // scale * log2(e): the exponentials are base 2
    int splits;         // workgroups sharing the keys of one query block (blockIdx.z); > 1 needs `partial`
    float *partial;     // [stack][query block][split][64 rows][4 + DP]: running maximum, sum, two unused, unnormalised output
};

constexpr int AT_BQ = 64, AT_BK = 64; // query rows of a workgroup; keys of a block of the eight-wavefront kernel (the unit the split heuristic counts in)
constexpr float kLog2e = 1.4426950408889634f;

// position (in 16-byte chunks) of chunk c of row r inside a packed block of rows of dvec chunks
__device__ __forceinline__ int at_chunk_pos(int r, int c, int dvec) {
    if (dvec == 8) c ^= (r >> 1) & 7;    // 128-byte rows: two rows cover all banks
    else if (dvec == 16) c ^= r & 15;    // 256-byte rows: every row starts on the same bank
    return r * dvec + c;
}

// s_waitcnt vmcnt(n) lgkmcnt(0): at most n of this wavefront's loads outstanding, all LDS reads returned
__device__ __forceinline__ constexpr int at_waitcnt(int n) { return 0x0070 | (n & 0xF) | (((n >> 4) & 0x3) << 14); }

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the four lane groups that share a query row),
// left in all of them: v_permlane16_swap and v_permlane32_swap of a register with itself put the partner
// row's (half's) value beside the lane's own, so each step is two vector instructions and no trip through
// the LDS crossbar (ds_bpermute, which __shfl_xor is, costs an LDS round trip per step).
__device__ __forceinline__ float at_groups_max(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    // the instruction itself: fmaxf() of values that come out of a bit cast first quiets each of them (two more instructions)
    float w;
    asm("v_max_f32 %0, %1, %2" : "=v"(w) : "v"((uint32_t)a[0]), "v"((uint32_t)a[1]));
    const uint32_t x = __builtin_bit_cast(uint32_t, w);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return fmaxf(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}
__device__ __forceinline__ float at_groups_sum(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float w = __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
    const uint32_t x = __builtin_bit_cast(uint32_t, w);
    const auto b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __builtin_bit_cast(float, (uint32_t)b[0]) + __builtin_bit_cast(float, (uint32_t)b[1]);
}

// stages of the key / value ring: blocks of 32 nkq keys, at most 160 KB
constexpr int at_stages(int dp, int nkq) { return nkq == 4 ? 3 : (dp <= 96 ? 4 : 3); }

// four transposing reads at two addresses with immediate offsets; nothing waits here
template <int O0, int O1, int O2, int O3>
__device__ __forceinline__ void at_tr_read4(uint64_t &v0, uint64_t &v1, uint64_t &v2, uint64_t &v3, uint32_t a0, uint32_t a1) {
    asm volatile("ds_read_b64_tr_b16 %0, %4 offset:%6\n\tds_read_b64_tr_b16 %1, %4 offset:%7\n\t"
                 "ds_read_b64_tr_b16 %2, %5 offset:%8\n\tds_read_b64_tr_b16 %3, %5 offset:%9"
                 : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
                 : "v"(a0), "v"(a1), "n"(O0), "n"(O1), "n"(O2), "n"(O3)
                 : "memory");
}

template <int O0, int O1> __device__ __forceinline__ void at_tr_read2(uint64_t &v0, uint64_t &v1, uint32_t a0) {
    asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4" : "=&v"(v0), "=&v"(v1) : "v"(a0), "n"(O0), "n"(O1) : "memory");
}

// DP: head_dim padded to a multiple of 32.  MK: 0 no mask tensor; 1 an additive mask tensor, read from memory where it is
// used; 2 the same, its [64 queries x 64 keys] block travelling through the ring with the keys and values (see below).  DC: head_dim itself when the
// kernel is built for one (64, 80, 96, 128), else 0 and head_dim is the argument's: with a constant row length the
// fragment addresses inside a stage differ by constants, which the LDS instructions carry as immediate offsets, so
// a block costs three address additions instead of eighteen.
// 4 NKQ wavefronts: wavefront (qt, kh) owns query tile qt (16 rows) and part kh (32 keys) of every block of
// 32 NKQ keys, with its own running maximum, sum and output; the NKQ parts of a row are merged through LDS at the
// end.  NKQ = 2: eight wavefronts, blocks of 64 keys.  NKQ = 4: sixteen wavefronts, blocks of 128 keys; a wavefront
// issues an instruction every four cycles at best and a step is some 130 of them whatever their kind, so with two
// wavefronts per SIMD the vector unit is busy a third of the time: four per SIMD, each taking a quarter of a
// block twice as long, do the same work in the same number of instructions per wavefront and half as many steps.
// It needs the registers of a wavefront to stay within 128 and three stages of 128 keys within the LDS
// (head_dim up to 96).
// The mask tensor.  Read where it is used (eight loads per lane in the middle of a step, which the compiler has to
// await with every load into LDS still in flight: the ring drains on every step, 25.7 us at 32 x 512 x 512 x 80 where
// the causal flag takes 10.0) it is the slow path, yet a tensor is what the reference's callers pass
// (phi3/attn.rs:148-151).  With rows of whole 16-byte vectors (MK == 2) the block's 64 x 64 mask values are two more
// LDS-DMA instructions per wavefront and block, counted with the others, stored behind the values in the stage with
// the row's 16-byte chunks XOR-swizzled like the keys', and read back as two vectors per lane.
template <int DP, int MK, int DC, int NKQ>
__global__ __launch_bounds__(256 * NKQ) void attention_kernel(AttnArgs g) {
    constexpr bool MASK = MK != 0, MST = MK == 2;
    static_assert(NKQ == 2 || (NKQ == 4 && DP <= 96 && !MST), "eight wavefronts, or sixteen for head_dim up to 96 (not with a staged mask)");
    constexpr int BK = 32 * NKQ, WAVES = 4 * NKQ; // keys of a block; wavefronts
    static_assert(DC == 0 || (DC % 8 == 0 && DC <= DP && DC > DP - 32), "a fixed head_dim belongs to its padded size");
    constexpr int KK = DP / 32;             // MFMA steps over head_dim
    constexpr int DT = DP / 16;             // 16-column tiles of the output
    // load instructions per wavefront per block: a block is 2 ipo instructions (64 chunks each, ipo = dvec NKQ / 2
    // for the keys, then as many for the values); instruction j belongs to wavefront j % WAVES, surplus ones
    // repeat the last
    constexpr int NI = ((DP / 8) * NKQ + WAVES - 1) / WAVES;
    constexpr int NIM = MST ? 2 : 0;        // the mask block's instructions per wavefront (16 of 1 KB for f32, 8 for f16: the rest repeat the last)
    constexpr int STAGES = MST ? 3 : at_stages(DP, NKQ);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int qt = wave & 3, kh = wave >> 2;
    const int fr = lane & 15, fg = lane >> 4;
    // Which (query block, head, split) this workgroup takes.  Workgroups go to the eight XCDs round-robin by their
    // linear number; taken as it comes, the query blocks of one head would land on eight XCDs and every one of the
    // eight L2s would fetch that head's keys and values.  When the grid divides by eight, XCD x instead takes the
    // x-th eighth of the work items in (split, head, query block) order: all query blocks of a head share an L2.
    uint32_t qbi = blockIdx.x, bhi = blockIdx.y, spi = blockIdx.z;
    {
        const uint64_t total64 = (uint64_t)gridDim.x * gridDim.y * gridDim.z;
        if (total64 < (1u << 31) && (total64 & 7u) == 0) {
            const uint32_t total = (uint32_t)total64;
            const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
            const uint32_t w = (lin & 7u) * (total >> 3) + (lin >> 3);
            const uint32_t wy = w / gridDim.x;
            qbi = w - wy * gridDim.x, spi = wy / gridDim.y, bhi = wy - spi * gridDim.y;
        }
    }
    const int q0 = (int)qbi * AT_BQ;
    const int bh = (int)bhi, b = bh / g.heads, h = bh - b * g.heads;
    const half_t *Q = g.Q + b * g.q_bs + h * g.q_hs;
    const half_t *K = g.K + b * g.k_bs + h * g.k_hs;
    const half_t *V = g.V + b * g.v_bs + h * g.v_hs;
    half_t *O = g.O + b * g.o_bs + h * g.o_hs;
    const int D = DC ? DC : g.D;
    const int dvec = D >> 3;                // 16-byte chunks per row (head_dim % 8 == 0)
    const int off = g.kv_len - g.q_len;     // causal: query i sees keys <= i + off
    const uint4_t zero4 = {0u, 0u, 0u, 0u};
    const int blk_halfs = BK * D;           // one packed block of keys (or values)
    const int mesz = g.mask_f32 ? 4 : 2, mcpr = BK * mesz / 16;            // mask: bytes per value, 16-byte chunks per row of a block
    const int stage_halfs = 2 * blk_halfs + (MST ? AT_BQ * BK * mesz / 2 : 0); // keys, values (, mask)
    const int ipo = dvec * NKQ / 2;         // load instructions per operand and block
    half_t *ring = (half_t *)smem;          // [STAGES][keys | values][64 rows][D]

    // this wavefront's Q fragments: row q0 + 16 qt + fr, head_dim 32 kk + 8 fg .. + 7 (zero past head_dim)
    const int qrow = q0 + 16 * qt + fr;
    half8_t fq[KK];
    {
        const half_t *qp = Q + (int64_t)min(qrow, g.q_len - 1) * g.q_rs;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const int d = 32 * kk + 8 * fg;
            fq[kk] = d < D ? __builtin_bit_cast(half8_t, *(const uint4_t *)(qp + d)) : __builtin_bit_cast(half8_t, zero4);
        }
    }

    // This wavefront's load instructions.  Instruction j of a block fills LDS chunks 64 j' .. 64 j' + 63
    // of the keys (j' = j < dvec) or the values (j' = j - dvec); lane l supplies chunk 64 j' + l, i.e.
    // (row, position) = divmod(64 j' + l, dvec), and fetches the source chunk that the swizzle puts there.
    int lrow[NI];          // row inside the block
    uint32_t lcol[NI];     // source column (halfs) inside the row
    bool lval[NI];         // values (true) or keys
    int ldst[NI];          // LDS offset (halfs) of the instruction's 64 chunks inside a stage
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const int j = min(wave + WAVES * i, 2 * ipo - 1);      // surplus instructions repeat the block's last one
        lval[i] = j >= ipo;
        const int jj = lval[i] ? j - ipo : j;
        const int q = 64 * jj + lane;
        lrow[i] = q / dvec;
        const int pos = q - lrow[i] * dvec;                        // position inside the row ...
        const int src = at_chunk_pos(lrow[i], pos, dvec) - lrow[i] * dvec; // ... holds this source chunk (the XOR is its own inverse)
        lcol[i] = 8u * (uint32_t)src;
        ldst[i] = (lval[i] ? blk_halfs : 0) + 512 * jj;
    }
    // block `src_kb` into the stage of ring position `pos_kb` (they differ only past the end).  A block that lies
    // wholly inside the keys is addressed as the lane's pointer into block 0 plus the block's byte offset, one
    // scalar multiplication (the launcher keeps a head's keys and values within 2^32 bytes) and one vector addition.
    const uint8_t *lptr[NI]; // the lane's chunk in block 0
    uint32_t lstep[NI];      // bytes from a block to the next (uniform)
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const uint32_t rs = (uint32_t)(lval[i] ? g.v_rs : g.k_rs);
        lptr[i] = (const uint8_t *)(lval[i] ? V : K) + (size_t)(((uint32_t)lrow[i] * rs + lcol[i]) * 2u);
        lstep[i] = (uint32_t)BK * rs * 2u;
    }
    const uint8_t *mptr[MST ? NIM : 1]; // the lane's mask row
    uint32_t mcol[MST ? NIM : 1];       // byte offset of its source chunk inside a block's columns
    int mdst[MST ? NIM : 1];            // LDS offset (halfs) of the instruction's 64 chunks inside the mask block
    if constexpr (MST) {
#pragma unroll
        for (int i = 0; i < NIM; i++) {
            const int m = min(wave + WAVES * i, mcpr - 1);
            const int c = 64 * m + lane, row = c / mcpr, pos = c - row * mcpr;
            const int src = at_chunk_pos(row, pos, mcpr) - row * mcpr;
            mptr[i] = (const uint8_t *)g.mask + (int64_t)min(q0 + row, g.q_len - 1) * g.mask_rs * mesz;
            mcol[i] = 16u * (uint32_t)src;
            mdst[i] = 512 * m;
        }
    }
    auto issue_loads_at = [&](int pos_kb, int src_kb) {
        half_t *st = ring + (pos_kb % STAGES) * stage_halfs;
        const int k0 = src_kb * BK;
        if constexpr (MST) {
            // lane l of instruction m fills chunk 64 m + l of the mask block: row (64 m + l) / mcpr, and the source chunk the
            // swizzle puts at that position; past the row's end (a last, partial block) the row's last chunk again
#pragma unroll
            for (int i = 0; i < NIM; i++) {
                const uint32_t mo = min((uint32_t)(k0 * mesz) + mcol[i], (uint32_t)(g.mask_rs * mesz) - 16u);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(mptr[i] + mo),
                                                 (__attribute__((address_space(3))) void *)(st + 2 * blk_halfs + mdst[i]), 16, 0, 0);
            }
        }
        if (k0 + BK <= g.kv_len) { // uniform
#pragma unroll
            for (int i = 0; i < NI; i++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(lptr[i] + (size_t)((uint32_t)src_kb * lstep[i])),
                                                 (__attribute__((address_space(3))) void *)(st + ldst[i]), 16, 0, 0);
            return;
        }
#pragma unroll
        for (int i = 0; i < NI; i++) {
            // rows past the last key re-read the last key: finite data, and their scores are masked
            const uint32_t key = (uint32_t)min(k0 + lrow[i], g.kv_len - 1);
            const half_t *src = lval[i] ? V + (key * (uint32_t)g.v_rs + lcol[i]) : K + (key * (uint32_t)g.k_rs + lcol[i]);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)(st + ldst[i]), 16, 0, 0);
        }
    };
    // all but the newest `keep` blocks' loads of this wavefront have landed, all LDS reads have returned;
    // then everybody's have
    auto publish = [&](auto keep) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(at_waitcnt(decltype(keep)::value * (NI + NIM)));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    float4_t acc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++) acc[d] = float4_t{0.f, 0.f, 0.f, 0.f};
    // of query row fr over this wavefront's keys, in base-2 units; l is this lane's share of the sum
    float m_run = -INFINITY, l_run = 0.f;

    // causal: key blocks wholly above the diagonal of this query block are never visited
    int k_end = g.kv_len;
    if (g.causal) k_end = max(0, min(g.kv_len, q0 + AT_BQ + off));
    const int nkb_all = (k_end + BK - 1) / BK;
    // this workgroup's share of the key blocks: [kb_lo, kb_hi), an even split over gridDim.z
    const int split = (int)spi;
    int kb_lo = 0, kb_hi = nkb_all;
    if (g.splits > 1) kb_lo = (int)((uint32_t)(nkb_all * split) / (uint32_t)g.splits), kb_hi = (int)((uint32_t)(nkb_all * (split + 1)) / (uint32_t)g.splits);
    const int nkb = kb_hi - kb_lo;
    const int last = max(kb_hi - 1, 0);
    // prologue: the first STAGES - 1 blocks requested (an index past the end repeats the last block, so
    // that every step issues and awaits the same number of loads), the first one landed
    if (nkb > 0) {
#pragma unroll
        for (int sidx = 0; sidx < STAGES - 1; sidx++) issue_loads_at(sidx, min(kb_lo + sidx, last));
    }
    const half_t *mrow = nullptr;
    if constexpr (MASK && !MST) mrow = (const half_t *)g.mask; // indexed below by its own element type
    if (nkb > 0) publish(std::integral_constant<int, STAGES - 2>{});
    // fragment addressing inside a stage (halfs).  Sixteen rows further down the swizzle repeats, so the second key
    // tile and the second half of the value rows are 16 dvec chunks away from the first.
    const int tile_halfs = 128 * dvec;
    int koff[KK];          // key fragments: row 32 kh + fr (+ 16), chunk 4 kk + fg (clamped into the row: Q is zero there)
#pragma unroll
    for (int kk = 0; kk < KK; kk++) koff[kk] = 8 * at_chunk_pos(32 * kh + fr, min(4 * kk + fg, dvec - 1), dvec);
    int voff[DT];          // value fragments: rows 32 kh + 4 fg + fr / 4 (+ 16), halfs 16 d + 4 (fr % 4) .. + 3
#pragma unroll
    for (int d = 0; d < DT; d++) {
        const int r = 32 * kh + 4 * fg + (fr >> 2);
        const int c = min(2 * d + ((fr & 3) >> 1), dvec - 1);
        voff[d] = blk_halfs + 8 * at_chunk_pos(r, c, dvec) + 4 * (fr & 1);
    }
    // with a fixed unswizzled row length the value fragments of all tiles inside head_dim are 32 bytes apart
    constexpr bool VIMM = DC != 0 && DC != 64 && DC != 128;
    constexpr int DTL = DC ? (DC + 15) / 16 : DT; // output tiles that hold a column of head_dim
    // One step: ring position `it` holds key block kb_lo + it.  LEAN: the block crosses neither the end of the keys nor
    // the causal diagonal of this wavefront's rows, there is no mask tensor and the scale is positive, so the step
    // carries none of the tests for those (a wavefront issues an instruction every four cycles at best, whatever its
    // kind: the scalar bookkeeping of a step costs as much time as its vector arithmetic).
    auto step = [&](int it, auto lean_c) {
        constexpr bool LEAN = decltype(lean_c)::value;
        const int kb = kb_lo + it;
        const int k0 = kb * BK;
        // the stage the previous step used is free (everybody passed the barrier that ended it)
        issue_loads_at(it + STAGES - 1, min(kb + STAGES - 1, last));
        const half_t *st = ring + (it % STAGES) * stage_halfs;

        // S = Q K^T for this wavefront's 16 rows and its 32 keys of the block (key tiles 2 kh, 2 kh + 1): all key
        // fragments are requested before the first MFMA (one trip to LDS, not one per fragment), and the two
        // tiles' chains of dependent MFMAs alternate
        half8_t fk[2][KK];
#pragma unroll
        for (int b2 = 0; b2 < 2; b2++)
#pragma unroll
            for (int kk = 0; kk < KK; kk++) fk[b2][kk] = __builtin_bit_cast(half8_t, *(const uint4_t *)(st + koff[kk] + b2 * tile_halfs));
        __builtin_amdgcn_sched_barrier(0);
        float4_t S[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int kk = 0; kk < KK; kk++)
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++) S[b2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fk[b2][kk], fq[kk], S[b2], 0, 0, 0);
        // this lane's mask values: row 16 qt + fr, keys 32 kh + 16 b2 + 4 fg .. + 3 of the block, one vector per key tile
        float mvals[2][4];
        if constexpr (MST) {
            const uint8_t *mb = (const uint8_t *)(st + 2 * blk_halfs);
            const int row = 16 * qt + fr;
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++) {
                if (g.mask_f32) { // uniform
                    const float4_t mv = *(const float4_t *)(mb + 16 * at_chunk_pos(row, 8 * kh + 4 * b2 + fg, 16));
#pragma unroll
                    for (int r = 0; r < 4; r++) mvals[b2][r] = mv[r];
                } else {
                    const uint64_t raw = *(const uint64_t *)(mb + 16 * at_chunk_pos(row, 4 * kh + 2 * b2 + (fg >> 1), 8) + 8 * (fg & 1));
                    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
                    const half4_t mh = __builtin_bit_cast(half4_t, raw);
#pragma unroll
                    for (int r = 0; r < 4; r++) mvals[b2][r] = (float)mh[r];
                }
            }
        }
        // The value fragments of O += P V do not depend on the scores: they are requested here and awaited after
        // the softmax arithmetic, which hides their trip.  The transposing reads are issued from assembly: as a
        // builtin the compiler orders them after every outstanding load into LDS (vmcnt(0)), which would drain
        // the ring on every step.  Every tile is read and multiplied, also one wholly past head_dim (the clamped
        // addresses stay inside the block, its columns are never stored).
        const uint32_t st_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const half_t *)st;
        uint64_t fv[DT][2];
        if constexpr (DC != 0) {
            // a pair of tiles: two address registers (the same one twice, VIMM) and immediate offsets
            constexpr int TB2 = 2 * 128 * (DC / 8); // bytes between the two halves of the value rows
            constexpr int VS = VIMM ? 32 : 0;       // bytes from a tile to the next
#define RT_AT_PAIR(d0)                                                                                                         \
    if constexpr (DTL > d0 + 1) {                                                                                              \
        at_tr_read4<VS * d0, VS * d0 + TB2, VS * (d0 + 1), VS * (d0 + 1) + TB2>(fv[d0][0], fv[d0][1], fv[d0 + 1][0], fv[d0 + 1][1], \
                                                                                st_addr + 2 * voff[VIMM ? 0 : d0], st_addr + 2 * voff[VIMM ? 0 : d0 + 1]); \
    } else if constexpr (DTL > d0) {                                                                                           \
        at_tr_read2<VS * d0, VS * d0 + TB2>(fv[d0][0], fv[d0][1], st_addr + 2 * voff[VIMM ? 0 : d0]);                          \
    }
            RT_AT_PAIR(0)
            RT_AT_PAIR(2)
            RT_AT_PAIR(4)
            RT_AT_PAIR(6)
#undef RT_AT_PAIR
        } else {
#pragma unroll
            for (int d0 = 0; d0 < DT; d0 += 2)
                asm volatile("ds_read_b64_tr_b16 %0, %4\n\tds_read_b64_tr_b16 %1, %5\n\t"
                             "ds_read_b64_tr_b16 %2, %6\n\tds_read_b64_tr_b16 %3, %7"
                             : "=&v"(fv[d0][0]), "=&v"(fv[d0][1]), "=&v"(fv[d0 + 1][0]), "=&v"(fv[d0 + 1][1])
                             : "v"(st_addr + 2 * voff[d0]), "v"(st_addr + 2 * (voff[d0] + tile_halfs)),
                               "v"(st_addr + 2 * voff[d0 + 1]), "v"(st_addr + 2 * (voff[d0 + 1] + tile_halfs))
                             : "memory");
        }
        // scale, mask, bounds; then the row maximum over the wavefront's keys.  Only a block that
        // crosses the end of the keys or the causal diagonal of this wavefront's rows needs the
        // per-element tests (uniform).
        const int kw0 = k0 + 32 * kh; // first of this wavefront's keys
        const bool edge = !LEAN && (kw0 + 32 > g.kv_len || (g.causal && kw0 + 31 > q0 + 16 * qt + off));
        // Fast path (scale > 0, no mask, no edge): the maximum is taken on the raw scores and the scale
        // is folded into the exponent's argument, exp2(S * c - m).
        const bool raw = LEAN || (!MASK && !edge && g.scale_log2e > 0.f); // uniform
        float bmax = -INFINITY;
        if (raw) {
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++)
#pragma unroll
                for (int r = 0; r < 4; r++) bmax = fmaxf(bmax, S[b2][r]);
            bmax *= g.scale_log2e;
        } else {
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int key = kw0 + 16 * b2 + 4 * fg + r;
                    float s = S[b2][r] * g.scale_log2e;
                    if constexpr (MST) {
                        s += mvals[b2][r] * kLog2e;
                    } else if constexpr (MASK) {
                        const int64_t mi = (int64_t)min(qrow, g.q_len - 1) * g.mask_rs + min(key, g.kv_len - 1);
                        const float mv = g.mask_f32 ? ((const float *)mrow)[mi] : (float)mrow[mi];
                        s += mv * kLog2e;
                    }
                    if (key >= g.kv_len || (g.causal && key > qrow + off)) s = -INFINITY;
                    S[b2][r] = s;
                    bmax = fmaxf(bmax, s);
                }
        }
        bmax = at_groups_max(bmax);
        const float m_new = fmaxf(m_run, bmax);
        // a row that has seen no finite score yet keeps a reference of 0: exp2(-inf - 0) = 0
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use); // m_run = -inf -> 0
        m_run = m_new;
        const float sc = raw ? g.scale_log2e : 1.f;
        float psum = 0.f;
        half8_t fp;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float p = __builtin_amdgcn_exp2f(fmaf(S[e >> 2][e & 3], sc, -m_use));
            psum += p;
            fp[e] = (half_t)p;
        }
        l_run = l_run * alpha + psum;
        // the running maximum rarely moves after the first blocks: rescale only if some row's did
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
            for (int d = 0; d < DT; d++) acc[d] *= alpha;
        }
        // O += P V over this wavefront's 32 keys.  The wait names every fragment register, so nothing that uses
        // one can be placed before it.
        constexpr int DTU = DTL; // tiles read and multiplied
#pragma unroll
        for (int d0 = 0; d0 < DTU; d0 += 2) {
            if (d0 == 0)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fv[d0][0]), "+v"(fv[d0][1]), "+v"(fv[d0 + 1][0]), "+v"(fv[d0 + 1][1])::"memory");
            else if (d0 + 1 < DTU)
                asm volatile("" : "+v"(fv[d0][0]), "+v"(fv[d0][1]), "+v"(fv[d0 + 1][0]), "+v"(fv[d0 + 1][1])::"memory");
            else
                asm volatile("" : "+v"(fv[d0][0]), "+v"(fv[d0][1])::"memory");
        }
        typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int d = 0; d < DTU; d++)
            acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, u64x2_t{fv[d][0], fv[d][1]}), fp, acc[d], 0, 0, 0);
        // block kb + 1 has landed for everybody, and nobody reads block kb's stage any more
        publish(std::integral_constant<int, STAGES - 2>{});
    };
    // the leading blocks of this wavefront's share that are lean: kw0 + 32 <= kv_len, and causal: kw0 + 31 <= first row + off
    int n_lean = 0;
    if (!MASK && g.scale_log2e > 0.f) {
        auto blocks_upto = [](int num) { return num < 0 ? 0 : num / BK + 1; }; // block numbers kb with BK kb <= num
        int n = blocks_upto(g.kv_len - 32 - 32 * kh);
        if (g.causal) n = min(n, blocks_upto(q0 + 16 * qt + off - 31 - 32 * kh));
        n_lean = max(0, min(n - kb_lo, nkb));
    }
    {
        int it = 0;
        for (; it < n_lean; it++) step(it, std::true_type{});
        for (; it < nkb; it++) step(it, std::false_type{});
    }
    // no load may land in LDS once the merge below reuses it
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(at_waitcnt(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // merge the key parts of every row: the kh > 0 wavefronts hand (m, l, O) to their kh = 0 partner through LDS,
    // lane to lane
    constexpr int EXW = (2 + 4 * DT) * 64; // floats one wavefront hands over
    float *exb = (float *)smem + (size_t)qt * EXW + lane; // [kh - 1][qt][2 + 4 DT][64 lanes]
    if (kh > 0) {
        float *ex = exb + (size_t)(kh - 1) * 4 * EXW;
        ex[0] = m_run;
        ex[64] = l_run;
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 4; r++) ex[(2 + 4 * d + r) * 64] = acc[d][r];
    }
    __syncthreads();
    if (kh > 0) return;
    {
        float mp[NKQ - 1], lp[NKQ - 1];
        float m_new = m_run;
#pragma unroll
        for (int p = 0; p < NKQ - 1; p++) {
            mp[p] = exb[(size_t)p * 4 * EXW], lp[p] = exb[(size_t)p * 4 * EXW + 64];
            m_new = fmaxf(m_new, mp[p]);
        }
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float a0 = __builtin_amdgcn_exp2f(m_run - m_use);
        l_run *= a0;
#pragma unroll
        for (int d = 0; d < DT; d++) acc[d] *= a0;
#pragma unroll
        for (int p = 0; p < NKQ - 1; p++) {
            const float ap = __builtin_amdgcn_exp2f(mp[p] - m_use);
            l_run += lp[p] * ap;
#pragma unroll
            for (int d = 0; d < DT; d++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[d][r] += exb[(size_t)p * 4 * EXW + (2 + 4 * d + r) * 64] * ap;
        }
        m_run = m_new; // what the sums and outputs are now relative to (a split launch hands it on)
    }
    // the row's sum over its four lanes, then O / l; lane (fr, fg) holds columns 16 d + 4 fg + r of row fr
    l_run = at_groups_sum(l_run);
    if (g.splits > 1) {
        // this workgroup saw only its share of the keys: hand (m, l, O) of every row to the merge kernel
        // (rows past q_len are never merged: a decode step has one live row of 64)
        float *pr = g.partial + ((((size_t)bhi * gridDim.x + qbi) * g.splits + split) * AT_BQ + 16 * qt + fr) * (4 + DP);
        if (qrow < g.q_len) {
            if (fg == 0) pr[0] = m_run, pr[1] = l_run;
#pragma unroll
            for (int d = 0; d < DT; d++) *(float4_t *)(pr + 4 + 16 * d + 4 * fg) = acc[d];
        }
        return;
    }
    const float inv = 1.f / l_run; // no visible key: 0 / 0 = NaN, what the unfused sequence yields
    if (qrow < g.q_len) {
        half_t *op = O + (int64_t)qrow * g.o_rs;
#pragma unroll
        for (int d = 0; d < DT; d++) {
            const int c = 16 * d + 4 * fg;
            if (c < D) { // head_dim % 8 == 0 and c % 4 == 0: a group of four is inside or outside as a whole
                const half_t o4[4] = {(half_t)(acc[d][0] * inv), (half_t)(acc[d][1] * inv), (half_t)(acc[d][2] * inv),
                                      (half_t)(acc[d][3] * inv)};
                *(uint64_t *)(op + c) = *(const uint64_t *)o4;
            }
        }
    }
}

// Second pass of a split launch: per row, the partial (maximum, sum, output) triples of the splits are
// combined exactly as the two key halves are inside the kernel, then normalised and rounded once.
// One workgroup per (stack, query block); a thread owns four columns of one row and reads every split's
// share of them with all loads issued up front (the loops are unrolled over the most splits there can be).
constexpr int AT_MAX_SPLITS = 16;
template <int DP>
__global__ __launch_bounds__(256) void attention_merge_kernel(AttnArgs g) {
    const int cg = g.D >> 2;                                   // groups of four columns per row
    const int rows = min(AT_BQ, g.q_len - (int)blockIdx.x * AT_BQ);
    const int bh = blockIdx.y, b = bh / g.heads, h = bh - b * g.heads;
    const float *base = g.partial + (((size_t)blockIdx.y * gridDim.x + blockIdx.x) * g.splits) * AT_BQ * (4 + DP);
    const size_t sstride = (size_t)AT_BQ * (4 + DP);
    for (int item = threadIdx.x; item < rows * cg; item += blockDim.x) {
        const int row = item / cg, c = 4 * (item - row * cg);
        const float *pr = base + (size_t)row * (4 + DP);
        float ms[AT_MAX_SPLITS], ls[AT_MAX_SPLITS];
        float4_t vs[AT_MAX_SPLITS];
#pragma unroll
        for (int s = 0; s < AT_MAX_SPLITS; s++) {
            const int sc = min(s, g.splits - 1);               // past the last split: re-read it, weight zero below
            ms[s] = pr[sc * sstride], ls[s] = pr[sc * sstride + 1];
            vs[s] = *(const float4_t *)(pr + sc * sstride + 4 + c);
        }
        float m = -INFINITY;
#pragma unroll
        for (int s = 0; s < AT_MAX_SPLITS; s++) m = fmaxf(m, ms[s]);
        const float m_use = m == -INFINITY ? 0.f : m;
        float l = 0.f;
        float4_t o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < AT_MAX_SPLITS; s++) {
            const float w = s < g.splits ? __builtin_amdgcn_exp2f(ms[s] - m_use) : 0.f;
            l += ls[s] * w;
            o += vs[s] * w;
        }
        const float inv = 1.f / l; // no visible key anywhere: 0 / 0 = NaN, as in the single pass
        half_t *op = g.O + b * g.o_bs + h * g.o_hs + (int64_t)(blockIdx.x * AT_BQ + row) * g.o_rs;
        const half_t o4[4] = {(half_t)(o[0] * inv), (half_t)(o[1] * inv), (half_t)(o[2] * inv), (half_t)(o[3] * inv)};
        *(uint64_t *)(op + c) = *(const uint64_t *)o4;
    }
}


// ---------------------------------------------------------------------------------------------
// Decoding: one query row per head against a long cache.  The tiled kernel above would spend a 64-row
// query block and its matrix instructions on one live row; this one is a stream over the keys and
// values, like the GEMV of a decode step.  A workgroup of four wavefronts takes 128 consecutive keys
// of one head: 16 lanes share a key (lane `seg` holds dimensions 8 seg .. + 7: 16 bytes of the key and
// 16 of the value, lanes past head_dim / 8 idle), so a wavefront's load covers four whole keys, and
// all 8 + 8 loads of a lane are requested before the first is used.  The score is 4 v_dot2_f32_f16
// and four DPP additions inside the 16-lane row; the softmax of the 128 keys is local (maximum and
// sum through LDS), the probabilities stay f32, and the 16 key slots' shares of the output meet in
// LDS.  Every workgroup writes (maximum, sum, unnormalised output) of its keys; a second small
// kernel merges the splits of a head exactly as the tiled kernel's merge does.
// ---------------------------------------------------------------------------------------------
constexpr int AD_THREADS = 256, AD_L = 8, AD_KEYS = 16 * AD_L; // key slots per load x loads = keys per workgroup
constexpr int AD_PSTRIDE = 4 + 128;                            // floats per (head, split) in the workspace

template <int CTRL> __device__ __forceinline__ float ad_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// sum over the 16 lanes of a row, left in all of them
__device__ __forceinline__ float ad_row_sum(float v) {
    v += ad_dpp<0x128>(v); // row_ror:8
    v += ad_dpp<0x124>(v); // row_ror:4
    v += ad_dpp<0x122>(v); // row_ror:2
    v += ad_dpp<0x121>(v); // row_ror:1
    return v;
}

__global__ __launch_bounds__(AD_THREADS) void attention_decode_kernel(AttnArgs g) {
    __shared__ float sm[4], sl[4];
    __shared__ __attribute__((aligned(16))) float so[16][16][8]; // [key slot][seg][8 dimensions]
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int seg = lane & 15, slot = wave * 4 + (lane >> 4);
    const int ns = g.D >> 3;
    const int segc = min(seg, ns - 1); // idle lanes repeat the last live lane's addresses (no extra traffic) and contribute zeros
    const int split = blockIdx.x, bh = blockIdx.y, b = bh / g.heads, h = bh - b * g.heads;
    const half_t *Q = g.Q + b * g.q_bs + h * g.q_hs;
    const half_t *K = g.K + b * g.k_bs + h * g.k_hs;
    const half_t *V = g.V + b * g.v_bs + h * g.v_hs;
    const uint4_t zero4 = {0u, 0u, 0u, 0u};
    const int key0 = split * AD_KEYS + slot;

    uint4_t kr[AD_L], vr[AD_L];
#pragma unroll
    for (int i = 0; i < AD_L; i++) {
        const uint32_t kc = (uint32_t)min(key0 + 16 * i, g.kv_len - 1); // past the last key: a valid one, masked below
        kr[i] = __builtin_nontemporal_load((const uint4_t *)(K + (kc * (uint32_t)g.k_rs + 8u * segc)));
    }
#pragma unroll
    for (int i = 0; i < AD_L; i++) {
        const uint32_t kc = (uint32_t)min(key0 + 16 * i, g.kv_len - 1);
        vr[i] = __builtin_nontemporal_load((const uint4_t *)(V + (kc * (uint32_t)g.v_rs + 8u * segc)));
    }
    uint4_t qv = *(const uint4_t *)(Q + 8 * segc);
    if (seg >= ns) qv = zero4;

    // scores in base-2 units, the same in all 16 lanes of a key
    float sc[AD_L], m = -INFINITY;
#pragma unroll
    for (int i = 0; i < AD_L; i++) {
        float p = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t qa = qv[e], ka = kr[i][e];
            p = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, qa), __builtin_bit_cast(half2_t, ka), p, false);
        }
        p = ad_row_sum(p);
        sc[i] = key0 + 16 * i < g.kv_len ? p * g.scale_log2e : -INFINITY;
        m = fmaxf(m, sc[i]);
    }
    m = wave_max(m);
    if (lane == 0) sm[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
    const float m_use = m == -INFINITY ? 0.f : m; // no visible key here: every weight is exp2(-inf) = 0

    // probabilities (f32) and this lane's 8 dimensions of sum_k p_k v_k over its key slot
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, l = 0.f;
#pragma unroll
    for (int i = 0; i < AD_L; i++) {
        const float p = __builtin_amdgcn_exp2f(sc[i] - m_use);
        l += p;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t va = vr[i][e];
            const half2_t v2 = __builtin_bit_cast(half2_t, va);
            acc[2 * e] = fmaf(p, (float)v2[0], acc[2 * e]);
            acc[2 * e + 1] = fmaf(p, (float)v2[1], acc[2 * e + 1]);
        }
    }
    // a key's probability sits in all 16 lanes of its row: the wavefront's sum counts it 16 times
    l = wave_sum(l) * (1.f / 16.f);
    if (lane == 0) sl[wave] = l;
    *(float4_t *)&so[slot][seg][0] = float4_t{acc[0], acc[1], acc[2], acc[3]};
    *(float4_t *)&so[slot][seg][4] = float4_t{acc[4], acc[5], acc[6], acc[7]};
    __syncthreads();
    float *pr = g.partial + ((size_t)bh * g.splits + split) * AD_PSTRIDE;
    if (t == 0) pr[0] = m, pr[1] = (sl[0] + sl[1]) + (sl[2] + sl[3]);
    if (t < g.D) {
        float o = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) o += so[k][t >> 3][t & 7];
        pr[4 + t] = o;
    }
}

// One workgroup per head: thread d combines dimension d of the head's splits.
__global__ __launch_bounds__(128) void attention_decode_merge_kernel(AttnArgs g) {
    const int bh = blockIdx.x, b = bh / g.heads, h = bh - b * g.heads, d = threadIdx.x;
    const float *base = g.partial + (size_t)bh * g.splits * AD_PSTRIDE;
    // (maximum, sum, output) over the splits, sixteen splits' values requested at a time: the partial results come
    // from other XCDs' workgroups, so every round of loads is a trip to memory, and a cache of 2048 keys is one round.
    // Within a round the sixteen weights are independent of each other (one maximum first, then sixteen
    // exponentials side by side), not a chain of sixteen rescalings.
    float m = -INFINITY, l = 0.f, o = 0.f;
    const int dc = min(d, g.D - 1);
    for (int s0 = 0; s0 < g.splits; s0 += 16) {
        float ms[16], ls[16], os[16];
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const float *ps = base + (size_t)min(s0 + u, g.splits - 1) * AD_PSTRIDE; // past the last split: re-read it, weight 0 below
            ms[u] = s0 + u < g.splits ? ps[0] : -INFINITY, ls[u] = ps[1], os[u] = ps[4 + dc];
        }
        float m_new = m;
#pragma unroll
        for (int u = 0; u < 16; u++) m_new = fmaxf(m_new, ms[u]);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float a = __builtin_amdgcn_exp2f(m - m_use);
        float lr = 0.f, orr = 0.f;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const float w = __builtin_amdgcn_exp2f(ms[u] - m_use); // exp2(-inf) = 0: a split past the end, or one with no visible key
            lr = fmaf(ls[u], w, lr), orr = fmaf(os[u], w, orr);
        }
        l = fmaf(l, a, lr), o = fmaf(o, a, orr);
        m = m_new;
    }
    if (d < g.D) g.O[b * g.o_bs + h * g.o_hs + d] = (half_t)(o / l); // no visible key anywhere: 0 / 0 = NaN, as in the single pass
}

// splits of the decode kernel for this problem, or 0 when it does not apply: one query row (the causal rule
// then hides nothing), a cache long enough to be worth two kernels; a launch with a mask tensor stays tiled
static int attention_decode_splits(const rt_attention_desc &d) {
    if (d.q_len != 1 || d.kv_len < 256 || d.head_dim % 8 != 0 || d.head_dim > 128) return 0;
    return (d.kv_len + AD_KEYS - 1) / AD_KEYS;
}
static uint64_t attention_decode_workspace_bytes(const rt_attention_desc &d) {
    return (uint64_t)d.batch * d.heads * attention_decode_splits(d) * AD_PSTRIDE * sizeof(float);
}

template <int DP, int MK, int DC, int NKQ> static hipError_t launch_attention_k(const AttnArgs &g, int stacks, hipStream_t st) {
    constexpr int STAGES = MK == 2 ? 3 : at_stages(DP, NKQ);
    // the ring of packed key + value (+ mask) blocks; the merge of the key parts reuses it
    const size_t stage = (size_t)2 * (32 * NKQ) * g.D * sizeof(half_t) + (MK == 2 ? (size_t)AT_BQ * (32 * NKQ) * (g.mask_f32 ? 4 : 2) : 0);
    const size_t ring = STAGES * stage;
    const size_t merge = (size_t)(NKQ - 1) * 4 * (2 + 4 * (DP / 16)) * 64 * sizeof(float);
    const size_t lds = ring > merge ? ring : merge;
    if (lds > 160 * 1024) return hipErrorNotSupported;
    if (lds > 48 * 1024) {
        if (const hipError_t e = ensure_lds_limit<&attention_kernel<DP, MK, DC, NKQ>>(); e != hipSuccess) return e;
    }
    const unsigned qb = (unsigned)((g.q_len + AT_BQ - 1) / AT_BQ);
    hipLaunchKernelGGL((attention_kernel<DP, MK, DC, NKQ>), dim3(qb, (unsigned)stacks, (unsigned)g.splits), dim3(256 * NKQ), lds, st, g);
    if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (g.splits > 1) {
        hipLaunchKernelGGL((attention_merge_kernel<DP>), dim3(qb, (unsigned)stacks), dim3(256), 0, st, g);
        return hipGetLastError();
    }
    return hipSuccess;
}

// keys from which a launch in one pass takes the sixteen-wavefront kernel (head_dim up to 96).  32 heads x 512 queries x
// head_dim 80, eight / sixteen wavefronts: 512 keys 10.0 / 10.7 us, 1024: 15.1 / 15.1, 1536: 21.3 / 20.1, 4096: 43.6 / 41.6;
// 6 heads x 1500 x 1500 x 64 (Whisper): 17.8 / 15.8; 32 x 2048 x 2048 x 96 causal: 78.3 / 71.8
RT_TUNABLE(g_attention_wide_from, 1280);
RT_TUNABLE(g_attention_mask_direct, 0); // non-zero: a mask tensor is always read from memory where it is used (for comparisons)

template <int DP, int MK, int DC> static hipError_t launch_attention_dm(const AttnArgs &g, int stacks, hipStream_t st) {
    if constexpr (DP <= 96 && MK != 2) {
        if (g.splits == 1 && g.kv_len >= g_attention_wide_from) return launch_attention_k<DP, MK, DC, 4>(g, stacks, st);
    }
    return launch_attention_k<DP, MK, DC, 2>(g, stacks, st);
}

// the kernel built for this head_dim (Whisper 64, Phi-2 80, Phi-3 96, Llama-class 128), else the one that takes it as an argument
template <int DP, int DC> static hipError_t launch_attention_dp(const AttnArgs &g, int stacks, hipStream_t st) {
    // a mask tensor whose rows are whole 16-byte vectors travels through the ring; any other is read where it is used
    const int64_t mrb = g.mask_rs * (g.mask_f32 ? 4 : 2);
    const int mk = !g.mask ? 0 : ((((uintptr_t)g.mask & 15u) == 0 && mrb % 16 == 0 && mrb >= 16 && mrb < (int64_t(1) << 31) && !g_attention_mask_direct) ? 2 : 1);
    if (g.D == DC) {
        if (mk == 2) return launch_attention_dm<DP, 2, DC>(g, stacks, st);
        return mk ? launch_attention_dm<DP, 1, DC>(g, stacks, st) : launch_attention_dm<DP, 0, DC>(g, stacks, st);
    }
    if (mk == 2) return launch_attention_dm<DP, 2, 0>(g, stacks, st);
    return mk ? launch_attention_dm<DP, 1, 0>(g, stacks, st) : launch_attention_dm<DP, 0, 0>(g, stacks, st);
}

static int attention_dp(int head_dim) { return head_dim <= 64 ? 64 : (head_dim <= 96 ? 96 : 128); }

// Workgroups per query block.  A launch with few query blocks (decoding: one query against a long
// cache) leaves most compute units idle; the keys of a block are then shared out, every workgroup
// gets at least two key blocks, and a second small kernel merges the partial results.
int attention_splits(const rt_attention_desc &d) {
    const int64_t wgs = (int64_t)((d.q_len + AT_BQ - 1) / AT_BQ) * d.batch * d.heads;
    const int nkb = (d.kv_len + AT_BK - 1) / AT_BK;
    if (wgs <= 0 || wgs >= 128 || nkb < 4) return 1;
    int s = (int)(256 / wgs);
    if (s > nkb / 2) s = nkb / 2;
    if (s > AT_MAX_SPLITS) s = AT_MAX_SPLITS;
    return s < 2 ? 1 : s;
}

// bytes of workspace a split launch of this problem needs (0: it runs in one pass)
uint64_t attention_workspace_bytes(const rt_attention_desc &d) {
    const int s = attention_splits(d);
    const uint64_t qb = (uint64_t)((d.q_len + AT_BQ - 1) / AT_BQ);
    const uint64_t tiled = s <= 1 ? 0 : qb * (uint64_t)d.batch * d.heads * s * AT_BQ * (4 + attention_dp(d.head_dim)) * sizeof(float);
    return std::max(tiled, attention_decode_workspace_bytes(d)); // whichever of the two split paths the launch takes
}

// f16 tensors, head_dim a multiple of 8 up to 128, rows 16-byte aligned.  `workspace` may be null
// (or too small): the launch then runs in one pass.
hipError_t launch_attention(const rt_attention_desc &d, const void *q, const void *k, const void *v, const void *mask,
                            void *out, void *workspace, uint64_t workspace_bytes, hipStream_t stream) {
    AttnArgs g{};
    g.Q = (const half_t *)q, g.K = (const half_t *)k, g.V = (const half_t *)v, g.mask = mask, g.O = (half_t *)out;
    g.heads = d.heads, g.q_len = d.q_len, g.kv_len = d.kv_len, g.D = d.head_dim;
    g.q_bs = d.q_strides[0], g.q_hs = d.q_strides[1], g.q_rs = d.q_strides[2];
    g.k_bs = d.k_strides[0], g.k_hs = d.k_strides[1], g.k_rs = d.k_strides[2];
    g.v_bs = d.v_strides[0], g.v_hs = d.v_strides[1], g.v_rs = d.v_strides[2];
    g.o_bs = d.o_strides[0], g.o_hs = d.o_strides[1], g.o_rs = d.o_strides[2];
    g.mask_rs = d.mask_row_stride, g.mask_f32 = d.mask_dtype == RT_F32;
    g.causal = d.causal != 0;
    g.scale_log2e = d.scale * kLog2e;
    g.splits = 1, g.partial = nullptr;
    if (const uint64_t need = attention_workspace_bytes(d); need > 0 && workspace && workspace_bytes >= need && !((uintptr_t)workspace & 15u))
        g.splits = attention_splits(d), g.partial = (float *)workspace;
    const int64_t stacks = (int64_t)d.batch * d.heads;
    if (stacks > 65535) return hipErrorNotSupported;
    // 32-bit element offsets inside one head's keys and values
    if ((int64_t)d.kv_len * g.k_rs >= (int64_t(1) << 31) || (int64_t)d.kv_len * g.v_rs >= (int64_t(1) << 31))
        return hipErrorNotSupported;
    // one query against a long cache: the streaming kernel, when the caller gave the workspace for it
    if (const int ds = attention_decode_splits(d); ds > 0 && ds <= 65535 && !mask && workspace && !((uintptr_t)workspace & 15u) &&
                                                   workspace_bytes >= attention_decode_workspace_bytes(d)) {
        g.splits = ds, g.partial = (float *)workspace;
        hipLaunchKernelGGL(attention_decode_kernel, dim3((unsigned)ds, (unsigned)stacks), dim3(AD_THREADS), 0, stream, g);
        if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        hipLaunchKernelGGL(attention_decode_merge_kernel, dim3((unsigned)stacks), dim3(128), 0, stream, g);
        return hipGetLastError();
    }
    if (d.head_dim <= 64) return launch_attention_dp<64, 64>(g, (int)stacks, stream);
    if (d.head_dim == 80) return launch_attention_dp<96, 80>(g, (int)stacks, stream);
    if (d.head_dim <= 96) return launch_attention_dp<96, 96>(g, (int)stacks, stream);
    return launch_attention_dp<128, 128>(g, (int)stacks, stream);
}

} // namespace rt
