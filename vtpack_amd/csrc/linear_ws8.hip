// Packed-M Linear for bf16 operands with a short K (K * 2 bytes = 768: the C = 384 models), weight-stationary, two
// waves per SIMD.
//
// A workgroup is 8 waves and owns 384 output columns for its whole life: every wave keeps its 48 rows of W (all of
// K) in registers as ready-made operands of the 16x16x32 MFMA (3 column blocks x 12 K steps = 36 fragments of 4
// registers, most of them in accumulation registers, which the MFMA reads directly), so the only operand that
// moves is A.  A streams HBM/L2 -> LDS in 32-row tiles by direct loads (no VGPR staging) into a ring several tiles
// deep, and every wave multiplies every tile against its own columns:  D = W_strip * A_tile^T, so a lane owns four
// consecutive output columns of one row per block.  The address unit takes a store of 16 rows x 32 bytes about as
// long as one of 16 rows x 64 bytes, so the first two column blocks of a row block leave in one store of 16 bytes a
// lane (the four lanes of a row regroup their halves with two row swaps) and the third in one of 8 bytes.
//
// Why two waves per SIMD: a single wave issues at most one vector instruction every other issue cycle (measured:
// an FMA every ~7.5 clocks from one wave, every ~3.7 from two) and keeps the matrix pipe 64 % busy with back-to-back
// MFMAs; two waves together reach 1.8 - 1.9 times the throughput of one on MFMA + VALU mixes.  With 256 registers a
// wave its strip is 48 columns.  Every wave runs the same stream, in half steps of one 16-row block: the 36 MFMAs
// of a row block, three per K step, and behind each K step one element of the epilogue of the row block finished
// half a step earlier (twelve K steps, twelve elements: scale, bias, residual, GELU, pack, store), so matrix and
// vector work alternate at the finest grain without a second set of accumulators.
//
// Epilogues: bias (fp32 add), residual (its tile comes through LDS with A's, same layout), GELU, and the two
// LayerNorm helpers:
//   HAS_LN: the rows of A are to be layer-normalised first, out = act(LayerNorm(A) W^T + bias), without a normalised
//   copy of A.  With gamma folded into W (W' = W * gamma, rounded to bf16) and b' = bias + W beta,
//       LayerNorm(a) W^T + bias = rstd * (a W'^T - mean * colsum(W') + sigma * b'),   sigma = 1 / rstd,
//   so the tile loop multiplies the raw rows by W' and one more K step adds the two rank-one terms: its A-side
//   fragment is the row's 32-byte statistics record (mean and sigma, each split into bf16 parts so that the products
//   carry 24 and 16 significant bits; written by whoever produced the row, see ln_record in common.h), its W-side
//   fragment the column's record of -colsum(W') and b' in the matching order (`lnw`, two 16-byte halves per output
//   column).  The records of a tile arrive in LDS with the tile (one more direct load); the epilogue multiplies by
//   rstd = 1 / (sigma_1 + sigma_2).  A separate bias is not taken (it is part of b').
//   HAS_STAT (one column group, N = 384: the workgroup owns whole output rows): also writes the statistics records
//   of the output rows (fp32 values before their rounding to bf16), for a HAS_LN Linear that takes `out` next: sums
//   about a pivot taken from the row itself (the first element of its residual; without a residual each wave's first
//   output element of the row, the waves' sums being moved to one pivot when they are merged), added up over the four
//   lanes of a row and, one barrier later, over the eight waves by a few lanes per wave, which write 128 contiguous
//   bytes of records.
//
// Synchronisation: one s_barrier per tile.  Vector-memory operations retire in issue order; each wave keeps a tally
// of the ones it has issued and, per tile, the tally right after that tile's direct loads, and waits with a counted
// s_waitcnt vmcnt for its own loads of the tile about to be read; younger loads and the stores stay in flight.
// Rows >= M of the last tile are clamped to row M-1 on every read and on the store (those lanes recompute row M-1
// and store the same bytes), and the last tile of the matrix is moved back to end at row M.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

namespace vtdge {

__device__ __forceinline__ void w8_mma_a(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void w8_mma_v(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(wfrag), "v"(afrag));
}
// for operands written by vector instructions just before: the wait states the MFMA needs after such a write
__device__ __forceinline__ void w8_mma_v_fresh(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void w8_mma_az(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(d) : "a"(wfrag), "v"(afrag));
}

// GELU(x) = x * Phi(x), Phi - 1/2 as a degree-15 odd minimax polynomial on [-4, 4] (x clamped there):
// |error| <= 1.3e-4, below 1/30 of a bf16 rounding step of the result.
__device__ __forceinline__ float w8_gelu(float f)
{
    const float x = __builtin_amdgcn_fmed3f(f, -4.0f, 4.0f);
    const float t = x * x;
    float q = -1.580785487e-09f * t + 1.217110604e-07f;
    q = q * t - 4.100865225e-06f;
    q = q * t + 8.066737963e-05f;
    q = q * t - 1.048204291e-03f;
    q = q * t + 9.664873803e-03f;
    q = q * t - 6.617537860e-02f;
    q = q * t + 3.988475095e-01f;
    return f * (x * q + 0.5f);
}

// The work of one workgroup: column group g of the matrix, position p among the P workgroups of that group.
template <int ACT, bool HAS_BIAS, bool HAS_RES, bool HAS_LN, bool HAS_STAT>
__device__ __forceinline__ void ws8_workgroup(
    const bf16_t *__restrict__ A, int64_t lda, const bf16_t *__restrict__ Wt, const bf16_t *__restrict__ bias,
    const bf16_t *__restrict__ res, int64_t ldr, bf16_t *__restrict__ out, int64_t ldo,
    const int64_t *__restrict__ rows_dev, int64_t rows, int g, int p, int P, const u32x4 *__restrict__ Wp,
    const u32x4 *__restrict__ lnrec, const u32x4 *__restrict__ lnw, u32x4 *__restrict__ stat_out, float stat_eps)
{
    constexpr int KB = 768;                     // bytes of one operand row
    constexpr int TILE = 32 * KB;               // bytes of one 32-row tile (A or residual) in LDS
    constexpr int KS = 12;                      // K steps of 32
    constexpr int CB = 3;                       // 16-column blocks per wave
    constexpr int NA = 32;                      // fragments (in the order cb * KS + ks) that live in accumulation registers
    constexpr int D = HAS_RES ? 3 : 4;          // ring depth (tiles)
    constexpr int PA = D - 1;                   // step t issues the loads of tile t + PA
    constexpr int SLOT = TILE * (HAS_RES ? 2 : 1);
    constexpr int OFF_L = D * SLOT;             // HAS_LN: the statistics records of the tiles in the ring, 1 KB each
    constexpr int OFF_S = OFF_L + (HAS_LN ? D * 1024 : 0);   // HAS_STAT: 3 buffers of [8 waves][32 rows] x 16 B
    constexpr int NLA = 3;                      // direct loads of A per wave and tile
    static_assert(!(HAS_LN && (HAS_BIAS || HAS_RES)), "with HAS_LN the bias is part of the column records");
    static_assert(!(HAS_RES && ACT != VTDGE_ACT_NONE), "residual after an activation is not built");
    static_assert(!HAS_STAT || ACT == VTDGE_ACT_NONE, "records are written for rows without activation");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15, kg = lane >> 4;
    const int col0 = g * 384 + w * 48;               // first output column of this wave

    // ---- the stationary operand: fragment (cb, ks) = columns 16cb.. of the strip, K step ks: lane (c16, kg) holds
    // W[col0 + 16cb + c16][32ks + 8kg .. + 7].  From a copy in fragment order (vtdge_linear_prepack) with contiguous
    // 1 KB loads, else straight from W.
    u32x4 wfa[NA], wfv[CB * KS - NA];
    {
        const u32x4 *wp = Wp != nullptr ? Wp + ((size_t)(g * 8 + w) * (CB * KS)) * 64 + lane : nullptr;
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                u32x4 v;
                if (wp != nullptr) v = wp[(cb * KS + ks) * 64];
                else v = *reinterpret_cast<const u32x4 *>(Wt + (size_t)(col0 + 16 * cb + c16) * 384 + 32 * ks + 8 * kg);
                if (cb * KS + ks < NA) wfa[cb * KS + ks] = v;
                else wfv[cb * KS + ks - NA] = v;
            }
    }

    const int64_t M = live_rows(rows_dev, rows);
    const int tiles_m = (int)((M + 31) / 32);
    const int nt = tiles_m > p ? (tiles_m - p + P - 1) / P : 0;
    if (nt == 0) return;
    const int M32 = (int)M;

    // ---- per-lane constants
    u32x2 bv[CB];                    // bias of the lane's columns (packed)
    u32x4 wl[CB];                    // HAS_LN: the column records, W-side fragments of the statistics K step
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        wl[cb] = z;
        if constexpr (HAS_LN) {
            if (kg < 2) wl[cb] = lnw[(col0 + 16 * cb + c16) * 2 + kg];
        }
        bv[cb] = u32x2{0u, 0u};
        if constexpr (HAS_BIAS) bv[cb] = *reinterpret_cast<const u32x2 *>(bias + col0 + 16 * cb + 4 * kg);
    }
    // fragment reads: row c16 (+16 for the second row block) of a 128-byte slab, chunk 4 (ks % 2) + kg, the chunk
    // position XOR-swizzled with the row's low bits (eight consecutive lanes read eight different bank groups)
    const int cs = c16 * 128 + ((kg ^ (c16 & 7)) * 16);
    // direct loads of a 32-row tile: instruction i covers slab i / 4 and rows (i % 4) * 8 + lane / 8; the lane
    // fetches chunk (lane % 8) ^ (row % 8) = (lane % 8) ^ (lane / 8) of its row.  Wave w issues i = 3w .. 3w + 2.
    const int l8 = lane >> 3;
    const int gx16 = ((lane & 7) ^ (lane >> 3)) * 16;
    const uint32_t lda2 = (uint32_t)lda * 2, ldr2 = (uint32_t)ldr * 2, ldo2 = (uint32_t)ldo * 2;
    const int m_last = M32 > 32 ? M32 - 32 : 0;
    auto tile_row0 = [&](int k) -> int { const int m = (p + k * P) * 32; return m < m_last ? m : m_last; };
    auto clamp_row = [&](int gm) -> int { return gm < M32 ? gm : M32 - 1; };
    // the residual's 8 bytes of a lane: columns 48w + 16cb + 4kg .. + 3 of the group's 384, same slab layout as A
    int rsoff[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const int off = 96 * w + 32 * cb + 8 * kg;           // byte offset in the 768-byte row
        rsoff[cb] = (off >> 7) * 4096 + c16 * 128 + ((((off >> 4) & 7) ^ (c16 & 7)) * 16) + (off & 15);
    }

    // tally of vector-memory operations issued by this wave and, per tile, the tally right after its loads
    int issued = 0;
    uint64_t marks = 0;
    auto set_mark = [&](int k) {
        const int sh = (k & 7) * 8;
        marks = (marks & ~(0xffull << sh)) | ((uint64_t)(issued & 0xff) << sh);
    };
    auto after_mark = [&](int k) -> int { return (issued - (int)((marks >> ((k & 7) * 8)) & 0xff)) & 0xff; };

    // the direct loads of tile k (this wave's share) into its ring slot; tiles past the last are not loaded
    auto issue_tile = [&](int k) {
        if (k >= nt) return;
        const int m0 = tile_row0(k);
        const uint32_t dst = lds0 + (k % D) * SLOT;
#pragma unroll
        for (int ii = 0; ii < NLA; ii++) {
            const int i = w * NLA + ii;
            const int gm = clamp_row(m0 + (i & 3) * 8 + l8);
            dma16(A, (uint32_t)gm * lda2 + (i >> 2) * 128 + gx16, dst + i * 1024);
            if constexpr (HAS_RES)
                dma16(res, (uint32_t)gm * ldr2 + g * KB + (i >> 2) * 128 + gx16, dst + TILE + i * 1024);
        }
        issued += NLA * (HAS_RES ? 2 : 1);
        if constexpr (HAS_LN) {
            // the records of the tile's 32 rows (lane i: half i % 2 of row i / 2): 1 KB, one load; the waves take
            // turns (a wave waits for its own loads of a tile before the tile's barrier, so the barrier covers it)
            if (w == (k & 7)) {
                const int gm = clamp_row(m0 + (lane >> 1));
                dma16(lnrec, (uint32_t)gm * 32u + (lane & 1) * 16u, lds0 + OFF_L + (k % D) * 1024);
                issued += 1;
            }
        }
        set_mark(k);
    };

    f32x4 acc[2][CB];                     // [row block][column block]
    float rs[2] = {1.0f, 1.0f};           // HAS_LN: rstd of the lane's rows
    u32x2 rv1[CB];                        // HAS_RES: the residual's values for row block 1 (kept past its slot's life)
    float pv[2] = {0.f, 0.f};             // HAS_STAT: the rows' pivots

    // One element of the epilogue: output column 16cb + 4kg + i of the lane's row in row block RB, taken from the
    // accumulator, finished in fp32 and kept until its group of four is stored.  E = 4 * cb + i counts the twelve
    // elements of a half tile.
    float f4[4], sa = 0.f, sq = 0.f;
    uint32_t rw = 0u;
    u32x2 o0 = {0u, 0u};
    // byte offset, from the lane's own first column (4 kg), of its 16 bytes of the pair of column blocks 0 and 1
    const int pair_off = (16 * (kg & 1) + 8 * (kg >> 1) - 4 * kg) * 2;
    auto epi_element = [&](auto rb_tag, auto e_tag, const unsigned char *rtile, unsigned char *orow, int part) {
        constexpr int RB = decltype(rb_tag)::value, E = decltype(e_tag)::value, cb = E / 4, i = E % 4;
        float f = acc[RB][cb][i];
        if constexpr (HAS_LN) f *= rs[RB];
        if constexpr (HAS_BIAS) f += (i & 1) ? bf16hi(i < 2 ? bv[cb].x : bv[cb].y) : bf16lo(i < 2 ? bv[cb].x : bv[cb].y);
        if constexpr (HAS_RES) {
            uint32_t word;
            if constexpr (RB == 1) {
                word = i < 2 ? rv1[cb].x : rv1[cb].y;
            } else {
                // row block 0 is finished while its tile's slot is still there
                if (i == 0 || i == 2)
                    rw = *reinterpret_cast<const uint32_t *>(rtile + rsoff[cb] + (i >> 1) * 4);
                word = rw;
            }
            f += (i & 1) ? bf16hi(word) : bf16lo(word);
        }
        if constexpr (ACT == VTDGE_ACT_GELU) f = w8_gelu(f);
        if constexpr (HAS_STAT) {
            if (E == 0) sa = sq = 0.f;
            if constexpr (!HAS_RES) {
                // no residual to take the pivot from: the row's first output element of this wave's strip (lane
                // kg = 0, E = 0), handed to the row's other lanes; the eight waves' pivots differ and are brought
                // to a common one when their sums are merged
                if (E == 0) pv[RB] = __shfl(f, c16, WAVE);
            }
            const float dl = f - pv[RB];
            sa += dl;
            sq = fmaf(dl, dl, sq);
        }
        f4[i] = f;
        if (i == 3) {
            u32x2 o;
            o.x = pack_bf16x2(f4[0], f4[1]);
            o.y = pack_bf16x2(f4[2], f4[3]);
            if (cb == 0) {
                o0 = o;            // waits for its neighbour
            } else if (cb == 1) {
                // Column blocks 0 and 1 leave together, 16 bytes a lane: the lanes kg = 1, 3 of a row hand their
                // half of block 0 to kg = 0, 2 and take those lanes' half of block 1 (rows of 16 lanes swapped
                // between the two registers), so lane kg holds columns 16 (kg % 2) + 8 (kg / 2) .. + 7 of the 32
                // and a store instruction covers 64 contiguous bytes of each of its 16 rows instead of 32.
                const auto sx = __builtin_amdgcn_permlane16_swap(o0.x, o.x, false, false);
                const auto sy = __builtin_amdgcn_permlane16_swap(o0.y, o.y, false, false);
                const u32x4 v = {sx[0], sy[0], sx[1], sy[1]};
                *reinterpret_cast<u32x4 *>(orow + pair_off) = v;
            } else {
                *reinterpret_cast<u32x2 *>(orow + cb * 32) = o;
            }
        }
        if constexpr (HAS_STAT) {
            if (E == 11) {
                // the four lanes of a row (kg = 0..3) hold sums about the same pivot: add them up
                sa += __shfl_xor(sa, 16, WAVE);
                sq += __shfl_xor(sq, 16, WAVE);
                sa += __shfl_xor(sa, 32, WAVE);
                sq += __shfl_xor(sq, 32, WAVE);
                if (kg == 0) {
                    const u32x4 v = {__float_as_uint(pv[RB]), __float_as_uint(sa), __float_as_uint(sq), 0u};
                    *reinterpret_cast<u32x4 *>(smem + OFF_S + part * 4096 + (w * 32 + 16 * RB + c16) * 16) = v;
                }
            }
        }
    };

    // ---- half a step: the 36 MFMAs of row block RB of tile k, three per K step, and behind each K step one element
    // of the epilogue of the row block finished half a step ago (row block 1 of tile k-1 for RB = 0, row block 0 of
    // tile k for RB = 1) - twelve K steps, twelve elements.  Every wave runs the same stream; the two waves of a SIMD
    // fill each other's issue gaps.
    auto half_step = [&](auto rb_tag, int k, bool with_epilogue) {
        constexpr int RB = decltype(rb_tag)::value;
        using OTHER = std::integral_constant<int, 1 - RB>;
        const unsigned char *at = smem + (k % D) * SLOT;
        const int ke = RB == 0 ? k - 1 : k;                       // the tile whose other row block is finished here
        unsigned char *orow = nullptr;
        if (with_epilogue) {
            const int gm = clamp_row(tile_row0(ke) + 16 * (1 - RB) + c16);
            orow = reinterpret_cast<unsigned char *>(out) + (uint64_t)(uint32_t)gm * ldo2 + (col0 + 4 * kg) * 2;
        }
        const unsigned char *rtile = at + TILE;                   // residual of tile k (used for row block 0 only)
        u32x4 fa[2];
        fa[0] = *reinterpret_cast<const u32x4 *>(at + RB * 2048 + cs);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            if (ks + 1 < KS)
                fa[(ks + 1) & 1] = *reinterpret_cast<const u32x4 *>(at + ((ks + 1) >> 1) * 4096 + RB * 2048 +
                                                                    (cs ^ (((ks + 1) & 1) * 64)));
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const int fi = cb * KS + ks;
                if (ks == 0) w8_mma_az(acc[RB][cb], wfa[fi], fa[0]);
                else if (fi < NA) w8_mma_a(acc[RB][cb], wfa[fi], fa[ks & 1]);
                else w8_mma_v_fresh(acc[RB][cb], wfv[fi - NA], fa[ks & 1]);   // may just have been moved
            }
            if (ks == 0) {
                // The other row block's last MFMAs were issued before the three above; with these wait states their
                // results have reached the registers.  The accumulators pass through the statement, which keeps
                // every read of them (the epilogue below, or a copy of the compiler's) behind it.
                asm volatile("s_nop 7" : "+v"(acc[1 - RB][0]), "+v"(acc[1 - RB][1]), "+v"(acc[1 - RB][2]));
            }
            if (with_epilogue) {
                static_for<KS>([&](auto e_tag) {
                    if (decltype(e_tag)::value == ks) epi_element(OTHER{}, e_tag, rtile, orow, ke % 3);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (HAS_LN) {
            const unsigned char *rec = smem + OFF_L + (k % D) * 1024;
            const int r = 16 * RB + c16;
            u32x4 fl = {0u, 0u, 0u, 0u};
            if (kg < 2) fl = *reinterpret_cast<const u32x4 *>(rec + r * 32 + kg * 16);
            const uint32_t sg = *reinterpret_cast<const uint32_t *>(rec + r * 32 + 12);     // (sigma_1, sigma_2)
            rs[RB] = __builtin_amdgcn_rcpf(bf16lo(sg) + bf16hi(sg));
#pragma unroll
            for (int cb = 0; cb < CB; cb++) w8_mma_v_fresh(acc[RB][cb], wl[cb], fl);
        }
        // the same wait states for this row block's own last MFMAs, ahead of any copy of the accumulators that the
        // compiler may put at the end of the loop body
        asm volatile("s_nop 7\n\ts_nop 3" : "+v"(acc[RB][0]), "+v"(acc[RB][1]), "+v"(acc[RB][2]));
        if constexpr (HAS_RES) {
            if constexpr (RB == 1) {
                // row block 1 is finished in the next step, when the slot is being overwritten: its residual values
                // (and pivot) leave with it
#pragma unroll
                for (int cb = 0; cb < CB; cb++)
                    rv1[cb] = *reinterpret_cast<const u32x2 *>(at + TILE + 2048 + rsoff[cb]);
            }
            if constexpr (HAS_STAT) {
                // first element of the row's residual: chunk 0 of slab 0, at position 0 ^ (row % 8)
                const int r = 16 * RB + c16;
                pv[RB] = bf16_to_f32(*reinterpret_cast<const bf16_t *>(at + TILE + r * 128 + (r & 7) * 16));
            }
        }
    };
    auto count_stores = [&]() { issued += CB - 1; };      // blocks 0 and 1 in one store, block 2 in another

    // HAS_STAT: the records of tile k from the eight waves' sums: wave w merges rows 4w .. 4w+3, lane l < 8 writing
    // half l % 2 of row 4w + l / 2 (128 contiguous bytes per wave)
    auto stat_finish = [&](int k) {
        const int r = w * 4 + ((lane >> 1) & 3);
        const unsigned char *pb = smem + OFF_S + (k % 3) * 4096 + r * 16;
        float sa = 0.f, sq = 0.f, pivot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(pb + i * 512);
            if constexpr (HAS_RES) {
                pivot = __uint_as_float(v.x);      // the same in all eight
                sa += __uint_as_float(v.y);
                sq += __uint_as_float(v.z);
            } else {
                // sums of 48 values about the wave's own pivot p_i, moved to wave 0's pivot P (d = p_i - P):
                //   sum (x - P) = sa_i + 48 d,   sum (x - P)^2 = sq_i + 2 d sa_i + 48 d^2
                if (i == 0) pivot = __uint_as_float(v.x);
                const float d = __uint_as_float(v.x) - pivot, si = __uint_as_float(v.y);
                sa += fmaf(48.0f, d, si);
                sq += fmaf(d, fmaf(48.0f, d, 2.0f * si), __uint_as_float(v.z));
            }
        }
        const float m = sa * (1.0f / 384.0f);
        const float var = fmaxf(sq * (1.0f / 384.0f) - m * m, 0.f);
        u32x4 lo, hi;
        ln_record(pivot + m, sqrtf(var + stat_eps), lo, hi);
        const int gm = clamp_row(tile_row0(k) + r);
        if (lane < 8) stat_out[(int64_t)gm * 2 + (lane & 1)] = (lane & 1) ? hi : lo;
        issued += 1;
    };

    // ---- prologue: the first tiles
#pragma unroll
    for (int k = 0; k < PA; k++) issue_tile(k);

    // ---- the tile loop
    using R0 = std::integral_constant<int, 0>;
    using R1 = std::integral_constant<int, 1>;
    for (int k = 0; k < nt; k++) {
        // everything issued so far stays before the wait: the count below is of operations really in flight
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt_dyn(after_mark(k));
        if constexpr (HAS_STAT) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the sums put last step
        block_barrier();       // tile k is in LDS for every wave; the slot read last step is free
        if constexpr (HAS_STAT) {
            if (k >= 2) stat_finish(k - 2);
        }
        issue_tile(k + PA);
        half_step(R0{}, k, k > 0);
        if (k > 0) count_stores();
        half_step(R1{}, k, true);
        count_stores();
    }
    {
        // row block 1 of the last tile
        asm volatile("s_nop 7\n\ts_nop 7" : "+v"(acc[1][0]), "+v"(acc[1][1]), "+v"(acc[1][2]));
        const int ke = nt - 1;
        const int gm = clamp_row(tile_row0(ke) + 16 + c16);
        unsigned char *orow = reinterpret_cast<unsigned char *>(out) + (uint64_t)(uint32_t)gm * ldo2 + (col0 + 4 * kg) * 2;
        static_for<KS>([&](auto e_tag) { epi_element(R1{}, e_tag, nullptr, orow, ke % 3); });
        count_stores();
    }
    if constexpr (HAS_STAT) {
        lds_barrier();          // the sums of the last two tiles are in LDS for every wave
        if (nt >= 2) stat_finish(nt - 2);
        stat_finish(nt - 1);
    }
}

template <int ACT, bool HAS_BIAS, bool HAS_RES, bool HAS_LN, bool HAS_STAT>
__global__ __launch_bounds__(512) void linear_ws8_kernel(
    const bf16_t *__restrict__ A, int64_t lda, const bf16_t *__restrict__ Wt, const bf16_t *__restrict__ bias,
    const bf16_t *__restrict__ res, int64_t ldr, bf16_t *__restrict__ out, int64_t ldo,
    const int64_t *__restrict__ rows_dev, int64_t rows, int groups, int P, const u32x4 *__restrict__ Wp,
    const u32x4 *__restrict__ lnrec, const u32x4 *__restrict__ lnw, u32x4 *__restrict__ stat_out, float stat_eps)
{
    // the P workgroups of a column group are spread over the 8 XCDs (consecutive workgroup numbers go to consecutive
    // XCDs), and the workgroups that share A tiles (same position in different groups) sit on the same XCD
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int g = slot % groups;                     // column group
    const int p = xcd + 8 * (slot / groups);         // position among the P workgroups of the group
    ws8_workgroup<ACT, HAS_BIAS, HAS_RES, HAS_LN, HAS_STAT>(A, lda, Wt, bias, res, ldr, out, ldo, rows_dev, rows, g, p,
                                                            P, Wp, lnrec, lnw, stat_out, stat_eps);
}

// Two Linears with folded LayerNorms in ONE launch (the key/value projection of all tokens and the query projection
// of the packed rows: same K, same epilogue, different operands and row counts).  Alone, the smaller of the two
// gives every workgroup three or four tiles behind the fixed cost of fetching its strip of W; here the grid is
// dealt out between the two in proportion to their tiles, so that every workgroup has a long run of one of them.
// The live row counts are on the device, so every workgroup works the split out for itself (the same integers in
// all of them): units of 8 workgroups (one per XCD), na units per column group of the first problem, nb per column
// group of the second, na * groups_a + nb * groups_b = gridDim.x / 8, chosen to minimise the longer of the two runs.
struct Ws8Problem {
    const bf16_t *A;
    int64_t lda;
    const bf16_t *Wt;
    bf16_t *out;
    int64_t ldo;
    const int64_t *rows_dev;
    int64_t rows;
    int groups;
    const u32x4 *Wp, *lnrec, *lnw;
};

template <int ACT>
__global__ __launch_bounds__(512) void linear_ws8_pair_kernel(const Ws8Problem a, const Ws8Problem b)
{
    const int ta = (int)((live_rows(a.rows_dev, a.rows) + 31) / 32), tb = (int)((live_rows(b.rows_dev, b.rows) + 31) / 32);
    const int units = (int)(gridDim.x >> 3);
    // nearest split to the proportional one, then its neighbours
    const float wa = (float)ta * a.groups, wb = (float)tb * b.groups;
    int na = (int)((float)units * wa / fmaxf(wa + wb, 1.f) / (float)a.groups + 0.5f);
    int best_na = 0, best_steps = 0x7fffffff;
#pragma unroll 1
    for (int c = na - 1; c <= na + 1; c++) {
        if (c < 1 || c * a.groups >= units) continue;
        const int rem = units - c * a.groups;
        if (rem % b.groups) continue;
        const int nb = rem / b.groups;
        const int sa = (ta + 8 * c - 1) / (8 * c), sb = (tb + 8 * nb - 1) / (8 * nb);
        const int steps = sa > sb ? sa : sb;
        if (steps < best_steps) {
            best_steps = steps;
            best_na = c;
        }
    }
    if (best_na == 0) {                      // no neighbour fits (tiny grids, awkward group counts): first valid split
#pragma unroll 1
        for (int c = 1; c * a.groups < units; c++)
            if ((units - c * a.groups) % b.groups == 0) {
                best_na = c;
                break;
            }
    }
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int slots_a = best_na * a.groups;
    const bool first = slot < slots_a;
    const Ws8Problem &m = first ? a : b;
    const int s2 = first ? slot : slot - slots_a;
    const int n_units = first ? best_na : (units - slots_a) / b.groups;
    const int g = s2 % m.groups, p = xcd + 8 * (s2 / m.groups);
    ws8_workgroup<ACT, false, false, true, false>(m.A, m.lda, m.Wt, nullptr, nullptr, 0, m.out, m.ldo, m.rows_dev, m.rows, g,
                                                  p, 8 * n_units, m.Wp, m.lnrec, m.lnw, nullptr, 0.f);
}

// ----------------------------------------------------------------------------- host
bool linear_ws_applicable(int64_t lda, int64_t ldr, int64_t ldo, int64_t rows, int N, int K, int esz, int act,
                          const void *bias, const void *res, const void *out)
{
    // the residual is added ahead of an activation: such a pair goes elsewhere
    if (res != nullptr && act != VTDGE_ACT_NONE) return false;
    return esz == 2 && K == 384 && lda < (1ll << 31) && ldo < (1ll << 31) && ldr < (1ll << 31) && N % 384 == 0 &&
           N / 384 <= 8 && rows >= 2048 && rows * lda < (1ll << 31) && (res == nullptr || rows * ldr < (1ll << 31)) &&
           lda % 8 == 0 && ldo % 8 == 0 && (res == nullptr || ldr % 8 == 0) &&
           (((uintptr_t)bias | (uintptr_t)res | (uintptr_t)out) & 15) == 0;
}

template <int ACT, bool HB, bool HR, bool LN, bool STAT>
static int go_ws8(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                  int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, hipStream_t st,
                  const void *lnrec, const void *lnw, void *stat_out, float stat_eps)
{
    constexpr size_t tile = 32 * 768;
    constexpr size_t lds = (HR ? 3 * 2 * tile : 4 * tile) + (LN ? 4 * 1024 : 0) + (STAT ? 3 * 4096 : 0);
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = linear_ws8_kernel<ACT, HB, HR, LN, STAT>;
    VT_RESERVE_LDS(kern, lds, "linear");
    const int groups = N / 384;
    // one workgroup per CU; the P workgroups of a column group are spread over the 8 XCDs, and the workgroups that
    // share A tiles (same position in different groups) sit on the same XCD
    int P = (compute_units() / groups) & ~7;
    if (P < 8) P = 8;
    const int64_t tiles_m = ceil_div(rows, 32);
    if (P > tiles_m) P = (int)((tiles_m + 7) & ~7);
    dim3 grid((unsigned)(P * groups)), block(512);
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<grid, block, lds, st>>>((const bf16_t *)A, lda, (const bf16_t *)W, (const bf16_t *)bias, (const bf16_t *)res,
                                   ldr, (bf16_t *)out, ldo, rows_dev, rows, groups, P, (const u32x4 *)Wp,
                                   (const u32x4 *)lnrec, (const u32x4 *)lnw, (u32x4 *)stat_out, stat_eps);
    return check_launch("linear");
}

int launch_linear_ws8(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                      int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int act,
                      hipStream_t st)
{
    const bool hb = bias != nullptr, hr = res != nullptr;
#define VT_WS(ACT, HB, HR)                                                                                       \
    return go_ws8<ACT, HB, HR, false, false>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st, nullptr, \
                                             nullptr, nullptr, 0.f)
    if (act == VTDGE_ACT_GELU) {
        if (hr) {
            set_error("linear: activation with residual is not built in the weight-stationary kernel");
            return VTDGE_ERR_UNSUPPORTED;
        }
        if (hb) VT_WS(VTDGE_ACT_GELU, true, false);
        VT_WS(VTDGE_ACT_GELU, false, false);
    }
    if (hb && hr) VT_WS(VTDGE_ACT_NONE, true, true);
    if (hb) VT_WS(VTDGE_ACT_NONE, true, false);
    if (hr) VT_WS(VTDGE_ACT_NONE, false, true);
    VT_WS(VTDGE_ACT_NONE, false, false);
#undef VT_WS
}

// out = act(LayerNorm(A) W^T + bias) from the raw rows, their statistics records and the folded weights
int launch_linear_ws8_ln(const void *A, int64_t lda, const void *lnrec, const void *Wf, const void *Wfp,
                         const void *lnw, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N,
                         int act, hipStream_t st)
{
    if (act == VTDGE_ACT_GELU)
        return go_ws8<VTDGE_ACT_GELU, false, false, true, false>(A, lda, Wf, Wfp, nullptr, nullptr, 0, out, ldo,
                                                                  rows_dev, rows, N, st, lnrec, lnw, nullptr, 0.f);
    return go_ws8<VTDGE_ACT_NONE, false, false, true, false>(A, lda, Wf, Wfp, nullptr, nullptr, 0, out, ldo, rows_dev,
                                                              rows, N, st, lnrec, lnw, nullptr, 0.f);
}

// two such Linears in one launch (see linear_ws8_pair_kernel)
int launch_linear_ws8_ln_pair(const void *A0, int64_t lda0, const void *lnrec0, const void *Wf0, const void *Wfp0,
                              const void *lnw0, void *out0, int64_t ldo0, const int64_t *rows_dev0, int64_t rows0,
                              int N0, const void *A1, int64_t lda1, const void *lnrec1, const void *Wf1,
                              const void *Wfp1, const void *lnw1, void *out1, int64_t ldo1, const int64_t *rows_dev1,
                              int64_t rows1, int N1, hipStream_t st)
{
    constexpr size_t lds = 4 * 32 * 768 + 4 * 1024;
    auto kern = linear_ws8_pair_kernel<VTDGE_ACT_NONE>;
    VT_RESERVE_LDS(kern, lds, "linear");
    const Ws8Problem a = {(const bf16_t *)A0, lda0, (const bf16_t *)Wf0, (bf16_t *)out0, ldo0, rows_dev0, rows0, N0 / 384,
                          (const u32x4 *)Wfp0, (const u32x4 *)lnrec0, (const u32x4 *)lnw0};
    const Ws8Problem b = {(const bf16_t *)A1, lda1, (const bf16_t *)Wf1, (bf16_t *)out1, ldo1, rows_dev1, rows1, N1 / 384,
                          (const u32x4 *)Wfp1, (const u32x4 *)lnrec1, (const u32x4 *)lnw1};
    // one workgroup per CU in units of 8 (one per XCD); at least one unit per column group of either problem
    int units = compute_units() / 8;
    if (units < a.groups + b.groups) units = a.groups + b.groups;
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<dim3((unsigned)(units * 8)), dim3(512), lds, st>>>(a, b);
    return check_launch("linear");
}

// out = A W^T + bias + residual for N = 384, with the statistics records of the rows of out
int launch_linear_ws8_stats(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias,
                            const void *res, int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev,
                            int64_t rows, void *records, float eps, hipStream_t st)
{
    const bool hb = bias != nullptr, hr = res != nullptr;
#define VT_WS(HB, HR)                                                                                              \
    return go_ws8<VTDGE_ACT_NONE, HB, HR, false, true>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, 384, st, \
                                                       nullptr, nullptr, records, eps)
    if (hb && hr) VT_WS(true, true);
    if (hb) VT_WS(true, false);
    if (hr) VT_WS(false, true);
    VT_WS(false, false);
#undef VT_WS
}

}  // namespace vtdge
