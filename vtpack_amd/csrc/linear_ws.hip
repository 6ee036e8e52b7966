// Packed-M Linear for bf16 operands with a short K (K * 2 bytes = 768: the C = 384 models), weight-stationary.
//
// A workgroup is 4 waves, one per SIMD, and owns a strip of BN = 4 * NB * 32 output columns for its whole life:
// every wave keeps its NB * 32 rows of W (all of K) in registers as ready-made MFMA operands (NB * K/16 fragments
// of 4 registers: 288 for NB = 3, K = 384; half of them in accumulation registers, which the MFMA reads directly),
// so the only operand that moves while the kernel runs is A.
// A streams HBM/L2 -> LDS in 32-row tiles by direct loads (no VGPR staging) into a ring that is several tiles
// deep; each wave multiplies every A tile against its own columns:  D = W_strip * A_tile^T, 32 x 32 x 16 MFMAs,
// so a lane owns one output row and bias / GELU / residual are applied in fp32 on 8-column vectors.
// Per output tile the memory system delivers 24 KB for 72 MFMAs per wave: ~10 B/clk per CU, against the ~46
// B/clk a CU can pull from L2, and the MFMA pipe never waits on the second operand.
//
// With one wave per SIMD nothing overlaps by itself, so the instruction stream is woven by hand: the fragment of
// A for substep s+3 is read from LDS before the MFMAs of substep s, and the epilogue of tile t (24 units of two
// output elements per lane) is spread over the 24 substeps of tile t+1, which accumulates into a second register
// set; a few vector instructions follow each MFMA and run while it executes.
//
// W reaches the registers through LDS as well (before the first A tile needs the space): coalesced direct loads of
// 32-row blocks in the same slab layout as A, two half-rings of three blocks, each wave reading its own blocks as
// fragments while the next blocks are in flight.
//
// Synchronisation: one s_barrier per tile.  Vector-memory operations retire in issue order, so before the barrier
// a wave waits with a *counted* s_waitcnt vmcnt until its own direct loads of the tile about to be consumed have
// landed; younger prefetches and stores stay in flight.  The count is kept exactly: a per-wave tally of issued
// operations and, per tile, the tally right after its loads.  The direct loads and the MFMAs are issued from inline
// assembly (the LDS reads of the fragments then need no vmcnt wait of the compiler's own, and the stationary
// fragments stay where they were put).
//
// Rows >= M of the last tile are clamped to row M-1 on every read and on the store: those lanes recompute row M-1
// bit for bit and store the same bytes, so the tile loop has no predicated memory operation.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

namespace vtdge {

// D = W_frag * A_frag^T (+ D).  The stationary fragment sits in accumulation registers (A) or vector registers (V);
// Z starts a new sum.  Issued from assembly so the register classes are exactly these.
__device__ __forceinline__ void mma_a(f32x16 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void mma_v(f32x16 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(wfrag), "v"(afrag));
}
// for operands written by vector instructions just before: the two wait states the MFMA needs after such a write
// (the compiler adds them for its own MFMAs, not inside assembly)
__device__ __forceinline__ void mma_v_fresh(f32x16 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void mma_az(f32x16 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(d) : "a"(wfrag), "v"(afrag));
}

// State of one epilogue unit: two output elements of a lane on their way from the accumulator to bf16.
struct EpiUnit {
    float f0, f1;   // values
    float x0, x1, t0, t1, q0, q1;   // GELU: clamped argument, its square, Horner accumulator
};

// GELU(x) = x * Phi(x), Phi - 1/2 as a degree-15 odd minimax polynomial on [-4, 4] (x clamped there):
// |error| <= 1.3e-4, below 1/30 of a bf16 rounding step of the result.  Three parts of about equal length.
__device__ __forceinline__ void gelu_part1(EpiUnit &u)
{
    u.x0 = __builtin_amdgcn_fmed3f(u.f0, -4.0f, 4.0f);
    u.x1 = __builtin_amdgcn_fmed3f(u.f1, -4.0f, 4.0f);
    u.t0 = u.x0 * u.x0;
    u.t1 = u.x1 * u.x1;
    u.q0 = -1.580785487e-09f * u.t0 + 1.217110604e-07f;
    u.q1 = -1.580785487e-09f * u.t1 + 1.217110604e-07f;
    u.q0 = u.q0 * u.t0 - 4.100865225e-06f;
    u.q1 = u.q1 * u.t1 - 4.100865225e-06f;
}
__device__ __forceinline__ void gelu_part2(EpiUnit &u)
{
    u.q0 = u.q0 * u.t0 + 8.066737963e-05f;
    u.q1 = u.q1 * u.t1 + 8.066737963e-05f;
    u.q0 = u.q0 * u.t0 - 1.048204291e-03f;
    u.q1 = u.q1 * u.t1 - 1.048204291e-03f;
    u.q0 = u.q0 * u.t0 + 9.664873803e-03f;
    u.q1 = u.q1 * u.t1 + 9.664873803e-03f;
    u.q0 = u.q0 * u.t0 - 6.617537860e-02f;
    u.q1 = u.q1 * u.t1 - 6.617537860e-02f;
}
__device__ __forceinline__ void gelu_part3(EpiUnit &u)
{
    u.q0 = u.q0 * u.t0 + 3.988475095e-01f;
    u.q1 = u.q1 * u.t1 + 3.988475095e-01f;
    u.f0 = u.f0 * (u.x0 * u.q0 + 0.5f);
    u.f1 = u.f1 * (u.x1 * u.q1 + 0.5f);
}

// HAS_LN: the rows of A are to be layer-normalised first, out = act(LayerNorm(A) W^T + bias), without a normalised
// copy of A.  With gamma folded into W (W' = W * gamma, rounded to bf16) and b' = bias + W beta,
//     LayerNorm(a) W^T + bias = rstd * (a W'^T - mean * colsum(W') + sigma * b'),   sigma = 1 / rstd,
// so the tile loop multiplies the raw rows by W' and one more K step adds the two rank-one terms: its A-side
// fragment is the row's 32-byte statistics record (mean and sigma, each split into bf16 parts so that the products
// carry 24 and 16 significant bits; written by whoever produced the row, see ln_record in common.h), its W-side
// fragment the column's record of -colsum(W') and b' in the matching order (`lnw`, two 16-byte halves per output
// column).  The records of a tile arrive in LDS with the tile (one more direct load, issued by wave 0); the
// epilogue multiplies by rstd = 1 / (sigma_1 + sigma_2).  A separate bias is not taken (it is part of b').
//
// HAS_STAT (one column group, i.e. N = 384: the workgroup owns whole output rows): also writes the statistics record
// of every output row (fp32 values before their rounding to bf16), for a HAS_LN Linear that takes `out` next.  A
// lane sums its 48 elements of the row about the first of them while the epilogue units pass; the eight partial sums
// of a row (two lane halves, four waves) meet in LDS and, one step later, sixteen lanes per wave merge them for eight
// rows each (pairwise-exact merge of means and squared deviations) and write 256 contiguous bytes of records.
template <int KS, int NB, int ACT, bool HAS_BIAS, bool HAS_RES, bool HAS_LN = false, bool HAS_STAT = false>
__global__ __launch_bounds__(256) void linear_ws_kernel(
    const bf16_t *__restrict__ A, int64_t lda, const bf16_t *__restrict__ Wt, const bf16_t *__restrict__ bias,
    const bf16_t *__restrict__ res, int64_t ldr, bf16_t *__restrict__ out, int64_t ldo,
    const int64_t *__restrict__ rows_dev, int64_t rows, int groups, int P, const u32x4 *__restrict__ Wp,
    const u32x4 *__restrict__ lnrec = nullptr, const u32x4 *__restrict__ lnw = nullptr,
    u32x4 *__restrict__ stat_out = nullptr, float stat_eps = 0.f)
{
    constexpr int KB = KS * 32;                 // bytes of one operand row
    constexpr int TILE = 32 * KB;               // bytes of one 32-row tile (A, W block or residual) in LDS
    constexpr int STRIP = NB * 32;              // output columns per wave
    constexpr int BN = 4 * STRIP;               // output columns per workgroup
    constexpr int DA = HAS_RES ? 3 : 4;         // A ring depth (tiles): deeper gains nothing and lengthens the start;
                                                // behind a residual its ring takes three of the six slots
    constexpr int DR = 3;
    constexpr int PA = DA - 1;                  // step k issues the loads of A(k + PA)
    constexpr int PR = DR - 1;                  // ... and of the residual of tile k + PR
    // Without a residual a step waits for the tile after its own, whose first fragments it reads at its end, so no
    // MFMA waits for LDS behind the barrier; with only two tiles of A in flight that wait would come too early.
    constexpr bool XT = !HAS_RES;
    constexpr int NL = TILE / 1024 / 4;         // direct loads per wave and tile
    constexpr int NU = NB * 8;                  // epilogue units per tile (two elements each)
    constexpr int KA = KS - 3;                  // substeps whose W fragments live in accumulation registers
    constexpr int FD = (HAS_RES || ACT != VTDGE_ACT_NONE) ? 2 : 3;         // fragments of A are read FD substeps ahead of their MFMAs
    constexpr int EARLY = 2;                    // A tiles issued while the last W blocks are still being read
    static_assert(KS % 4 == 0 && NL * 4 * 1024 == TILE && BN * 2 == KB, "tile geometry (residual rows = A rows)");
    static_assert(!(HAS_RES && ACT != VTDGE_ACT_NONE), "the residual is summed in the accumulator, ahead of an activation");
    static_assert(NL == 6 && NB == 3, "the vmcnt bookkeeping counts in units of 6");
    static_assert(NU == KS, "one epilogue unit per K substep");
    static_assert(KS % (FD + 1) == 0, "the fragment ring keeps its phase from tile to tile");
    static_assert(EARLY <= PA && 2 * NL <= KS, "prologue / direct loads inside the K loop");
    constexpr int OFF_R = DA * TILE;
    constexpr int OFF_L = 6 * TILE;             // statistics records of the tiles in the A ring, 1 KB each
    constexpr int OFF_S = OFF_L + (HAS_LN ? DA * 1024 : 0);   // HAS_STAT: two buffers of 8 x 32 partial sums, 16 B each
    static_assert(!(HAS_LN && HAS_BIAS), "with HAS_LN the bias is part of the column records");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int g = slot % groups;                     // column group
    const int p = xcd + 8 * (slot / groups);         // position among the P workgroups of the group
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- the stationary operand: fragment (j, s) of this wave's strip of W, s < KA in accumulation registers.
    // Given a copy of W in fragment order (vtdge_linear_prepack: 64 lanes x 16 B per fragment, contiguous), the
    // registers are loaded straight from it, first thing: nothing here depends on the row count.
    u32x4 wfa[NB][KA], wfv[NB][KS - KA];
    if (Wp != nullptr) {
        const u32x4 *wp = Wp + ((size_t)(g * 4 + w) * (NB * KS)) * 64 + lane;
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const u32x4 v = wp[(j * KS + s) * 64];
                if (s < KA) wfa[j][s] = v;
                else wfv[j][s - KA] = v;
            }
    }

    const int64_t M = live_rows(rows_dev, rows);
    const int tiles_m = (int)((M + 31) / 32);
    const int nt = tiles_m > p ? (tiles_m - p + P - 1) / P : 0;
    if (nt == 0) return;

    const int M32 = (int)M;
    const int lr = lane & 31, lg = lane >> 5;
    const int col0 = g * BN + w * STRIP;             // first output column of this wave

    // ---- constant MFMA operands
    // bias: one more K step whose W-side fragment holds bias[col] at k = 0 and whose A-side fragment is 1 at k = 0;
    // residual: K steps whose W-side fragment is a 16-column slice of the identity and whose A-side fragments are
    // read from the residual tile like fragments of A.  bf16 x 1 is exact, so the sum is (A W^T + bias) + residual,
    // each rounded once in fp32, as with separate additions.
    uint32_t wb[NB];
    u32x4 wl[NB];         // HAS_LN: the column records, W-side fragments of the statistics K step
    u32x4 eye[2];
    {
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < NB; j++) {
            wb[j] = 0u;
            if constexpr (HAS_BIAS) wb[j] = lg == 0 ? (uint32_t)bias[col0 + j * 32 + lr] : 0u;
            wl[j] = z;
            if constexpr (HAS_LN) wl[j] = lnw[(col0 + j * 32 + lr) * 2 + lg];
        }
#pragma unroll
        for (int h = 0; h < 2; h++) {
            eye[h] = z;
            if constexpr (HAS_RES) {
                // element e of lane (lr, lg) is k = 8*lg + e of W-side row lr: 1 where 16*h + k == lr
                const bool mine = (lr >> 4) == h && lg == ((lr & 15) >> 3);
                const uint32_t one = 0x3f80u << (16 * (lr & 1));
                const int wd = (lr & 7) >> 1;
                eye[h].x = mine && wd == 0 ? one : 0u;
                eye[h].y = mine && wd == 1 ? one : 0u;
                eye[h].z = mine && wd == 2 ? one : 0u;
                eye[h].w = mine && wd == 3 ? one : 0u;
            }
        }
    }

    // ---- per-lane constants
    // fragment reads: row lr of the tile, 16-byte chunk (2c + lg) of a 128-byte slab, slot-swizzled; cs[c] = cs[0] ^ 32c
    int cs[4];
#pragma unroll
    for (int c = 0; c < 4; c++) cs[c] = lr * 128 + (((2 * c + lg) ^ ((lr >> 1) & 7)) * 16);
    // direct loads of a 32-row tile (A, a W block, the residual): instruction i = w*NL + ii covers slab i/4 and rows
    // (i%4)*8 + lane/8; the lane fetches chunk (lane%8) ^ ((row/2)%8) = ((lane%8) ^ (lane/16)) ^ 4*(i%2).
    // Everything that depends on i is wave-uniform: byte offset = uniform part + one of two lane constants.
    const int l8 = lane >> 3;
    const int ax16 = ((lane & 7) ^ (lane >> 4)) * 16;
    const uint32_t lda2 = (uint32_t)lda * 2, ldr2 = (uint32_t)ldr * 2, ldo2 = (uint32_t)ldo * 2;   // row pitches, bytes
    const uint32_t va[2] = {l8 * lda2 + ax16, l8 * lda2 + (ax16 ^ 64)};
    const uint32_t vr[2] = {l8 * ldr2 + ax16, l8 * ldr2 + (ax16 ^ 64)};
    // First row of this workgroup's k-th tile.  The last tile of the matrix is moved back so that it ends at row M
    // (its first rows repeat rows of the tile before, recomputed bit for bit), so no tile but a lone first one
    // (M < 32) reaches past the end.
    const int m_last = M32 > 32 ? M32 - 32 : 0;
    auto tile_row0 = [&](int k) -> int { const int m = (p + k * P) * 32; return m < m_last ? m : m_last; };
    // one direct load of tile rows m0.. from `base` (row pitch `pitch`, `col` bytes into the row) to LDS `dst`;
    // ii = which of the wave's NL loads, par = ii % 2
    auto tile_dma = [&](const void *base, uint32_t pitch, uint32_t col, const uint32_t (&v)[2], int m0, int ii, int par,
                        uint32_t dst) {
        const int i = w * NL + ii;
        dma16(base, (uint32_t)(m0 + (i & 3) * 8) * pitch + col + (i >> 2) * 128 + v[par], dst + i * 1024);
    };
    // the same for a lone tile of fewer than 32 rows: rows past the end are clamped to the last one
    auto tile_dma_short = [&](const void *base, uint32_t pitch, uint32_t col, int ii, uint32_t dst) {
        const int i = w * NL + ii;
        int gm = (i & 3) * 8 + l8;
        gm = gm < M32 ? gm : M32 - 1;
        dma16(base, (uint32_t)gm * pitch + col + (i >> 2) * 128 + (ax16 ^ ((i & 1) * 64)), dst + i * 1024);
    };

    // tally of vector-memory operations issued by this wave and, per tile, the tally right after its loads
    int issued = 0;
    uint64_t marks_a = 0, marks_r = 0;
    auto set_mark = [](uint64_t &m, int k, int v) {
        const int sh = (k & 7) * 8;
        m = (m & ~(0xffull << sh)) | ((uint64_t)(v & 0xff) << sh);
    };
    auto after_mark = [&](uint64_t m, int k) -> int { return (issued - (int)((m >> ((k & 7) * 8)) & 0xff)) & 0xff; };
    // the statistics records of tile k's 32 rows (lane i: half i % 2 of row i / 2), wave 0 only
    auto rec_dma = [&](int k) {
        int gm = tile_row0(k) + (lane >> 1);
        gm = gm < M32 ? gm : M32 - 1;
        dma16(lnrec, (uint32_t)gm * 32u + (lane & 1) * 16u, lds0 + OFF_L + (k % DA) * 1024);
    };
    auto issue_a_all = [&](int k) {      // prologue only; inside the K loop the six loads are spread out
        if constexpr (HAS_LN) {
            if (w == 0) {
                rec_dma(k);
                issued += 1;
            }
        }
#pragma unroll
        for (int ii = 0; ii < NL; ii++) {
            if (M32 >= 32) tile_dma(A, lda2, 0, va, tile_row0(k), ii, ii & 1, lds0 + (k % DA) * TILE);
            else tile_dma_short(A, lda2, 0, ii, lds0 + (k % DA) * TILE);
        }
        issued += NL;
        set_mark(marks_a, k, issued);
    };

    // ---- the stationary operand: 12 blocks of 32 W rows (block 3 * wave + j holds wave's j-th column block) pass
    // through the six LDS slots.  Pass j brings every wave its j-th block, so all four waves read at once; the
    // loads of the next pass are in flight meanwhile (slots: pass 0 -> 0..3; pass 1 -> 4, 5, 0, 1;
    // pass 2 -> 2, 3, 4, 5), and the first two tiles of A follow into slots 0 and 1 as soon as those are free.
    if (Wp != nullptr) {
        // the registers are being loaded from the packed copy: LDS is free and the first tiles of A go out at once
#pragma unroll
        for (int k = 0; k < EARLY; k++)
            if (k < nt) issue_a_all(k);
    } else {
        // Every workgroup of a column group reads the same 288 KB, and the workgroups of an XCD would walk them in
        // step, all on the same few L2 channels at any moment: each starts its walk somewhere else.
        const int rot = slot % NL, rot4 = (slot / NL) & 3;
        auto issue_w = [&](int wave, int j, int lds_slot) {   // this wave's share (NL loads) of block (wave, j)
            const uint32_t src = (uint32_t)(g * BN + (wave * NB + j) * 32) * KB;
            const uint32_t dst = lds0 + lds_slot * TILE;
#pragma unroll
            for (int ii = 0; ii < NL; ii++) {
                int i2 = ii + rot;
                i2 = i2 >= NL ? i2 - NL : i2;
                const int i = w * NL + i2;
                dma16(Wt, src + ((i & 3) * 8 + l8) * KB + (i >> 2) * 128 + (ax16 ^ ((i & 1) * 64)), dst + i * 1024);
            }
        };
        auto read_w = [&](int j, int slot) {
            const unsigned char *base = smem + slot * TILE;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(base + (s >> 2) * 4096 + cs[s & 3]);
                if (s < KA) wfa[j][s] = v;
                else wfv[j][s - KA] = v;
            }
        };
#pragma unroll
        for (int v = 0; v < 4; v++) issue_w((v + rot4) & 3, 0, (v + rot4) & 3);
        issue_w(0, 1, 4);
        issue_w(1, 1, 5);
        wait_vmcnt<2 * NL>();                  // pass 0 has landed
        lds_barrier();
        // the bias values are consumed here as far as the compiler is concerned: their loads are issued above and
        // waited for now, not next to their first real use in the middle of the pipeline
#pragma unroll
        for (int j = 0; j < NB; j++) asm volatile("" : "+v"(wb[j]));
        read_w(0, w);
        lds_barrier();                       // slots 0..3 are free
        issue_w(2, 1, 0);
        issue_w(3, 1, 1);
        issue_w(0, 2, 2);
        issue_w(1, 2, 3);
        wait_vmcnt<2 * NL>();                  // pass 1 has landed
        lds_barrier();
        read_w(1, w < 2 ? 4 + w : w - 2);
        lds_barrier();                       // slots 4, 5, 0, 1 are free
        issue_w(2, 2, 4);
        issue_w(3, 2, 5);
#pragma unroll
        for (int k = 0; k < EARLY; k++)
            if (k < nt) issue_a_all(k);
        wait_vmcnt_dyn(issued);                // pass 2 has landed (all but the tiles of A)
        lds_barrier();
        read_w(2, 2 + w);
        lds_barrier();                       // slots 2..5 are free
    }
    // ---- rest of the prologue: first residual tiles, remaining first tiles of A
    if constexpr (HAS_RES) {
#pragma unroll
        for (int k = 0; k < PR; k++) {
            if (k < nt) {
#pragma unroll
                for (int ii = 0; ii < NL; ii++) {
                    if (M32 >= 32) tile_dma(res, ldr2, g * KB, vr, tile_row0(k), ii, ii & 1, lds0 + OFF_R + k * TILE);
                    else tile_dma_short(res, ldr2, g * KB, ii, lds0 + OFF_R + k * TILE);
                }
                issued += NL;
                set_mark(marks_r, k, issued);
            }
        }
    }
#pragma unroll
    for (int k = EARLY; k < PA; k++)
        if (k < nt) issue_a_all(k);
    f32x16 acc[2][NB];
    u32x4 fa[FD + 1];

    // ---- epilogue of one tile, in NU units.  Unit n = 4 * (2j + q) + e turns the accumulator pair
    // (8q + e, 8q + 4 + e) of block j into elements e and 4 + e of the lane's 8-column vector (j, q).
    uint32_t e_w[4];        // packed pairs of the current vector
    float rs_prev = 1.0f;   // HAS_LN: rstd of the lane's row in the tile whose epilogue is due
    float st_p = 0.f, st_a = 0.f, st_q = 0.f;   // HAS_STAT: pivot, sum and sum of squares about it (48 elements)
    float h0, h1;           // elements of an even unit waiting for their odd neighbours
    EpiUnit un;
    auto epi_part1 = [&](auto pp_tag, int n) {
        constexpr int PP = decltype(pp_tag)::value;
        const int j = n / 8, q = (n / 4) % 2, e = n % 4;
        auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[PP][j][8 * q + e]),
                                                  __float_as_uint(acc[PP][j][8 * q + 4 + e]), false, false);
        un.f0 = __uint_as_float(r[0]);
        un.f1 = __uint_as_float(r[1]);
        if constexpr (HAS_LN) {
            un.f0 *= rs_prev;
            un.f1 *= rs_prev;
        }
        if constexpr (ACT == VTDGE_ACT_GELU) gelu_part1(un);
    };
    auto epi_part2 = [&](int n) {
        if constexpr (ACT == VTDGE_ACT_GELU) gelu_part2(un);
        if constexpr (HAS_STAT && ACT == VTDGE_ACT_NONE) {
            if (n == 0) {
                st_p = un.f0;
                st_a = st_q = 0.f;
            }
            const float d0 = un.f0 - st_p, d1 = un.f1 - st_p;
            st_a += d0;
            st_q = fmaf(d0, d0, st_q);
            st_a += d1;
            st_q = fmaf(d1, d1, st_q);
        }
    };
    // the lane's partial sums of tile t go to LDS ...
    auto stat_put = [&](int t) {
        const u32x4 v = {__float_as_uint(st_p), __float_as_uint(st_a), __float_as_uint(st_q), 0u};
        *reinterpret_cast<u32x4 *>(smem + OFF_S + (t & 1) * 4096 + ((w * 2 + lg) * 32 + lr) * 16) = v;
    };
    // ... and, once every wave's are there (a barrier later), become the records of the tile's rows: wave w merges rows
    // 8w .. 8w+7, lane l < 16 writing half l % 2 of row 8w + l / 2
    auto stat_finish = [&](int t) {
        const int row = w * 8 + ((lane >> 1) & 7);
        const unsigned char *pb = smem + OFF_S + (t & 1) * 4096 + row * 16;
        float mi[8], m2 = 0.f, ms = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const u32x4 pv = *reinterpret_cast<const u32x4 *>(pb + i * 512);
            const float a = __uint_as_float(pv.y) * (1.0f / 48.0f);
            mi[i] = __uint_as_float(pv.x) + a;
            m2 += __uint_as_float(pv.z) - __uint_as_float(pv.y) * a;
            ms += mi[i];
        }
        const float mean = ms * 0.125f;
        float dev = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) dev = fmaf(mi[i] - mean, mi[i] - mean, dev);
        const float var = fmaxf((m2 + 48.0f * dev) * (1.0f / 384.0f), 0.f);
        u32x4 lo, hi;
        ln_record(mean, sqrtf(var + stat_eps), lo, hi);
        int gm = tile_row0(t) + row;
        gm = gm < M32 ? gm : M32 - 1;
        if (lane < 16) stat_out[(int64_t)gm * 2 + (lane & 1)] = (lane & 1) ? hi : lo;
        issued += 1;
    };
    auto epi_part3 = [&](int n, unsigned char *orow) {
        const int j = n / 8, q = (n / 4) % 2, e = n % 4;
        if constexpr (ACT == VTDGE_ACT_GELU) gelu_part3(un);
        if (e % 2 == 0) {
            h0 = un.f0;
            h1 = un.f1;
        } else {
            e_w[e / 2] = pack_bf16x2(h0, un.f0);        // elements e-1, e
            e_w[2 + e / 2] = pack_bf16x2(h1, un.f1);    // elements 4+e-1, 4+e
        }
        if (e == 3) {
            u32x4 v;
            v.x = e_w[0]; v.y = e_w[1]; v.z = e_w[2]; v.w = e_w[3];
            *reinterpret_cast<u32x4 *>(orow + (j * 32 + 8 * 2 * q) * 2) = v;
        }
    };
    auto out_row = [&](int k) -> unsigned char * {
        int gm = tile_row0(k) + lr;
        gm = gm < M32 ? gm : M32 - 1;
        return reinterpret_cast<unsigned char *>(out) + (uint64_t)(uint32_t)gm * ldo2 + (col0 + 8 * lg) * 2;
    };

    // wait until this wave's loads of what step k needs have landed: A(k+1) (its first fragments are read at the
    // end of step k), or A(k) and the residual of tile k
    auto wait_step = [&](int k) {
        int after = 255;
        if constexpr (XT) {
            if (k + 1 < nt) after = after_mark(marks_a, k + 1);
        } else {
            after = after_mark(marks_a, k);
        }
        if constexpr (HAS_RES) {
            const int ar = after_mark(marks_r, k);
            after = ar < after ? ar : after;
        }
        if (after != 255) wait_vmcnt_dyn(after);
    };

    // ---- one tile: multiplies A(k) into acc[PP]; when EPI, finishes tile k-1 (in acc[1-PP]) on the way.
    auto tile_step = [&](auto pp_tag, auto epi_tag, int k) {
        constexpr int PP = decltype(pp_tag)::value;
        constexpr bool EPI = decltype(epi_tag)::value;
        using PQ = std::integral_constant<int, 1 - PP>;
        const bool more = k + 1 < nt;
        wait_step(k);
        if constexpr (HAS_STAT) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the partial sums put last step
        block_barrier();   // what was awaited is in LDS for every wave; the slots read last step are free
        if constexpr (HAS_STAT) {
            if (k >= 2) stat_finish(k - 2);
        }

        // Direct loads of this step: the residual of tile k+PR and A(k+PA), six each per wave.  The waves take turns
        // (wave w issues in substeps 6w .. 6w+5: load number s of each tile in substep s, the residual's first), so
        // the loads of different waves do not queue behind each other at the address unit.  Stores (when EPI) follow
        // the MFMAs of substeps 3, 7, .., 23.  The tallies count, for this wave, what is issued up to the last load
        // of each tile.
        const bool has_a = k + PA < nt;
        const bool has_r = HAS_RES && k + PR < nt;
        const int w6 = w * NL;
        const uint32_t mask_a = has_a ? 0x3fu << w6 : 0u, mask_r = has_r ? 0x3fu << w6 : 0u;
        // wave 0 also brings the statistics records of tile k+PA: in its last substep, between the residual's load
        // and A's
        const bool has_l = HAS_LN && has_a && w == 0;
        {
            const int start = issued, n = (has_a ? 1 : 0) + (has_r ? 1 : 0), x = has_l ? 1 : 0;
            const int st = EPI ? (w6 + 1) / 4 + 1 : 0;        // stores before the loads of substep 6w+5
            if (has_r) set_mark(marks_r, k + PR, start + (NL - 1) * n + 1 + st);
            if (has_a) set_mark(marks_a, k + PA, start + NL * n + x + st);
            issued = start + NL * n + x + (EPI ? NB * 2 : 0);
        }
        const uint32_t dst_a = lds0 + ((k + PA) % DA) * TILE, dst_r = lds0 + OFF_R + ((k + PR) % DR) * TILE;
        const uint32_t sa = (uint32_t)tile_row0(k + PA) * lda2, sr = (uint32_t)tile_row0(k + PR) * ldr2 + g * KB;
        auto step_dma = [&](int s) {      // s is a compile-time constant at every call
            if constexpr (HAS_RES) {
                if ((mask_r >> s) & 1) dma16(res, sr + (s & 3) * 8 * ldr2 + (s >> 2) * 128 + vr[s & 1], dst_r + s * 1024);
            }
            if constexpr (HAS_LN) {
                if (s == NL - 1 && has_l) rec_dma(k + PA);
            }
            if ((mask_a >> s) & 1) dma16(A, sa + (s & 3) * 8 * lda2 + (s >> 2) * 128 + va[s & 1], dst_a + s * 1024);
        };

        // fragment addresses of this step: only cs[0] is kept between steps
        const int cs0 = fresh(cs[0]);
        const int csl[4] = {cs0, cs0 ^ 32, cs0 ^ 64, cs0 ^ 96};
        const unsigned char *at = smem + (k % DA) * TILE;
        const unsigned char *an = smem + ((k + 1) % DA) * TILE;
        unsigned char *orow = nullptr;
        if constexpr (EPI) orow = out_row(k - 1);
        u32x4 fl = {0u, 0u, 0u, 0u};
        float rs_cur = 1.0f;
        if constexpr (HAS_LN) {
            fl = *reinterpret_cast<const u32x4 *>(smem + OFF_L + (k % DA) * 1024 + lr * 32 + lg * 16);
            const uint32_t sg = lg ? fl.x : fl.w;      // (sigma_1, sigma_2) sits in both halves of the record
            rs_cur = __builtin_amdgcn_rcpf(__uint_as_float(sg << 16) + __uint_as_float(sg & 0xffff0000u));
        }
        // residual fragments: K steps 6w .. 6w+5 of the residual tile, through a ring of four registers sets
        u32x4 fr[4];
        auto read_fr = [&](int i) {            // i-th fragment in the order the MFMAs take them
            const int t = w * 2 * NB + (i % NB) * 2 + i / NB;
            fr[i % 4] = *reinterpret_cast<const u32x4 *>(smem + OFF_R + (k % DR) * TILE + (t >> 2) * 4096 +
                                                          (cs0 ^ ((t & 3) * 32)));
        };
        if constexpr (!XT) {
#pragma unroll
            for (int s = 0; s < FD; s++) fa[s] = *reinterpret_cast<const u32x4 *>(at + (s >> 2) * 4096 + csl[s & 3]);
        }
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const u32x4 &f = fa[s % (FD + 1)];
#pragma unroll
            for (int j = 0; j < NB; j++) {
                if (s == 0) mma_az(acc[PP][j], wfa[j][0], f);
                else if (s < KA) mma_a(acc[PP][j], wfa[j][s], f);
                else mma_v(acc[PP][j], wfv[j][s - KA], f);
                // behind every MFMA a few other instructions, which issue while it runs
                if (j == 0) {
                    // the fragment of A for substep s + FD (the next tile's when this one has no more)
                    if (s + FD < KS)
                        fa[(s + FD) % (FD + 1)] =
                            *reinterpret_cast<const u32x4 *>(at + ((s + FD) >> 2) * 4096 + csl[(s + FD) & 3]);
                    else if (XT && more)
                        fa[(s + FD) % (FD + 1)] =
                            *reinterpret_cast<const u32x4 *>(an + ((s + FD - KS) >> 2) * 4096 + csl[(s + FD - KS) & 3]);
                    if constexpr (HAS_RES) {
                        if (s >= KS - 2) read_fr(s - (KS - 2));    // the first two residual fragments
                    }
                    if constexpr (EPI) epi_part1(PQ{}, s);
                }
                if (j == 1) {
                    step_dma(s);
                    if constexpr (EPI) epi_part2(s);
                }
                if (j == 2) {
                    if constexpr (EPI) {
                        epi_part3(s, orow);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (HAS_STAT && EPI) stat_put(k - 1);
        if constexpr (HAS_LN) {
#pragma unroll
            for (int j = 0; j < NB; j++) mma_v_fresh(acc[PP][j], wl[j], fl);
            rs_prev = rs_cur;       // for this tile's epilogue, which runs during the next step
        }
        if constexpr (HAS_BIAS) {
            const u32x4 ones = {fresh(lane) < 32 ? 0x3f80u : 0u, 0u, 0u, 0u};   // made here: no registers held
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const u32x4 wbj = {wb[j], 0u, 0u, 0u};
                mma_v_fresh(acc[PP][j], wbj, ones);
            }
        }
        if constexpr (HAS_RES) {
            // in the order 0, 2, 4, 1, 3, 5 of K steps, so that consecutive MFMAs go to different accumulators
            read_fr(2);
            read_fr(3);
#pragma unroll
            for (int i = 0; i < 2 * NB; i++) {
                const int kk = (i % NB) * 2 + i / NB;
                __builtin_amdgcn_sched_barrier(0);
                mma_v(acc[PP][kk / 2], eye[kk % 2], fr[i % 4]);
                if (i < 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    read_fr(i + 4);
                }
            }
        }
    };

    if constexpr (XT) {
        // first tile: its own wait, and its first fragments
        wait_vmcnt_dyn(after_mark(marks_a, 0));
        block_barrier();
#pragma unroll
        for (int s = 0; s < FD; s++) fa[s] = *reinterpret_cast<const u32x4 *>(smem + (s >> 2) * 4096 + cs[s & 3]);
    }
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    tile_step(I0{}, std::false_type{}, 0);
    int k = 1;
    for (; k + 1 < nt; k += 2) {
        tile_step(I1{}, std::true_type{}, k);
        tile_step(I0{}, std::true_type{}, k + 1);
    }
    if (k < nt) tile_step(I1{}, std::true_type{}, k);
    // ---- last tile's epilogue
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs' results must have reached the registers
    unsigned char *orow = out_row(nt - 1);
    if ((nt - 1) & 1) {
#pragma unroll
        for (int j = 0; j < NB; j++) acc[0][j] = acc[1][j];
    }
#pragma unroll
    for (int n = 0; n < NU; n++) {
        epi_part1(I0{}, n);
        epi_part2(n);
        epi_part3(n, orow);
    }
    if constexpr (HAS_STAT) {
        stat_put(nt - 1);
        lds_barrier();          // the sums of the last two tiles are in LDS for every wave
        if (nt >= 2) stat_finish(nt - 2);
        stat_finish(nt - 1);
    }
}

// ----------------------------------------------------------------------------- host
bool linear_ws_applicable(int64_t lda, int64_t ldr, int64_t ldo, int64_t rows, int N, int K, int esz, int act,
                          const void *bias, const void *res, const void *out)
{
    // the residual is added inside the accumulator, i.e. before an activation: such a pair goes elsewhere
    if (res != nullptr && act != VTDGE_ACT_NONE) return false;
    return esz == 2 && K == 384 && lda < (1ll << 31) && ldo < (1ll << 31) && ldr < (1ll << 31) && N % 384 == 0 &&
           N / 384 <= 8 && rows >= 2048 && rows * lda < (1ll << 31) && (res == nullptr || rows * ldr < (1ll << 31)) &&
           lda % 8 == 0 && ldo % 8 == 0 && (res == nullptr || ldr % 8 == 0) &&
           (((uintptr_t)bias | (uintptr_t)res | (uintptr_t)out) & 15) == 0;
}

template <int ACT, bool HB, bool HR, bool LN = false, bool STAT = false>
static int go_ws(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                 int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, hipStream_t st,
                 const void *lnrec = nullptr, const void *lnw = nullptr, void *stat_out = nullptr, float stat_eps = 0.f)
{
    constexpr int KS = 24, NB = 3;
    // six 32-row tiles (+ four tiles' records) (+ two buffers of partial sums)
    constexpr size_t lds = (size_t)6 * 32 * KS * 32 + (LN ? 4 * 1024 : 0) + (STAT ? 2 * 4096 : 0);
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = linear_ws_kernel<KS, NB, ACT, HB, HR, LN, STAT>;
    VT_RESERVE_LDS(kern, lds, "linear");
    const int groups = N / (4 * NB * 32);
    // one workgroup per CU; the P workgroups of a column group are spread over the 8 XCDs, and the workgroups
    // that share A tiles (same position in different groups) sit on the same XCD
    int P = (256 / groups) & ~7;
    const int64_t tiles_m = ceil_div(rows, 32);
    if (P > tiles_m) P = (int)((tiles_m + 7) & ~7);
    dim3 grid((unsigned)(P * groups)), block(256);
    kern<<<grid, block, lds, st>>>((const bf16_t *)A, lda, (const bf16_t *)W, (const bf16_t *)bias, (const bf16_t *)res,
                                   ldr, (bf16_t *)out, ldo, rows_dev, rows, groups, P, (const u32x4 *)Wp,
                                   (const u32x4 *)lnrec, (const u32x4 *)lnw, (u32x4 *)stat_out, stat_eps);
    return check_launch("linear");
}

// out = A W^T + bias + residual for N = 384, with the statistics records of the rows of out
int launch_linear_ws_stats(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                           int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows,
                           void *records, float eps, hipStream_t st)
{
    const bool hb = bias != nullptr, hr = res != nullptr;
#define VT_WS(HB, HR)                                                                                               \
    return go_ws<VTDGE_ACT_NONE, HB, HR, false, true>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, 384, st, \
                                                      nullptr, nullptr, records, eps)
    if (hb && hr) VT_WS(true, true);
    if (hb) VT_WS(true, false);
    if (hr) VT_WS(false, true);
    VT_WS(false, false);
#undef VT_WS
}

// out = act(LayerNorm(A) W^T + bias) from the raw rows, their statistics records and the folded weights
int launch_linear_ws_ln(const void *A, int64_t lda, const void *lnrec, const void *Wf, const void *Wfp,
                        const void *lnw, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int act,
                        hipStream_t st)
{
    if (act == VTDGE_ACT_GELU)
        return go_ws<VTDGE_ACT_GELU, false, false, true>(A, lda, Wf, Wfp, nullptr, nullptr, 0, out, ldo, rows_dev, rows,
                                                          N, st, lnrec, lnw);
    return go_ws<VTDGE_ACT_NONE, false, false, true>(A, lda, Wf, Wfp, nullptr, nullptr, 0, out, ldo, rows_dev, rows, N,
                                                      st, lnrec, lnw);
}

int launch_linear_ws(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                     int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int act,
                     hipStream_t st)
{
    const bool hb = bias != nullptr, hr = res != nullptr;
#define VT_WS(ACT, HB, HR) return go_ws<ACT, HB, HR>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st)
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

}  // namespace vtdge
