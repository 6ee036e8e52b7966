// Packed-M Linear for bf16 operands with a long K and a narrow output (K = 1536, N a multiple of 96: the second
// Linear of the MLP of the C = 384 models), weight-stationary with the K dimension split over the waves.
//
// W (N x 1536) is too large for the registers of one CU, and a narrow N leaves a streaming kernel too few tiles to
// fill the chip evenly.  Here a workgroup owns 96 output columns for its whole life and its four waves (one per
// SIMD) split K: wave w keeps W[96 columns][k in 384w .. 384w+383] in registers (72 fragments of the 16x16x32 MFMA:
// 288 registers, 240 of them accumulation registers, which the MFMA reads directly) and multiplies it with the
// same quarter of every 16-row tile of A.  A fragment of A then feeds six MFMAs and is read by one wave only: each
// wave streams its own quarter of the tiles HBM/L2 -> LDS by direct loads into a private ring of five half stages
// (16 rows x 384 B) and needs no barrier to consume it.  The four partial sums of a tile meet in LDS: every wave
// writes its 16 x 96 partials, and after a barrier each wave adds up two of the six 16-column blocks in a fixed
// order, adds bias and residual (the residual tile comes through a small LDS ring, each wave loading four of its
// rows), rounds once and stores: (A W^T + bias) + residual in fp32.  All of this is interleaved with the MFMAs of
// the next tile, which accumulate into a second register set: writes in its first half, reads in its second.
//
// Synchronisation: two barriers per tile, in the middle (the previous tile's partial sums are visible) and at the
// end (their readers are done).  Vector-memory operations retire in issue order and every tile issues the same
// ones in the same order (no load is conditional: tiles past the end are clamped into the matrix and loaded
// unused), so a wave waits for its own loads of the tile it starts with a constant s_waitcnt vmcnt.
// Direct loads and MFMAs are issued from inline assembly (the compiler then adds no vmcnt wait of its own before the LDS reads of the fragments, and the stationary fragments stay in the registers they were put in).
// The last tile of the matrix is moved back to end at row M, so no tile but a lone first one reaches past the end.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

namespace vtdge {

// D = W_frag * A_frag^T (+ D) on 16 x 16 x 32; the stationary fragment in accumulation (A) or vector (V) registers;
// Z starts a new sum.
__device__ __forceinline__ void mma16_a(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void mma16_v(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(wfrag), "v"(afrag));
}
__device__ __forceinline__ void mma16_az(f32x4 &d, const u32x4 &wfrag, const u32x4 &afrag)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=v"(d) : "a"(wfrag), "v"(afrag));
}
template <bool HAS_BIAS, bool HAS_RES>
__global__ __launch_bounds__(256) void linear_ks_kernel(
    const bf16_t *__restrict__ A, int64_t lda, const bf16_t *__restrict__ Wt, const bf16_t *__restrict__ bias,
    const bf16_t *__restrict__ res, int64_t ldr, bf16_t *__restrict__ out, int64_t ldo,
    const int64_t *__restrict__ rows_dev, int64_t rows, int groups, int P, const u32x4 *__restrict__ Wp)
{
    constexpr int KQ = 768;                  // bytes of a wave's K quarter of a row
    constexpr int KROW = 4 * KQ;             // bytes of a row of W
    constexpr int CB = 6;                    // 16-column blocks per workgroup
    constexpr int BN = CB * 16;
    constexpr int KS = KQ / 64;              // K steps (of 32) per wave and tile: 12
    constexpr int KA = 10;                   // K steps whose W fragments live in accumulation registers
    constexpr int HS = 16 * KQ / 2;          // bytes of a half stage: 16 rows x 384 B = 3 slabs of 2 KB
    constexpr int DH = 5;                    // half stages in a wave's ring
    constexpr int RING = DH * HS;
    constexpr int OFF_X = 4 * RING;          // partial sums: [4 waves][CB blocks][64 lanes x 16 B]
    constexpr int OFF_R = OFF_X + 4 * CB * 1024;   // residual ring: 3 tiles of [16 rows][256 B]
    constexpr int WTILE = 32 * KQ;           // a W staging block: 32 rows x 768 B
    constexpr int FD = 3;                    // fragments of A are read FD K steps ahead of their MFMAs
    static_assert(OFF_R + 3 * 4096 <= 160 * 1024 && 6 * WTILE <= OFF_R + 3 * 4096, "LDS budget");
    static_assert(KS == 12 && HS == 6144 && KS % (FD + 1) == 0, "geometry");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int g = slot % groups;                     // column group
    const int p = xcd + 8 * (slot / groups);         // position among the P workgroups of the group
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15, kg = lane >> 4;

    // ---- the stationary operand: fragment (cb, ks) = rows 16cb.. of the strip, K step ks of this wave's quarter,
    // ks < KA in accumulation registers.  Given a copy of W in fragment order (vtdge_linear_prepack: 64 lanes x
    // 16 B per fragment, contiguous), the registers are loaded straight from it, first thing: nothing here depends
    // on the row count.
    u32x4 wfa[CB][KA], wfv[CB][KS - KA];
    if (Wp != nullptr) {
        const u32x4 *wp = Wp + ((size_t)(g * 4 + w) * (CB * KS)) * 64 + lane;
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const u32x4 v = wp[(cb * KS + ks) * 64];
                if (ks < KA) wfa[cb][ks] = v;
                else wfv[cb][ks - KA] = v;
            }
    }

    const int64_t M = live_rows(rows_dev, rows);
    const int M32 = (int)M;
    const int tiles_m = (M32 + 15) / 16;
    const int nt = tiles_m > p ? (tiles_m - p + P - 1) / P : 0;
    if (nt == 0) return;

    // ---- per-lane constants
    // fragment reads (16 rows x 4 chunks of a 128-byte slab): row c16, chunk (4p + kg) ^ ((c16/2)%8), p = K step % 2
    const int cs16 = c16 * 128 + ((kg ^ ((c16 >> 1) & 7)) * 16);
    // direct loads of 8 rows x 128 B: the lane fetches chunk (lane%8) ^ ((row/2)%8) of row lane/8 (+8 for odd i)
    const int l8 = lane >> 3;
    const int ax16 = ((lane & 7) ^ (lane >> 4)) * 16;
    const uint32_t lda2 = (uint32_t)lda * 2, ldr2 = (uint32_t)ldr * 2, ldo2 = (uint32_t)ldo * 2;
    const int m_last = M32 > 16 ? M32 - 16 : 0;
    auto tile_row0 = [&](int k) -> int { const int m = (p + k * P) * 16; return m < m_last ? m : m_last; };
    const uint32_t ring0 = lds0 + w * RING;
    const unsigned char *A8 = reinterpret_cast<const unsigned char *>(A);
    const unsigned char *R8 = reinterpret_cast<const unsigned char *>(res);

    // Direct loads of A.  Per lane and for the whole kernel: the byte offset of its 16 bytes inside a tile, for the
    // even (rows 0..7) and odd (rows 8..15) instructions; rows past the end of a lone short tile are clamped to the
    // last one.  Per tile: a wave-uniform base (tile row, this wave's K quarter).  Per instruction: an immediate
    // (the 128-byte slab), which the hardware adds to the LDS address as well: dma16_imm takes it off again.
    uint32_t voa[2][2];      // [K half of the tile][even / odd instruction]
#pragma unroll
    for (int e = 0; e < 2; e++) {
        int r = e * 8 + l8;
        r = r < M32 ? r : M32 - 1;
        voa[0][e] = (uint32_t)r * lda2 + (ax16 ^ (e * 64));
        voa[1][e] = voa[0][e] + KQ / 2;
    }
    auto a_base = [&](int k) -> const unsigned char * { return A8 + (uint32_t)tile_row0(k) * lda2 + w * KQ; };
    // Direct loads of a residual tile: [16 rows][256 B], chunk slots XOR-swizzled with the row; wave w brings rows
    // 4w .. 4w+3, slot lane%16 (slots whose chunk lies past the 12 real ones re-read the last one and are never
    // used)
    uint32_t vor = 0;
    if constexpr (HAS_RES) {
        const int row = w * 4 + (lane >> 4);
        int gc = (lane & 15) ^ row;
        gc = gc < 2 * CB ? gc : 2 * CB - 1;
        const int r = row < M32 ? row : M32 - 1;
        vor = (uint32_t)r * ldr2 + gc * 16;
    }
    auto r_base = [&](int k) -> const unsigned char * { return R8 + (uint32_t)tile_row0(k) * ldr2 + g * (BN * 2); };
    auto wrap5 = [](int x) -> int { return x >= RING ? x - RING : x; };          // ring of DH half stages
    auto wrap3 = [](int x) -> int { return x >= 3 * 4096 ? x - 3 * 4096 : x; };  // ring of 3 residual tiles

    // ---- without a packed copy: 12 blocks of 32 W rows x 768 B (block (v, j): rows 32j.. of the strip, K quarter
    // v) pass through six 24 KB slots; pass j brings every wave its j-th block (slots: pass 0 -> 0..3;
    // pass 1 -> 4, 5, 0, 1; pass 2 -> 2, 3, 4, 5)
    if (Wp == nullptr) {
        auto issue_w = [&](int v, int j, int lds_slot) {   // this wave's share (6 loads) of block (v, j)
            const uint32_t src = (uint32_t)(g * BN + j * 32) * KROW + v * KQ;
            const uint32_t dst = lds0 + lds_slot * WTILE;
#pragma unroll
            for (int ii = 0; ii < 6; ii++) {
                const int i = w * 6 + ii;
                dma16(Wt, src + ((i & 3) * 8 + l8) * KROW + (i >> 2) * 128 + (ax16 ^ ((i & 1) * 64)), dst + i * 1024);
            }
        };
        auto read_w = [&](int j, int lds_slot) {
            const unsigned char *base = smem + lds_slot * WTILE;
#pragma unroll
            for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    const u32x4 v =
                        *reinterpret_cast<const u32x4 *>(base + (ks >> 1) * 4096 + h2 * 2048 + (cs16 ^ ((ks & 1) * 64)));
                    if (ks < KA) wfa[2 * j + h2][ks] = v;
                    else wfv[2 * j + h2][ks - KA] = v;
                }
        };
#pragma unroll
        for (int v = 0; v < 4; v++) issue_w(v, 0, v);
        issue_w(0, 1, 4);
        issue_w(1, 1, 5);
        wait_vmcnt<12>();                      // pass 0 has landed
        lds_barrier();
        read_w(0, w);
        lds_barrier();                       // slots 0..3 are free
        issue_w(2, 1, 0);
        issue_w(3, 1, 1);
        issue_w(0, 2, 2);
        issue_w(1, 2, 3);
        wait_vmcnt<12>();                      // pass 1 has landed
        lds_barrier();
        read_w(1, w < 2 ? 4 + w : w - 2);
        lds_barrier();                       // slots 4, 5, 0, 1 are free
        issue_w(2, 2, 4);
        issue_w(3, 2, 5);
        wait_vmcnt<0>();
        lds_barrier();
        read_w(2, 2 + w);
        lds_barrier();                       // LDS is free
    }

    // ---- prologue: this wave's rows of residual tile 0, then half stages 0..3 (tiles 0, 1).  Tiles past this workgroup's
    // last one are loaded all the same (their rows are clamped into the matrix) and never used: no load in this
    // kernel is conditional, so the number of operations in flight at any point is known at compile time.
    if constexpr (HAS_RES) dma16(r_base(0), vor, lds0 + OFF_R + w * 1024);
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const unsigned char *ab = a_base(k);
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i = 0; i < 6; i++)
                dma16(ab, voa[h][i & 1] + (i >> 1) * 128, ring0 + (2 * k + h) * HS + i * 1024);
    }
    int hb = 0;      // ring offset of half stage 2k (tile k, first K half)
    int rs = 0;      // residual ring offset of tile k

    f32x4 acc[2][CB];
    u32x4 fa[FD + 1];

    // ---- reduction + epilogue of tile k: this wave adds up blocks w and 4 + w/2 (waves 2v and 2v+1 both finish
    // block 4 + v and store the same bytes), in the fixed order of the waves, then bias, then residual, in fp32,
    // and rounds once.  All of it rides on the MFMAs of the next tile: the partial sums are written in K steps
    // 0..2, block A is read (its residual too) in steps 6 and 7 and finished in step 9, block B in steps 8, 9, 11.
    const int blk[2] = {w, 4 + (w >> 1)};
    float bv[2][4];
    int rofs[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
        for (int e = 0; e < 4; e++)
            bv[j][e] = HAS_BIAS ? bf16_to_f32(bias[g * BN + blk[j] * 16 + 4 * kg + e]) : 0.f;
        // row c16 of the residual tile, chunk 2*block + kg/2 (swizzled with the row), half kg%2
        rofs[j] = c16 * 256 + (((2 * blk[j] + (kg >> 1)) ^ c16) * 16) + (kg & 1) * 8;
    }
    u32x4 px[2][4];
    u32x2 rr[2] = {{0u, 0u}, {0u, 0u}};
    unsigned char *orow = nullptr;
    int rs_red = 0;          // residual ring offset of the tile being reduced
    auto red_read = [&](int j, int v) {
        px[j][v] = *reinterpret_cast<const u32x4 *>(smem + OFF_X + (v * CB + blk[j]) * 1024 + lane * 16);
        if constexpr (HAS_RES) {
            if (v == 0) rr[j] = *reinterpret_cast<const u32x2 *>(smem + OFF_R + rs_red + rofs[j]);
        }
    };
    auto red_finish = [&](int j) {
        float f[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            f[e] = ((__uint_as_float(px[j][0][e]) + __uint_as_float(px[j][1][e])) + __uint_as_float(px[j][2][e])) +
                   __uint_as_float(px[j][3][e]);
            if constexpr (HAS_BIAS) f[e] += bv[j][e];
        }
        if constexpr (HAS_RES) {
            f[0] += bf16lo(rr[j].x);
            f[1] += bf16hi(rr[j].x);
            f[2] += bf16lo(rr[j].y);
            f[3] += bf16hi(rr[j].y);
        }
        u32x2 o;
        o.x = pack_bf16x2(f[0], f[1]);
        o.y = pack_bf16x2(f[2], f[3]);
        *reinterpret_cast<u32x2 *>(orow + blk[j] * 32) = o;
    };
    auto out_row = [&](int k) -> unsigned char * {
        int gm = tile_row0(k) + c16;
        gm = gm < M32 ? gm : M32 - 1;
        return reinterpret_cast<unsigned char *>(out) + (uint64_t)(uint32_t)gm * ldo2 + (g * BN + 4 * kg) * 2;
    };
    auto red_all = [&](int j) {
#pragma unroll
        for (int v = 0; v < 4; v++) red_read(j, v);
    };

    // ---- one tile: multiplies this wave's K quarter of A(k) into acc[PP]; when EPI, finishes tile k-1 on the way.
    // Vector-memory operations of a tile, in issue order: first this wave's rows of the residual of tile k+1, then
    // in K step s one load of half stage 2k+4 (s < 6) or 2k+5 (s >= 6), when EPI a store in steps 9 and 11: whatever
    // was issued before the last twelve of them belongs to tile k or before.
    auto tile_step = [&](auto pp_tag, auto epi_tag, int k) {
        constexpr int PP = decltype(pp_tag)::value;
        constexpr bool EPI = decltype(epi_tag)::value;
        wait_vmcnt<12>();                     // this wave's loads of tile k and of the residual of tile k have landed
        const int cs0 = fresh(cs16);
        const int o0 = hb, o1 = wrap5(hb + HS), o4 = wrap5(hb + 4 * HS);   // half stages 2k (and 2k+5), 2k+1, 2k+4
        hb = wrap5(hb + 2 * HS);
        rs_red = wrap3(rs + 2 * 4096);        // tile k-1
        rs = wrap3(rs + 4096);                // tile k+1
        const unsigned char *a_next = a_base(k + 2);
        if constexpr (HAS_RES) dma16(r_base(k + 1), vor, lds0 + OFF_R + rs + w * 1024);
        const unsigned char *at = smem + w * RING;
        auto frag = [&](int ks) -> const u32x4 * {      // address of fragment ks of this tile
            const int kk = ks % 6;
            return reinterpret_cast<const u32x4 *>(at + (ks < 6 ? o0 : o1) + (kk >> 1) * 2048 + (cs0 ^ ((kk & 1) * 64)));
        };
        if constexpr (EPI) orow = out_row(k - 1);
#pragma unroll
        for (int s = 0; s < FD; s++) fa[s] = *frag(s);
        static_for<KS>([&](auto s_tag) {
            constexpr int s = decltype(s_tag)::value;
            const u32x4 &f = fa[s % (FD + 1)];
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                if (s == 0) mma16_az(acc[PP][cb], wfa[cb][0], f);
                else if (s < KA) mma16_a(acc[PP][cb], wfa[cb][s < KA ? s : 0], f);
                else mma16_v(acc[PP][cb], wfv[cb][s >= KA ? s - KA : 0], f);
                // behind the MFMAs a few other instructions, which issue while they run
                if (cb == 0) {
                    if (s + FD < KS) fa[(s + FD) % (FD + 1)] = *frag(s + FD);
                }
                if (cb == 1) {
                    dma16_imm<((s % 6) >> 1) * 128>(a_next, voa[s / 6][s & 1], ring0 + (s < 6 ? o4 : o0) + (s % 6) * 1024);
                }
                if (cb == 3) {
                    if constexpr (EPI) {
                        // tile k-1: its partial sums go out in the first half of this tile and are added up in
                        // the second
                        if constexpr (s < CB / 2) {
                            *reinterpret_cast<f32x4 *>(smem + OFF_X + (w * CB + 2 * s) * 1024 + lane * 16) =
                                acc[PP ^ 1][2 * s];
                            *reinterpret_cast<f32x4 *>(smem + OFF_X + (w * CB + 2 * s + 1) * 1024 + lane * 16) =
                                acc[PP ^ 1][2 * s + 1];
                        }
                        if constexpr (s == 6) { red_read(0, 0); red_read(0, 1); }
                        if constexpr (s == 7) { red_read(0, 2); red_read(0, 3); }
                        if constexpr (s == 8) { red_read(1, 0); red_read(1, 1); }
                        if constexpr (s == 9) { red_finish(0); red_read(1, 2); red_read(1, 3); }
                        if constexpr (s == 11) red_finish(1);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (EPI && s == 5) {
                // LDS operations complete in order and three fragment reads were issued after the last write
                asm volatile("s_waitcnt lgkmcnt(3)" ::: "memory");
                block_barrier();                         // the partial sums of tile k-1 are visible
            }
        });
        if constexpr (EPI) block_barrier();              // every wave has read the partial sums of tile k-1
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    tile_step(I0{}, std::false_type{}, 0);
    int k = 1;
    for (; k + 1 < nt; k += 2) {
        tile_step(I1{}, std::true_type{}, k);
        tile_step(I0{}, std::true_type{}, k + 1);
    }
    if (k < nt) tile_step(I1{}, std::true_type{}, k);
    // ---- last tile's partial sums and reduction
    asm volatile("s_nop 15" ::: "memory");              // the last MFMAs' results have reached the registers
    if ((nt - 1) & 1) {
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
            *reinterpret_cast<f32x4 *>(smem + OFF_X + (w * CB + cb) * 1024 + lane * 16) = acc[1][cb];
    } else {
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
            *reinterpret_cast<f32x4 *>(smem + OFF_X + (w * CB + cb) * 1024 + lane * 16) = acc[0][cb];
    }
    lds_barrier();
    orow = out_row(nt - 1);
    rs_red = wrap3(rs + 2 * 4096);
    red_all(0);
    red_finish(0);
    red_all(1);
    red_finish(1);
    wait_vmcnt<0>();      // the loads issued for tiles past the last one must not outlive the workgroup's LDS
}

// ----------------------------------------------------------------------------- host
bool linear_ks_applicable(int64_t lda, int64_t ldr, int64_t ldo, int64_t rows, int N, int K, int esz, int act,
                          const void *bias, const void *res, const void *out)
{
    return esz == 2 && K == 1536 && act == VTDGE_ACT_NONE && N % 96 == 0 && N / 96 <= 8 && rows >= 2048 &&
           rows * lda < (1ll << 31) && (res == nullptr || rows * ldr < (1ll << 31)) && ldo < (1ll << 31) &&
           lda % 8 == 0 && ldo % 4 == 0 && (res == nullptr || ldr % 8 == 0) &&
           (((uintptr_t)res) & 15) == 0 && (((uintptr_t)out) & 7) == 0;
}

template <bool HB, bool HR>
static int go_ks(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                 int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, hipStream_t st)
{
    constexpr size_t lds = 4 * 5 * 6144 + 4 * 6 * 1024 + 3 * 4096;   // rings + partial sums + residual ring
    static_assert(lds <= 160 * 1024, "LDS budget");
    auto kern = linear_ks_kernel<HB, HR>;
    VT_RESERVE_LDS(kern, lds, "linear");
    const int groups = N / 96;
    int P = (256 / groups) & ~7;
    const int64_t tiles_m = ceil_div(rows, 16);
    if (P > tiles_m) P = (int)((tiles_m + 7) & ~7);
    dim3 grid((unsigned)(P * groups)), block(256);
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<grid, block, lds, st>>>((const bf16_t *)A, lda, (const bf16_t *)W, (const bf16_t *)bias, (const bf16_t *)res,
                                   ldr, (bf16_t *)out, ldo, rows_dev, rows, groups, P, (const u32x4 *)Wp);
    return check_launch("linear");
}

int launch_linear_ks(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                     int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, hipStream_t st)
{
    const bool hb = bias != nullptr, hr = res != nullptr;
    if (hb && hr) return go_ks<true, true>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st);
    if (hb) return go_ks<true, false>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st);
    if (hr) return go_ks<false, true>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st);
    return go_ks<false, false>(A, lda, W, Wp, bias, res, ldr, out, ldo, rows_dev, rows, N, st);
}

}  // namespace vtdge
