// Packed-M Linear, pipelined variant: operands go HBM/L2 -> LDS by direct loads
// (global_load_lds_dwordx4, no VGPR staging) into a 3-deep ring, so the loads of
// the next two stages are in flight while the MFMAs of the current one run.
//
// Geometry (bytes, shared by bf16 and fp32 -- see Slab<> in common.h):
//   stage   = (BM + BN) rows x 128 B of K;  row r of the stage lives at r*128 in LDS
//   chunk   = 16 B; a direct load writes 64 lanes x 16 B = 8 consecutive rows.
//   swizzle : LDS chunk slot c of row r holds K-chunk  c ^ ((r >> 1) & 7)  of that row,
//             which makes the 16-lane phases of the MFMA fragment reads
//             (32 rows x 16 B at one K offset) bank-conflict free without padding.
// The product is formed transposed (D = W_blk * A_blk^T): a lane then owns 4
// consecutive output columns of one row, and bias, GELU and residual are applied
// in fp32 on 16-byte vectors on the way out.
//
// Synchronisation: one raw s_barrier per K stage.  Before it every wave waits
// (s_waitcnt vmcnt) for its own direct loads of the stage about to be consumed;
// after it the ring slot consumed in the previous iteration is free for the next
// prefetch.  __syncthreads() is not used in the loop because its fence would also
// wait for the prefetches still in flight.  The epilogue stays in registers
// (a half-wave swap gives each lane 8 consecutive bf16 columns), so LDS holds
// nothing but the operand ring.
#include "common.h"
#include <stdlib.h>

namespace vtdge {

constexpr int DKB = 128;  // K bytes per stage

// GELU(x) = x * Phi(x).  fp32 keeps the exact erf form.  For bf16 outputs Phi is a degree-15 odd minimax
// polynomial on [-4, 4] (x clamped there): no transcendental, 11 VALU instructions; |error| <= 1.3e-4 for
// |x| <= 4 and <= 5.3e-5 * |x| beyond, i.e. below 1/30 of a bf16 rounding step of the result.
template <typename T> __device__ __forceinline__ float gelu_fn(float v);
template <> __device__ __forceinline__ float gelu_fn<float>(float v)
{
    return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
}
template <> __device__ __forceinline__ float gelu_fn<bf16_t>(float v)
{
    const float x = __builtin_amdgcn_fmed3f(v, -4.0f, 4.0f);
    const float t = x * x;
    float q = -1.580785487e-09f;
    q = q * t + 1.217110604e-07f;
    q = q * t - 4.100865225e-06f;
    q = q * t + 8.066737963e-05f;
    q = q * t - 1.048204291e-03f;
    q = q * t + 9.664873803e-03f;
    q = q * t - 6.617537860e-02f;
    q = q * t + 3.988475095e-01f;
    return v * (x * q + 0.5f);
}

// Persistent, wave-specialised kernel.  A workgroup = WGM*WGN MFMA waves + NWP loader waves.  It walks a static
// list of output tiles; the 3-deep operand ring keeps running across tile boundaries, so the first stages of the
// next tile are already in flight during the epilogue of the current one.  The loader waves issue nothing but
// the direct loads of stage g+2 (and block in the memory pipeline, which sustains ~46 B/clk per CU, while the
// MFMA waves keep multiplying); the MFMA waves never wait on vector memory inside the K loop.
//
// Tile order: m-tile t belongs to XCD t % 8 (consecutive workgroup ids are dealt to the 8 XCDs in turn), and
// inside an XCD the (m-tile, n-tile) pairs are walked n-fastest, so the n-tiles sharing an A tile run
// concurrently on CUs that share an L2.  The mapping does not depend on the live row count, which only
// trims each XCD's list.
// NSTAGE = depth of the operand ring (3, or 2 for tiles whose stages are too large for three); LATE = fetch bias and
// residual in the epilogue itself instead of during the last stage (large wave tiles have no registers to park them).
//
// PATCH: the kernel is a patch embedding (a convolution whose stride is its kernel size, as a Linear over the
// patches).  A is the image batch [B, Cin, S, S] itself: row (b, gy, gx) of the product is patch (gy, gx) of image b
// and its K index runs over (channel, row of the patch, pixel), so a 128-byte K slab of a row is a few consecutive
// pixel rows of one channel of the patch and the loader waves fetch them straight from the image - nothing but
// their per-lane source addresses differs from the plain kernel, no unfolded copy of the images exists.  The output
// row goes to token `extra + gy G + gx` of sample b in [B, extra + G G, N], and the residual is row
// `extra + gy G + gx` of one [extra + G G, N] table for every sample (the position embedding).
//
// The same mode reads patches of a channels-last token grid (cl_C > 0): A is [B, cl_H cl_W, cl_C] tokens, row
// (b, gy, gx) of the product is the P x P block of tokens at (gy P, gx P) and its K index runs over (token row of
// the block, token of that row, channel), i.e. a 128-byte K slab is a piece of one token's channels (cl_C values
// must fill whole slabs).  This is a stride-P P x P convolution over the grid with its weight in [O, kh, kw, C]
// order; rows of the product are stored densely (extra = 0) and there is no residual.
struct PatchGeom {
    int P, S, G, Cin, extra;     // patch edge, image edge, patches per edge, input channels, tokens in front
    int cl_C, cl_H, cl_W;        // channels-last source: channels and token grid (cl_C = 0: an image batch)
};

template <typename T, int BM, int BN, int WGM, int WGN, int NWP, int ACT, bool HAS_BIAS, bool HAS_RES, int NSTAGE = 3,
          bool LATE = false, bool PATCH = false>
__global__ __launch_bounds__((WGM * WGN + NWP) * 64) void linear_dma_kernel(
    const T *__restrict__ A, int64_t lda, const T *__restrict__ Wt, const T *__restrict__ bias,
    const T *__restrict__ res, int64_t ldr, T *__restrict__ out, int64_t ldo, const int64_t *__restrict__ rows_dev,
    int64_t rows, int N, int K, PatchGeom pg)
{
    constexpr int ESZ = sizeof(T);
    static_assert(NSTAGE == 2 || NSTAGE == 3, "ring depth");
    constexpr int NWC = WGM * WGN;                   // MFMA waves
    constexpr int TM = BM / WGM, TN = BN / WGN;      // wave tile
    constexpr int IM = TM / 32, JN = TN / 32;        // 32x32 MFMA blocks per wave
    constexpr int STAGE = (BM + BN) * DKB;           // bytes
    constexpr int NLW = (BM + BN) / 8 / NWP;         // direct loads per loader wave per stage
    static_assert((BM + BN) % (8 * NWP) == 0 && TM % 32 == 0 && TN % 32 == 0 && BM % 16 == 0, "tile shape");
    static_assert(NLW < 64, "6-bit vmcnt");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int64_t M = live_rows(rows_dev, rows);
    const int tiles_n = (N + BN - 1) / BN;
    const int tiles_m = (int)((M + BM - 1) / BM);
    const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3, nwg = gridDim.x >> 3;
    const int mt_x = tiles_m > xcd ? (tiles_m - xcd + 7) / 8 : 0;   // m-tiles owned by this XCD
    const int U = mt_x * tiles_n;                                    // tiles owned by this XCD
    const int nt = U > wg ? (U - wg + nwg - 1) / nwg : 0;            // tiles of this workgroup: u = wg + k*nwg
    if (nt == 0) return;
    const int nk = (int)(((int64_t)K * ESZ) / DKB);
    const int G = nt * nk;                                           // stages this workgroup consumes

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;

    if (wid >= NWC) {
        // ------------------------------------------------------------------ loader waves
        // They issue nothing but direct loads, so a wave blocked on the memory pipeline never holds up an MFMA,
        // and their vmcnt sees loads only.
        const int lw = wid - NWC;
        const unsigned char *src[NLW];
        auto set_tile = [&](int k) {
            const int u = wg + k * nwg;
            const int64_t m0 = (int64_t)((u / tiles_n) * 8 + xcd) * BM;
            const int n0 = (u % tiles_n) * BN;
#pragma unroll
            for (int i = 0; i < NLW; i++) {
                const int r = (lw * NLW + i) * 8 + (lane >> 3);
                const int chunk = (lane & 7) ^ ((r >> 1) & 7);
                if (r < BM) {
                    int64_t gm = m0 + r;
                    gm = gm < M ? gm : M - 1;
                    if constexpr (PATCH) {
                        if (pg.cl_C > 0) {
                            // block (b, gy, gx) of the token grid: its first token; the slab's piece is added per stage
                            const int gw = pg.cl_W / pg.P, g2 = (pg.cl_H / pg.P) * gw;
                            const int gmi = (int)gm, b = gmi / g2, t = gmi - b * g2, gy = t / gw, gx = t - gy * gw;
                            src[i] = reinterpret_cast<const unsigned char *>(
                                         A + (((int64_t)b * pg.cl_H + gy * pg.P) * pg.cl_W + gx * pg.P) * pg.cl_C) +
                                     chunk * 16;
                        } else {
                            // patch (b, gy, gx); the chunk is pixels `cc` of patch row `cr` of the slab's first rows
                            const int g2 = pg.G * pg.G, cpr = pg.P * ESZ / 16;      // chunks per patch row
                            const int gmi = (int)gm, b = gmi / g2, t = gmi - b * g2, gy = t / pg.G, gx = t - gy * pg.G;
                            const int cr = chunk / cpr, cc = chunk % cpr;
                            src[i] = reinterpret_cast<const unsigned char *>(
                                         A + ((int64_t)b * pg.Cin * pg.S + gy * pg.P + cr) * pg.S + gx * pg.P) + cc * 16;
                        }
                    } else {
                        src[i] = reinterpret_cast<const unsigned char *>(A + gm * lda) + chunk * 16;
                    }
                } else {
                    int gn = n0 + r - BM;
                    gn = gn < N ? gn : N - 1;
                    src[i] = reinterpret_cast<const unsigned char *>(Wt + (int64_t)gn * K) + chunk * 16;
                }
            }
        };
        int it_tile = 0, it_kt = 0, issued = 0;      // next stage to issue
        set_tile(0);
        auto issue_next = [&]() {
            unsigned char *dst = smem + (issued % NSTAGE) * STAGE + lw * NLW * 1024;
            int64_t a_off = (int64_t)it_kt * DKB;
            if constexpr (PATCH) {
                if (pg.cl_C > 0) {
                    // slab it_kt of a block of tokens: which token of the block and where in its channels
                    const int spt = pg.cl_C * ESZ / DKB;                       // slabs per token
                    const int tk = it_kt / spt, dy = tk / pg.P, dx = tk - dy * pg.P;
                    a_off = ((int64_t)(dy * pg.cl_W + dx) * pg.cl_C) * ESZ + (int64_t)(it_kt - tk * spt) * DKB;
                } else {
                    // slab it_kt of a patch: its channel and its first row in the patch
                    const int rps = DKB / (pg.P * ESZ), spc = pg.P / rps;      // rows per slab, slabs per channel
                    a_off = ((int64_t)(it_kt / spc) * pg.S + (it_kt % spc) * rps) * pg.S * ESZ;
                }
            }
#pragma unroll
            for (int i = 0; i < NLW; i++) {
                const bool a_rows = (lw * NLW + i) * 8 < BM;
                VT_GLOBAL_TO_LDS(src[i] + (a_rows ? a_off : (int64_t)it_kt * DKB), dst + i * 1024);
            }
            issued++;
            if (++it_kt == nk) {
                it_kt = 0;
                if (++it_tile < nt) set_tile(it_tile);
            }
        };
#pragma unroll
        for (int i = 0; i < NSTAGE - 1; i++)
            if (issued < G) issue_next();
        for (int g = 0; g < G; g++) {
            // stage g has landed once at most the loads of the younger stages in flight are outstanding (loads
            // retire in order)
            if (g + NSTAGE - 2 < G) wait_vmcnt<(NSTAGE - 2) * NLW>();
            else wait_vmcnt<0>();
            block_barrier();                         // stage g visible to the MFMA waves; slot of g-1 is free
            if (issued < G) issue_next();            // stage g + NSTAGE - 1
        }
        return;
    }

    // ---- MFMA side
    // where row `row` of the product is stored and which row of the residual it takes
    // (32-bit arithmetic: the patch count of a batch fits, and a 64-bit division costs a hundred instructions)
    auto out_row = [&](int64_t row) -> int64_t {
        if constexpr (PATCH) { const int g2 = pg.G * pg.G; return row + ((int)row / g2 + 1) * pg.extra; }
        else return row;
    };
    auto res_row = [&](int64_t row) -> int64_t {
        if constexpr (PATCH) { const int g2 = pg.G * pg.G; return (int)row % g2 + pg.extra; }
        else return row;
    };
    const int wm = wid / WGN, wn = wid % WGN;
    const int lr = lane & 31, lg = lane >> 5;
    const int sw = (lr >> 1) & 7;
    int cs[4];
#pragma unroll
    for (int s = 0; s < 4; s++) cs[s] = ((2 * s + lg) ^ sw) * 16;
    const int a_row = (wm * TM + lr) * DKB;
    const int w_row = (BM + wn * TN + lr) * DKB;

    f32x16 acc[IM][JN];
#pragma unroll
    for (int i = 0; i < IM; i++)
#pragma unroll
        for (int j = 0; j < JN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    constexpr int EPL = 16 / ESZ;          // output elements per lane and store
    constexpr int NQ = 32 / (2 * EPL);     // stores per 32x32 block and lane: bf16 2 (8 columns each), fp32 4
    u32x4 braw[JN][NQ], rraw[IM][JN][NQ];  // bias / residual vectors of the tile, fetched during its last stage
    int kt = 0, tk = 0;
    for (int g = 0; g < G; g++) {
        const bool last = kt == nk - 1;
        block_barrier();
        // output coordinates of the tile being accumulated
        const int u = wg + tk * nwg;
        const int64_t m0 = (int64_t)((u / tiles_n) * 8 + xcd) * BM;
        const int n0 = (u % tiles_n) * BN;
        if (last && !LATE) {
            // issue the epilogue's reads now; they return while the last stage is multiplied
#pragma unroll
            for (int j = 0; j < JN; j++)
#pragma unroll
                for (int q = 0; q < NQ; q++) {
                    const int col = n0 + wn * TN + j * 32 + (ESZ == 2 ? 8 * (2 * q + lg) : 8 * q + 4 * lg);
                    const u32x4 z = {0u, 0u, 0u, 0u};
                    braw[j][q] = z;
                    if constexpr (HAS_BIAS)
                        if (col < N) braw[j][q] = *reinterpret_cast<const u32x4 *>(bias + col);
#pragma unroll
                    for (int i = 0; i < IM; i++) {
                        const int64_t row = m0 + wm * TM + i * 32 + lr;
                        rraw[i][j][q] = z;
                        if constexpr (HAS_RES)
                            if (row < M && col < N)
                                rraw[i][j][q] = *reinterpret_cast<const u32x4 *>(res + res_row(row) * ldr + col);
                    }
                }
        }
        const unsigned char *st = smem + (g % NSTAGE) * STAGE;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            u32x4 fa[IM], fw[JN];
#pragma unroll
            for (int i = 0; i < IM; i++) fa[i] = *reinterpret_cast<const u32x4 *>(st + a_row + i * 32 * DKB + cs[s]);
#pragma unroll
            for (int j = 0; j < JN; j++) fw[j] = *reinterpret_cast<const u32x4 *>(st + w_row + j * 32 * DKB + cs[s]);
#pragma unroll
            for (int i = 0; i < IM; i++)
#pragma unroll
                for (int j = 0; j < JN; j++) Slab<T>::mma(fw[j], fa[i], acc[i][j]);   // D = W_blk * A_blk^T
        }
        if (++kt < nk) continue;
        kt = 0;
        tk++;
        // ---- epilogue, registers only.  acc[i][j][v] = C[row i*32 + lr][col j*32 + 8*(v/4) + 4*lg + v%4];
        // for bf16 a half-wave swap of the column groups (2q, 2q+1) leaves 8 consecutive columns in each lane.
#pragma unroll
        for (int i = 0; i < IM; i++) {
            const int64_t row = m0 + wm * TM + i * 32 + lr;
            const int64_t orow = out_row(row), rrow = res_row(row);
#pragma unroll
            for (int j = 0; j < JN; j++) {
#pragma unroll
                for (int q = 0; q < NQ; q++) {
                    float f[EPL];
                    int col;
                    if constexpr (ESZ == 2) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[i][j][8 * q + e]),
                                                                      __float_as_uint(acc[i][j][8 * q + 4 + e]), false,
                                                                      false);
                            f[e] = __uint_as_float(r[0]);
                            f[4 + e] = __uint_as_float(r[1]);
                        }
                        col = n0 + wn * TN + j * 32 + 8 * (2 * q + lg);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++) f[e] = acc[i][j][4 * q + e];
                        col = n0 + wn * TN + j * 32 + 8 * q + 4 * lg;
                    }
                    if constexpr (LATE) {
                        const u32x4 z = {0u, 0u, 0u, 0u};
                        braw[j][q] = z;
                        rraw[i][j][q] = z;
                        if constexpr (HAS_BIAS)
                            if (col < N) braw[j][q] = *reinterpret_cast<const u32x4 *>(bias + col);
                        if constexpr (HAS_RES)
                            if (row < M && col < N)
                                rraw[i][j][q] = *reinterpret_cast<const u32x4 *>(res + rrow * ldr + col);
                    }
                    if constexpr (HAS_BIAS) {
                        float bv[EPL];
                        Elem<T>::unpack(braw[j][q], bv);
#pragma unroll
                        for (int e = 0; e < EPL; e++) f[e] += bv[e];
                    }
                    if constexpr (ACT == VTDGE_ACT_GELU) {
#pragma unroll
                        for (int e = 0; e < EPL; e++) f[e] = gelu_fn<T>(f[e]);
                    }
                    if constexpr (HAS_RES) {
                        float rv[EPL];
                        Elem<T>::unpack(rraw[i][j][q], rv);
#pragma unroll
                        for (int e = 0; e < EPL; e++) f[e] += rv[e];
                    }
                    if (row < M && col < N) *reinterpret_cast<u32x4 *>(out + orow * ldo + col) = Elem<T>::pack(f);
                }
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
            }
        }
    }
}

// ----------------------------------------------------------------------------- host
struct LinArgs {
    const void *A; int64_t lda; const void *W; const void *bias; const void *res; int64_t ldr;
    void *out; int64_t ldo; const int64_t *rows_dev; int64_t rows; int N; int K; int act; hipStream_t st;
};

template <typename T, int BM, int BN, int WGM, int WGN, int NWP, int ACT, bool HB, bool HR, bool PATCH = false>
static int go(const LinArgs &a, const PatchGeom &pg = PatchGeom{0, 0, 0, 0, 0, 0, 0, 0})
{
    constexpr int NW = WGM * WGN + NWP;
    constexpr int NSTAGE = (size_t)3 * (BM + BN) * DKB <= 160 * 1024 ? 3 : 2;
    constexpr bool LATE = (BM / WGM) * (BN / WGN) > 64 * 64;      // wave tiles beyond 64 x 64
    constexpr size_t lds = (size_t)NSTAGE * (BM + BN) * DKB;
    static_assert(lds <= 160 * 1024, "LDS budget");
    constexpr int WGS_PER_CU = lds <= 80 * 1024 ? 2 : 1;
    auto kern = linear_dma_kernel<T, BM, BN, WGM, WGN, NWP, ACT, HB, HR, NSTAGE, LATE, PATCH>;
    VT_RESERVE_LDS(kern, lds, "linear");
    // persistent grid: what fits on the 256 CUs at once, but never more workgroups than tiles per XCD
    const int64_t tiles_per_xcd = ceil_div(ceil_div(a.rows, BM), 8) * ceil_div(a.N, BN);
    int64_t wgs_per_xcd = 32 * WGS_PER_CU;
    if (wgs_per_xcd > tiles_per_xcd) wgs_per_xcd = tiles_per_xcd;
    dim3 grid((unsigned)(wgs_per_xcd * 8)), block(NW * 64);
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<grid, block, lds, a.st>>>((const T *)a.A, a.lda, (const T *)a.W, (const T *)a.bias, (const T *)a.res,
                                     a.ldr, (T *)a.out, a.ldo, a.rows_dev, a.rows, a.N, a.K, pg);
    return check_launch("linear");
}

template <typename T, int BM, int BN, int WGM, int WGN, int NWP>
static int pick_epilogue(const LinArgs &a)
{
    const bool hb = a.bias != nullptr, hr = a.res != nullptr;
    if (a.act == VTDGE_ACT_GELU) {
        if (hb && !hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_GELU, true, false>(a);
        if (hb && hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_GELU, true, true>(a);
        if (hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_GELU, false, true>(a);
        return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_GELU, false, false>(a);
    }
    if (hb && !hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_NONE, true, false>(a);
    if (hb && hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_NONE, true, true>(a);
    if (hr) return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_NONE, false, true>(a);
    return go<T, BM, BN, WGM, WGN, NWP, VTDGE_ACT_NONE, false, false>(a);
}

// Whether the pipelined kernel can take the problem (the generic kernel takes the rest).
bool linear_dma_applicable(int64_t lda, int64_t ldr, int64_t ldo, int N, int K, int esz, const void *bias,
                           const void *res, const void *out)
{
    const int vec = 16 / esz;
    return ((int64_t)K * esz) % DKB == 0 && N % vec == 0 && lda % vec == 0 && ldo % vec == 0 &&
           (res == nullptr || ldr % vec == 0) && (((uintptr_t)bias | (uintptr_t)res | (uintptr_t)out) & 15) == 0;
}

template <typename T>
int launch_linear_dma(const void *A, int64_t lda, const void *W, const void *bias, const void *res, int64_t ldr,
                      void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int K, int act,
                      hipStream_t st)
{
    LinArgs a{A, lda, W, bias, res, ldr, out, ldo, rows_dev, rows, N, K, act, st};
    // wide outputs: 256x128 tiles on 8 MFMA waves; narrow ones (N <= 512), and matrices that have fewer large tiles
    // than the chip has compute units (a classifier on 256 rows): 128x128 on 4, for more tiles.  Other shapes of the
    // same template (2 loader waves, 128x256 and 128x384 tiles on a two-stage ring) measured no faster.
    if (N >= 768 && ceil_div(rows, 256) * ceil_div(N, 128) >= 256) return pick_epilogue<T, 256, 128, 4, 2, 4>(a);
    return pick_epilogue<T, 128, 128, 2, 2, 4>(a);
}

// The patch embedding: images [B, Cin, S, S] -> tokens [B, extra + G G, N] rows extra.., = conv + bias + pos.
bool patch_embed_applicable(int P, int S, int Cin, int N, int esz, const void *images, const void *weight,
                            const void *bias, const void *pos, const void *out)
{
    const int row = P * esz;                 // bytes of a patch row
    return P > 0 && S % P == 0 && row % 16 == 0 && DKB % row == 0 && P % (DKB / row) == 0 &&
           ((int64_t)S * esz) % 16 == 0 && N % (16 / esz) == 0 && bias != nullptr && pos != nullptr &&
           (((uintptr_t)images | (uintptr_t)weight | (uintptr_t)bias | (uintptr_t)pos | (uintptr_t)out) & 15) == 0;
}

template <typename T>
int launch_patch_embed(const void *images, const void *W, const void *bias, const void *pos, void *out, int B, int Cin,
                       int S, int P, int N, int extra, hipStream_t st)
{
    const int G = S / P;
    const PatchGeom pg{P, S, G, Cin, extra, 0, 0, 0};
    LinArgs a{images, 0, W, bias, pos, N, out, N, nullptr, (int64_t)B * G * G, N, Cin * P * P, VTDGE_ACT_NONE, st};
    // 128x128 tiles, two workgroups per CU, unless the output is wide.  At 256 x 256 patches and N = 384 a launch takes
    // 80 - 88 us against 125 - 138 us on 256x128 tiles with one workgroup per CU (which only looks faster, 67 against
    // 78 us, when launches are timed back to back and the tail of one hides under the head of the next).
    // Eight loader waves instead of four (they also work out the patch addresses): 77.5 against 83.5 us; with two,
    // 201 us.  64x128 tiles: 108 us, 256x128 with eight loaders: 98 us.
    if (N >= 768) return go<T, 256, 128, 4, 2, 4, VTDGE_ACT_NONE, true, true, true>(a, pg);
    return go<T, 128, 128, 2, 2, 8, VTDGE_ACT_NONE, true, true, true>(a, pg);
}

// A stride-P P x P convolution over a channels-last token grid [B, H W, C] (weight in [N, kh, kw, C] order) + bias:
// rows (b, gy, gx) of out [B (H/P) (W/P), N].
bool patch_linear_applicable(int P, int H, int W, int C, int N, int esz, const void *tokens, const void *weight,
                             const void *bias, const void *out)
{
    return P > 0 && H > 0 && W > 0 && H % P == 0 && W % P == 0 && ((int64_t)C * esz) % DKB == 0 &&
           N % (16 / esz) == 0 && bias != nullptr &&
           (((uintptr_t)tokens | (uintptr_t)weight | (uintptr_t)bias | (uintptr_t)out) & 15) == 0;
}

template <typename T>
int launch_patch_linear(const void *tokens, const void *W, const void *bias, void *out, int B, int H, int Wd, int C,
                        int P, int N, hipStream_t st)
{
    const PatchGeom pg{P, 0, 1, 0, 0, C, H, Wd};
    const int64_t rows = (int64_t)B * (H / P) * (Wd / P);
    LinArgs a{tokens, 0, W, bias, nullptr, 0, out, N, nullptr, rows, N, P * P * C, VTDGE_ACT_NONE, st};
    if (N >= 768 || ceil_div(rows, 256) * ceil_div(N, 128) >= 512)
        return go<T, 256, 128, 4, 2, 4, VTDGE_ACT_NONE, true, false, true>(a, pg);
    return go<T, 128, 128, 2, 2, 4, VTDGE_ACT_NONE, true, false, true>(a, pg);
}

template int launch_patch_linear<float>(const void *, const void *, const void *, void *, int, int, int, int, int, int,
                                        hipStream_t);
template int launch_patch_linear<bf16_t>(const void *, const void *, const void *, void *, int, int, int, int, int, int,
                                         hipStream_t);

template int launch_patch_embed<float>(const void *, const void *, const void *, const void *, void *, int, int, int,
                                       int, int, int, hipStream_t);
template int launch_patch_embed<bf16_t>(const void *, const void *, const void *, const void *, void *, int, int, int,
                                        int, int, int, hipStream_t);

template int launch_linear_dma<float>(const void *, int64_t, const void *, const void *, const void *, int64_t, void *,
                                      int64_t, const int64_t *, int64_t, int, int, int, hipStream_t);
template int launch_linear_dma<bf16_t>(const void *, int64_t, const void *, const void *, const void *, int64_t,
                                       void *, int64_t, const int64_t *, int64_t, int, int, int, hipStream_t);

}  // namespace vtdge
