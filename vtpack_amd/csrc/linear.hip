// Packed-M Linear for gfx950: out = act(A W^T + bias) + residual on MFMA.
//
// Both operands are K-contiguous (A [M,K], W [N,K]), which is exactly what the
// gfx950 MFMA wants: every lane feeds 16 bytes of one operand row per
// instruction group.  In bytes the two precisions share one geometry: a 32-byte
// K-slab of a row is consumed by
//   bf16: one  v_mfma_f32_32x32x16_bf16 (lane group g holds elements 8g..8g+7)
//   fp32: four v_mfma_f32_32x32x2_f32   (lane group g holds floats 4g..4g+3;
//         instruction j takes float j of both groups -- the contraction index
//         is merely permuted identically for both operands)
// so one kernel template serves both.
//
// Tiling: 128x128 output tile per 256-thread workgroup (2x2 waves of 64x64,
// each 2x2 MFMA blocks of 32x32), K advanced 128 bytes per step through a
// double-buffered LDS stage (row pitch 144 B: the 16-byte pad makes the
// 16-lane phases of ds_read_b128 conflict free).  Workgroups are renumbered so
// that the eight XCDs (round-robin over consecutive workgroup ids) each walk a
// contiguous range of tiles and the N-tiles that share an A tile meet in one L2.
#include "common.h"

namespace vtdge {

constexpr int BM = 128, BN = 128;
constexpr int KB = 128;               // K bytes per stage
constexpr int PITCH = KB + 16;        // LDS row pitch in bytes
constexpr int NXCD = 8;

__device__ __forceinline__ float gelu_erf(float v) { return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f)); }

template <typename T, int ACT, bool HAS_BIAS, bool HAS_RES>
__global__ __launch_bounds__(256) void linear_kernel(const T *__restrict__ A, int64_t lda, const T *__restrict__ Wt,
                                                      const T *__restrict__ bias, const T *__restrict__ res,
                                                      int64_t ldr, T *__restrict__ out, int64_t ldo,
                                                      const int64_t *__restrict__ rows_dev, int64_t rows, int N,
                                                      int K)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int ESZ = sizeof(T);
    constexpr int STAGE = (BM + BN) * PITCH;

    const int64_t M = live_rows(rows_dev, rows);
    const int tiles_n = (N + BN - 1) / BN;
    const int64_t tiles_m = (M + BM - 1) / BM;
    const int64_t total = tiles_m * tiles_n;
    const int64_t per_xcd = (total + NXCD - 1) / NXCD;
    const int64_t local = blockIdx.x / NXCD;
    const int64_t tile = (int64_t)(blockIdx.x % NXCD) * per_xcd + local;
    if (local >= per_xcd || tile >= total) return;
    const int64_t m0 = (tile / tiles_n) * BM;
    const int n0 = (int)(tile % tiles_n) * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wid = tid >> 6;
    const int wm = wid >> 1, wn = wid & 1;
    const int lr = lane & 31, lg = lane >> 5;

    const int64_t kbytes = (int64_t)K * ESZ;
    const int nk = (int)((kbytes + KB - 1) / KB);

    // global -> register staging: 4 A chunks + 4 W chunks of 16 B per thread
    u32x4 ra[4], rw[4];
    auto load_global = [&](int kt) {
        const int64_t kb0 = (int64_t)kt * KB;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 256 * i;
            const int r = idx >> 3, ch = idx & 7;
            const int64_t kb = kb0 + ch * 16;
            const int64_t gm = m0 + r;
            u32x4 z = {0u, 0u, 0u, 0u};
            ra[i] = z;
            rw[i] = z;
            if (gm < M && kb < kbytes)
                ra[i] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const unsigned char *>(A + gm * lda) + kb);
            const int gn = n0 + r;
            if (gn < N && kb < kbytes)
                rw[i] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const unsigned char *>(Wt + (int64_t)gn * K) +
                                                        kb);
        }
    };
    auto store_lds = [&](int buf) {
        unsigned char *sa = smem + buf * STAGE;
        unsigned char *sw = sa + BM * PITCH;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 256 * i;
            const int r = idx >> 3, ch = idx & 7;
            *reinterpret_cast<u32x4 *>(sa + r * PITCH + ch * 16) = ra[i];
            *reinterpret_cast<u32x4 *>(sw + r * PITCH + ch * 16) = rw[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        if (kt + 1 < nk) load_global(kt + 1);
        const unsigned char *sa = smem + (kt & 1) * STAGE + (wm * 64 + lr) * PITCH + lg * 16;
        const unsigned char *sw = smem + (kt & 1) * STAGE + BM * PITCH + (wn * 64 + lr) * PITCH + lg * 16;
#pragma unroll
        for (int s = 0; s < KB / 32; s++) {
            u32x4 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = *reinterpret_cast<const u32x4 *>(sa + i * 32 * PITCH + s * 32);
                fb[i] = *reinterpret_cast<const u32x4 *>(sw + i * 32 * PITCH + s * 32);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) Slab<T>::mma(fa[i], fb[j], acc[i][j]);
        }
        if (kt + 1 < nk) store_lds((kt + 1) & 1);
        __syncthreads();
    }

    // epilogue: lane holds column lr of each 32x32 block, rows 8*(v/4) + 4*lg + v%4
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + lr;
        if (col >= N) continue;
        float bv = 0.f;
        if constexpr (HAS_BIAS) bv = Elem<T>::load(bias + col);
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lg + (v & 3);
                if (row < M) {
                    float val = acc[i][j][v] + bv;
                    if constexpr (ACT == VTDGE_ACT_GELU) val = gelu_erf(val);
                    if constexpr (HAS_RES) val += Elem<T>::load(res + row * ldr + col);
                    Elem<T>::store(out + row * ldo + col, val);
                }
            }
        }
    }
}

template <typename T>
static int launch_linear(const void *A, int64_t lda, const void *W, const void *bias, const void *res, int64_t ldr,
                         void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int K, int act,
                         hipStream_t st)
{
    const int64_t tiles = ceil_div(rows, BM) * ceil_div(N, BN);
    const int64_t per_xcd = ceil_div(tiles, NXCD);
    dim3 grid((unsigned)(per_xcd * NXCD)), block(256);
    const size_t lds = 2 * (BM + BN) * PITCH;
#define VT_GO(ACT, HB, HR)                                                                                      \
    do {                                                                                                        \
        auto kern = linear_kernel<T, ACT, HB, HR>;                                                              \
        VT_RESERVE_LDS(kern, lds, "linear");                                                                    \
        note_kernel(reinterpret_cast<const void *>(kern)),                                                      \
        kern<<<grid, block, lds, st>>>((const T *)A, lda, (const T *)W, (const T *)bias, (const T *)res, ldr,   \
                                       (T *)out, ldo, rows_dev, rows, N, K);                                    \
    } while (0)
    const bool hb = bias != nullptr, hr = res != nullptr;
    if (act == VTDGE_ACT_GELU) {
        if (hb && hr) VT_GO(VTDGE_ACT_GELU, true, true);
        else if (hb) VT_GO(VTDGE_ACT_GELU, true, false);
        else if (hr) VT_GO(VTDGE_ACT_GELU, false, true);
        else VT_GO(VTDGE_ACT_GELU, false, false);
    } else {
        if (hb && hr) VT_GO(VTDGE_ACT_NONE, true, true);
        else if (hb) VT_GO(VTDGE_ACT_NONE, true, false);
        else if (hr) VT_GO(VTDGE_ACT_NONE, false, true);
        else VT_GO(VTDGE_ACT_NONE, false, false);
    }
#undef VT_GO
    return check_launch("linear");
}

// pipelined direct-to-LDS variant (linear_dma.hip)
bool linear_dma_applicable(int64_t lda, int64_t ldr, int64_t ldo, int N, int K, int esz, const void *bias,
                           const void *res, const void *out);
template <typename T>
int launch_linear_dma(const void *A, int64_t lda, const void *W, const void *bias, const void *res, int64_t ldr,
                      void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int K, int act,
                      hipStream_t st);

// the patch embedding on the same kernel (linear_dma.hip)
bool patch_embed_applicable(int P, int S, int Cin, int N, int esz, const void *images, const void *weight,
                            const void *bias, const void *pos, const void *out);
template <typename T>
int launch_patch_embed(const void *images, const void *W, const void *bias, const void *pos, void *out, int B, int Cin,
                       int S, int P, int N, int extra, hipStream_t st);

// a strided convolution over a channels-last token grid on the same kernel (linear_dma.hip)
bool patch_linear_applicable(int P, int H, int W, int C, int N, int esz, const void *tokens, const void *weight,
                             const void *bias, const void *out);
template <typename T>
int launch_patch_linear(const void *tokens, const void *W, const void *bias, void *out, int B, int H, int Wd, int C,
                        int P, int N, hipStream_t st);

// weight-stationary variant for bf16, K = 384 (linear_ws8.hip)
bool linear_ws_applicable(int64_t lda, int64_t ldr, int64_t ldo, int64_t rows, int N, int K, int esz, int act,
                          const void *bias, const void *res, const void *out);
int launch_linear_ws8(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                      int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int act,
                      hipStream_t st);
int launch_linear_ws8_ln_pair(const void *A0, int64_t lda0, const void *lnrec0, const void *Wf0, const void *Wfp0,
                              const void *lnw0, void *out0, int64_t ldo0, const int64_t *rows_dev0, int64_t rows0,
                              int N0, const void *A1, int64_t lda1, const void *lnrec1, const void *Wf1,
                              const void *Wfp1, const void *lnw1, void *out1, int64_t ldo1, const int64_t *rows_dev1,
                              int64_t rows1, int N1, hipStream_t st);
int launch_linear_ws8_ln(const void *A, int64_t lda, const void *lnrec, const void *Wf, const void *Wfp,
                         const void *lnw, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N,
                         int act, hipStream_t st);
int launch_linear_ws8_stats(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias,
                            const void *res, int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev,
                            int64_t rows, void *records, float eps, hipStream_t st);

// K-split weight-stationary variant for bf16, K = 1536, narrow N (linear_ks.hip)
bool linear_ks_applicable(int64_t lda, int64_t ldr, int64_t ldo, int64_t rows, int N, int K, int esz, int act,
                          const void *bias, const void *res, const void *out);
int launch_linear_ks(const void *A, int64_t lda, const void *W, const void *Wp, const void *bias, const void *res,
                     int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, hipStream_t st);

}  // namespace vtdge

using namespace vtdge;

// ---------------------------------------------------------------------------------------------------------
// Packed copies of W for the weight-stationary kernels: the 16-byte register images of the MFMA fragments, in the
// order [column group][wave][fragment][lane], so a wave fills its registers with contiguous 1 KB loads.
//   layout 1 (K = 384, linear_ws8.hip): group = 384 columns; wave w, fragment (cb, ks), lane (c16, kg) holds
//            W[384 g + 48 w + 16 cb + c16][32 ks + 8 kg .. + 7]                    (w < 8, cb < 3, ks < 12)
//   layout 2 (K = 1536, linear_ks.hip): group = 96 columns; wave w, fragment (cb, ks), lane (c16, kg) holds
//            W[96 g + 16 cb + c16][384 w + 32 ks + 8 kg .. + 7]                    (cb < 6, ks < 12)
static int packed_layout(int N, int K, int dtype)
{
    if (dtype != VTDGE_BF16) return 0;
    if (K == 384 && N % 384 == 0 && N / 384 <= 8) return 1;
    if (K == 1536 && N % 96 == 0 && N / 96 <= 8) return 2;
    return 0;
}

__global__ __launch_bounds__(256) void linear_prepack_kernel(const bf16_t *__restrict__ W, u32x4 *__restrict__ packed,
                                                              int N, int K, int layout)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;       // one 16-byte unit each
    if (idx >= (int64_t)N * K / 8) return;
    const int lane = (int)(idx & 63);
    int row, k;
    if (layout == 1) {
        const int f = (int)((idx >> 6) % 36), gw = (int)((idx >> 6) / 36);
        const int w = gw & 7, g = gw >> 3;
        const int cb = f / 12, ks = f % 12, c16 = lane & 15, kg = lane >> 4;
        row = 384 * g + 48 * w + 16 * cb + c16;
        k = 32 * ks + 8 * kg;
    } else {
        const int f = (int)((idx >> 6) % 72), gw = (int)((idx >> 6) / 72);
        const int w = gw & 3, g = gw >> 2;
        const int cb = f / 12, ks = f % 12, c16 = lane & 15, kg = lane >> 4;
        row = 96 * g + 16 * cb + c16;
        k = 384 * w + 32 * ks + 8 * kg;
    }
    packed[idx] = *reinterpret_cast<const u32x4 *>(W + (int64_t)row * K + k);
}

extern "C" int vtdge_linear_packed_size(int N, int K, int dtype, int64_t *bytes)
{
    VT_REQUIRE(bytes != nullptr, VTDGE_ERR_ARG, "linear_packed_size: NULL result");
    VT_REQUIRE(N > 0 && K > 0, VTDGE_ERR_ARG, "linear_packed_size: bad sizes N=%d K=%d", N, K);
    *bytes = packed_layout(N, K, dtype) ? (int64_t)N * K * 2 : 0;
    return VTDGE_OK;
}

extern "C" int vtdge_linear_prepack(const void *W, int N, int K, int dtype, void *packed, void *stream)
{
    VT_REQUIRE(W && packed, VTDGE_ERR_ARG, "linear_prepack: NULL operand");
    VT_REQUIRE(N > 0 && K > 0, VTDGE_ERR_ARG, "linear_prepack: bad sizes N=%d K=%d", N, K);
    const int layout = packed_layout(N, K, dtype);
    VT_REQUIRE(layout != 0, VTDGE_ERR_UNSUPPORTED, "linear_prepack: no packed layout for N=%d K=%d dtype=%d", N, K,
               dtype);
    VT_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)packed & 15) == 0, VTDGE_ERR_ARG,
               "linear_prepack: W and packed must be 16-byte aligned");
    const int64_t units = (int64_t)N * K / 8;
    note_kernel(reinterpret_cast<const void *>(linear_prepack_kernel));
    linear_prepack_kernel<<<(unsigned)ceil_div(units, 256), 256, 0, (hipStream_t)stream>>>(
        (const bf16_t *)W, (u32x4 *)packed, N, K, layout);
    return check_launch("linear_prepack");
}

// ---------------------------------------------------------------------------------------------------------
// LayerNorm folded into the Linear that follows it:  LayerNorm(a) W^T + bias = rstd * (a W'^T - mean * colsum(W')
// + sigma * b')  with W' = W * gamma (rounded to bf16, the value the MFMAs multiply by) and b' = bias + W beta.
// One wave per output column writes the row of W' and the column's record (see ln_column_record).
__global__ __launch_bounds__(256) void layernorm_fold_kernel(const bf16_t *__restrict__ W, const bf16_t *__restrict__ bias,
                                                              const bf16_t *__restrict__ gamma,
                                                              const bf16_t *__restrict__ beta, bf16_t *__restrict__ Wf,
                                                              u32x4 *__restrict__ colrec, int N, int K)
{
    const int col = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (col >= N) return;
    float cs = 0.f, wb = 0.f;
    for (int k = lane; k < K; k += 64) {
        const float w = bf16_to_f32(W[(int64_t)col * K + k]);
        const bf16_t f = f32_to_bf16(w * bf16_to_f32(gamma[k]));
        Wf[(int64_t)col * K + k] = f;
        cs += bf16_to_f32(f);
        wb += w * bf16_to_f32(beta[k]);
    }
    cs = wave_sum(cs);
    wb = wave_sum(wb);
    if (lane == 0) {
        u32x4 lo, hi;
        ln_column_record(cs, wb + (bias ? bf16_to_f32(bias[col]) : 0.f), lo, hi);
        colrec[col * 2] = lo;
        colrec[col * 2 + 1] = hi;
    }
}

extern "C" int vtdge_layernorm_fold(const void *W, const void *bias, const void *ln_weight, const void *ln_bias, int N,
                                    int K, int dtype, void *W_folded, void *col_records, void *stream)
{
    VT_REQUIRE(W && ln_weight && ln_bias && W_folded && col_records, VTDGE_ERR_ARG, "layernorm_fold: NULL operand");
    VT_REQUIRE(N > 0 && K > 0, VTDGE_ERR_ARG, "layernorm_fold: bad sizes N=%d K=%d", N, K);
    VT_REQUIRE(dtype == VTDGE_BF16, VTDGE_ERR_UNSUPPORTED, "layernorm_fold: built for bf16 weights only");
    VT_REQUIRE(((uintptr_t)col_records & 15) == 0, VTDGE_ERR_ARG, "layernorm_fold: records must be 16-byte aligned");
    note_kernel(reinterpret_cast<const void *>(layernorm_fold_kernel));
    layernorm_fold_kernel<<<(unsigned)ceil_div(N, 4), 256, 0, (hipStream_t)stream>>>(
        (const bf16_t *)W, (const bf16_t *)bias, (const bf16_t *)ln_weight, (const bf16_t *)ln_bias, (bf16_t *)W_folded,
        (u32x4 *)col_records, N, K);
    return check_launch("layernorm_fold");
}

extern "C" int vtdge_linear_layernorm(const void *A, int64_t lda, const void *row_records, const void *W_folded,
                                      const void *packed, const void *col_records, void *out, int64_t ldo,
                                      const int64_t *rows_dev, int64_t rows, int N, int K, int act, int dtype,
                                      void *stream)
{
    VT_REQUIRE(A && row_records && W_folded && col_records && out, VTDGE_ERR_ARG, "linear_layernorm: NULL operand");
    VT_REQUIRE(act == VTDGE_ACT_NONE || act == VTDGE_ACT_GELU, VTDGE_ERR_ARG, "linear_layernorm: unknown activation %d",
               act);
    VT_REQUIRE(rows >= 0 && N > 0 && K > 0, VTDGE_ERR_ARG, "linear_layernorm: bad sizes rows=%lld N=%d K=%d",
               (long long)rows, N, K);
    VT_REQUIRE(lda >= K && ldo >= N, VTDGE_ERR_ARG, "linear_layernorm: leading dim too small");
    VT_REQUIRE((((uintptr_t)A | (uintptr_t)W_folded | (uintptr_t)packed | (uintptr_t)row_records |
                 (uintptr_t)col_records) & 15) == 0,
               VTDGE_ERR_ARG, "linear_layernorm: operands must be 16-byte aligned");
    VT_REQUIRE(dtype == VTDGE_BF16 && linear_ws_applicable(lda, 0, ldo, rows, N, K, 2, act, nullptr, nullptr, out),
               VTDGE_ERR_UNSUPPORTED,
               "linear_layernorm: built for bf16, K = 384, N a multiple of 384 (at most 3072) and 2048 rows or more "
               "(rows=%lld N=%d K=%d dtype=%d)", (long long)rows, N, K, dtype);
    return launch_linear_ws8_ln(A, lda, row_records, W_folded, packed, col_records, out, ldo, rows_dev, rows, N, act,
                                (hipStream_t)stream);
}

extern "C" int vtdge_linear_layernorm_pair(const void *A0, int64_t lda0, const void *row_records0, const void *W_folded0,
                                           const void *packed0, const void *col_records0, void *out0, int64_t ldo0,
                                           const int64_t *rows_dev0, int64_t rows0, int N0, const void *A1,
                                           int64_t lda1, const void *row_records1, const void *W_folded1,
                                           const void *packed1, const void *col_records1, void *out1, int64_t ldo1,
                                           const int64_t *rows_dev1, int64_t rows1, int N1, int K, int dtype,
                                           void *stream)
{
    VT_REQUIRE(A0 && row_records0 && W_folded0 && col_records0 && out0 && A1 && row_records1 && W_folded1 &&
                   col_records1 && out1,
               VTDGE_ERR_ARG, "linear_layernorm_pair: NULL operand");
    VT_REQUIRE(rows0 >= 0 && rows1 >= 0 && N0 > 0 && N1 > 0 && K > 0, VTDGE_ERR_ARG, "linear_layernorm_pair: bad sizes");
    VT_REQUIRE(lda0 >= K && ldo0 >= N0 && lda1 >= K && ldo1 >= N1, VTDGE_ERR_ARG,
               "linear_layernorm_pair: leading dim too small");
    VT_REQUIRE((((uintptr_t)A0 | (uintptr_t)W_folded0 | (uintptr_t)packed0 | (uintptr_t)row_records0 |
                 (uintptr_t)col_records0 | (uintptr_t)A1 | (uintptr_t)W_folded1 | (uintptr_t)packed1 |
                 (uintptr_t)row_records1 | (uintptr_t)col_records1) & 15) == 0,
               VTDGE_ERR_ARG, "linear_layernorm_pair: operands must be 16-byte aligned");
    VT_REQUIRE(dtype == VTDGE_BF16 &&
                   linear_ws_applicable(lda0, 0, ldo0, rows0, N0, K, 2, VTDGE_ACT_NONE, nullptr, nullptr, out0) &&
                   linear_ws_applicable(lda1, 0, ldo1, rows1, N1, K, 2, VTDGE_ACT_NONE, nullptr, nullptr, out1) &&
                   N0 / 384 + N1 / 384 <= 16,
               VTDGE_ERR_UNSUPPORTED,
               "linear_layernorm_pair: both Linears as vtdge_linear_layernorm takes them (bf16, K = 384, N a multiple of "
               "384, 2048 rows or more; rows=%lld,%lld N=%d,%d K=%d)", (long long)rows0, (long long)rows1, N0, N1, K);
    return launch_linear_ws8_ln_pair(A0, lda0, row_records0, W_folded0, packed0, col_records0, out0, ldo0, rows_dev0,
                                     rows0, N0, A1, lda1, row_records1, W_folded1, packed1, col_records1, out1, ldo1,
                                     rows_dev1, rows1, N1, (hipStream_t)stream);
}

extern "C" int vtdge_linear_stats(const void *A, int64_t lda, const void *W, const void *packed, const void *bias,
                                  const void *residual, int64_t ldr, void *out, int64_t ldo, void *out_records,
                                  float records_eps, const int64_t *rows_dev, int64_t rows, int N, int K, int dtype,
                                  void *stream)
{
    VT_REQUIRE(A && W && out && out_records, VTDGE_ERR_ARG, "linear_stats: NULL operand");
    VT_REQUIRE(rows >= 0 && N > 0 && K > 0, VTDGE_ERR_ARG, "linear_stats: bad sizes rows=%lld N=%d K=%d",
               (long long)rows, N, K);
    VT_REQUIRE(lda >= K && ldo >= N && (!residual || ldr >= N), VTDGE_ERR_ARG, "linear_stats: leading dim too small");
    VT_REQUIRE((((uintptr_t)A | (uintptr_t)W | (uintptr_t)packed | (uintptr_t)out_records) & 15) == 0, VTDGE_ERR_ARG,
               "linear_stats: operands must be 16-byte aligned");
    VT_REQUIRE(dtype == VTDGE_BF16 && N == 384 &&
                   linear_ws_applicable(lda, ldr, ldo, rows, N, K, 2, VTDGE_ACT_NONE, bias, residual, out),
               VTDGE_ERR_UNSUPPORTED,
               "linear_stats: built for bf16, K = 384, N = 384 and 2048 rows or more (rows=%lld N=%d K=%d dtype=%d)",
               (long long)rows, N, K, dtype);
    return launch_linear_ws8_stats(A, lda, W, packed, bias, residual, ldr, out, ldo, rows_dev, rows, out_records,
                                   records_eps, (hipStream_t)stream);
}

extern "C" int vtdge_linear(const void *A, int64_t lda, const void *W, const void *bias, const void *residual,
                            int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int K,
                            int act, int dtype, void *stream)
{
    return vtdge_linear_prepacked(A, lda, W, nullptr, bias, residual, ldr, out, ldo, rows_dev, rows, N, K, act, dtype,
                                  stream);
}

extern "C" int vtdge_linear_prepacked(const void *A, int64_t lda, const void *W, const void *packed, const void *bias,
                                      const void *residual, int64_t ldr, void *out, int64_t ldo,
                                      const int64_t *rows_dev, int64_t rows, int N, int K, int act, int dtype,
                                      void *stream)
{
    VT_REQUIRE(A && W && out, VTDGE_ERR_ARG, "linear: NULL operand");
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "linear: unknown dtype %d", dtype);
    VT_REQUIRE(act == VTDGE_ACT_NONE || act == VTDGE_ACT_GELU, VTDGE_ERR_ARG, "linear: unknown activation %d", act);
    VT_REQUIRE(rows >= 0 && N > 0 && K > 0, VTDGE_ERR_ARG, "linear: bad sizes rows=%lld N=%d K=%d", (long long)rows,
               N, K);
    const int esz = dtype == VTDGE_BF16 ? 2 : 4;
    VT_REQUIRE(((int64_t)K * esz) % 16 == 0 && (lda * esz) % 16 == 0, VTDGE_ERR_UNSUPPORTED,
               "linear: K=%d and lda=%lld must be multiples of %d elements", K, (long long)lda, 16 / esz);
    VT_REQUIRE(lda >= K && ldo >= N && (!residual || ldr >= N), VTDGE_ERR_ARG, "linear: leading dim too small");
    VT_REQUIRE(((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)packed & 15) == 0, VTDGE_ERR_ARG,
               "linear: A, W and the packed copy of W must be 16-byte aligned");
    if (rows == 0) return VTDGE_OK;
    hipStream_t st = (hipStream_t)stream;
    if (linear_ws_applicable(lda, ldr, ldo, rows, N, K, esz, act, bias, residual, out))
        return launch_linear_ws8(A, lda, W, packed, bias, residual, ldr, out, ldo, rows_dev, rows, N, act, st);
    if (linear_ks_applicable(lda, ldr, ldo, rows, N, K, esz, act, bias, residual, out))
        return launch_linear_ks(A, lda, W, packed, bias, residual, ldr, out, ldo, rows_dev, rows, N, st);
    if (linear_dma_applicable(lda, ldr, ldo, N, K, esz, bias, residual, out)) {
        if (dtype == VTDGE_F32)
            return launch_linear_dma<float>(A, lda, W, bias, residual, ldr, out, ldo, rows_dev, rows, N, K, act, st);
        return launch_linear_dma<bf16_t>(A, lda, W, bias, residual, ldr, out, ldo, rows_dev, rows, N, K, act, st);
    }
    if (dtype == VTDGE_F32)
        return launch_linear<float>(A, lda, W, bias, residual, ldr, out, ldo, rows_dev, rows, N, K, act, st);
    return launch_linear<bf16_t>(A, lda, W, bias, residual, ldr, out, ldo, rows_dev, rows, N, K, act, st);
}

extern "C" int vtdge_patch_embed(const void *images, const void *weight, const void *bias, const void *pos_embed,
                                 void *tokens, int B, int Cin, int S, int P, int C, int extra, int dtype, void *stream)
{
    VT_REQUIRE(images && weight && tokens, VTDGE_ERR_ARG, "patch_embed: NULL operand");
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "patch_embed: unknown dtype %d", dtype);
    VT_REQUIRE(B > 0 && Cin > 0 && S > 0 && P > 0 && C > 0 && extra >= 0, VTDGE_ERR_ARG, "patch_embed: bad sizes");
    const int esz = dtype == VTDGE_F32 ? 4 : 2;
    VT_REQUIRE(patch_embed_applicable(P, S, Cin, C, esz, images, weight, bias, pos_embed, tokens), VTDGE_ERR_UNSUPPORTED,
               "patch_embed: no kernel for patch %d, image %d, %d channels, width %d (or bias / position table missing, "
               "or an operand not 16-byte aligned)", P, S, Cin, C);
    VT_REQUIRE((int64_t)B * Cin * S * S < (1ll << 40), VTDGE_ERR_UNSUPPORTED, "patch_embed: batch too large");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VTDGE_F32)
        return launch_patch_embed<float>(images, weight, bias, pos_embed, tokens, B, Cin, S, P, C, extra, st);
    return launch_patch_embed<bf16_t>(images, weight, bias, pos_embed, tokens, B, Cin, S, P, C, extra, st);
}

extern "C" int vtdge_patch_linear(const void *tokens, const void *weight, const void *bias, void *out, int B, int H,
                                  int W, int C, int P, int N, int dtype, void *stream)
{
    VT_REQUIRE(tokens && weight && out, VTDGE_ERR_ARG, "patch_linear: NULL operand");
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "patch_linear: unknown dtype %d", dtype);
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && C > 0 && P > 0 && N > 0, VTDGE_ERR_ARG, "patch_linear: bad sizes");
    const int esz = dtype == VTDGE_F32 ? 4 : 2;
    VT_REQUIRE(patch_linear_applicable(P, H, W, C, N, esz, tokens, weight, bias, out), VTDGE_ERR_UNSUPPORTED,
               "patch_linear: no kernel for a %d x %d block of a %d x %d grid of %d channels, width %d (or bias missing, "
               "or an operand not 16-byte aligned)", P, P, H, W, C, N);
    VT_REQUIRE((int64_t)B * H * W < (1ll << 31) && (int64_t)B * H * W * C < (1ll << 40), VTDGE_ERR_UNSUPPORTED,
               "patch_linear: batch too large");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VTDGE_F32) return launch_patch_linear<float>(tokens, weight, bias, out, B, H, W, C, P, N, st);
    return launch_patch_linear<bf16_t>(tokens, weight, bias, out, B, H, W, C, P, N, st);
}
