// Per-sample variable-length batched matmul over heads (gfx950), on the matrix cores.
//
// The reference loops over samples on the host and calls at::bmm / cuBLAS once per sample
// (batched_sparse_gemm.cu:150-195, :83-148).  Here one launch covers every (sample, head, output tile): a
// workgroup decodes its tile from a flat index (no grid-dimension limit on batch x heads) and resolves its own
// operand slices from the device-side offsets, so no length ever has to visit the host.
//
// Tile: 64 x 64 outputs per workgroup of four waves (2 x 2, one 32 x 32 MFMA block each), K in stages of 64 bytes
// per operand row (32 bf16 / 16 fp32 values = two 32-byte slabs of the MFMA helper in common.h: 32x32x16 bf16, or
// four 32x32x2 fp32 instructions per slab - fp32 storage multiplies in fp32).  Either operand may be transposed in
// its last two dimensions and no extent has to be a multiple of anything: an operand whose rows start on 16-byte
// boundaries comes in by 16-byte loads, any other element by element, both with bounds checks (zero beyond the
// edges) and a thread -> element map that runs along the source's contiguous dimension.  Both land in LDS in one
// canonical form, [tile row][k] in the storage type, from which the MFMA operands are 16-byte fragment reads (row
// pitch 80 bytes: the 16 rows that read together start in 16 different bank groups).
#include "common.h"

namespace vtdge {

constexpr int GT = 64;       // output tile edge
constexpr int GSB = 64;      // bytes of K per operand row and stage
constexpr int GPITCH = 80;   // LDS row pitch in bytes

template <typename T>
__global__ __launch_bounds__(256) void sparse_gemm_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                           const int64_t *__restrict__ a_off,
                                                           const int64_t *__restrict__ b_off, T *__restrict__ out,
                                                           int h, int64_t La, int ka, int64_t Lb, int kb, int ta,
                                                           int tb, int64_t out_rows, int64_t out_cols, int tiles_m,
                                                           int tiles_n, bool vec_a, bool vec_b)
{
    constexpr int KT = GSB / (int)sizeof(T);     // K values per stage
    constexpr int PER = GT * KT / 256;           // elements of each operand a thread brings per stage
    __shared__ __attribute__((aligned(16))) unsigned char As[GT * GPITCH];
    __shared__ __attribute__((aligned(16))) unsigned char Bs[GT * GPITCH];

    // flat index -> (sample, head, m tile, n tile), n fastest
    int64_t bid = blockIdx.x;
    const int tn = (int)(bid % tiles_n);
    bid /= tiles_n;
    const int tm = (int)(bid % tiles_m);
    bid /= tiles_m;
    const int hd = (int)(bid % h);
    const int i = (int)(bid / h);

    const int64_t sa = a_off[i], la = a_off[i + 1] - sa;
    const int64_t sb = b_off[i], lb = b_off[i + 1] - sb;
    const int64_t m = ta ? ka : la, kk = ta ? la : ka;
    const int64_t nn = tb ? lb : kb;
    const int64_t ro = ta ? (int64_t)i * ka : sa;
    const int64_t r0 = (int64_t)tm * GT, c0 = (int64_t)tn * GT;
    if (r0 >= m || c0 >= nn || c0 >= out_cols) return;      // the whole workgroup
    const T *ai = a + ((int64_t)hd * La + sa) * ka;
    const T *bi = b + ((int64_t)hd * Lb + sb) * kb;

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = wv >> 1, wn = wv & 1;                    // this wave's 32 x 32 block of the tile
    const int fr = lane & 31, fg = lane >> 5;               // fragment row and 16-byte half of a slab

    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;

    // One operand's stage: tile rows rows0 .. of `nrows`, K values t0 .. of kk, from `base` with leading dimension
    // ld.  along_k: the source is contiguous along K (element (r, t) = base[(rows0 + r) ld + t0 + t]), else along the
    // tile row (base[(t0 + t) ld + rows0 + r]).  vec: 16-byte loads (rows of the source 16-byte aligned, which also
    // makes the contiguous extent a whole number of vectors), else element by element.
    auto stage = [&](const T *base, int64_t ld, bool along_k, bool vec, int64_t rows0, int64_t nrows, int64_t t0,
                     unsigned char *S) {
        constexpr int VEC = Elem<T>::VEC;
        if (vec) {
            // GT * KT / VEC = 256 vectors: one a thread
            if (along_k) {
                const int r = tid / (KT / VEC), t = (tid % (KT / VEC)) * VEC;
                u32x4 v = {0u, 0u, 0u, 0u};
                if (rows0 + r < nrows && t0 + t < kk) v = *reinterpret_cast<const u32x4 *>(base + (rows0 + r) * ld + t0 + t);
                *reinterpret_cast<u32x4 *>(S + r * GPITCH + t * (int)sizeof(T)) = v;
            } else {
                const int r = (tid % (GT / VEC)) * VEC, t = tid / (GT / VEC);
                alignas(16) T v[VEC];
#pragma unroll
                for (int j = 0; j < VEC; j++) v[j] = T(0);
                if (rows0 + r < nrows && t0 + t < kk)
                    *reinterpret_cast<u32x4 *>(v) = *reinterpret_cast<const u32x4 *>(base + (t0 + t) * ld + rows0 + r);
#pragma unroll
                for (int j = 0; j < VEC; j++) *reinterpret_cast<T *>(S + (r + j) * GPITCH + t * (int)sizeof(T)) = v[j];
            }
            return;
        }
#pragma unroll
        for (int e = 0; e < PER; e++) {
            const int idx = tid + 256 * e;
            // the index runs along the contiguous dimension of the source
            int r, t;
            if (along_k) { t = idx % KT; r = idx / KT; } else { r = idx % GT; t = idx / GT; }
            T v = T(0);
            if (rows0 + r < nrows && t0 + t < kk) v = along_k ? base[(rows0 + r) * ld + t0 + t] : base[(t0 + t) * ld + rows0 + r];
            *reinterpret_cast<T *>(S + r * GPITCH + t * (int)sizeof(T)) = v;
        }
    };

    for (int64_t t0 = 0; t0 < kk; t0 += KT) {
        stage(ai, ka, !ta, vec_a, r0, m, t0, As);       // op(A): tile rows are output rows
        stage(bi, kb, tb, vec_b, c0, nn, t0, Bs);       // op(B)^T: tile rows are output columns
        __syncthreads();
#pragma unroll
        for (int s = 0; s < GSB / 32; s++) {
            const u32x4 fa = *reinterpret_cast<const u32x4 *>(As + (wm * 32 + fr) * GPITCH + s * 32 + fg * 16);
            const u32x4 fb = *reinterpret_cast<const u32x4 *>(Bs + (wn * 32 + fr) * GPITCH + s * 32 + fg * 16);
            Slab<T>::mma(fa, fb, acc);
        }
        __syncthreads();
    }

    // the 32 x 32 block: lane (column fr, row group fg) holds rows 8 (v / 4) + 4 fg + v % 4 in acc[v]
    const int64_t c = c0 + wn * 32 + fr;
    if (c < nn && c < out_cols) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int64_t r = r0 + wm * 32 + 8 * (v >> 2) + 4 * fg + (v & 3);
            if (r < m) Elem<T>::store(out + ((int64_t)hd * out_rows + ro + r) * out_cols + c, acc[v]);
        }
    }
}

}  // namespace vtdge

using namespace vtdge;

extern "C" int vtdge_batched_sparse_gemm(const void *a, const void *b, const int64_t *a_offsets,
                                         const int64_t *b_offsets, void *out, int B, int h, int64_t La, int ka,
                                         int64_t Lb, int kb, int trans_a, int trans_b, int64_t out_rows,
                                         int64_t out_cols, int64_t max_m, int dtype, void *stream)
{
    VT_REQUIRE(a && b && a_offsets && b_offsets && out, VTDGE_ERR_ARG, "batched_sparse_gemm: NULL operand");
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "batched_sparse_gemm: unknown dtype %d",
               dtype);
    VT_REQUIRE(B > 0 && h > 0 && ka > 0 && kb > 0 && La >= 0 && Lb >= 0 && out_rows >= 0 && out_cols >= 0 &&
                   max_m >= 0,
               VTDGE_ERR_ARG, "batched_sparse_gemm: bad sizes");
    if (max_m == 0 || out_cols == 0) return VTDGE_OK;
    const int64_t tiles_m = ceil_div(max_m, GT), tiles_n = ceil_div(out_cols, GT);
    const int64_t total = tiles_m * tiles_n * B * h;
    VT_REQUIRE(tiles_m < (1ll << 31) && tiles_n < (1ll << 31) && total < (1ll << 31), VTDGE_ERR_UNSUPPORTED,
               "batched_sparse_gemm: %lld output tiles exceed one launch", (long long)total);
    dim3 grid((unsigned)total), block(256);
    hipStream_t st = (hipStream_t)stream;
    // 16-byte loads for an operand whose rows start on 16-byte boundaries
    const int64_t esz = dtype == VTDGE_F32 ? 4 : 2;
    const bool vec_a = (ka * esz) % 16 == 0 && ((uintptr_t)a & 15) == 0;
    const bool vec_b = (kb * esz) % 16 == 0 && ((uintptr_t)b & 15) == 0;
    if (dtype == VTDGE_F32)
        note_kernel(reinterpret_cast<const void *>(sparse_gemm_kernel<float>)),
        sparse_gemm_kernel<float><<<grid, block, 0, st>>>((const float *)a, (const float *)b, a_offsets, b_offsets,
                                                          (float *)out, h, La, ka, Lb, kb, trans_a, trans_b, out_rows,
                                                          out_cols, (int)tiles_m, (int)tiles_n, vec_a, vec_b);
    else
        note_kernel(reinterpret_cast<const void *>(sparse_gemm_kernel<bf16_t>)),
        sparse_gemm_kernel<bf16_t><<<grid, block, 0, st>>>((const bf16_t *)a, (const bf16_t *)b, a_offsets,
                                                           b_offsets, (bf16_t *)out, h, La, ka, Lb, kb, trans_a,
                                                           trans_b, out_rows, out_cols, (int)tiles_m, (int)tiles_n, vec_a, vec_b);
    return check_launch("batched_sparse_gemm");
}
