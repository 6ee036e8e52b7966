// Per-sample variable-length batched matmul over heads (gfx950).
//
// The reference loops over samples on the host and calls at::bmm / cuBLAS once
// per sample (batched_sparse_gemm.cu:150-195, :83-148).  Here one launch covers
// every (sample, head): blockIdx.z = sample * h + head, and each workgroup
// resolves its own operand slices from the device-side offsets, so no length
// ever has to visit the host.  The inference path of the models never calls
// this operator (only the unequal-length training branch does), so it is a
// plain LDS-tiled fp32-FMA kernel: 64x64 output tile, 16-deep K steps,
// 4x4 outputs per thread.
#include "common.h"

namespace vtdge {

constexpr int GT = 64;  // output tile edge
constexpr int GK = 16;  // K step

template <typename T>
__global__ __launch_bounds__(256) void sparse_gemm_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                           const int64_t *__restrict__ a_off,
                                                           const int64_t *__restrict__ b_off, T *__restrict__ out,
                                                           int h, int64_t La, int ka, int64_t Lb, int kb, int ta,
                                                           int tb, int64_t out_rows, int64_t out_cols)
{
    __shared__ float As[GK][GT + 1];
    __shared__ float Bs[GK][GT + 1];
    const int i = blockIdx.z / h, hd = blockIdx.z % h;
    const int64_t sa = a_off[i], la = a_off[i + 1] - sa;
    const int64_t sb = b_off[i], lb = b_off[i + 1] - sb;
    const int64_t m = ta ? ka : la, kk = ta ? la : ka;
    const int64_t nn = tb ? lb : kb;
    const int64_t ro = ta ? (int64_t)i * ka : sa;
    const int64_t r0 = (int64_t)blockIdx.x * GT, c0 = (int64_t)blockIdx.y * GT;
    if (r0 >= m || c0 >= nn || c0 >= out_cols) return;
    const T *ai = a + ((int64_t)hd * La + sa) * ka;
    const T *bi = b + ((int64_t)hd * Lb + sb) * kb;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    float acc[4][4];
#pragma unroll
    for (int p = 0; p < 4; p++)
#pragma unroll
        for (int q = 0; q < 4; q++) acc[p][q] = 0.f;

    for (int64_t t0 = 0; t0 < kk; t0 += GK) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int idx = threadIdx.x + 256 * e;
            // A tile: element (r, t).  Index so that the contiguous dimension of the source varies fastest.
            int r, t;
            if (ta) { r = idx % GT; t = idx / GT; } else { t = idx % GK; r = idx / GK; }
            float av = 0.f;
            if (r0 + r < m && t0 + t < kk)
                av = Elem<T>::load(ta ? ai + (t0 + t) * ka + (r0 + r) : ai + (r0 + r) * ka + (t0 + t));
            As[t][r] = av;
            int c, t2;
            if (tb) { t2 = idx % GK; c = idx / GK; } else { c = idx % GT; t2 = idx / GT; }
            float bv = 0.f;
            if (c0 + c < nn && t0 + t2 < kk)
                bv = Elem<T>::load(tb ? bi + (c0 + c) * kb + (t0 + t2) : bi + (t0 + t2) * kb + (c0 + c));
            Bs[t2][c] = bv;
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < GK; t++) {
            float av[4], bv[4];
#pragma unroll
            for (int p = 0; p < 4; p++) av[p] = As[t][ty * 4 + p];
#pragma unroll
            for (int q = 0; q < 4; q++) bv[q] = Bs[t][tx * 4 + q];
#pragma unroll
            for (int p = 0; p < 4; p++)
#pragma unroll
                for (int q = 0; q < 4; q++) acc[p][q] += av[p] * bv[q];
        }
        __syncthreads();
    }
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int64_t r = r0 + ty * 4 + p;
        if (r >= m) continue;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int64_t c = c0 + tx * 4 + q;
            if (c < nn && c < out_cols) Elem<T>::store(out + ((int64_t)hd * out_rows + ro + r) * out_cols + c, acc[p][q]);
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
    VT_REQUIRE((int64_t)B * h <= 65535, VTDGE_ERR_UNSUPPORTED, "batched_sparse_gemm: B*h=%lld exceeds 65535",
               (long long)B * h);
    if (max_m == 0 || out_cols == 0) return VTDGE_OK;
    dim3 grid((unsigned)ceil_div(max_m, GT), (unsigned)ceil_div(out_cols, GT), (unsigned)(B * h)), block(256);
    VT_REQUIRE(grid.y <= 65535, VTDGE_ERR_UNSUPPORTED, "batched_sparse_gemm: output too wide");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VTDGE_F32)
        sparse_gemm_kernel<float><<<grid, block, 0, st>>>((const float *)a, (const float *)b, a_offsets, b_offsets,
                                                          (float *)out, h, La, ka, Lb, kb, trans_a, trans_b, out_rows,
                                                          out_cols);
    else
        sparse_gemm_kernel<bf16_t><<<grid, block, 0, st>>>((const bf16_t *)a, (const bf16_t *)b, a_offsets,
                                                           b_offsets, (bf16_t *)out, h, La, ka, Lb, kb, trans_a,
                                                           trans_b, out_rows, out_cols);
    return check_launch("batched_sparse_gemm");
}
