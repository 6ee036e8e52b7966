// Sparse attention of packed queries against each sample's full K/V (gfx950).
//
// One 256-thread workgroup = (sample, head, chunk of 128 packed query rows);
// each of its 4 waves owns 32 query rows.  K/V of the sample are streamed
// through LDS 128 keys at a time with an online (running max / running sum)
// softmax, so the [h, L, n] score tensor the reference materialises in HBM
// (batched_sparse_gemm.cu:249) never exists.
//
// MFMA mapping (32x32 blocks, see Slab<> for the operand geometry):
//   S^T = K Q^T : keys are the M dimension, queries the N dimension.  A lane
//         then owns ONE query (column lane%32) and 16 keys per block, so the
//         softmax row reductions are in-register plus one exchange with
//         lane^32, and P never has to move between lanes before the second
//         product.
//   O^T = V^T P^T : head-dim is M, queries N, keys the contraction.  The P
//         values a lane holds after the first product are exactly the B
//         fragment of the second (the key order inside a fragment is a fixed
//         permutation, applied identically to the V^T fragment read from LDS).
//   V is transposed into LDS ([d][key]) while it is staged.
#include "common.h"

namespace vtdge {

constexpr int QROWS = 128;   // query rows per workgroup
constexpr int KSTAGE = 128;  // keys per LDS stage (4 blocks of 32)

template <typename T> struct ExpFn;
template <> struct ExpFn<float> {
    static __device__ __forceinline__ float f(float x) { return expf(x); }
};
template <> struct ExpFn<bf16_t> {
    static __device__ __forceinline__ float f(float x) { return __expf(x); }
};

template <typename T, int D>
__global__ __launch_bounds__(256) void sparse_attention_kernel(
    const T *__restrict__ q, int64_t q_rs, int64_t q_hs, const T *__restrict__ k, const T *__restrict__ v,
    int64_t kv_bs, int64_t kv_ts, int64_t kv_hs, const int64_t *__restrict__ offsets, T *__restrict__ out,
    int64_t o_rs, int64_t o_hs, int n, int qchunks, float scale)
{
    constexpr int ESZ = sizeof(T);
    constexpr int ROWB = D * ESZ;            // bytes of one K/V row (one head)
    constexpr int NSLAB = ROWB / 32;         // 32-byte slabs along d
    constexpr int KP = ROWB + 16;            // K row pitch in LDS
    constexpr int VP = KSTAGE * ESZ + 16;    // V^T row pitch in LDS
    constexpr int CPR = ROWB / 16;           // 16-byte chunks per K/V row
    constexpr int DB = D / 32;               // 32-wide head-dim blocks
    constexpr int VEC = 16 / ESZ;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem;
    unsigned char *Vt = smem + KSTAGE * KP;

    const int b = blockIdx.x / qchunks, qc = blockIdx.x % qchunks;
    const int head = blockIdx.y;
    const int64_t row0 = offsets[b];
    const int Lb = (int)(offsets[b + 1] - row0);
    if (qc * QROWS >= Lb) return;

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const int qrow = qc * QROWS + wid * 32 + lr;     // row of this lane's query inside the sample
    const bool wave_live = qc * QROWS + wid * 32 < Lb;
    const bool row_live = qrow < Lb;

    // Q fragments (B operand of S^T): bytes [32 s + 16 g, +16) of the query row
    u32x4 qf[NSLAB];
    {
        const unsigned char *qp =
            reinterpret_cast<const unsigned char *>(q + (row0 + qrow) * q_rs + (int64_t)head * q_hs) + lg * 16;
#pragma unroll
        for (int s = 0; s < NSLAB; s++) {
            u32x4 z = {0u, 0u, 0u, 0u};
            qf[s] = row_live ? *reinterpret_cast<const u32x4 *>(qp + s * 32) : z;
        }
    }

    f32x16 o[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const T *kb_ptr = k + (int64_t)b * kv_bs + (int64_t)head * kv_hs;
    const T *vb_ptr = v + (int64_t)b * kv_bs + (int64_t)head * kv_hs;

    for (int key0 = 0; key0 < n; key0 += KSTAGE) {
        // ---- stage K rows and V^T into LDS (zero beyond n)
        for (int idx = tid; idx < KSTAGE * CPR; idx += 256) {
            const int kr = idx / CPR, ch = idx % CPR;
            const int key = key0 + kr;
            u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
            if (key < n) {
                kk = *reinterpret_cast<const u32x4 *>(kb_ptr + (int64_t)key * kv_ts + ch * VEC);
                vv = *reinterpret_cast<const u32x4 *>(vb_ptr + (int64_t)key * kv_ts + ch * VEC);
            }
            *reinterpret_cast<u32x4 *>(Ks + kr * KP + ch * 16) = kk;
            if constexpr (ESZ == 2) {
                const uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint16_t h16 = (uint16_t)(e & 1 ? w[e >> 1] >> 16 : w[e >> 1] & 0xffffu);
                    *reinterpret_cast<uint16_t *>(Vt + (ch * 8 + e) * VP + kr * 2) = h16;
                }
            } else {
                const uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
                for (int e = 0; e < 4; e++) *reinterpret_cast<uint32_t *>(Vt + (ch * 4 + e) * VP + kr * 4) = w[e];
            }
        }
        __syncthreads();

        if (wave_live) {
            const int nb = min(KSTAGE / 32, (n - key0 + 31) / 32);
            // ---- S^T blocks
            f32x16 s[KSTAGE / 32];
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < KSTAGE / 32; kb++) {
                if (kb < nb) {
#pragma unroll
                    for (int e = 0; e < 16; e++) s[kb][e] = 0.f;
                    const unsigned char *kp = Ks + (kb * 32 + lr) * KP + lg * 16;
#pragma unroll
                    for (int sl = 0; sl < NSLAB; sl++) {
                        const u32x4 kf = *reinterpret_cast<const u32x4 *>(kp + sl * 32);
                        Slab<T>::mma(kf, qf[sl], s[kb]);
                    }
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const int key = key0 + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3);
                        const float sv = key < n ? s[kb][e] * scale : -INFINITY;
                        s[kb][e] = sv;
                        mx = fmaxf(mx, sv);
                    }
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(m_run, mx);
            const float alpha = ExpFn<T>::f(m_run - m_new);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < DB; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) o[i][e] *= alpha;
            // ---- P = exp(S - m), O^T += V^T P^T
#pragma unroll
            for (int kb = 0; kb < KSTAGE / 32; kb++) {
                if (kb < nb) {
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const float p = ExpFn<T>::f(s[kb][e] - m_new);
                        s[kb][e] = p;
                        l_run += p;
                    }
                    if constexpr (ESZ == 2) {
#pragma unroll
                        for (int t = 0; t < 2; t++) {
                            u32x4 pf;
                            pf.x = pack_bf16x2(s[kb][8 * t + 0], s[kb][8 * t + 1]);
                            pf.y = pack_bf16x2(s[kb][8 * t + 2], s[kb][8 * t + 3]);
                            pf.z = pack_bf16x2(s[kb][8 * t + 4], s[kb][8 * t + 5]);
                            pf.w = pack_bf16x2(s[kb][8 * t + 6], s[kb][8 * t + 7]);
#pragma unroll
                            for (int db = 0; db < DB; db++) {
                                const unsigned char *vp = Vt + (db * 32 + lr) * VP + (kb * 32 + 16 * t + 4 * lg) * 2;
                                const u32x2 lo = *reinterpret_cast<const u32x2 *>(vp);
                                const u32x2 hi = *reinterpret_cast<const u32x2 *>(vp + 16);
                                u32x4 vf;
                                vf.x = lo.x; vf.y = lo.y; vf.z = hi.x; vf.w = hi.y;
                                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf),
                                                                               __builtin_bit_cast(bf16x8, pf), o[db],
                                                                               0, 0, 0);
                            }
                        }
                    } else {
#pragma unroll
                        for (int g4 = 0; g4 < 4; g4++) {
#pragma unroll
                            for (int db = 0; db < DB; db++) {
                                const unsigned char *vp = Vt + (db * 32 + lr) * VP + (kb * 32 + 8 * g4 + 4 * lg) * 4;
                                const u32x4 vf = *reinterpret_cast<const u32x4 *>(vp);
                                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(vf.x), s[kb][4 * g4 + 0],
                                                                            o[db], 0, 0, 0);
                                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(vf.y), s[kb][4 * g4 + 1],
                                                                            o[db], 0, 0, 0);
                                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(vf.z), s[kb][4 * g4 + 2],
                                                                            o[db], 0, 0, 0);
                                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(vf.w), s[kb][4 * g4 + 3],
                                                                            o[db], 0, 0, 0);
                            }
                        }
                    }
                }
            }
        }
        __syncthreads();
    }

    if (!wave_live) return;
    const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    if (!row_live) return;
    const float inv = 1.0f / l_tot;
    T *op = out + (row0 + qrow) * o_rs + (int64_t)head * o_hs;
#pragma unroll
    for (int db = 0; db < DB; db++) {
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
            const int d0 = db * 32 + 8 * g4 + 4 * lg;
            float f[4];
#pragma unroll
            for (int e = 0; e < 4; e++) f[e] = o[db][4 * g4 + e] * inv;
            if constexpr (ESZ == 2) {
                u32x2 w;
                w.x = pack_bf16x2(f[0], f[1]);
                w.y = pack_bf16x2(f[2], f[3]);
                *reinterpret_cast<u32x2 *>(op + d0) = w;
            } else {
                *reinterpret_cast<f32x4 *>(op + d0) = f32x4{f[0], f[1], f[2], f[3]};
            }
        }
    }
}

template <typename T, int D>
static int launch_attention(const void *q, int64_t q_rs, int64_t q_hs, const void *k, const void *v, int64_t kv_bs,
                            int64_t kv_ts, int64_t kv_hs, const int64_t *offsets, void *out, int64_t o_rs,
                            int64_t o_hs, int B, int h, int n, int max_rows, float scale, hipStream_t st)
{
    constexpr int ESZ = sizeof(T);
    const size_t lds = (size_t)KSTAGE * (D * ESZ + 16) + (size_t)D * (KSTAGE * ESZ + 16);
    const int qchunks = (int)ceil_div(max_rows, QROWS);
    auto kern = sparse_attention_kernel<T, D>;
    VT_RESERVE_LDS(kern, lds, "sparse_attention");
    dim3 grid((unsigned)((int64_t)B * qchunks), (unsigned)h), block(256);
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<grid, block, lds, st>>>((const T *)q, q_rs, q_hs, (const T *)k, (const T *)v, kv_bs, kv_ts, kv_hs, offsets,
                                   (T *)out, o_rs, o_hs, n, qchunks, scale);
    return check_launch("sparse_attention");
}

// bf16 / head_dim 64 fast path (attention_dma.hip)
int launch_attention_bf16_d64(const void *q, int64_t q_rs, int64_t q_hs, const void *k, const void *v, int64_t kv_bs,
                              int64_t kv_ts, int64_t kv_hs, const int64_t *offsets, void *out, int64_t o_rs,
                              int64_t o_hs, int B, int h, int n, int max_rows, float scale, hipStream_t st);

}  // namespace vtdge

using namespace vtdge;

extern "C" int vtdge_sparse_attention(const void *q, int64_t q_row_stride, int64_t q_head_stride, const void *k,
                                      const void *v, int64_t kv_batch_stride, int64_t kv_tok_stride,
                                      int64_t kv_head_stride, const int64_t *offsets, void *out, int64_t o_row_stride,
                                      int64_t o_head_stride, int B, int h, int d, int n, int max_rows_per_sample,
                                      float scale, int dtype, void *stream)
{
    VT_REQUIRE(q && k && v && offsets && out, VTDGE_ERR_ARG, "sparse_attention: NULL operand");
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "sparse_attention: unknown dtype %d", dtype);
    VT_REQUIRE(B > 0 && h > 0 && n > 0 && max_rows_per_sample >= 0, VTDGE_ERR_ARG, "sparse_attention: bad sizes");
    VT_REQUIRE(d == 64 || d == 32, VTDGE_ERR_UNSUPPORTED, "sparse_attention: head_dim %d (only 32 and 64 are built)",
               d);
    VT_REQUIRE(h <= 65535, VTDGE_ERR_UNSUPPORTED, "sparse_attention: too many heads");
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(q_row_stride % vec == 0 && q_head_stride % vec == 0 && kv_batch_stride % vec == 0 &&
                   kv_tok_stride % vec == 0 && kv_head_stride % vec == 0 && o_row_stride % 4 == 0 &&
                   o_head_stride % 4 == 0,
               VTDGE_ERR_UNSUPPORTED, "sparse_attention: strides must keep 16-byte alignment");
    VT_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0, VTDGE_ERR_ARG,
               "sparse_attention: operands must be 16-byte aligned");
    if (max_rows_per_sample == 0) return VTDGE_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == VTDGE_BF16 && d == 64 && scale > 0.f && (int64_t)n * kv_tok_stride * 2 < (1LL << 31))
        return launch_attention_bf16_d64(q, q_row_stride, q_head_stride, k, v, kv_batch_stride, kv_tok_stride,
                                         kv_head_stride, offsets, out, o_row_stride, o_head_stride, B, h, n,
                                         max_rows_per_sample, scale, st);
#define VT_ATT(T, D)                                                                                                 \
    return launch_attention<T, D>(q, q_row_stride, q_head_stride, k, v, kv_batch_stride, kv_tok_stride,             \
                                  kv_head_stride, offsets, out, o_row_stride, o_head_stride, B, h, n,               \
                                  max_rows_per_sample, scale, st)
    if (dtype == VTDGE_F32) {
        if (d == 64) VT_ATT(float, 64);
        VT_ATT(float, 32);
    } else {
        if (d == 64) VT_ATT(bf16_t, 64);
        VT_ATT(bf16_t, 32);
    }
#undef VT_ATT
}
