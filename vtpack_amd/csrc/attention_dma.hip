// Sparse attention, bf16 / head_dim 64 fast path (gfx950).
//
// Same mathematics and MFMA mapping as attention.hip (S^T = K Q^T, O^T = V^T P^T, online softmax, a lane owns one
// query), restructured around what limits this operator at head_dim 64: the softmax VALU work (about 8 lane-ops
// per score against 0.25 MFMA cycles) and the K/V staging.
//   * K/V stages of 128 keys are double buffered in LDS: while stage s is multiplied, K of stage s+1 arrives by
//     direct loads (global_load_lds, 128-byte rows, XOR-swizzled 16-byte chunks, no padding) and V of stage s+1
//     sits in registers, to be written transposed ([d][key], key groups XOR-swizzled by d to spread the 2-byte
//     writes over the banks) after the multiply.  One barrier per stage.
//   * the softmax works in the log2 domain: p = exp2(fma(s, scale*log2(e), -m)); the running maximum is taken on
//     the raw scores (scale > 0), and key masking is only applied in a stage that contains the end of the keys.
#include "common.h"
#include <stdlib.h>

namespace vtdge {

constexpr int AQ = 128;    // query rows per workgroup (4 waves x 32)
constexpr int AK = 128;    // keys per stage
constexpr int AVP = AK * 2 + 16;                    // V^T row pitch (bytes)
constexpr int ABUF = AK * 128 + 64 * AVP;           // one K + V^T buffer

// One stage of up to 128 keys for a wave's 32 queries (online softmax update + O^T += V^T P^T).
//   ks: first K row of the stage in LDS (128-byte rows, XOR-swizzled chunks);  vt: V^T base in LDS, rows of
//   `vpitch` bytes whose key columns start at `vcol`;  key0: index of the stage's first key;  FULL: all 128 exist.
template <bool FULL>
__device__ __forceinline__ void attn_stage(const unsigned char *ks, const unsigned char *vt, int vpitch, int vcol,
                                           int key0, int n, int lr, int lg, const int (&cs)[4], const u32x4 (&qf)[4],
                                           f32x16 (&o)[2], float &m_run, float &l_run, float c)
{
    const int nb = FULL ? 4 : (n - key0 + 31) / 32;
    int vsw[2];                                                  // key-group swizzle of this lane's two V^T rows
#pragma unroll
    for (int db = 0; db < 2; db++) vsw[db] = 8 * (((db * 32 + lr) >> 4) & 3);
    f32x16 s[4];
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 4; kb++) {
        if (FULL || kb < nb) {
#pragma unroll
            for (int e = 0; e < 16; e++) s[kb][e] = 0.f;
            const unsigned char *kp = ks + (kb * 32 + lr) * 128;
#pragma unroll
            for (int sl = 0; sl < 4; sl++) {
                const u32x4 kf = *reinterpret_cast<const u32x4 *>(kp + cs[sl]);
                Slab<bf16_t>::mma(kf, qf[sl], s[kb]);
            }
            if constexpr (!FULL) {
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int key = key0 + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3);
                    if (key >= n) s[kb][e] = -INFINITY;
                }
            }
#pragma unroll
            for (int e = 0; e < 16; e++) mx = fmaxf(mx, s[kb][e]);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m_run, mx * c);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[i][e] *= alpha;
#pragma unroll
    for (int kb = 0; kb < 4; kb++) {
        if (FULL || kb < nb) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], c, -m_new));
                s[kb][e] = p;
                l_run += p;
            }
#pragma unroll
            for (int t = 0; t < 2; t++) {
                u32x4 pf;
                pf.x = pack_bf16x2(s[kb][8 * t + 0], s[kb][8 * t + 1]);
                pf.y = pack_bf16x2(s[kb][8 * t + 2], s[kb][8 * t + 3]);
                pf.z = pack_bf16x2(s[kb][8 * t + 4], s[kb][8 * t + 5]);
                pf.w = pack_bf16x2(s[kb][8 * t + 6], s[kb][8 * t + 7]);
#pragma unroll
                for (int db = 0; db < 2; db++) {
                    const unsigned char *vp = vt + (db * 32 + lr) * vpitch + vcol * 2;
                    const int k0 = kb * 32 + 16 * t + 4 * lg;
                    const u32x2 lo = *reinterpret_cast<const u32x2 *>(vp + ((k0) ^ vsw[db]) * 2);
                    const u32x2 hi = *reinterpret_cast<const u32x2 *>(vp + ((k0 + 8) ^ vsw[db]) * 2);
                    u32x4 vf;
                    vf.x = lo.x; vf.y = lo.y; vf.z = hi.x; vf.w = hi.y;
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf),
                                                                   __builtin_bit_cast(bf16x8, pf), o[db], 0, 0, 0);
                }
            }
        }
    }
}

// normalise and store this lane's query row
__device__ __forceinline__ void attn_store(bf16_t *op, const f32x16 (&o)[2], float l_tot, int lg)
{
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < 2; db++) {
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
            const int d0 = db * 32 + 8 * g4 + 4 * lg;
            u32x2 w;
            w.x = pack_bf16x2(o[db][4 * g4 + 0] * inv, o[db][4 * g4 + 1] * inv);
            w.y = pack_bf16x2(o[db][4 * g4 + 2] * inv, o[db][4 * g4 + 3] * inv);
            *reinterpret_cast<u32x2 *>(op + d0) = w;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Resident variant for short key sequences (n <= 288, e.g. 257 tokens at 256 px): one workgroup per (sample,
// head) stages that sample's whole K and V^T once (one exposed memory latency, no re-staging per query chunk),
// then its four waves walk the sample's 32-row query tiles independently, without further barriers.
//
// V^T layout in LDS: row d holds the keys in groups of 16; inside a group key 8h + 4g + j sits at position
// 8g + 4h + j, so the 8 keys a lane feeds to one MFMA (its P fragment holds keys 4g + j and 8 + 4g + j) are 16
// contiguous bytes; the group index is XOR-ed with (d >> 4) & 3, which spreads the 2-byte transposing writes over
// all banks; rows are padded by 16 B, which keeps the 16-byte fragment reads conflict free.
//
// Softmax: the keys are cut into equal stages of at most 4 blocks of 32 (257 keys: 3 stages of 3 blocks).  The
// running reference m of a row is only raised when a stage's maximum exceeds it by more than 8 (log2 units), so
// p = exp2(s*c - m) <= 256 and the rescaling of the output accumulators is skipped in most stages; the result is
// the same softmax (any reference cancels in the final division).
constexpr float ATT_RESCALE = 8.0f;

// acc + lo + hi of a packed bf16 pair in fp32 (v_dot2c_f32_bf16 against (1, 1))
__device__ __forceinline__ float bf16_pair_sum(uint32_t pair, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), __builtin_bit_cast(bf16x2, 0x3f803f80u),
                                           acc, false);
}

template <int NB, bool FULL>
__device__ __forceinline__ void attn_stage_resident(const unsigned char *kp, const unsigned char *vrow0,
                                                    const unsigned char *vrow1, int vsw0, int vsw1, int key0, int n,
                                                    int lg, const int (&cs)[4], const u32x4 (&qf)[4], f32x16 (&o)[2],
                                                    float &m_used, float &l_run, float c)
{
    // byte offsets of this stage's 16-key groups in the two V^T rows of the lane
    int voff0[2 * NB], voff1[2 * NB];
#pragma unroll
    for (int g = 0; g < 2 * NB; g++) {
        voff0[g] = ((key0 + 16 * g) ^ vsw0) * 2;
        voff1[g] = ((key0 + 16 * g) ^ vsw1) * 2;
    }
    f32x16 s[NB];
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NB; kb++) {
#pragma unroll
        for (int e = 0; e < 16; e++) s[kb][e] = 0.f;
#pragma unroll
        for (int sl = 0; sl < 4; sl++) {
            const u32x4 kf = *reinterpret_cast<const u32x4 *>(kp + kb * 32 * 128 + cs[sl]);
            Slab<bf16_t>::mma(kf, qf[sl], s[kb]);
        }
        if constexpr (!FULL) {
            if (kb == NB - 1) {        // only the last block of the last stage can run past the keys
                const int lim = n - key0 - kb * 32 - 4 * lg;
#pragma unroll
                for (int e = 0; e < 16; e++)
                    if (8 * (e >> 2) + (e & 3) >= lim) s[kb][e] = -INFINITY;
            }
        }
#pragma unroll
        for (int e = 0; e < 16; e++) mx = fmaxf(mx, s[kb][e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE)) * c;
    if (__builtin_amdgcn_ballot_w64(mx > m_used + ATT_RESCALE) != 0) {      // wave-uniform; rare after stage 0
        const float m_new = mx > m_used + ATT_RESCALE ? mx : m_used;
        const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);           // 0 on the first stage (m_used = -inf)
        l_run *= alpha;
        if (__builtin_amdgcn_ballot_w64(m_used > -INFINITY) != 0) {          // nothing accumulated yet on stage 0
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) o[i][e] *= alpha;
        }
        m_used = m_new;
    }
#pragma unroll
    for (int kb = 0; kb < NB; kb++) {
#pragma unroll
        for (int e = 0; e < 16; e++) s[kb][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], c, -m_used));
#pragma unroll
        for (int t = 0; t < 2; t++) {
            u32x4 pf;
            pf.x = pack_bf16x2(s[kb][8 * t + 0], s[kb][8 * t + 1]);
            pf.y = pack_bf16x2(s[kb][8 * t + 2], s[kb][8 * t + 3]);
            pf.z = pack_bf16x2(s[kb][8 * t + 4], s[kb][8 * t + 5]);
            pf.w = pack_bf16x2(s[kb][8 * t + 6], s[kb][8 * t + 7]);
            // the row sum is taken over the rounded probabilities, the values the second MFMA multiplies with
            l_run = bf16_pair_sum(pf.x, l_run);
            l_run = bf16_pair_sum(pf.y, l_run);
            l_run = bf16_pair_sum(pf.z, l_run);
            l_run = bf16_pair_sum(pf.w, l_run);
            const u32x4 v0 = *reinterpret_cast<const u32x4 *>(vrow0 + voff0[2 * kb + t]);
            const u32x4 v1 = *reinterpret_cast<const u32x4 *>(vrow1 + voff1[2 * kb + t]);
            o[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, v0),
                                                          __builtin_bit_cast(bf16x8, pf), o[0], 0, 0, 0);
            o[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, v1),
                                                          __builtin_bit_cast(bf16x8, pf), o[1], 0, 0, 0);
        }
    }
}

template <bool FULL>
__device__ __forceinline__ void attn_stage_resident_nb(int nb, const unsigned char *kp, const unsigned char *vrow0,
                                                       const unsigned char *vrow1, int vsw0, int vsw1, int key0,
                                                       int n, int lg, const int (&cs)[4], const u32x4 (&qf)[4],
                                                       f32x16 (&o)[2], float &m_used, float &l_run, float c)
{
    switch (nb) {
    case 4: attn_stage_resident<4, FULL>(kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c); break;
    case 3: attn_stage_resident<3, FULL>(kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c); break;
    case 2: attn_stage_resident<2, FULL>(kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c); break;
    default: attn_stage_resident<1, FULL>(kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c); break;
    }
}

__global__ __launch_bounds__(256, 2) void sparse_attention_bf16_d64_resident_kernel(
    const bf16_t *__restrict__ q, int64_t q_rs, int64_t q_hs, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, int64_t kv_bs, int64_t kv_ts, int64_t kv_hs, const int64_t *__restrict__ offsets,
    bf16_t *__restrict__ out, int64_t o_rs, int64_t o_hs, int n, float scale, int B, int h)
{
    constexpr int MAXV = 9;          // 16-byte V chunks per thread: covers n_pad = 288
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int b = blockIdx.x % B, head = blockIdx.x / B;
    const int64_t row0 = offsets[b];
    const int Lb = (int)(offsets[b + 1] - row0);
    if (Lb <= 0) return;
    const int npad = (n + 31) & ~31;
    const int vpitch = ((n + 63) & ~63) * 2 + 16;
    unsigned char *ks = smem;
    unsigned char *vt = smem + npad * 128;

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const unsigned char *kbase = reinterpret_cast<const unsigned char *>(k + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const unsigned char *vbase = reinterpret_cast<const unsigned char *>(v + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const int64_t row_bytes = kv_ts * 2;

    // Q fragments (B operand of S^T: bytes [32 s + 16 g, +16) of the query row) of this wave's first tile; the
    // fragments of tile rt + 4 are fetched while tile rt is processed
    auto load_q = [&](int rt, u32x4 (&dst)[4]) {
        const int qrow = rt * 32 + lr;
        const unsigned char *qp =
            reinterpret_cast<const unsigned char *>(q + (row0 + qrow) * q_rs + (int64_t)head * q_hs) + lg * 16;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            dst[s] = qrow < Lb ? *reinterpret_cast<const u32x4 *>(qp + s * 32) : z;
        }
    };
    u32x4 qf[4];
    load_q(wid, qf);

    // K by direct loads (wave-load j covers keys 8j..8j+7), V through registers
    for (int j = wid; j < npad / 8; j += 4) {
        const int r = j * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((r >> 1) & 7);
        const int key = r < n ? r : n - 1;
        VT_GLOBAL_TO_LDS(kbase + key * row_bytes + chunk * 16, ks + j * 1024);
    }
    u32x4 vreg[MAXV];
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int idx = tid + 256 * i;
        int key = idx >> 3;
        key = key < n ? key : n - 1;
        vreg[i] = *reinterpret_cast<const u32x4 *>(vbase + key * row_bytes + (idx & 7) * 16);
    }
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int idx = tid + 256 * i;
        const int kr = idx >> 3, ch = idx & 7;
        if (kr < npad) {
            // position of key kr in its row: bits 2 and 3 swapped inside the group of 16, group XOR-ed by d >> 4
            const int kpos = ((kr & ~12) | ((kr & 4) << 1) | ((kr & 8) >> 1)) ^ (16 * ((ch >> 1) & 3));
            const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint16_t h16 = (uint16_t)(e & 1 ? w[e >> 1] >> 16 : w[e >> 1] & 0xffffu);
                *reinterpret_cast<uint16_t *>(vt + (ch * 8 + e) * vpitch + kpos * 2) = h16;
            }
        }
    }
    wait_vmcnt<0>();
    __syncthreads();

    const int sw = (lr >> 1) & 7;
    int cs[4];
#pragma unroll
    for (int s = 0; s < 4; s++) cs[s] = ((2 * s + lg) ^ sw) * 16;
    const float c = scale * 1.44269504088896340736f;
    const int nblk = npad / 32;
    const int nstage = (nblk + 3) / 4;
    const int nbs = (nblk + nstage - 1) / nstage;          // blocks per stage (the last stage takes the rest)
    const unsigned char *vrow0 = vt + lr * vpitch + lg * 16;
    const unsigned char *vrow1 = vt + (32 + lr) * vpitch + lg * 16;
    const int vsw0 = 16 * ((lr >> 4) & 3), vsw1 = 16 * ((2 + (lr >> 4)) & 3);

    for (int rt = wid; rt * 32 < Lb; rt += 4) {
        const int qrow = rt * 32 + lr;
        const bool row_live = qrow < Lb;
        u32x4 qn[4];
        load_q(rt + 4, qn);            // zeros past the last tile
        f32x16 o[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) o[i][e] = 0.f;
        float m_used = -INFINITY, l_run = 0.f;
        for (int st = 0; st < nstage; st++) {
            const int key0 = st * nbs * 32;
            const int nb = st + 1 < nstage ? nbs : nblk - st * nbs;
            const unsigned char *kp = ks + (key0 + lr) * 128;
            if (key0 + nb * 32 <= n)
                attn_stage_resident_nb<true>(nb, kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c);
            else
                attn_stage_resident_nb<false>(nb, kp, vrow0, vrow1, vsw0, vsw1, key0, n, lg, cs, qf, o, m_used, l_run, c);
        }
        const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
        if (row_live) attn_store(out + (row0 + qrow) * o_rs + (int64_t)head * o_hs, o, l_tot, lg);
#pragma unroll
        for (int s = 0; s < 4; s++) qf[s] = qn[s];
    }
}

// ---------------------------------------------------------------------------------------------------------
// Streaming variant (any n): K/V stages of 128 keys double buffered in LDS, workgroup = 128 query rows.
__global__ __launch_bounds__(256, 2) void sparse_attention_bf16_d64_kernel(
    const bf16_t *__restrict__ q, int64_t q_rs, int64_t q_hs, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, int64_t kv_bs, int64_t kv_ts, int64_t kv_hs, const int64_t *__restrict__ offsets,
    bf16_t *__restrict__ out, int64_t o_rs, int64_t o_hs, int n, int qchunks, float scale)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int b = blockIdx.x / qchunks, qc = blockIdx.x % qchunks;
    const int head = blockIdx.y;
    const int64_t row0 = offsets[b];
    const int Lb = (int)(offsets[b + 1] - row0);
    if (qc * AQ >= Lb) return;

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const int qrow = qc * AQ + wid * 32 + lr;
    const bool wave_live = qc * AQ + wid * 32 < Lb;
    const bool row_live = qrow < Lb;

    // Q fragments (B operand of S^T): bytes [32 s + 16 g, +16) of the query row
    u32x4 qf[4];
    {
        const unsigned char *qp =
            reinterpret_cast<const unsigned char *>(q + (row0 + qrow) * q_rs + (int64_t)head * q_hs) + lg * 16;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            qf[s] = row_live ? *reinterpret_cast<const u32x4 *>(qp + s * 32) : z;
        }
    }

    const unsigned char *kbase = reinterpret_cast<const unsigned char *>(k + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const unsigned char *vbase = reinterpret_cast<const unsigned char *>(v + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const int64_t row_bytes = kv_ts * 2;
    const int nstage = (n + AK - 1) / AK;

    // K direct loads: wave-load j = wid*4 + i covers keys 8j..8j+7 of the stage
    auto issue_k = [&](int st) {
        unsigned char *dst = smem + (st & 1) * ABUF + wid * 4 * 1024;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int r = (wid * 4 + i) * 8 + (lane >> 3);
            const int chunk = (lane & 7) ^ ((r >> 1) & 7);
            int key = st * AK + r;
            key = key < n ? key : n - 1;
            VT_GLOBAL_TO_LDS(kbase + key * row_bytes + chunk * 16, dst + i * 1024);
        }
    };
    // V: thread -> (key, 16-byte chunk of d); registers now, transposed LDS writes later
    u32x4 vreg[4];
    auto load_v = [&](int st) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 256 * i;
            int key = st * AK + (idx >> 3);
            key = key < n ? key : n - 1;
            vreg[i] = *reinterpret_cast<const u32x4 *>(vbase + key * row_bytes + (idx & 7) * 16);
        }
    };
    auto store_v = [&](int st) {
        unsigned char *vt = smem + (st & 1) * ABUF + AK * 128;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 256 * i;
            const int kr = idx >> 3, ch = idx & 7;
            const int kpos = kr ^ (8 * ((ch >> 1) & 3));       // (d >> 4) & 3 with d = 8*ch + e
            const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint16_t h16 = (uint16_t)(e & 1 ? w[e >> 1] >> 16 : w[e >> 1] & 0xffffu);
                *reinterpret_cast<uint16_t *>(vt + (ch * 8 + e) * AVP + kpos * 2) = h16;
            }
        }
    };

    f32x16 o[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float c = scale * 1.44269504088896340736f;

    // fragment addressing
    const int sw = (lr >> 1) & 7;
    int cs[4];
#pragma unroll
    for (int s = 0; s < 4; s++) cs[s] = ((2 * s + lg) ^ sw) * 16;
    issue_k(0);
    load_v(0);
    store_v(0);
    for (int st = 0; st < nstage; st++) {
        wait_vmcnt<0>();                 // K of this stage (and nothing else is outstanding)
        __syncthreads();                 // K and V^T of stage st visible; the other buffer is free
        if (st + 1 < nstage) {
            issue_k(st + 1);
            load_v(st + 1);
        }
        if (wave_live) {
            const int key0 = st * AK;
            const unsigned char *ks = smem + (st & 1) * ABUF;
            if (key0 + AK <= n) attn_stage<true>(ks, ks + AK * 128, AVP, 0, key0, n, lr, lg, cs, qf, o, m_run, l_run, c);
            else attn_stage<false>(ks, ks + AK * 128, AVP, 0, key0, n, lr, lg, cs, qf, o, m_run, l_run, c);
        }
        if (st + 1 < nstage) store_v(st + 1);    // buffer (st+1)&1 was last read in iteration st-1
    }

    if (!wave_live) return;
    const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    if (row_live) attn_store(out + (row0 + qrow) * o_rs + (int64_t)head * o_hs, o, l_tot, lg);
}

int launch_attention_bf16_d64(const void *q, int64_t q_rs, int64_t q_hs, const void *k, const void *v, int64_t kv_bs,
                              int64_t kv_ts, int64_t kv_hs, const int64_t *offsets, void *out, int64_t o_rs,
                              int64_t o_hs, int B, int h, int n, int max_rows, float scale, hipStream_t st)
{
    if (n <= 288) {
        const int npad = (n + 31) & ~31;
        const size_t lds_r = (size_t)npad * 128 + 64 * ((size_t)((n + 63) & ~63) * 2 + 16);
        auto kern_r = sparse_attention_bf16_d64_resident_kernel;
        VT_RESERVE_LDS(kern_r, 80 * 1024, "sparse_attention");
        dim3 grid_r((unsigned)(B * h)), block_r(256);
        kern_r<<<grid_r, block_r, lds_r, st>>>((const bf16_t *)q, q_rs, q_hs, (const bf16_t *)k, (const bf16_t *)v,
                                               kv_bs, kv_ts, kv_hs, offsets, (bf16_t *)out, o_rs, o_hs, n, scale, B, h);
        return check_launch("sparse_attention");
    }
    const size_t lds = 2 * (size_t)ABUF;
    const int qchunks = (int)ceil_div(max_rows, AQ);
    auto kern = sparse_attention_bf16_d64_kernel;
    VT_RESERVE_LDS(kern, lds, "sparse_attention");
    dim3 grid((unsigned)((int64_t)B * qchunks), (unsigned)h), block(256);
    kern<<<grid, block, lds, st>>>((const bf16_t *)q, q_rs, q_hs, (const bf16_t *)k, (const bf16_t *)v, kv_bs, kv_ts,
                                   kv_hs, offsets, (bf16_t *)out, o_rs, o_hs, n, qchunks, scale);
    return check_launch("sparse_attention");
}

}  // namespace vtdge
