// Grained sampling kernels for gfx950: router, index->patch compaction,
// compress (gather + window mean) and decompress (scatter back).
//
// All four are HBM-bandwidth or latency bound.  The element kernels give a
// group of GS lanes (64, 32, 16 or 8: the smallest that covers C with 16 bytes
// per lane) to one packed query row, so a row of C channels is read/written
// with fully coalesced 16-byte accesses and narrow rows (C = 64, 128: the
// first PVT stages) still keep every lane of the wavefront busy.
#include "common.h"
#include "region_pack.h"
#include <atomic>
#include <type_traits>

namespace vtdge {

constexpr int ROWS_PER_BLOCK = 4;  // one wave per row (GS = 64) or 64/GS rows per wave, 256 threads
constexpr int MAX_IT = 3;          // 16-byte vectors per lane: C <= 64*3*VEC

// lanes per row for a row of nvec 16-byte vectors
static int group_size(int nvec) { return nvec > 32 ? 64 : nvec > 16 ? 32 : nvec > 8 ? 16 : 8; }

// sum over the GS lanes of a row's group, returned in each of them
template <int GS, int NV> __device__ __forceinline__ void group_sum_n(float (&v)[NV])
{
    if constexpr (GS == 64) {
        wave_sum_n<NV>(v);
    } else {
#pragma unroll
        for (int o = GS / 2; o > 0; o >>= 1)
#pragma unroll
            for (int i = 0; i < NV; i++) v[i] += __shfl_xor(v[i], o, WAVE);
    }
}
template <int GS> __device__ __forceinline__ float group_sum(float v)
{
    if constexpr (GS == 64) {
        return wave_sum(v);
    } else {
#pragma unroll
        for (int o = GS / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
        return v;
    }
}

// LayerNorm of NR rows at once, one 16-byte vector of each row per lane of a GS-lane group (`active` false: the
// lane holds no channels and only takes part in the sums).  dst(t) is where the lane's vector of row t goes.
template <typename T, int GS, int NR, class F>
__device__ __forceinline__ void layernorm_rows(const u32x4 (&raw)[NR], bool active, const T *__restrict__ w,
                                               const T *__restrict__ bsrc, float eps, int C, F &&dst)
{
    constexpr int VEC = Elem<T>::VEC;
    float s[NR];
#pragma unroll
    for (int t = 0; t < NR; t++) {
        float f[VEC];
        Elem<T>::unpack(raw[t], f);
        s[t] = 0.f;
#pragma unroll
        for (int c = 0; c < VEC; c++) s[t] += f[c];
    }
    group_sum_n<GS, NR>(s);
    float q[NR];
#pragma unroll
    for (int t = 0; t < NR; t++) {
        s[t] = s[t] / (float)C;      // mean
        float f[VEC];
        Elem<T>::unpack(raw[t], f);
        q[t] = 0.f;
        if (active) {
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float dlt = f[c] - s[t];
                q[t] += dlt * dlt;
            }
        }
    }
    group_sum_n<GS, NR>(q);
    if (!active) return;          // after the last reduction
    float ww[VEC], bb[VEC];
    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(w), ww);
    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(bsrc), bb);
#pragma unroll
    for (int t = 0; t < NR; t++) {
        const float rstd = 1.0f / sqrtf(q[t] / (float)C + eps);
        float f[VEC], y[VEC];
        Elem<T>::unpack(raw[t], f);
#pragma unroll
        for (int c = 0; c < VEC; c++) y[c] = (f[c] - s[t]) * rstd * ww[c] + bb[c];
        *reinterpret_cast<u32x4 *>(dst(t)) = Elem<T>::pack(y);
    }
}

// ------------------------------------------------------------------ router
// One wave per region.  Replaces AvgPool2d(R,R) -> Linear(C,S) -> argmax
// (vtpack/layers/dge.py:145-150, :75).
//
// LNF: the wave also writes LayerNorm(x) of the tokens it has just read (and the wave of a sample's first region
// that of the sample's extra tokens): the block's first LayerNorm (vtpack/models/dge/deit_dge.py:127) without a
// second pass over x.  Same arithmetic as layernorm_kernel (two-pass statistics in fp32, the same reduction
// tree).  Needs RS > 0 and a row that fits one 16-byte vector per lane of the group.
template <typename T, int RS, int GS, bool LNF = false>   // RS = region size known at compile time (all window loads in flight), 0 = generic
__global__ __launch_bounds__(256) void router_kernel(const T *__restrict__ x, const T *__restrict__ weight,
                                                      const T *__restrict__ bias, T *__restrict__ gate,
                                                      int64_t *__restrict__ indices, int B, int H, int W,
                                                      int C, int extra, int R, int S,
                                                      const T *__restrict__ ln_w = nullptr,
                                                      const T *__restrict__ ln_b = nullptr, float eps = 0.f,
                                                      T *__restrict__ ln_out = nullptr)
{
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & (GS - 1);
    const int Hr = H / R, Wr = W / R;
    const int64_t region = ((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS;
    if (region >= (int64_t)B * Hr * Wr) return;
    const int b = (int)(region / (Hr * Wr));
    const int rr = (int)(region % (Hr * Wr));
    const int ry = rr / Wr, rx = rr % Wr;
    const int N = extra + H * W;
    const int nvec = C / VEC;
    const T *xb = x + (int64_t)b * N * C;
    const float area = (float)(R * R);

    float part[VTDGE_MAX_SPLITS];
#pragma unroll
    for (int s = 0; s < VTDGE_MAX_SPLITS; s++) part[s] = 0.f;

    if constexpr (LNF) {
        // one vector per lane (the host launches this variant only when nvec <= GS); every lane of the group takes
        // part in the reductions, lanes past the row with zeros
        static_assert(RS > 0, "the fused LayerNorm needs the region size at compile time");
        const bool act = lane < nvec;
        const int v = act ? lane : 0;
        const int64_t tok0 = (int64_t)(ry * R) * W + rx * R + extra;
        const T *base = xb + tok0 * C + v * VEC;
        u32x4 raw[RS * RS];
#pragma unroll
        for (int t = 0; t < RS * RS; t++) {
            raw[t] = u32x4{0u, 0u, 0u, 0u};
            if (act) raw[t] = *reinterpret_cast<const u32x4 *>(base + ((int64_t)(t / RS) * W + (t % RS)) * C);
        }
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = 0.f;
#pragma unroll
        for (int t = 0; t < RS * RS; t++) {
            float f[VEC];
            Elem<T>::unpack(raw[t], f);
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[i] += f[i];
        }
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = Elem<T>::round(acc[i] / area);
        if (act) {
#pragma unroll
            for (int s = 0; s < VTDGE_MAX_SPLITS; s++) {
                if (s < S) {
                    float w[VEC];
                    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(weight + (int64_t)s * C + v * VEC), w);
#pragma unroll
                    for (int i = 0; i < VEC; i++) part[s] += acc[i] * w[i];
                }
            }
        }
        T *ob = ln_out + (int64_t)b * N * C + tok0 * C + v * VEC;
        layernorm_rows<T, GS, RS * RS>(raw, act, ln_w + v * VEC, ln_b + v * VEC, eps, C,
                                       [&](int t) { return ob + ((int64_t)(t / RS) * W + (t % RS)) * C; });
        if (rr == 0) {           // the sample's extra tokens (a branch the whole group takes or not)
            for (int e = 0; e < extra; e++) {
                u32x4 one[1] = {u32x4{0u, 0u, 0u, 0u}};
                if (act) one[0] = *reinterpret_cast<const u32x4 *>(xb + (int64_t)e * C + v * VEC);
                T *oe = ln_out + (int64_t)b * N * C + (int64_t)e * C + v * VEC;
                layernorm_rows<T, GS, 1>(one, act, ln_w + v * VEC, ln_b + v * VEC, eps, C, [&](int) { return oe; });
            }
        }
    } else
    for (int v = lane; v < nvec; v += GS) {
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = 0.f;
        const T *base = xb + ((int64_t)(ry * R) * W + rx * R + extra) * C + v * VEC;
        if constexpr (RS > 0) {
            u32x4 raw[RS * RS];
#pragma unroll
            for (int dy = 0; dy < RS; dy++)
#pragma unroll
                for (int dx = 0; dx < RS; dx++)
                    raw[dy * RS + dx] = *reinterpret_cast<const u32x4 *>(base + ((int64_t)dy * W + dx) * C);
#pragma unroll
            for (int t = 0; t < RS * RS; t++) {
                float f[VEC];
                Elem<T>::unpack(raw[t], f);
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[i] += f[i];
            }
        } else {
            for (int dy = 0; dy < R; dy++) {
                for (int dx = 0; dx < R; dx++) {
                    u32x4 raw = *reinterpret_cast<const u32x4 *>(base + ((int64_t)dy * W + dx) * C);
                    float f[VEC];
                    Elem<T>::unpack(raw, f);
#pragma unroll
                    for (int i = 0; i < VEC; i++) acc[i] += f[i];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = Elem<T>::round(acc[i] / area);
#pragma unroll
        for (int s = 0; s < VTDGE_MAX_SPLITS; s++) {
            if (s < S) {
                u32x4 raw = *reinterpret_cast<const u32x4 *>(weight + (int64_t)s * C + v * VEC);
                float w[VEC];
                Elem<T>::unpack(raw, w);
#pragma unroll
                for (int i = 0; i < VEC; i++) part[s] += acc[i] * w[i];
            }
        }
    }
    float best = 0.f;
    int best_s = 0;
#pragma unroll
    for (int s = 0; s < VTDGE_MAX_SPLITS; s++) {
        if (s < S) {
            float logit = group_sum<GS>(part[s]) + Elem<T>::load(bias + s);
            logit = Elem<T>::round(logit);
            if (gate != nullptr && lane == 0) Elem<T>::store(gate + region * S + s, logit);
            if (s == 0 || logit > best) {  // strict >: lowest index wins a tie
                best = logit;
                best_s = s;
            }
        }
    }
    if (lane == 0) indices[region] = best_s;
}

// ------------------------------------------------------------ index->patch
// Step 1 (single workgroup): per-sample query counts and their exclusive scan, 1024 samples per pass.
// Counts: every thread reads gate indices with independent, coalesced loads and adds the query count of its
// region to its sample's LDS counter (integer atomics: order does not matter).
// Scan: wave-level shuffles + LDS for the wave totals.
__global__ __launch_bounds__(1024) void patch_count_scan_kernel(const int64_t *__restrict__ indices,
                                                                 const int64_t *__restrict__ splits, int B,
                                                                 int nreg, int S, int extra,
                                                                 int64_t *__restrict__ offsets,
                                                                 int64_t *__restrict__ lengths)
{
    __shared__ int64_t wave_tot[16];
    __shared__ int64_t carry_s;
    __shared__ int sq[VTDGE_MAX_SPLITS];
    __shared__ int cnt_s[1024];
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    if (threadIdx.x < VTDGE_MAX_SPLITS) {
        int ps = threadIdx.x < S ? (int)splits[threadIdx.x] : 0;
        sq[threadIdx.x] = ps * ps;
    }
    if (threadIdx.x == 0) carry_s = 0;
    for (int base = 0; base < B; base += 1024) {
        cnt_s[threadIdx.x] = 0;
        __syncthreads();
        const int nb = min(1024, B - base);
        for (int64_t i = threadIdx.x; i < (int64_t)nb * nreg; i += 1024) {
            int64_t g = indices[(int64_t)base * nreg + i];
            g = g < 0 ? 0 : (g >= S ? S - 1 : g);
            atomicAdd(&cnt_s[i / nreg], sq[g]);
        }
        __syncthreads();
        const int b = base + threadIdx.x;
        const int64_t v = b < B ? (int64_t)cnt_s[threadIdx.x] + extra : 0;
        if (b < B) lengths[b] = v;
        int64_t inc = v;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            int64_t up = __shfl_up(inc, o, WAVE);
            if (lane >= o) inc += up;
        }
        if (lane == 63) wave_tot[wid] = inc;
        __syncthreads();
        int64_t before = carry_s;
        for (int w = 0; w < wid; w++) before += wave_tot[w];
        if (b < B) offsets[b] = before + inc - v;
        __syncthreads();
        if (threadIdx.x == 1023) carry_s = before + inc;
        __syncthreads();
    }
    if (threadIdx.x == 0) offsets[B] = carry_s;
}

// Step 1 for batches of a few thousand samples: a wave per sample adds up the query counts of its regions ->
// lengths; the write kernel then finds each sample's first row from the lengths before it (no scan, and no single
// workgroup that reads every gate index of the batch).
__global__ __launch_bounds__(256) void patch_count_kernel(const int64_t *__restrict__ indices,
                                                           const int64_t *__restrict__ splits, int B, int nreg, int S,
                                                           int extra, int64_t *__restrict__ lengths)
{
    __shared__ int sq[VTDGE_MAX_SPLITS];
    if (threadIdx.x < VTDGE_MAX_SPLITS) {
        const int ps = threadIdx.x < S ? (int)splits[threadIdx.x] : 0;
        sq[threadIdx.x] = ps * ps;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= B) return;
    int part = 0;
    for (int i = lane; i < nreg; i += WAVE) {
        int64_t g = indices[(int64_t)b * nreg + i];
        g = g < 0 ? 0 : (g >= S ? S - 1 : g);
        part += sq[g];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, WAVE);
    if (lane == 0) lengths[b] = (int64_t)part + extra;
}

// Step 2: one workgroup per sample.  The per-region query counts go through an
// LDS-staged wavefront prefix sum (256 regions per pass); then every thread emits
// one descriptor per turn (row j of the sample: its region by binary search in the
// prefix sums), so a workgroup writes 256 consecutive 32-byte rows at a time.
//
// FUSED: the workgroup also finds its own first row, as the sum of the query counts of all samples before it (it
// reads their gate indices itself: a few KB out of L2 for the batch sizes this variant is launched for), and writes
// offsets / lengths; no first step then, and no dependency between workgroups.
// Not FUSED: the first row comes from `offsets` (written by the scan kernel) or, with from_lengths, is the sum of
// the lengths of the samples before this one (written by the count kernel), in which case the workgroup writes
// offsets as well.
typedef long long i64x2 __attribute__((ext_vector_type(2)));

template <bool FUSED>
__global__ __launch_bounds__(256) void patch_write_kernel(const int64_t *__restrict__ indices,
                                                           const int64_t *__restrict__ splits,
                                                           int64_t *__restrict__ offsets, int64_t *__restrict__ lengths,
                                                           int Hr, int Wr, int S, int R, int extra,
                                                           int64_t *__restrict__ patches, int64_t capacity,
                                                           int from_lengths)
{
    __shared__ int wave_tot[4];
    __shared__ int carry_s;
    __shared__ int split_s[VTDGE_MAX_SPLITS];
    __shared__ int64_t before_s[4];
    __shared__ int start_s[256], ps_s[256];
    const int b = blockIdx.x;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int nreg = Hr * Wr;
    // everything the workgroup reads is requested before anything is used: the splits, the first gate indices of
    // its own sample and (FUSED) sixteen per thread of the samples before it - one trip to memory instead of three
    const int sp = threadIdx.x < S ? (int)splits[threadIdx.x] : 1;
    int64_t g_first = 0;
    if (threadIdx.x < nreg) g_first = indices[(int64_t)b * nreg + threadIdx.x];
    constexpr int PRE = 16;
    const int64_t nbefore = FUSED ? (int64_t)b * nreg : 0;
    int64_t gq[PRE];
    if constexpr (FUSED) {
#pragma unroll
        for (int i = 0; i < PRE; i++) {
            const int64_t idx = threadIdx.x + 256 * (int64_t)i;
            gq[i] = idx < nbefore ? indices[idx] : 0;
        }
    }
    if (threadIdx.x < VTDGE_MAX_SPLITS) split_s[threadIdx.x] = sp;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    int64_t row0;
    if constexpr (FUSED) {
        int64_t part = 0;
#pragma unroll
        for (int i = 0; i < PRE; i++) {
            if (threadIdx.x + 256 * (int64_t)i < nbefore) {
                const int64_t g = gq[i] < 0 ? 0 : (gq[i] >= S ? S - 1 : gq[i]);
                const int ps = split_s[g];
                part += ps * ps;
            }
        }
        for (int64_t i = threadIdx.x + 256 * (int64_t)PRE; i < nbefore; i += 256) {
            int64_t g = indices[i];
            g = g < 0 ? 0 : (g >= S ? S - 1 : g);
            const int ps = split_s[g];
            part += ps * ps;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, WAVE);
        if (lane == 0) before_s[wid] = part;
        __syncthreads();
        row0 = before_s[0] + before_s[1] + before_s[2] + before_s[3] + (int64_t)b * extra;
        if (threadIdx.x == 0) offsets[b] = row0;
    } else if (from_lengths) {
        int64_t part = 0;
        for (int i = threadIdx.x; i < b; i += 256) part += lengths[i];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, WAVE);
        if (lane == 0) before_s[wid] = part;
        __syncthreads();
        row0 = before_s[0] + before_s[1] + before_s[2] + before_s[3];
        if (threadIdx.x == 0) {
            offsets[b] = row0;
            if (b == (int)gridDim.x - 1) offsets[b + 1] = row0 + lengths[b];
        }
    } else {
        row0 = offsets[b];
    }
    for (int e = threadIdx.x; e < extra; e += 256) {
        const int64_t row = row0 + e;
        if (row < capacity) {
            int64_t *p = patches + 4 * row;
            p[0] = b; p[1] = -(int64_t)e - 1; p[2] = 0; p[3] = 1;
        }
    }
    for (int base = 0; base < nreg; base += 256) {
        const int r = base + threadIdx.x;
        int ps = 0;
        if (r < nreg) {
            int64_t g = base == 0 ? g_first : indices[(int64_t)b * nreg + r];
            g = g < 0 ? 0 : (g >= S ? S - 1 : g);
            ps = split_s[g];
        }
        const int cnt = ps * ps;
        int inc = cnt;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            int up = __shfl_up(inc, o, WAVE);
            if (lane >= o) inc += up;
        }
        if (lane == 63) wave_tot[wid] = inc;
        __syncthreads();
        const int first = carry_s;                 // rows of the regions of earlier passes
        int before = first;
        for (int w = 0; w < wid; w++) before += wave_tot[w];
        // first row of the region (or, past the last region, one past the last row of the pass) and its split
        start_s[threadIdx.x] = before + inc - cnt;
        ps_s[threadIdx.x] = ps;
        __syncthreads();
        const int nr = min(256, nreg - base);
        const int last = start_s[nr - 1] + ps_s[nr - 1] * ps_s[nr - 1];
        // one descriptor per thread and turn: the region of row j is the last one that starts at or before j
        for (int j = first + threadIdx.x; j < last; j += 256) {
            int lo = 0, hi = nr - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (start_s[mid] <= j) lo = mid;
                else hi = mid - 1;
            }
            const int rps = ps_s[lo], local = j - start_s[lo];
            const int rg = base + lo, ry = rg / Wr, rx = rg % Wr;
            const int step = R / rps, dy = local / rps, dx = local - dy * rps;
            const int64_t row = row0 + extra + j;
            if (row < capacity) {
                i64x2 *p = reinterpret_cast<i64x2 *>(patches + 4 * row);
                const i64x2 lo2 = {(int64_t)b, (int64_t)ry * R + dy * step};
                const i64x2 hi2 = {(int64_t)rx * R + dx * step, (int64_t)step};
                p[0] = lo2;
                p[1] = hi2;
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) carry_s = last;
        __syncthreads();
    }
    if constexpr (FUSED) {
        if (threadIdx.x == 0) {
            const int64_t len = (int64_t)extra + carry_s;
            lengths[b] = len;
            if (b == (int)gridDim.x - 1) offsets[b + 1] = row0 + len;
        }
    }
}

struct DenseSplits {
    int n;
    int ps[VTDGE_MAX_SPLITS];
};

// One thread per descriptor; closed-form enumeration (grained_sample.cu:347-391).
__global__ __launch_bounds__(256) void patch_dense_kernel(DenseSplits sp, int B, int Hr, int Wr, int R, int extra,
                                                           int per_sample, int64_t *__restrict__ patches)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)B * per_sample) return;
    const int b = (int)(idx / per_sample);
    int j = (int)(idx % per_sample);
    int64_t *p = patches + 4 * idx;
    if (j < extra) {
        p[0] = b; p[1] = -(int64_t)j - 1; p[2] = 0; p[3] = 1;
        return;
    }
    j -= extra;
    for (int s = 0; s < sp.n; s++) {
        const int ps = sp.ps[s];
        const int len = Hr * Wr * ps * ps;
        if (j < len) {
            const int step = R / ps;
            p[0] = b;
            p[1] = (int64_t)(j / (Wr * ps)) * step;
            p[2] = (int64_t)(j % (Wr * ps)) * step;
            p[3] = step;
            return;
        }
        j -= len;
    }
}

// ---------------------------------------------------------------- compress
template <typename T, int SZ>
__device__ __forceinline__ void window_sum(const T *__restrict__ base, int W, int C, int sz,
                                           float (&acc)[Elem<T>::VEC])
{
    constexpr int VEC = Elem<T>::VEC;
    if constexpr (SZ > 0) {
        // at most eight loads in flight at a time (32 registers); the sum runs over the window in the same order
        constexpr int NT = SZ * SZ, NBATCH = NT > 8 ? 8 : NT;
#pragma unroll
        for (int t0 = 0; t0 < NT; t0 += NBATCH) {
            u32x4 raw[NBATCH];
#pragma unroll
            for (int i = 0; i < NBATCH; i++)
                raw[i] = *reinterpret_cast<const u32x4 *>(base + ((int64_t)((t0 + i) / SZ) * W + (t0 + i) % SZ) * C);
#pragma unroll
            for (int i = 0; i < NBATCH; i++) {
                float f[VEC];
                Elem<T>::unpack(raw[i], f);
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] += f[c];
            }
        }
    } else {
        for (int dy = 0; dy < sz; dy++)
            for (int dx = 0; dx < sz; dx++) {
                u32x4 raw = *reinterpret_cast<const u32x4 *>(base + ((int64_t)dy * W + dx) * C);
                float f[VEC];
                Elem<T>::unpack(raw, f);
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] += f[c];
            }
    }
}

// NIT = 16-byte vectors per lane (1 unless a row is longer than one vector per lane of a 64-lane group).  The
// one-vector variant is held to 64 registers so that its waves fit next to those of a weight-stationary Linear
// (one wave per SIMD and most of its registers), which the key/value projection keeps running on every CU meanwhile.
template <typename T, bool LN, int GS, int NIT>
__global__ __launch_bounds__(256, NIT == 1 ? 8 : 2) void compress_kernel(const T *__restrict__ x, const int64_t *__restrict__ patches,
                                                        const int64_t *__restrict__ rows_dev, int64_t rows,
                                                        T *__restrict__ out, T *__restrict__ ln_out,
                                                        const T *__restrict__ ln_w, const T *__restrict__ ln_b,
                                                        float eps, int N, int C, int W, int extra)
{
    constexpr int VEC = Elem<T>::VEC;
    static_assert(NIT == 1 || GS == 64, "several vectors per lane only with whole-wave groups");
    const int lane = threadIdx.x & (GS - 1);
    const int64_t row = ((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS;
    if (row >= live_rows(rows_dev, rows)) return;
    const int64_t *p = patches + 4 * row;
    const int64_t b = p[0], y0 = p[1], x0 = p[2];
    const int sz = (int)p[3];
    const int nvec = C / VEC;
    const T *xb = x + b * (int64_t)N * C;

    float vals[NIT][VEC];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int v = it * WAVE + lane;
        if (v < nvec) {
            float acc[VEC];
            if (y0 < 0) {
                u32x4 raw = *reinterpret_cast<const u32x4 *>(xb + (-y0 - 1) * (int64_t)C + v * VEC);
                Elem<T>::unpack(raw, acc);
            } else {
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] = 0.f;
                const T *base = xb + ((y0 * W + x0 + extra) * (int64_t)C + v * VEC);
                // mean = sum / area.  The areas of the usual windows are powers of two, whose reciprocals are exact:
                // the product is then the quotient, bit for bit, at a tenth of the instructions
                if (sz == 1) {
                    window_sum<T, 1>(base, W, C, sz, acc);
                } else if (sz == 2) {
                    window_sum<T, 2>(base, W, C, sz, acc);
#pragma unroll
                    for (int c = 0; c < VEC; c++) acc[c] *= 0.25f;
                } else if (sz == 4) {
                    window_sum<T, 4>(base, W, C, sz, acc);
#pragma unroll
                    for (int c = 0; c < VEC; c++) acc[c] *= 0.0625f;
                } else {
                    window_sum<T, 0>(base, W, C, sz, acc);
                    const float area = (float)(sz * sz);
#pragma unroll
                    for (int c = 0; c < VEC; c++) acc[c] = acc[c] / area;
                }
            }
            const u32x4 packed = Elem<T>::pack(acc);
            *reinterpret_cast<u32x4 *>(out + row * (int64_t)C + v * VEC) = packed;
            if constexpr (LN) Elem<T>::unpack(packed, vals[it]);        // the row as stored
        } else if constexpr (LN) {
#pragma unroll
            for (int c = 0; c < VEC; c++) vals[it][c] = 0.f;
        }
    }
    if constexpr (LN) {
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++)
#pragma unroll
            for (int c = 0; c < VEC; c++) s += vals[it][c];
        const float mean = group_sum<GS>(s) / (float)C;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            if (it * WAVE + lane < nvec) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float dlt = vals[it][c] - mean;
                    q += dlt * dlt;
                }
            }
        }
        const float rstd = 1.0f / sqrtf(group_sum<GS>(q) / (float)C + eps);
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int v = it * WAVE + lane;
            if (v < nvec) {
                float w[VEC], bb[VEC], y[VEC];
                Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ln_w + v * VEC), w);
                Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ln_b + v * VEC), bb);
#pragma unroll
                for (int c = 0; c < VEC; c++) y[c] = (vals[it][c] - mean) * rstd * w[c] + bb[c];
                *reinterpret_cast<u32x4 *>(ln_out + row * (int64_t)C + v * VEC) = Elem<T>::pack(y);
            }
        }
    }
}

// -------------------------------------------------------------- decompress
template <typename T, int SZ, bool ADD>
__device__ __forceinline__ void window_store(const T *__restrict__ ref, T *__restrict__ dst, int W, int C, int sz,
                                             const float (&d)[Elem<T>::VEC])
{
    constexpr int VEC = Elem<T>::VEC;
    if constexpr (SZ > 0) {
        u32x4 raw[SZ * SZ];
        if constexpr (ADD) {
#pragma unroll
            for (int dy = 0; dy < SZ; dy++)
#pragma unroll
                for (int dx = 0; dx < SZ; dx++)
                    raw[dy * SZ + dx] = *reinterpret_cast<const u32x4 *>(ref + ((int64_t)dy * W + dx) * C);
        }
#pragma unroll
        for (int dy = 0; dy < SZ; dy++)
#pragma unroll
            for (int dx = 0; dx < SZ; dx++) {
                float o[VEC];
                if constexpr (ADD) {
                    float r[VEC];
                    Elem<T>::unpack(raw[dy * SZ + dx], r);
#pragma unroll
                    for (int c = 0; c < VEC; c++) o[c] = d[c] + r[c];
                } else {
#pragma unroll
                    for (int c = 0; c < VEC; c++) o[c] = d[c];
                }
                *reinterpret_cast<u32x4 *>(dst + ((int64_t)dy * W + dx) * C) = Elem<T>::pack(o);
            }
    } else {
        for (int dy = 0; dy < sz; dy++)
            for (int dx = 0; dx < sz; dx++) {
                float o[VEC];
                if constexpr (ADD) {
                    float r[VEC];
                    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ref + ((int64_t)dy * W + dx) * C), r);
#pragma unroll
                    for (int c = 0; c < VEC; c++) o[c] = d[c] + r[c];
                } else {
#pragma unroll
                    for (int c = 0; c < VEC; c++) o[c] = d[c];
                }
                *reinterpret_cast<u32x4 *>(dst + ((int64_t)dy * W + dx) * C) = Elem<T>::pack(o);
            }
    }
}

template <typename T, bool SUB, bool ADD, int GS>
__global__ __launch_bounds__(256) void decompress_kernel(const T *__restrict__ in, const T *__restrict__ sub,
                                                          const int64_t *__restrict__ patches,
                                                          const int64_t *__restrict__ rows_dev, int64_t rows,
                                                          const T *__restrict__ ref, T *__restrict__ out, int N,
                                                          int C, int W, int extra)
{
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & (GS - 1);
    const int64_t row = ((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS;
    if (row >= live_rows(rows_dev, rows)) return;
    const int64_t *p = patches + 4 * row;
    const int64_t b = p[0], y0 = p[1], x0 = p[2];
    const int sz = (int)p[3];
    const int nvec = C / VEC;
    for (int v = lane; v < nvec; v += GS) {
        float d[VEC];
        Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(in + row * (int64_t)C + v * VEC), d);
        if constexpr (SUB) {
            float s[VEC];
            Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(sub + row * (int64_t)C + v * VEC), s);
#pragma unroll
            for (int c = 0; c < VEC; c++) d[c] = Elem<T>::round(d[c] - s[c]);
        }
        const int64_t tok = y0 < 0 ? (-y0 - 1) : (y0 * W + x0 + extra);
        const int64_t off = (b * N + tok) * (int64_t)C + v * VEC;
        const T *r = ADD ? ref + off : nullptr;
        T *o = out + off;
        if (y0 < 0 || sz == 1) window_store<T, 1, ADD>(r, o, W, C, 1, d);
        else if (sz == 2) window_store<T, 2, ADD>(r, o, W, C, sz, d);
        else if (sz == 4) window_store<T, 4, ADD>(r, o, W, C, sz, d);
        else window_store<T, 0, ADD>(r, o, W, C, sz, d);
    }
}

// Scatter back and LayerNorm in one pass: out = (in - sub) + ref as above, and ln_out = LayerNorm(out) of every
// token written (what the next block's first LayerNorm would read back and compute).  One group of GS lanes per
// packed row, one 16-byte vector per lane (rows of at most GS vectors); the tokens of the window are finished one
// after the other: sum, rounded as it is stored, then two-pass statistics over the group, affine, second store.
template <typename T, bool SUB, int GS>
__global__ __launch_bounds__(256) void decompress_ln_kernel(const T *__restrict__ in, const T *__restrict__ sub,
                                                             const int64_t *__restrict__ patches,
                                                             const int64_t *__restrict__ rows_dev, int64_t rows,
                                                             const T *__restrict__ ref, T *__restrict__ out,
                                                             T *__restrict__ ln_out, const T *__restrict__ ln_w,
                                                             const T *__restrict__ ln_b, float eps, int N, int C,
                                                             int W, int extra)
{
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & (GS - 1);
    const int64_t row = ((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS;
    if (row >= live_rows(rows_dev, rows)) return;
    const int64_t *p = patches + 4 * row;
    const int64_t b = p[0], y0 = p[1], x0 = p[2];
    const int sz = y0 < 0 ? 1 : (int)p[3];
    const int nvec = C / VEC;
    const bool act = lane < nvec;
    const int v = act ? lane : 0;        // idle lanes shadow lane 0's addresses and store nothing

    float d[VEC], w[VEC], bb[VEC];
    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(in + row * (int64_t)C + v * VEC), d);
    if constexpr (SUB) {
        float sv[VEC];
        Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(sub + row * (int64_t)C + v * VEC), sv);
#pragma unroll
        for (int c = 0; c < VEC; c++) d[c] = Elem<T>::round(d[c] - sv[c]);
    }
    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ln_w + v * VEC), w);
    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ln_b + v * VEC), bb);
    const int64_t tok = y0 < 0 ? (-y0 - 1) : (y0 * W + x0 + extra);
    const int64_t off = (b * N + tok) * (int64_t)C + v * VEC;

    // NT tokens at a time (their reductions interleave): raw = their vectors of ref, o = their element offsets
    auto finish = [&](auto nt_tag, const u32x4 *raw, const int64_t *o) {
        constexpr int NT = decltype(nt_tag)::value;
        float val[NT][VEC], s[NT], q[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float r[VEC];
            Elem<T>::unpack(raw[t], r);
#pragma unroll
            for (int c = 0; c < VEC; c++) r[c] += d[c];
            const u32x4 packed = Elem<T>::pack(r);
            if (act) *reinterpret_cast<u32x4 *>(out + o[t]) = packed;
            Elem<T>::unpack(packed, val[t]);                      // as stored
            s[t] = 0.f;
#pragma unroll
            for (int c = 0; c < VEC; c++) s[t] += act ? val[t][c] : 0.f;
        }
        group_sum_n<GS, NT>(s);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            s[t] = s[t] / (float)C;                               // mean
            q[t] = 0.f;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float dl = val[t][c] - s[t];
                q[t] += act ? dl * dl : 0.f;
            }
        }
        group_sum_n<GS, NT>(q);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float rstd = 1.0f / sqrtf(q[t] / (float)C + eps);
            float y[VEC];
#pragma unroll
            for (int c = 0; c < VEC; c++) y[c] = (val[t][c] - s[t]) * rstd * w[c] + bb[c];
            if (act) *reinterpret_cast<u32x4 *>(ln_out + o[t]) = Elem<T>::pack(y);
        }
    };
    auto window = [&](auto sz_tag) {
        constexpr int SZ = decltype(sz_tag)::value;
        constexpr int NT = SZ == 1 ? 1 : 4;
        u32x4 raw[SZ * SZ];
        int64_t o[SZ * SZ];
#pragma unroll
        for (int dy = 0; dy < SZ; dy++)
#pragma unroll
            for (int dx = 0; dx < SZ; dx++) {
                o[dy * SZ + dx] = off + ((int64_t)dy * W + dx) * C;
                raw[dy * SZ + dx] = *reinterpret_cast<const u32x4 *>(ref + o[dy * SZ + dx]);
            }
#pragma unroll
        for (int i = 0; i < SZ * SZ; i += NT) finish(std::integral_constant<int, NT>{}, raw + i, o + i);
    };
    if (sz == 1) window(std::integral_constant<int, 1>{});
    else if (sz == 2) window(std::integral_constant<int, 2>{});
    else if (sz == 4) window(std::integral_constant<int, 4>{});
    else {
        for (int dy = 0; dy < sz; dy++)
            for (int dx = 0; dx < sz; dx++) {
                const int64_t o = off + ((int64_t)dy * W + dx) * C;
                const u32x4 raw = *reinterpret_cast<const u32x4 *>(ref + o);
                finish(std::integral_constant<int, 1>{}, &raw, &o);
            }
    }
}

// ------------------------------------------------- decompress + next router
// Scatter back by REGION instead of by packed row, so that the same wave can route the next block: a group of GS
// lanes owns one R x R region (R = 4) of one sample.  The packed rows of a region are consecutive (regions in
// row-major order, sub-patches in row-major order inside a region), starting at
//   offsets[b] + extra + sum of the query counts of the sample's earlier regions,
// which the group adds up from the gate indices itself.  It writes out = (in - sub) + ref for the region's 16
// tokens (the same arithmetic and rounding as decompress_kernel), sums the values as stored, in the order the
// router sums them, and finishes with the router's Linear + argmax on the NEXT block's gate weights: the indices
// and logits it leaves are bit for bit those of router_kernel run on `out`, without a second pass over the tokens.
// The group of a sample's first region also scatters the sample's extra tokens.
// STAT (one wave per region, all 64 lanes present, `act` false for lanes past the row): also writes the
// statistics records of the 16 stored rows, `rec` pointing at the record of the region's first token.
template <typename T, int PS, bool SUB, bool STAT = false>
__device__ __forceinline__ void region_scatter(const T *__restrict__ in, const T *__restrict__ sub, int64_t r0,
                                               const T *__restrict__ refp, T *__restrict__ outp, int W, int C,
                                               float (&acc)[Elem<T>::VEC], bool act = true,
                                               u32x4 *__restrict__ rec = nullptr, float eps = 0.f)
{
    constexpr int VEC = Elem<T>::VEC;
    constexpr int STEP = 4 / PS;
    const int lane = threadIdx.x & 63;
#pragma unroll 1
    for (int dy = 0; dy < 4; dy++) {                       // one token row (4 tokens) at a time; not unrolled: the
                                                           // loads of one row are what a wave keeps in flight
        constexpr int NJ = PS;                              // packed rows these tokens take their values from
        const int j0 = (dy / STEP) * PS;
        float pivot[4], st[8];
        u32x4 xr[4], ir[NJ], sr[NJ];
        if constexpr (STAT) {
            const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int j = 0; j < NJ; j++) ir[j] = sr[j] = z;
#pragma unroll
            for (int dx = 0; dx < 4; dx++) xr[dx] = z;
        }
        if (act) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                ir[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in + (r0 + j0 + j) * (int64_t)C));
                if constexpr (SUB)
                    sr[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(sub + (r0 + j0 + j) * (int64_t)C));
            }
#pragma unroll
            for (int dx = 0; dx < 4; dx++)
                xr[dx] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(refp + ((int64_t)dy * W + dx) * C));
        }
        // in - sub, rounded to the storage type (kept packed: four registers per row)
        if constexpr (SUB) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                float dv[VEC], sv[VEC];
                Elem<T>::unpack(ir[j], dv);
                Elem<T>::unpack(sr[j], sv);
#pragma unroll
                for (int c = 0; c < VEC; c++) dv[c] -= sv[c];
                ir[j] = Elem<T>::pack(dv);
            }
        }
#pragma unroll
        for (int dx = 0; dx < 4; dx++) {
            float r[VEC], dv[VEC];
            Elem<T>::unpack(xr[dx], r);
            Elem<T>::unpack(ir[dx / STEP], dv);
#pragma unroll
            for (int c = 0; c < VEC; c++) r[c] += dv[c];
            const u32x4 packed = Elem<T>::pack(r);
            if (act) *reinterpret_cast<u32x4 *>(outp + ((int64_t)dy * W + dx) * C) = packed;
            float f[VEC];
            Elem<T>::unpack(packed, f);                   // as stored: what the next block's router reads
#pragma unroll
            for (int c = 0; c < VEC; c++) acc[c] += f[c];
            if constexpr (STAT) {
                pivot[dx] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(f[0])));
                float a = 0.f, q = 0.f;
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float d = f[c] - pivot[dx];
                    a += d;
                    q += d * d;
                }
                st[2 * dx] = act ? a : 0.f;
                st[2 * dx + 1] = act ? q : 0.f;
            }
        }
        if constexpr (STAT) write_records4(st, pivot[0], pivot[1], pivot[2], pivot[3], C, eps, rec + (int64_t)dy * W * 2);
    }
}

// The same pass over a region without the scatter (SCATTER = false below): the tokens are read, summed for the
// router and, with STAT, their records written; nothing is stored to the tokens.
template <typename T, bool STAT>
__device__ __forceinline__ void region_read(const T *__restrict__ refp, int W, int C, float (&acc)[Elem<T>::VEC],
                                            bool act, u32x4 *__restrict__ rec, float eps)
{
    constexpr int VEC = Elem<T>::VEC;
#pragma unroll 1
    for (int dy = 0; dy < 4; dy++) {
        float pivot[4], st[8];
        u32x4 xr[4];
#pragma unroll
        for (int dx = 0; dx < 4; dx++) {
            xr[dx] = u32x4{0u, 0u, 0u, 0u};
            if (act) xr[dx] = *reinterpret_cast<const u32x4 *>(refp + ((int64_t)dy * W + dx) * C);
        }
#pragma unroll
        for (int dx = 0; dx < 4; dx++) {
            float f[VEC];
            Elem<T>::unpack(xr[dx], f);
#pragma unroll
            for (int c = 0; c < VEC; c++) acc[c] += f[c];
            if constexpr (STAT) {
                pivot[dx] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(f[0])));
                float a = 0.f, q = 0.f;
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float d = f[c] - pivot[dx];
                    a += d;
                    q += d * d;
                }
                st[2 * dx] = act ? a : 0.f;
                st[2 * dx + 1] = act ? q : 0.f;
            }
        }
        if constexpr (STAT) write_records4(st, pivot[0], pivot[1], pivot[2], pivot[3], C, eps, rec + (int64_t)dy * W * 2);
    }
}

// CHAIN = true: the kernel goes on to pack the NEXT block's queries (what vtdge_compress_regions would do in a launch
// of its own, reading the tokens back): the wave that has just written a region's tokens and chosen its next split has
// everything for that but the region's first packed row, which is the number of queries of ALL regions before it.
// The workgroups pass that number along in launch order through one 64-bit status word each (two flag bits + a
// count): a workgroup publishes the queries of its four regions ("aggregate"), looks back over the words of the
// workgroups before it - 64 of them per step, one per lane - until it meets one that already knows its total
// ("prefix"), adds up what lies between and publishes its own prefix.  A workgroup only ever waits for workgroups
// with smaller numbers, which were dispatched before it and wait for nobody behind them, so the chain always moves;
// the wait is bounded all the same (a workgroup that gives up raises the error word and places its rows past the
// capacity, where nothing is written).  The status words must be zero at launch; nothing else of them is kept.
struct ChainArgs {
    bf16_t *comp;                 // [capacity, C] the next block's packed queries
    u32x4 *comp_records;          // [capacity, 2] their statistics records
    float comp_eps;
    int64_t *patches;             // [capacity, 4] (nullable)
    int64_t capacity;
    int64_t *offsets;             // [B + 1]
    int32_t *region_rows;         // [B * regions] first packed row of every region (nullable)
    unsigned long long *status;   // [1 + workgroups]: word 0 = error flag, then one word per workgroup
};
constexpr unsigned long long CHAIN_AGGREGATE = 1ull << 62, CHAIN_PREFIX = 2ull << 62;
constexpr int CHAIN_SPIN_LIMIT = 1 << 20;

// SCATTER = false: no packed rows at all - the kernel routes on `ref` as it stands and writes the records of its
// rows (the first block of a model, which no scatter-back precedes); `in` then points, if anywhere, at `extra`
// rows [extra, C] that are first copied into the extra-token rows of every sample of `out` (class / distillation
// token plus their position embedding, the same for every sample).
template <typename T, int GS, bool SUB, bool STAT = false, bool SCATTER = true, bool CHAIN = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(CHAIN ? 4 : 1, CHAIN ? 4 : 8)))
void decompress_route_kernel(
    const T *__restrict__ in, const T *__restrict__ sub, const int64_t *__restrict__ cur_indices,
    const int64_t *__restrict__ splits, const int64_t *__restrict__ offsets, const T *__restrict__ ref,
    T *__restrict__ out, const T *__restrict__ weight, const T *__restrict__ bias, T *__restrict__ gate,
    int64_t *__restrict__ indices, int B, int H, int W, int C, int extra, int S, int S2,
    u32x4 *__restrict__ records = nullptr, float eps = 0.f, const int64_t *__restrict__ next_splits = nullptr,
    uint8_t *__restrict__ next_counts = nullptr, const int32_t *__restrict__ region_rows = nullptr,
    const uint8_t *__restrict__ cur_counts = nullptr, const ChainArgs chain = ChainArgs{})
{
    static_assert(!STAT || (GS == WAVE && std::is_same<T, bf16_t>::value), "records: one wave per region, bf16 rows");
    static_assert(!CHAIN || (STAT && SCATTER), "the chained variant is the bf16 scatter-back with records");
    constexpr int VEC = Elem<T>::VEC;
    constexpr int R = 4;
    const int lane = threadIdx.x & (GS - 1);
    const int Hr = H / R, Wr = W / R, nreg = Hr * Wr;
    if constexpr (!SCATTER) {
        // the first kernel of a forward also clears `chain.capacity` 64-bit words at `chain.status` (the status words
        // of the chained scatter-backs that follow it on the stream)
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < chain.capacity;
             i += (int64_t)gridDim.x * blockDim.x)
            chain.status[i] = 0ull;
    }
    const int64_t region = ((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS;
    if (region >= (int64_t)B * nreg) return;
    const int b = (int)(region / nreg);
    const int rr = (int)(region % nreg);
    const int ry = rr / Wr, rx = rr % Wr;
    const int N = extra + H * W;
    const int nvec = C / VEC;

    auto split_of = [&](int64_t reg) {
        int64_t g = cur_indices[reg];
        g = g < 0 ? 0 : (g >= S ? S - 1 : g);
        return (int)splits[g];
    };
    // first packed row of this region (query counts are small integers: exact in fp32)
    int64_t row_b = 0, r0 = 0;
    int ps = 1;
    if constexpr (SCATTER) {
        if (region_rows != nullptr) {
            // the kernel that packed the rows has left every region's first row and query count: one load each
            r0 = region_rows[region];
            row_b = r0 - extra;          // read for a sample's first region only
            const int cnt = cur_counts[region];
            ps = cnt == 16 ? 4 : cnt == 4 ? 2 : 1;
        } else {
            float before = 0.f;
            for (int r2 = lane; r2 < rr; r2 += GS) {
                const int ps2 = split_of((int64_t)b * nreg + r2);
                before += (float)(ps2 * ps2);
            }
            row_b = offsets[b];
            r0 = row_b + extra + (int64_t)group_sum<GS>(before);
            ps = split_of(region);
        }
        if constexpr (GS == WAVE) ps = __builtin_amdgcn_readfirstlane(ps);      // one region per wave: a scalar branch
    }

    float part[VTDGE_MAX_SPLITS];
#pragma unroll
    for (int s = 0; s < VTDGE_MAX_SPLITS; s++) part[s] = 0.f;
    const int64_t tok0 = (int64_t)(ry * R) * W + rx * R + extra;
    // STAT: the host sends rows of at most GS vectors, and every lane makes the one trip (lanes past the row idle
    // inside it, present for the sums over the wave)
    const int vend = STAT ? GS : nvec;
    u32x4 pooled = {0u, 0u, 0u, 0u};      // CHAIN: this lane's vector of the region's mean as the router rounds it
    for (int v0 = lane; v0 < vend; v0 += GS) {
        const bool act = !STAT || v0 < nvec;
        const int v = act ? v0 : 0;
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] = 0.f;
        const int64_t off = ((int64_t)b * N + tok0) * C + v * VEC;
        const T *inv = in + v * VEC;
        const T *subv = SUB ? sub + v * VEC : nullptr;
        u32x4 *rec = STAT ? records + ((int64_t)b * N + tok0) * 2 : nullptr;
        if constexpr (!SCATTER) region_read<T, STAT>(ref + off, W, C, acc, act, rec, eps);
        else if (ps == 4) region_scatter<T, 4, SUB, STAT>(inv, subv, r0, ref + off, out + off, W, C, acc, act, rec, eps);
        else if (ps == 2) region_scatter<T, 2, SUB, STAT>(inv, subv, r0, ref + off, out + off, W, C, acc, act, rec, eps);
        else region_scatter<T, 1, SUB, STAT>(inv, subv, r0, ref + off, out + off, W, C, acc, act, rec, eps);
        if (rr == 0) {          // the sample's extra tokens: packed rows row_b .. row_b + extra - 1
            for (int e = 0; e < extra; e++) {
                float d[VEC], r[VEC];
#pragma unroll
                for (int c = 0; c < VEC; c++) d[c] = r[c] = 0.f;
                const int64_t oe = ((int64_t)b * N + e) * C + v * VEC;
                u32x4 packed = {0u, 0u, 0u, 0u};
                if constexpr (SCATTER) {
                    if (act) {
                        Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(inv + (row_b + e) * (int64_t)C), d);
                        if constexpr (SUB) {
                            float sv[VEC];
                            Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(subv + (row_b + e) * (int64_t)C), sv);
#pragma unroll
                            for (int c = 0; c < VEC; c++) d[c] -= sv[c];
                            Elem<T>::unpack(Elem<T>::pack(d), d);      // rounded to the storage type
                        }
                        Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(ref + oe), r);
                    }
#pragma unroll
                    for (int c = 0; c < VEC; c++) r[c] += d[c];
                    packed = Elem<T>::pack(r);
                    if (act) *reinterpret_cast<u32x4 *>(out + oe) = packed;
                } else if (act) {
                    // the row as it stands, or the row given for every sample, which is put in place first
                    if (in != nullptr) {
                        packed = *reinterpret_cast<const u32x4 *>(inv + (int64_t)e * C);
                        *reinterpret_cast<u32x4 *>(out + oe) = packed;
                    } else {
                        packed = *reinterpret_cast<const u32x4 *>(ref + oe);
                    }
                }
                if constexpr (STAT) {
                    float f[VEC], st[2] = {0.f, 0.f};
                    Elem<T>::unpack(packed, f);
                    const float pivot = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(f[0])));
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        const float dl = f[c] - pivot;
                        st[0] += act ? dl : 0.f;
                        st[1] += act ? dl * dl : 0.f;
                    }
                    wave_sum_n<2>(st);
                    u32x4 lo, hi;
                    row_record(pivot, st[0], st[1], C, eps, lo, hi);
                    if (lane < 2) records[((int64_t)b * N + e) * 2 + lane] = lane ? hi : lo;
                }
            }
        }
        if (weight != nullptr && act) {
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[i] = Elem<T>::round(acc[i] / (float)(R * R));
            if constexpr (CHAIN) pooled = Elem<T>::pack(acc);
#pragma unroll
            for (int s = 0; s < VTDGE_MAX_SPLITS; s++) {
                if (s < S2) {
                    float w[VEC];
                    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(weight + (int64_t)s * C + v * VEC), w);
#pragma unroll
                    for (int i = 0; i < VEC; i++) part[s] += acc[i] * w[i];
                }
            }
        }
    }
    if (weight == nullptr) return;
    float best = 0.f;
    int best_s = 0;
#pragma unroll
    for (int s = 0; s < VTDGE_MAX_SPLITS; s++) {
        if (s < S2) {
            float logit = group_sum<GS>(part[s]) + Elem<T>::load(bias + s);
            logit = Elem<T>::round(logit);
            if (gate != nullptr && lane == 0) Elem<T>::store(gate + region * S2 + s, logit);
            if (s == 0 || logit > best) {  // strict >: lowest index wins a tie
                best = logit;
                best_s = s;
            }
        }
    }
    if (lane == 0) {
        indices[region] = best_s;
        if (next_counts != nullptr) {        // queries the next block takes from this region: its split, squared
            const int ps2 = (int)next_splits[best_s];
            next_counts[region] = (uint8_t)(ps2 * ps2);
        }
    }
    if constexpr (CHAIN) {
        // ---- the next block's packed rows of this region (the host launches whole workgroups of four regions)
        __shared__ int cnt_s[4];
        __shared__ long long excl_s;
        const int wv = threadIdx.x >> 6;
        const int ps_n = __builtin_amdgcn_readfirstlane((int)next_splits[best_s]);
        const int nq = ps_n == 4 ? 16 : ps_n == 2 ? 4 : 1;
        if (lane == 0) cnt_s[wv] = nq;
        __syncthreads();
        unsigned long long *st = chain.status + 1;
        const int wg = (int)blockIdx.x;
        if (wv == 0) {
            const int agg = cnt_s[0] + cnt_s[1] + cnt_s[2] + cnt_s[3];
            if (lane == 0)
                __hip_atomic_store(st + wg, (wg == 0 ? CHAIN_PREFIX : CHAIN_AGGREGATE) | (unsigned long long)agg,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            long long excl = 0;
            if (wg > 0) {
                // Every step looks at LOOK x 64 words, nearest first.  One load a lane is the fastest: the nearest
                // workgroups are the last to publish, and a wider window only makes each retry dearer (measured at
                // 1024 workgroups: 52 us for the kernel with 64 words a step, 54 with 128, 57 with 512).
                constexpr int LOOK = 1;
                int j = wg - 1, spins = 0;
                bool gave_up = false;
                while (true) {
                    unsigned long long v[LOOK];
#pragma unroll
                    for (int k = 0; k < LOOK; k++) {
                        const int idx = j - lane - WAVE * k;   // lane 0 of k = 0: the workgroup just before this one
                        v[k] = CHAIN_PREFIX;                   // before the first workgroup: a prefix of zero
                        if (idx >= 0) v[k] = __hip_atomic_load(st + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    float part = 0.f;
                    bool found = false, wait = false;
#pragma unroll
                    for (int k = 0; k < LOOK; k++) {
                        if (!found && !wait) {
                            const int flag = (int)(v[k] >> 62);
                            const unsigned long long missing = __builtin_amdgcn_ballot_w64(flag == 0);
                            const unsigned long long known = __builtin_amdgcn_ballot_w64(flag == 2);
                            const int first_known = known ? __builtin_ctzll(known) : 64;
                            const int first_missing = missing ? __builtin_ctzll(missing) : 64;
                            if (first_missing < first_known) {
                                wait = true;     // somebody nearer than the first prefix has not published yet
                            } else {
                                const int upto = first_known < 64 ? first_known : 63;
                                part += lane <= upto ? (float)(unsigned)(v[k] & 0xffffffffull) : 0.f;
                                found = first_known < 64;
                            }
                        }
                    }
                    if (wait) {
                        if (++spins > CHAIN_SPIN_LIMIT) {
                            gave_up = true;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                        continue;
                    }
                    excl += (long long)wave_sum(part);
                    if (found) break;
                    j -= WAVE * LOOK;
                }
                if (gave_up) {
                    excl = chain.capacity;                 // every row of this workgroup falls past the capacity
                    if (lane == 0) __hip_atomic_store(chain.status, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (lane == 0)
                    __hip_atomic_store(st + wg, CHAIN_PREFIX | (unsigned long long)(excl + agg), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            }
            if (lane == 0) excl_s = excl;
        }
        __syncthreads();
        long long rows_before = excl_s;
        for (int w2 = 0; w2 < wv; w2++) rows_before += cnt_s[w2];
        const int64_t n0 = rows_before + (int64_t)extra * (b + 1);        // first packed row of the region, next block
        if (chain.region_rows != nullptr && lane == 0) chain.region_rows[region] = (int32_t)n0;
        // descriptors, offsets (lengths are the differences of the offsets)
        if (chain.patches != nullptr && lane < nq) {
            const int pq = ps_n, step = R / pq;
            const int dy = lane / pq, dx = lane - dy * pq;
            const int64_t row = n0 + lane;
            if (row >= 0 && row < chain.capacity) {
                i64x2 *pp = reinterpret_cast<i64x2 *>(chain.patches + 4 * row);
                pp[0] = i64x2{(long long)b, (long long)(ry * R + dy * step)};
                pp[1] = i64x2{(long long)(rx * R + dx * step), (long long)step};
            }
        }
        if (rr == 0) {
            if (lane == 0) chain.offsets[b] = n0 - extra;
            if (chain.patches != nullptr && lane < extra && n0 >= extra && n0 - extra + lane < chain.capacity) {
                int64_t *pp = chain.patches + 4 * (n0 - extra + lane);
                pp[0] = b; pp[1] = -(int64_t)lane - 1; pp[2] = 0; pp[3] = 1;
            }
        }
        if (region == (int64_t)B * nreg - 1 && lane == 0) chain.offsets[B] = n0 + nq;
        if (n0 < extra || n0 + nq > chain.capacity) return;   // never outside the buffers
        // The tokens are read back by the lanes that stored them (a lane reads what it wrote itself, in program
        // order): plain loads, served by the caches the stores went through.
        const bool act = lane < nvec;
        const int v = act ? lane : 0;
        const bf16_t *xs = out + (int64_t)b * N * C + v * 8;
        if (rr == 0)
            pack_front_rows<bf16_t, true>(xs, chain.comp + (n0 - extra) * (int64_t)C + v * 8,
                                          chain.comp_records + (n0 - extra) * 2, extra, C, chain.comp_eps, act, lane);
        if (ps_n == 1) {
            // one query for the whole region: the mean of its 16 tokens, which the router has just taken (the same
            // sum in the same order, the same single rounding) - nothing to read back
            if (act) *reinterpret_cast<u32x4 *>(chain.comp + n0 * (int64_t)C + v * 8) = pooled;
            float pivot, sums[2];
            lane_sums<bf16_t>(pooled, act, pivot, sums[0], sums[1]);
            wave_sum_n<2>(sums);
            u32x4 lo, hi;
            row_record(pivot, sums[0], sums[1], C, chain.comp_eps, lo, hi);
            if (lane < 2) chain.comp_records[n0 * 2 + lane] = lane ? hi : lo;
        } else {
            pack_region<bf16_t, true>(xs + tok0 * C, chain.comp + n0 * (int64_t)C + v * 8,
                                      chain.comp_records + n0 * 2, ps_n, W, C, chain.comp_eps, act, lane);
        }
    }
}

// --------------------------------------------------------------- layernorm
constexpr int LN_RPW = 4;   // rows per wave: their loads are issued together so that enough bytes are in flight

template <typename T, int NIT, int GS>   // NIT = 16-byte vectors per lane = ceil(C / VEC / 64) (1 when GS < 64)
__global__ __launch_bounds__(256) void layernorm_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                         const T *__restrict__ bsrc, T *__restrict__ out,
                                                         const int64_t *__restrict__ rows_dev, int64_t rows, int C,
                                                         float eps, int64_t x_group_stride, int x_group_rows,
                                                         const T *__restrict__ add = nullptr, int64_t add_rows = 1)
{
    // add (nullable) [add_rows, C]: row (r mod add_rows) of it is added to output row r after that row's rounding to
    // the storage type, and the sum rounded again - a LayerNorm module followed by `+ pos_embed`.
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & (GS - 1);
    const int64_t live = live_rows(rows_dev, rows);
    const int64_t row0 =
        (((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS) * LN_RPW;
    if (row0 >= live) return;
    const int nvec = C / VEC;
    u32x4 raw[LN_RPW][NIT];
#pragma unroll
    for (int r = 0; r < LN_RPW; r++)
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int v = it * WAVE + lane;
            // input rows come in groups of x_group_rows dense rows, the groups x_group_stride elements apart
            const int64_t rr = row0 + r;
            const int64_t src = x_group_rows > 0 ? (rr / x_group_rows) * x_group_stride + (rr % x_group_rows) * C : rr * C;
            if (v < nvec && rr < live) raw[r][it] = *reinterpret_cast<const u32x4 *>(x + src + v * VEC);
        }
    float ww[NIT][VEC], bb[NIT][VEC];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int v = it * WAVE + lane;
        if (v < nvec) {
            Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(w + v * VEC), ww[it]);
            Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(bsrc + v * VEC), bb[it]);
        }
    }
#pragma unroll
    for (int r = 0; r < LN_RPW; r++) {
        if (row0 + r >= live) break;
        float vals[NIT][VEC];
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            if (it * WAVE + lane < nvec) {
                Elem<T>::unpack(raw[r][it], vals[it]);
#pragma unroll
                for (int c = 0; c < VEC; c++) s += vals[it][c];
            }
        }
        const float mean = group_sum<GS>(s) / (float)C;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            if (it * WAVE + lane < nvec) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float dlt = vals[it][c] - mean;
                    q += dlt * dlt;
                }
            }
        }
        const float rstd = 1.0f / sqrtf(group_sum<GS>(q) / (float)C + eps);
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int v = it * WAVE + lane;
            if (v < nvec) {
                float y[VEC];
#pragma unroll
                for (int c = 0; c < VEC; c++) y[c] = (vals[it][c] - mean) * rstd * ww[it][c] + bb[it][c];
                if (add != nullptr) {
                    float a[VEC];
                    Elem<T>::unpack(*reinterpret_cast<const u32x4 *>(add + ((row0 + r) % add_rows) * C + v * VEC), a);
                    Elem<T>::unpack(Elem<T>::pack(y), y);
#pragma unroll
                    for (int c = 0; c < VEC; c++) y[c] += a[c];
                }
                *reinterpret_cast<u32x4 *>(out + (row0 + r) * (int64_t)C + v * VEC) = Elem<T>::pack(y);
            }
        }
    }
}

// The statistics half of layernorm_kernel: per row the 32-byte record (mean and sqrt(var + eps), see ln_record)
// that a Linear with a folded LayerNorm takes next to the raw rows.  Same two-pass arithmetic and reduction tree.
template <int NIT, int GS>
__global__ __launch_bounds__(256) void layernorm_stats_kernel(const bf16_t *__restrict__ x, u32x4 *__restrict__ rec,
                                                               const int64_t *__restrict__ rows_dev, int64_t rows,
                                                               int C, float eps)
{
    constexpr int VEC = 8;
    const int lane = threadIdx.x & (GS - 1);
    const int64_t live = live_rows(rows_dev, rows);
    const int64_t row0 =
        (((int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6)) * (WAVE / GS) + (threadIdx.x & 63) / GS) * LN_RPW;
    if (row0 >= live) return;
    const int nvec = C / VEC;
    u32x4 raw[LN_RPW][NIT];
#pragma unroll
    for (int r = 0; r < LN_RPW; r++)
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int v = it * WAVE + lane;
            if (v < nvec && row0 + r < live)
                raw[r][it] = *reinterpret_cast<const u32x4 *>(x + (row0 + r) * (int64_t)C + v * VEC);
        }
#pragma unroll
    for (int r = 0; r < LN_RPW; r++) {
        if (row0 + r >= live) break;
        float vals[NIT][VEC];
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            if (it * WAVE + lane < nvec) {
                Elem<bf16_t>::unpack(raw[r][it], vals[it]);
#pragma unroll
                for (int c = 0; c < VEC; c++) s += vals[it][c];
            }
        }
        const float mean = group_sum<GS>(s) / (float)C;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            if (it * WAVE + lane < nvec) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float dlt = vals[it][c] - mean;
                    q += dlt * dlt;
                }
            }
        }
        const float sigma = sqrtf(group_sum<GS>(q) / (float)C + eps);
        if (lane == 0) {
            u32x4 lo, hi;
            ln_record(mean, sigma, lo, hi);
            rec[(row0 + r) * 2] = lo;
            rec[(row0 + r) * 2 + 1] = hi;
        }
    }
}

// ------------------------------------------------------------- host side
static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T> static int elem_vec() { return Elem<T>::VEC; }

static int check_channels(int C, int dtype, const char *who)
{
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "%s: unknown dtype %d", who, dtype);
    VT_REQUIRE(C > 0 && C % vec == 0, VTDGE_ERR_UNSUPPORTED, "%s: C=%d must be a positive multiple of %d", who, C,
               vec);
    return VTDGE_OK;
}

}  // namespace vtdge

using namespace vtdge;

extern "C" int vtdge_router(const void *x, const void *weight, const void *bias, void *gate, int64_t *indices,
                            int B, int H, int W, int C, int extra, int R, int S, int dtype, void *stream)
{
    VT_REQUIRE(x && weight && bias && indices, VTDGE_ERR_ARG, "router: NULL operand");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && R > 0 && extra >= 0, VTDGE_ERR_ARG, "router: bad sizes");
    VT_REQUIRE(H % R == 0 && W % R == 0, VTDGE_ERR_ARG, "router: H=%d, W=%d not multiples of region %d", H, W, R);
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "router: S=%d outside [1,%d]", S,
               VTDGE_MAX_SPLITS);
    if (int rc = check_channels(C, dtype, "router")) return rc;
    VT_REQUIRE(aligned16(x) && aligned16(weight), VTDGE_ERR_ARG, "router: operands must be 16-byte aligned");
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    const int gs = group_size(C / (dtype == VTDGE_BF16 ? 8 : 4));
    dim3 grid((unsigned)ceil_div(regions, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, RS, GS)                                                                                     \
    note_kernel(reinterpret_cast<const void *>(router_kernel<T, RS, GS>)),                                        \
    router_kernel<T, RS, GS><<<grid, block, 0, st>>>((const T *)x, (const T *)weight, (const T *)bias, (T *)gate, \
                                                     indices, B, H, W, C, extra, R, S)
#define VT_REGION(T, GS) \
    do { if (R == 4) VT_LAUNCH(T, 4, GS); else if (R == 2) VT_LAUNCH(T, 2, GS); else VT_LAUNCH(T, 0, GS); } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) VT_REGION(T, 64); else if (gs == 32) VT_REGION(T, 32); else if (gs == 16) VT_REGION(T, 16); \
         else VT_REGION(T, 8); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_REGION
#undef VT_LAUNCH
    return check_launch("router");
}

extern "C" int vtdge_router_layernorm(const void *x, const void *weight, const void *bias, void *gate,
                                      int64_t *indices, const void *ln_weight, const void *ln_bias, float ln_eps,
                                      void *ln_out, int B, int H, int W, int C, int extra, int R, int S, int dtype,
                                      void *stream)
{
    VT_REQUIRE(x && weight && bias && indices && ln_weight && ln_bias && ln_out, VTDGE_ERR_ARG,
               "router_layernorm: NULL operand");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && extra >= 0, VTDGE_ERR_ARG, "router_layernorm: bad sizes");
    VT_REQUIRE(R == 4 || R == 2, VTDGE_ERR_UNSUPPORTED, "router_layernorm: region size %d (4 or 2 only)", R);
    VT_REQUIRE(H % R == 0 && W % R == 0, VTDGE_ERR_ARG, "router_layernorm: H=%d, W=%d not multiples of region %d", H,
               W, R);
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "router_layernorm: S=%d outside [1,%d]", S,
               VTDGE_MAX_SPLITS);
    if (int rc = check_channels(C, dtype, "router_layernorm")) return rc;
    const int nvec = C / (dtype == VTDGE_BF16 ? 8 : 4);
    VT_REQUIRE(nvec <= 64, VTDGE_ERR_UNSUPPORTED, "router_layernorm: C=%d exceeds one 16-byte vector per lane", C);
    VT_REQUIRE(aligned16(x) && aligned16(weight) && aligned16(ln_weight) && aligned16(ln_bias) && aligned16(ln_out),
               VTDGE_ERR_ARG, "router_layernorm: operands must be 16-byte aligned");
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    const int gs = group_size(nvec);
    dim3 grid((unsigned)ceil_div(regions, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, RS, GS)                                                                                  \
    note_kernel(reinterpret_cast<const void *>(router_kernel<T, RS, GS, true>)),                              \
    router_kernel<T, RS, GS, true><<<grid, block, 0, st>>>((const T *)x, (const T *)weight, (const T *)bias,  \
                                                           (T *)gate, indices, B, H, W, C, extra, R, S,       \
                                                           (const T *)ln_weight, (const T *)ln_bias, ln_eps,  \
                                                           (T *)ln_out)
#define VT_REGION(T, GS) \
    do { if (R == 4) VT_LAUNCH(T, 4, GS); else VT_LAUNCH(T, 2, GS); } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) VT_REGION(T, 64); else if (gs == 32) VT_REGION(T, 32); else if (gs == 16) VT_REGION(T, 16); \
         else VT_REGION(T, 8); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_REGION
#undef VT_LAUNCH
    return check_launch("router_layernorm");
}

extern "C" int vtdge_index_to_patch(const int64_t *indices, const int64_t *splits, int B, int Hr, int Wr, int S,
                                    int R, int extra, int64_t *patches, int64_t capacity_rows, int64_t *offsets,
                                    int64_t *lengths, void *stream)
{
    VT_REQUIRE(indices && splits && offsets && lengths, VTDGE_ERR_ARG, "index_to_patch: NULL operand");
    VT_REQUIRE(B > 0 && Hr > 0 && Wr > 0 && R > 0 && extra >= 0, VTDGE_ERR_ARG, "index_to_patch: bad sizes");
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "index_to_patch: S=%d outside [1,%d]", S,
               VTDGE_MAX_SPLITS);
    VT_REQUIRE(patches == nullptr || capacity_rows >= 0, VTDGE_ERR_ARG, "index_to_patch: negative capacity");
    VT_REQUIRE((reinterpret_cast<uintptr_t>(patches) & 15u) == 0, VTDGE_ERR_ARG,
               "index_to_patch: patches must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (patches != nullptr && (int64_t)B * Hr * Wr <= 16384) {
        // small batches: one launch, every sample's workgroup sums the counts before it on its own
        note_kernel(reinterpret_cast<const void *>(patch_write_kernel<true>));
        patch_write_kernel<true><<<B, 256, 0, st>>>(indices, splits, offsets, lengths, Hr, Wr, S, R, extra, patches,
                                                    capacity_rows, 0);
        return check_launch("index_to_patch");
    }
    if (patches != nullptr && B <= 4096) {
        // a wave per sample counts, then every sample's workgroup sums the lengths before it (a few KB)
        note_kernel(reinterpret_cast<const void *>(patch_count_kernel));
        patch_count_kernel<<<(B + 3) / 4, 256, 0, st>>>(indices, splits, B, Hr * Wr, S, extra, lengths);
        if (int rc = check_launch("index_to_patch(count)")) return rc;
        note_kernel(reinterpret_cast<const void *>(patch_write_kernel<false>));
        patch_write_kernel<false><<<B, 256, 0, st>>>(indices, splits, offsets, lengths, Hr, Wr, S, R, extra, patches,
                                                     capacity_rows, 1);
        return check_launch("index_to_patch(write)");
    }
    note_kernel(reinterpret_cast<const void *>(patch_count_scan_kernel));
    patch_count_scan_kernel<<<1, 1024, 0, st>>>(indices, splits, B, Hr * Wr, S, extra, offsets, lengths);
    if (int rc = check_launch("index_to_patch(count+scan)")) return rc;
    if (patches != nullptr) {
        note_kernel(reinterpret_cast<const void *>(patch_write_kernel<false>));
        patch_write_kernel<false><<<B, 256, 0, st>>>(indices, splits, offsets, lengths, Hr, Wr, S, R, extra, patches,
                                                     capacity_rows, 0);
        return check_launch("index_to_patch(write)");
    }
    return VTDGE_OK;
}

extern "C" int vtdge_index_to_patch_dense(const int64_t *splits_host, int B, int Hr, int Wr, int S, int R,
                                          int extra, int64_t *patches, void *stream)
{
    VT_REQUIRE(splits_host && patches, VTDGE_ERR_ARG, "index_to_patch_dense: NULL operand");
    VT_REQUIRE(B > 0 && Hr > 0 && Wr > 0 && R > 0 && extra >= 0, VTDGE_ERR_ARG, "index_to_patch_dense: bad sizes");
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "index_to_patch_dense: S=%d", S);
    DenseSplits sp;
    sp.n = S;
    int per = extra;
    for (int s = 0; s < S; s++) {
        VT_REQUIRE(splits_host[s] > 0 && R % splits_host[s] == 0, VTDGE_ERR_ARG,
                   "index_to_patch_dense: split %lld does not divide region %d", (long long)splits_host[s], R);
        sp.ps[s] = (int)splits_host[s];
        per += sp.ps[s] * sp.ps[s] * Hr * Wr;
    }
    const int64_t total = (int64_t)B * per;
    note_kernel(reinterpret_cast<const void *>(patch_dense_kernel));
    patch_dense_kernel<<<(unsigned)ceil_div(total, 256), 256, 0, (hipStream_t)stream>>>(sp, B, Hr, Wr, R, extra,
                                                                                        per, patches);
    return check_launch("index_to_patch_dense");
}

extern "C" int vtdge_compress(const void *x, const int64_t *patches, const int64_t *rows_dev, int64_t rows,
                              void *out, void *ln_out, const void *ln_weight, const void *ln_bias, float ln_eps,
                              int B, int N, int C, int W, int extra, int dtype, void *stream)
{
    VT_REQUIRE(x && patches && out, VTDGE_ERR_ARG, "compress: NULL operand");
    VT_REQUIRE(B > 0 && N > 0 && W > 0 && extra >= 0 && rows >= 0, VTDGE_ERR_ARG, "compress: bad sizes");
    VT_REQUIRE((N - extra) % W == 0, VTDGE_ERR_ARG, "compress: N-extra=%d is not a multiple of W=%d", N - extra, W);
    if (int rc = check_channels(C, dtype, "compress")) return rc;
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(C / vec <= WAVE * MAX_IT, VTDGE_ERR_UNSUPPORTED, "compress: C=%d exceeds %d", C, WAVE * MAX_IT * vec);
    VT_REQUIRE(aligned16(x) && aligned16(out), VTDGE_ERR_ARG, "compress: operands must be 16-byte aligned");
    const bool ln = ln_out != nullptr;
    VT_REQUIRE(!ln || (ln_weight && ln_bias && aligned16(ln_out)), VTDGE_ERR_ARG,
               "compress: fused LayerNorm needs weight and bias");
    if (rows == 0) return VTDGE_OK;
    const int gs = group_size(C / vec);
    dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, LNF, GS, NIT)                                                                                  \
    note_kernel(reinterpret_cast<const void *>(compress_kernel<T, LNF, GS, NIT>)),                                  \
    compress_kernel<T, LNF, GS, NIT><<<grid, block, 0, st>>>((const T *)x, patches, rows_dev, rows, (T *)out,       \
                                                             (T *)ln_out, (const T *)ln_weight, (const T *)ln_bias, \
                                                             ln_eps, N, C, W, extra)
#define VT_LNF(T, GS, NIT) do { if (ln) VT_LAUNCH(T, true, GS, NIT); else VT_LAUNCH(T, false, GS, NIT); } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) { if (C / vec > WAVE) VT_LNF(T, 64, MAX_IT); else VT_LNF(T, 64, 1); } \
         else if (gs == 32) VT_LNF(T, 32, 1); else if (gs == 16) VT_LNF(T, 16, 1); else VT_LNF(T, 8, 1); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_LNF
#undef VT_LAUNCH
    return check_launch("compress");
}

extern "C" int vtdge_decompress(const void *in, const void *sub, const int64_t *patches, const int64_t *rows_dev,
                                int64_t rows, const void *ref, void *out, int B, int N, int C, int W, int extra,
                                int dtype, void *stream)
{
    VT_REQUIRE(in && patches && out, VTDGE_ERR_ARG, "decompress: NULL operand");
    VT_REQUIRE(B > 0 && N > 0 && W > 0 && extra >= 0 && rows >= 0, VTDGE_ERR_ARG, "decompress: bad sizes");
    VT_REQUIRE((N - extra) % W == 0, VTDGE_ERR_ARG, "decompress: N-extra=%d is not a multiple of W=%d", N - extra,
               W);
    if (int rc = check_channels(C, dtype, "decompress")) return rc;
    VT_REQUIRE(aligned16(in) && aligned16(out) && aligned16(sub) && aligned16(ref), VTDGE_ERR_ARG,
               "decompress: operands must be 16-byte aligned");
    if (rows == 0) return VTDGE_OK;
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(C / vec <= WAVE * MAX_IT, VTDGE_ERR_UNSUPPORTED, "decompress: C=%d exceeds %d", C,
               WAVE * MAX_IT * vec);
    const int gs = group_size(C / vec);
    dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, SUBF, ADDF, GS)                                                                              \
    note_kernel(reinterpret_cast<const void *>(decompress_kernel<T, SUBF, ADDF, GS>)),                             \
    decompress_kernel<T, SUBF, ADDF, GS><<<grid, block, 0, st>>>((const T *)in, (const T *)sub, patches, rows_dev, \
                                                                 rows, (const T *)ref, (T *)out, N, C, W, extra)
#define VT_DISPATCH(T, GS)                                       \
    do {                                                         \
        if (sub && ref) VT_LAUNCH(T, true, true, GS);            \
        else if (sub) VT_LAUNCH(T, true, false, GS);             \
        else if (ref) VT_LAUNCH(T, false, true, GS);             \
        else VT_LAUNCH(T, false, false, GS);                     \
    } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) VT_DISPATCH(T, 64); else if (gs == 32) VT_DISPATCH(T, 32); else if (gs == 16) VT_DISPATCH(T, 16); \
         else VT_DISPATCH(T, 8); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_DISPATCH
#undef VT_LAUNCH
    return check_launch("decompress");
}

extern "C" int vtdge_decompress_layernorm(const void *in, const void *sub, const int64_t *patches,
                                          const int64_t *rows_dev, int64_t rows, const void *ref, void *out,
                                          void *ln_out, const void *ln_weight, const void *ln_bias, float ln_eps,
                                          int B, int N, int C, int W, int extra, int dtype, void *stream)
{
    VT_REQUIRE(in && patches && out && ref && ln_out && ln_weight && ln_bias, VTDGE_ERR_ARG,
               "decompress_layernorm: NULL operand");
    VT_REQUIRE(B > 0 && N > 0 && W > 0 && extra >= 0 && rows >= 0, VTDGE_ERR_ARG, "decompress_layernorm: bad sizes");
    VT_REQUIRE((N - extra) % W == 0, VTDGE_ERR_ARG, "decompress_layernorm: N-extra=%d is not a multiple of W=%d",
               N - extra, W);
    if (int rc = check_channels(C, dtype, "decompress_layernorm")) return rc;
    VT_REQUIRE(aligned16(in) && aligned16(out) && aligned16(sub) && aligned16(ref) && aligned16(ln_out) &&
                   aligned16(ln_weight) && aligned16(ln_bias),
               VTDGE_ERR_ARG, "decompress_layernorm: operands must be 16-byte aligned");
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(C / vec <= WAVE, VTDGE_ERR_UNSUPPORTED, "decompress_layernorm: C=%d exceeds %d (one vector per lane)",
               C, WAVE * vec);
    if (rows == 0) return VTDGE_OK;
    const int gs = group_size(C / vec);
    dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, SUBF, GS)                                                                                      \
    note_kernel(reinterpret_cast<const void *>(decompress_ln_kernel<T, SUBF, GS>)),                                 \
    decompress_ln_kernel<T, SUBF, GS><<<grid, block, 0, st>>>((const T *)in, (const T *)sub, patches, rows_dev,     \
                                                              rows, (const T *)ref, (T *)out, (T *)ln_out,          \
                                                              (const T *)ln_weight, (const T *)ln_bias, ln_eps, N,  \
                                                              C, W, extra)
#define VT_DISPATCH(T, GS) do { if (sub) VT_LAUNCH(T, true, GS); else VT_LAUNCH(T, false, GS); } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) VT_DISPATCH(T, 64); else if (gs == 32) VT_DISPATCH(T, 32); else if (gs == 16) VT_DISPATCH(T, 16); \
         else VT_DISPATCH(T, 8); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_DISPATCH
#undef VT_LAUNCH
    return check_launch("decompress_layernorm");
}

namespace vtdge {

// words of 64 bits the chained scatter-back needs for `regions` regions: the error word + one per workgroup
static inline int64_t chain_words(int64_t regions) { return 1 + ceil_div(regions, (int64_t)ROWS_PER_BLOCK); }

__global__ void clear_words_kernel(unsigned long long *p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}

static int decompress_router_launch(const void *in, const void *sub, const int64_t *cur_indices,
                                    const int64_t *splits, const int64_t *offsets, const void *ref, void *out,
                                    const void *next_weight, const void *next_bias, void *next_gate,
                                    int64_t *next_indices, void *out_records, float records_eps,
                                    const int64_t *next_splits, uint8_t *next_counts, const int32_t *region_rows,
                                    const uint8_t *cur_counts, const ChainArgs *chain, int B, int H, int W, int C,
                                    int extra, int R, int S, int S2, int dtype, void *stream)
{
    VT_REQUIRE((region_rows == nullptr) == (cur_counts == nullptr), VTDGE_ERR_ARG,
               "decompress_router: the regions' first rows and their query counts come together");
    VT_REQUIRE(next_counts == nullptr || (next_splits != nullptr && next_indices != nullptr), VTDGE_ERR_ARG,
               "decompress_router: the next block's query counts need its router and its splits");
    VT_REQUIRE(in && cur_indices && splits && offsets && ref && out, VTDGE_ERR_ARG, "decompress_router: NULL operand");
    VT_REQUIRE((next_weight == nullptr) == (next_bias == nullptr) && (next_weight == nullptr) == (next_indices == nullptr),
               VTDGE_ERR_ARG, "decompress_router: the next router needs weight, bias and indices together");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && extra >= 0, VTDGE_ERR_ARG, "decompress_router: bad sizes");
    VT_REQUIRE(R == 4, VTDGE_ERR_UNSUPPORTED, "decompress_router: region size %d (4 only)", R);
    VT_REQUIRE(H % R == 0 && W % R == 0, VTDGE_ERR_ARG, "decompress_router: H=%d, W=%d not multiples of region %d", H,
               W, R);
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS && S2 >= 1 && S2 <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED,
               "decompress_router: split counts %d / %d outside [1,%d]", S, S2, VTDGE_MAX_SPLITS);
    if (int rc = check_channels(C, dtype, "decompress_router")) return rc;
    VT_REQUIRE(aligned16(in) && aligned16(sub) && aligned16(ref) && aligned16(out) && aligned16(next_weight),
               VTDGE_ERR_ARG, "decompress_router: operands must be 16-byte aligned");
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    const int gs = group_size(C / (dtype == VTDGE_BF16 ? 8 : 4));
    dim3 grid((unsigned)ceil_div(regions, ROWS_PER_BLOCK * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
    if (out_records != nullptr) {
        VT_REQUIRE(dtype == VTDGE_BF16 && gs == WAVE && C / 8 <= WAVE, VTDGE_ERR_UNSUPPORTED,
                   "decompress_router: statistics records are written for bf16 rows of 264 to 512 channels (C=%d)", C);
        VT_REQUIRE(aligned16(out_records), VTDGE_ERR_ARG, "decompress_router: records must be 16-byte aligned");
        if (chain != nullptr) {
            // four regions to a workgroup, all present: the workgroups hand their query counts along
            VT_REQUIRE(regions % ROWS_PER_BLOCK == 0 && regions <= 65536 &&
                           (int64_t)B * (extra + (int64_t)H * W) < (1 << 24) && extra <= WAVE,
                       VTDGE_ERR_UNSUPPORTED,
                       "decompress_router_compress: %lld regions (a multiple of %d up to 65536), %d extra tokens (up to %d)",
                       (long long)regions, ROWS_PER_BLOCK, extra, WAVE);
            VT_REQUIRE(next_weight && next_splits && next_counts, VTDGE_ERR_ARG,
                       "decompress_router_compress: needs the next router, its splits and the count bytes");
#define VT_CHAIN(SUBF)                                                                                               \
    note_kernel(reinterpret_cast<const void *>(decompress_route_kernel<bf16_t, WAVE, SUBF, true, true, true>)),      \
    decompress_route_kernel<bf16_t, WAVE, SUBF, true, true, true><<<grid, block, 0, st>>>(                           \
        (const bf16_t *)in, (const bf16_t *)sub, cur_indices, splits, offsets, (const bf16_t *)ref, (bf16_t *)out,   \
        (const bf16_t *)next_weight, (const bf16_t *)next_bias, (bf16_t *)next_gate, next_indices, B, H, W, C, extra, \
        S, S2, (u32x4 *)out_records, records_eps, next_splits, next_counts, region_rows, cur_counts, *chain)
            if (sub) VT_CHAIN(true); else VT_CHAIN(false);
#undef VT_CHAIN
            return check_launch("decompress_router_compress");
        }
#define VT_STAT(SUBF)                                                                                                \
    note_kernel(reinterpret_cast<const void *>(decompress_route_kernel<bf16_t, WAVE, SUBF, true>)),                  \
    decompress_route_kernel<bf16_t, WAVE, SUBF, true><<<grid, block, 0, st>>>(                                       \
        (const bf16_t *)in, (const bf16_t *)sub, cur_indices, splits, offsets, (const bf16_t *)ref, (bf16_t *)out,   \
        (const bf16_t *)next_weight, (const bf16_t *)next_bias, (bf16_t *)next_gate, next_indices, B, H, W, C, extra, \
        S, S2, (u32x4 *)out_records, records_eps, next_splits, next_counts, region_rows, cur_counts)
        if (sub) VT_STAT(true); else VT_STAT(false);
#undef VT_STAT
        return check_launch("decompress_router");
    }
#define VT_LAUNCH2(T, GS, SUBF)                                                                                    \
    note_kernel(reinterpret_cast<const void *>(decompress_route_kernel<T, GS, SUBF>)),                             \
    decompress_route_kernel<T, GS, SUBF><<<grid, block, 0, st>>>(                                                  \
        (const T *)in, (const T *)sub, cur_indices, splits, offsets, (const T *)ref, (T *)out,                     \
        (const T *)next_weight, (const T *)next_bias, (T *)next_gate, next_indices, B, H, W, C, extra, S, S2,      \
        nullptr, 0.f, next_splits, next_counts, region_rows, cur_counts)
#define VT_LAUNCH(T, GS) do { if (sub) VT_LAUNCH2(T, GS, true); else VT_LAUNCH2(T, GS, false); } while (0)
#define VT_GROUP(T) \
    do { if (gs == 64) VT_LAUNCH(T, 64); else if (gs == 32) VT_LAUNCH(T, 32); else if (gs == 16) VT_LAUNCH(T, 16); \
         else VT_LAUNCH(T, 8); } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_LAUNCH
#undef VT_LAUNCH2
    return check_launch("decompress_router");
}

}  // namespace vtdge

extern "C" int vtdge_decompress_router(const void *in, const void *sub, const int64_t *cur_indices,
                                       const int64_t *splits, const int64_t *offsets, const void *ref, void *out,
                                       const void *next_weight, const void *next_bias, void *next_gate,
                                       int64_t *next_indices, void *out_records, float records_eps,
                                       const int64_t *next_splits, uint8_t *next_counts, const int32_t *region_rows,
                                       const uint8_t *cur_counts, int B, int H, int W, int C, int extra, int R, int S,
                                       int S2, int dtype, void *stream)
{
    return decompress_router_launch(in, sub, cur_indices, splits, offsets, ref, out, next_weight, next_bias, next_gate,
                                    next_indices, out_records, records_eps, next_splits, next_counts, region_rows,
                                    cur_counts, nullptr, B, H, W, C, extra, R, S, S2, dtype, stream);
}

extern "C" int64_t vtdge_decompress_router_compress_workspace(int B, int H, int W, int R)
{
    if (B <= 0 || H <= 0 || W <= 0 || R <= 0) return 0;
    return 8 * chain_words((int64_t)B * (H / R) * (W / R));
}

// ---- the same call for callers that cannot allocate device memory: the status words live in the library's image
namespace vtdge {
constexpr int64_t STATIC_CHAIN_REGIONS = 65536;      // the kernel's own limit
constexpr int64_t STATIC_CHAIN_WORDS = 1 + STATIC_CHAIN_REGIONS / ROWS_PER_BLOCK;
static __device__ __align__(256) unsigned long long scratch[STATIC_CHAIN_WORDS];     // 128 KB + 8 bytes per GPU
constexpr int MAX_DEVICES = 64;
static std::atomic<unsigned long long *> scratch_ptr[MAX_DEVICES];     // the array's address on every GPU seen so far
}  // namespace vtdge

extern "C" int vtdge_decompress_router_compress_static(
    const void *in, const void *sub, const int64_t *cur_indices, const int64_t *splits, const int64_t *offsets,
    const void *ref, void *out, const void *next_weight, const void *next_bias, void *next_gate,
    int64_t *next_indices, void *out_records, float records_eps, const int64_t *next_splits, uint8_t *next_counts,
    const int32_t *region_rows, const uint8_t *cur_counts, void *next_comp, void *next_comp_records,
    float next_records_eps, int64_t *next_patches, int64_t capacity_rows, int64_t *next_offsets,
    int32_t *next_region_rows, int B, int H, int W, int C, int extra, int R, int S, int S2, int dtype, void *stream)
{
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && R == 4, VTDGE_ERR_ARG, "decompress_router_compress_static: bad sizes");
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    VT_REQUIRE(regions <= STATIC_CHAIN_REGIONS, VTDGE_ERR_UNSUPPORTED,
               "decompress_router_compress_static: %lld regions, the built-in workspace holds %lld", (long long)regions,
               (long long)STATIC_CHAIN_REGIONS);
    int dev = -1;
    VT_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < MAX_DEVICES, VTDGE_ERR_LAUNCH,
               "decompress_router_compress_static: no current device (or more than %d)", MAX_DEVICES);
    unsigned long long *ws = scratch_ptr[dev].load(std::memory_order_acquire);
    if (ws == nullptr) {
        // every GPU holds its own copy of the array at its own address: ask for it once, with that GPU current
        const hipError_t rc = hipGetSymbolAddress((void **)&ws, HIP_SYMBOL(scratch));
        VT_REQUIRE(rc == hipSuccess && ws != nullptr, VTDGE_ERR_LAUNCH,
                   "decompress_router_compress_static: hipGetSymbolAddress: %s", hipGetErrorString(rc));
        scratch_ptr[dev].store(ws, std::memory_order_release);
    }
    // the words of this call start at zero (a fill kernel, not a memset: the call may be under stream capture)
    return vtdge_decompress_router_compress(in, sub, cur_indices, splits, offsets, ref, out, next_weight, next_bias,
                                            next_gate, next_indices, out_records, records_eps, next_splits,
                                            next_counts, region_rows, cur_counts, next_comp, next_comp_records,
                                            next_records_eps, next_patches, capacity_rows, next_offsets,
                                            next_region_rows, ws, 8 * STATIC_CHAIN_WORDS, 1, B, H, W, C, extra, R, S,
                                            S2, dtype, stream);
}

extern "C" int vtdge_decompress_router_compress(
    const void *in, const void *sub, const int64_t *cur_indices, const int64_t *splits, const int64_t *offsets,
    const void *ref, void *out, const void *next_weight, const void *next_bias, void *next_gate,
    int64_t *next_indices, void *out_records, float records_eps, const int64_t *next_splits, uint8_t *next_counts,
    const int32_t *region_rows, const uint8_t *cur_counts, void *next_comp, void *next_comp_records,
    float next_records_eps, int64_t *next_patches, int64_t capacity_rows, int64_t *next_offsets,
    int32_t *next_region_rows, void *workspace, int64_t workspace_bytes, int clear_workspace, int B, int H, int W,
    int C, int extra, int R, int S, int S2, int dtype, void *stream)
{
    VT_REQUIRE(next_comp && next_comp_records && next_offsets && workspace && out_records, VTDGE_ERR_ARG,
               "decompress_router_compress: NULL operand");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && R == 4 && capacity_rows >= 0, VTDGE_ERR_ARG,
               "decompress_router_compress: bad sizes");
    VT_REQUIRE(dtype == VTDGE_BF16, VTDGE_ERR_UNSUPPORTED, "decompress_router_compress: bf16 rows only");
    const int64_t words = chain_words((int64_t)B * (H / R) * (W / R));
    VT_REQUIRE(workspace_bytes >= 8 * words && (reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, VTDGE_ERR_ARG,
               "decompress_router_compress: the workspace holds %lld bytes, %lld needed (8-byte aligned)",
               (long long)workspace_bytes, (long long)(8 * words));
    VT_REQUIRE(aligned16(next_comp) && aligned16(next_comp_records) && aligned16(next_patches), VTDGE_ERR_ARG,
               "decompress_router_compress: operands must be 16-byte aligned");
    if (clear_workspace) {
        note_kernel(reinterpret_cast<const void *>(clear_words_kernel));
        clear_words_kernel<<<dim3((unsigned)ceil_div(words, (int64_t)256)), dim3(256), 0, (hipStream_t)stream>>>(
            (unsigned long long *)workspace, words);
        if (int rc = check_launch("decompress_router_compress")) return rc;
    }
    ChainArgs chain;
    chain.comp = (bf16_t *)next_comp;
    chain.comp_records = (u32x4 *)next_comp_records;
    chain.comp_eps = next_records_eps;
    chain.patches = next_patches;
    chain.capacity = capacity_rows;
    chain.offsets = next_offsets;
    chain.region_rows = next_region_rows;
    chain.status = (unsigned long long *)workspace;
    return decompress_router_launch(in, sub, cur_indices, splits, offsets, ref, out, next_weight, next_bias, next_gate,
                                    next_indices, out_records, records_eps, next_splits, next_counts, region_rows,
                                    cur_counts, &chain, B, H, W, C, extra, R, S, S2, dtype, stream);
}

extern "C" int vtdge_router_stats(void *x, const void *front_rows, const void *weight, const void *bias, void *gate,
                                  int64_t *indices, void *records, float records_eps, const int64_t *splits,
                                  uint8_t *counts, void *clear_words, int64_t n_clear_words, int B, int H, int W,
                                  int C, int extra, int R, int S, int dtype, void *stream)
{
    VT_REQUIRE(n_clear_words >= 0 && (n_clear_words == 0 || clear_words != nullptr) &&
                   (reinterpret_cast<uintptr_t>(clear_words) & 7u) == 0,
               VTDGE_ERR_ARG, "router_stats: the words to clear need an 8-byte aligned pointer");
    VT_REQUIRE(x && weight && bias && indices && records, VTDGE_ERR_ARG, "router_stats: NULL operand");
    VT_REQUIRE(counts == nullptr || splits != nullptr, VTDGE_ERR_ARG, "router_stats: the query counts need the splits");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && extra >= 0, VTDGE_ERR_ARG, "router_stats: bad sizes");
    VT_REQUIRE(R == 4, VTDGE_ERR_UNSUPPORTED, "router_stats: region size %d (4 only)", R);
    VT_REQUIRE(H % R == 0 && W % R == 0, VTDGE_ERR_ARG, "router_stats: H=%d, W=%d not multiples of region %d", H, W, R);
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "router_stats: S=%d outside [1,%d]", S,
               VTDGE_MAX_SPLITS);
    if (int rc = check_channels(C, dtype, "router_stats")) return rc;
    VT_REQUIRE(dtype == VTDGE_BF16 && group_size(C / 8) == WAVE && C / 8 <= WAVE, VTDGE_ERR_UNSUPPORTED,
               "router_stats: statistics records are written for bf16 rows of 264 to 512 channels (C=%d)", C);
    VT_REQUIRE(aligned16(x) && aligned16(front_rows) && aligned16(weight) && aligned16(records), VTDGE_ERR_ARG,
               "router_stats: operands must be 16-byte aligned");
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    dim3 grid((unsigned)ceil_div(regions, ROWS_PER_BLOCK)), block(256);
    ChainArgs side = {};            // no packing here: only the words this launch clears on the way
    side.status = (unsigned long long *)clear_words;
    side.capacity = n_clear_words;
    note_kernel(reinterpret_cast<const void *>(decompress_route_kernel<bf16_t, WAVE, false, true, false>));
    decompress_route_kernel<bf16_t, WAVE, false, true, false><<<grid, block, 0, (hipStream_t)stream>>>(
        (const bf16_t *)front_rows, nullptr, nullptr, splits, nullptr, (const bf16_t *)x, (bf16_t *)x,
        (const bf16_t *)weight, (const bf16_t *)bias, (bf16_t *)gate, indices, B, H, W, C, extra, S, S,
        (u32x4 *)records, records_eps, splits, counts, nullptr, nullptr, side);
    return check_launch("router_stats");
}

static int layernorm_launch(const void *x, int64_t x_group_stride, int x_group_rows, const void *weight,
                            const void *bias, void *out, const int64_t *rows_dev, int64_t rows, int C, float eps,
                            int dtype, void *stream, const void *add = nullptr, int64_t add_rows = 1);

extern "C" int vtdge_layernorm_add(const void *x, const void *weight, const void *bias, const void *add,
                                   int64_t add_rows, void *out, int64_t rows, int C, float eps, int dtype,
                                   void *stream)
{
    VT_REQUIRE(add != nullptr, VTDGE_ERR_ARG, "layernorm_add: NULL operand");
    return layernorm_launch(x, 0, 0, weight, bias, out, nullptr, rows, C, eps, dtype, stream, add, add_rows);
}

extern "C" int vtdge_layernorm(const void *x, const void *weight, const void *bias, void *out,
                               const int64_t *rows_dev, int64_t rows, int C, float eps, int dtype, void *stream)
{
    return layernorm_launch(x, 0, 0, weight, bias, out, rows_dev, rows, C, eps, dtype, stream);
}

extern "C" int vtdge_layernorm_rows(const void *x, int64_t x_group_stride, int x_group_rows, const void *weight,
                                    const void *bias, void *out, int64_t rows, int C, float eps, int dtype,
                                    void *stream)
{
    VT_REQUIRE(x_group_rows > 0 && x_group_stride >= (int64_t)x_group_rows * C, VTDGE_ERR_ARG,
               "layernorm_rows: groups of %d rows %lld elements apart overlap", x_group_rows, (long long)x_group_stride);
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(x_group_stride % vec == 0, VTDGE_ERR_ARG, "layernorm_rows: the group stride must keep rows 16-byte aligned");
    return layernorm_launch(x, x_group_stride, x_group_rows, weight, bias, out, nullptr, rows, C, eps, dtype, stream);
}

static int layernorm_launch(const void *x, int64_t x_group_stride, int x_group_rows, const void *weight,
                            const void *bias, void *out, const int64_t *rows_dev, int64_t rows, int C, float eps,
                            int dtype, void *stream, const void *add, int64_t add_rows)
{
    VT_REQUIRE(x && weight && bias && out, VTDGE_ERR_ARG, "layernorm: NULL operand");
    VT_REQUIRE(add == nullptr || (add_rows > 0 && aligned16(add)), VTDGE_ERR_ARG,
               "layernorm: the rows to add need a positive count and 16-byte alignment");
    VT_REQUIRE(rows >= 0, VTDGE_ERR_ARG, "layernorm: negative rows");
    if (int rc = check_channels(C, dtype, "layernorm")) return rc;
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(C / vec <= WAVE * MAX_IT, VTDGE_ERR_UNSUPPORTED, "layernorm: C=%d exceeds %d", C,
               WAVE * MAX_IT * vec);
    VT_REQUIRE(aligned16(x) && aligned16(out) && aligned16(weight) && aligned16(bias), VTDGE_ERR_ARG,
               "layernorm: operands must be 16-byte aligned");
    if (rows == 0) return VTDGE_OK;
    const int gs = group_size(C / vec);
    dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK * LN_RPW * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
    const int nit = (int)ceil_div(C / vec, WAVE);
#define VT_LAUNCH(T, NIT, GS)                                                                                        \
    note_kernel(reinterpret_cast<const void *>(layernorm_kernel<T, NIT, GS>)),                                       \
    layernorm_kernel<T, NIT, GS><<<grid, block, 0, st>>>((const T *)x, (const T *)weight, (const T *)bias, (T *)out, \
                                                         rows_dev, rows, C, eps, x_group_stride, x_group_rows,       \
                                                         (const T *)add, add_rows)
#define VT_GROUP(T)                                                                                       \
    do {                                                                                                  \
        if (gs == 64) { if (nit == 1) VT_LAUNCH(T, 1, 64); else if (nit == 2) VT_LAUNCH(T, 2, 64); else VT_LAUNCH(T, 3, 64); } \
        else if (gs == 32) VT_LAUNCH(T, 1, 32); else if (gs == 16) VT_LAUNCH(T, 1, 16); else VT_LAUNCH(T, 1, 8); \
    } while (0)
    if (dtype == VTDGE_F32) VT_GROUP(float); else VT_GROUP(bf16_t);
#undef VT_GROUP
#undef VT_LAUNCH
    return check_launch("layernorm");
}

extern "C" int vtdge_layernorm_stats(const void *x, void *records, const int64_t *rows_dev, int64_t rows, int C,
                                     float eps, int dtype, void *stream)
{
    VT_REQUIRE(x && records, VTDGE_ERR_ARG, "layernorm_stats: NULL operand");
    VT_REQUIRE(rows >= 0, VTDGE_ERR_ARG, "layernorm_stats: negative rows");
    VT_REQUIRE(dtype == VTDGE_BF16, VTDGE_ERR_UNSUPPORTED, "layernorm_stats: records exist for bf16 rows only");
    if (int rc = check_channels(C, dtype, "layernorm_stats")) return rc;
    VT_REQUIRE(C / 8 <= WAVE * MAX_IT, VTDGE_ERR_UNSUPPORTED, "layernorm_stats: C=%d exceeds %d", C, WAVE * MAX_IT * 8);
    VT_REQUIRE(aligned16(x) && aligned16(records), VTDGE_ERR_ARG, "layernorm_stats: operands must be 16-byte aligned");
    if (rows == 0) return VTDGE_OK;
    const int gs = group_size(C / 8);
    dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK * LN_RPW * (WAVE / gs))), block(256);
    hipStream_t st = (hipStream_t)stream;
    const int nit = (int)ceil_div(C / 8, WAVE);
#define VT_LAUNCH(NIT, GS) \
    note_kernel(reinterpret_cast<const void *>(layernorm_stats_kernel<NIT, GS>)), \
    layernorm_stats_kernel<NIT, GS><<<grid, block, 0, st>>>((const bf16_t *)x, (u32x4 *)records, rows_dev, rows, C, eps)
    if (gs == 64) { if (nit == 1) VT_LAUNCH(1, 64); else if (nit == 2) VT_LAUNCH(2, 64); else VT_LAUNCH(3, 64); }
    else if (gs == 32) VT_LAUNCH(1, 32); else if (gs == 16) VT_LAUNCH(1, 16); else VT_LAUNCH(1, 8);
#undef VT_LAUNCH
    return check_launch("layernorm_stats");
}
