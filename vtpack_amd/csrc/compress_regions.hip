// Grained sampling by REGION: index->patch and compress in one kernel, a wave per 4 x 4 region.
//
// The packed rows of a region are consecutive (samples in order, a sample's extra tokens first, then its regions in
// row-major order, sub-patches in row-major order inside a region), so a wave that knows how many rows come before
// its region needs no descriptor list to place the region's queries: it reads the region's 16 token rows once and
// writes the 16, 4 or 1 window means (the same fp32 sums in dy-outer / dx-inner order and the same single rounding
// as the row-wise compress kernel).  The rows before a region are the query counts of all regions before it: a byte
// per region when the kernel that chose the gate indices has left them (`counts`: a few KB per wave out of L2, summed
// four bytes per instruction), else worked out from the 64-bit gate indices themselves.
//
// The same wave writes the region's patch descriptors, the first wave of a sample the sample's offset, length and
// extra tokens, the wave of the last region the total - everything index->patch would - and, for bf16 rows, the
// statistics record of every packed row as stored (sums about a value of the row itself, four rows side by side),
// which is what a Linear with a folded LayerNorm takes next to the raw rows.
#include "common.h"
#include "region_pack.h"
#include <type_traits>

namespace vtdge {

template <typename T, bool REC>
__global__ __launch_bounds__(256) void compress_regions_kernel(
    const T *__restrict__ x, const int64_t *__restrict__ indices, const int64_t *__restrict__ splits,
    const uint8_t *__restrict__ counts, T *__restrict__ comp, u32x4 *__restrict__ records,
    int64_t *__restrict__ patches, int64_t capacity, int64_t *__restrict__ offsets, int64_t *__restrict__ lengths,
    int32_t *__restrict__ region_rows, int B, int H, int W, int C, int extra, int S, float eps)
{
    constexpr int VEC = Elem<T>::VEC;
    constexpr int R = 4;
    const int lane = threadIdx.x & 63;
    const int Hr = H / R, Wr = W / R, nreg = Hr * Wr;
    const int region = (int)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (region >= B * nreg) return;
    const int b = region / nreg, rr = region - b * nreg;
    const int ry = rr / Wr, rx = rr - ry * Wr;
    const int N = extra + H * W;
    const int nvec = C / VEC;

    auto count_of = [&](int reg) {
        int64_t g = indices[reg];
        g = g < 0 ? 0 : (g >= S ? S - 1 : g);
        const int ps = (int)splits[g];
        return ps * ps;
    };
    // ---- queries of all regions before this one (small integers: the float sums below are exact)
    float before = 0.f;
    if (counts != nullptr) {
        const u32x4 *c4 = reinterpret_cast<const u32x4 *>(counts);
        for (int i = lane; i * 16 < region; i += WAVE) {
            const u32x4 v = c4[i];
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            uint32_t sum = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int left = region - (i * 16 + 4 * k);          // bytes of this word that lie before the region
                const uint32_t word = left >= 4 ? w[k] : left <= 0 ? 0u : w[k] & ((1u << (8 * left)) - 1u);
                sum = __builtin_amdgcn_udot4(word, 0x01010101u, sum, false);
            }
            before += (float)sum;
        }
    } else {
        for (int i = lane; i < region; i += WAVE) before += (float)count_of(i);
    }
    const int64_t r0 = (int64_t)wave_sum(before) + (int64_t)extra * (b + 1);      // first packed row of the region
    // the region's own split: from its count byte when there is one (no trip through the indices and the splits)
    int ps;
    if (counts != nullptr) {
        const int cnt = __builtin_amdgcn_readfirstlane((int)counts[region]);
        ps = cnt == 16 ? 4 : cnt == 4 ? 2 : 1;
    } else {
        int64_t gi = indices[region];
        gi = gi < 0 ? 0 : (gi >= S ? S - 1 : gi);
        ps = __builtin_amdgcn_readfirstlane((int)splits[gi]);
    }
    const int nq = ps == 4 ? 16 : ps == 2 ? 4 : 1;
    if (region_rows != nullptr && lane == 0) region_rows[region] = (int32_t)r0;

    // ---- the bookkeeping index->patch leaves: descriptors, offsets, lengths
    if (patches != nullptr && lane < nq) {
        const int pq = nq == 16 ? 4 : nq == 4 ? 2 : 1, step = R / pq;       // windows per side, tokens per window side
        const int dy = lane / pq, dx = lane - dy * pq;
        const int64_t row = r0 + lane;
        if (row < capacity) {
            typedef long long i64x2 __attribute__((ext_vector_type(2)));
            i64x2 *p = reinterpret_cast<i64x2 *>(patches + 4 * row);
            p[0] = i64x2{(long long)b, (long long)(ry * R + dy * step)};
            p[1] = i64x2{(long long)(rx * R + dx * step), (long long)step};
        }
    }
    if (rr == 0) {
        const int64_t row_b = r0 - extra;
        float mine = 0.f;
        if (counts != nullptr) {
            for (int i = lane; i < nreg; i += WAVE) mine += (float)counts[region + i];
        } else {
            for (int i = lane; i < nreg; i += WAVE) mine += (float)count_of(region + i);
        }
        const int64_t len = (int64_t)wave_sum(mine) + extra;
        if (lane == 0) {
            offsets[b] = row_b;
            lengths[b] = len;
            if (b == B - 1) offsets[B] = row_b + len;
        }
        if (patches != nullptr && lane < extra && row_b + lane < capacity) {
            int64_t *p = patches + 4 * (row_b + lane);
            p[0] = b; p[1] = -(int64_t)lane - 1; p[2] = 0; p[3] = 1;
        }
    }

    // ---- the region's tokens -> its packed rows (never past the buffers, whatever the counts say)
    if (r0 + nq > capacity) return;
    const bool act = lane < nvec;
    const int v = act ? lane : 0;
    const T *xp = x + ((int64_t)b * N + extra + (int64_t)(ry * R) * W + rx * R) * C + v * VEC;
    T *cp = comp + r0 * (int64_t)C + v * VEC;
    u32x4 *rec = REC ? records + r0 * 2 : nullptr;
    if (rr == 0)             // the sample's extra tokens: packed rows r0 - extra .. r0 - 1, copied
        pack_front_rows<T, REC>(x + (int64_t)b * N * C + v * VEC, comp + (r0 - extra) * (int64_t)C + v * VEC,
                                REC ? records + (r0 - extra) * 2 : nullptr, extra, C, eps, act, lane);
    pack_region<T, REC>(xp, cp, rec, ps, W, C, eps, act, lane);
}

}  // namespace vtdge

using namespace vtdge;

extern "C" int vtdge_compress_regions(const void *x, const int64_t *indices, const int64_t *splits,
                                      const uint8_t *counts, void *comp, void *records, float records_eps,
                                      int64_t *patches, int64_t capacity_rows, int64_t *offsets, int64_t *lengths,
                                      int32_t *region_rows, int B, int H, int W, int C, int extra, int R, int S,
                                      int dtype, void *stream)
{
    VT_REQUIRE(x && indices && splits && comp && offsets && lengths, VTDGE_ERR_ARG, "compress_regions: NULL operand");
    VT_REQUIRE(B > 0 && H > 0 && W > 0 && extra >= 0 && capacity_rows >= 0, VTDGE_ERR_ARG, "compress_regions: bad sizes");
    VT_REQUIRE(R == 4, VTDGE_ERR_UNSUPPORTED, "compress_regions: region size %d (4 only)", R);
    VT_REQUIRE(H % R == 0 && W % R == 0, VTDGE_ERR_ARG, "compress_regions: H=%d, W=%d not multiples of region %d", H, W, R);
    VT_REQUIRE(S >= 1 && S <= VTDGE_MAX_SPLITS, VTDGE_ERR_UNSUPPORTED, "compress_regions: S=%d outside [1,%d]", S,
               VTDGE_MAX_SPLITS);
    VT_REQUIRE(dtype == VTDGE_F32 || dtype == VTDGE_BF16, VTDGE_ERR_ARG, "compress_regions: unknown dtype %d", dtype);
    const int vec = dtype == VTDGE_BF16 ? 8 : 4;
    VT_REQUIRE(C > 0 && C % vec == 0 && C / vec <= WAVE, VTDGE_ERR_UNSUPPORTED,
               "compress_regions: C=%d must be a multiple of %d up to %d (one 16-byte vector per lane)", C, vec, WAVE * vec);
    VT_REQUIRE(extra <= WAVE, VTDGE_ERR_UNSUPPORTED, "compress_regions: more than %d extra tokens", WAVE);
    const int64_t regions = (int64_t)B * (H / R) * (W / R);
    // a wave adds up the counts of every region before its own, and row numbers pass through fp32 sums
    VT_REQUIRE(regions <= 65536 && (int64_t)B * (extra + (int64_t)H * W) < (1 << 24), VTDGE_ERR_UNSUPPORTED,
               "compress_regions: %lld regions (at most 65536; use index_to_patch + compress)", (long long)regions);
    VT_REQUIRE(records == nullptr || dtype == VTDGE_BF16, VTDGE_ERR_UNSUPPORTED,
               "compress_regions: statistics records exist for bf16 rows only");
    const auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    VT_REQUIRE(a16(x) && a16(comp) && a16(records) && a16(patches) && a16(counts), VTDGE_ERR_ARG,
               "compress_regions: operands must be 16-byte aligned");
    dim3 grid((unsigned)ceil_div(regions, 4)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define VT_LAUNCH(T, RECF)                                                                                         \
    note_kernel(reinterpret_cast<const void *>(compress_regions_kernel<T, RECF>)),                                 \
    compress_regions_kernel<T, RECF><<<grid, block, 0, st>>>((const T *)x, indices, splits, counts, (T *)comp,     \
                                                             (u32x4 *)records, patches, capacity_rows, offsets,    \
                                                             lengths, region_rows, B, H, W, C, extra, S, records_eps)
    if (dtype == VTDGE_F32) VT_LAUNCH(float, false);
    else if (records != nullptr) VT_LAUNCH(bf16_t, true);
    else VT_LAUNCH(bf16_t, false);
#undef VT_LAUNCH
    return check_launch("compress_regions");
}
