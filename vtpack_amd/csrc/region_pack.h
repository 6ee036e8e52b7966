// Packing the tokens of 4 x 4 regions into query rows, for the kernels that do it a wave per region.
#pragma once
#include "common.h"

namespace vtdge {

// One row's lane sums about the row's first element (wave-uniform pivot); zero in lanes that hold nothing.
template <typename T>
__device__ __forceinline__ void lane_sums(const u32x4 &packed, bool act, float &pivot, float &a, float &q)
{
    constexpr int VEC = Elem<T>::VEC;
    float f[VEC];
    Elem<T>::unpack(packed, f);
    pivot = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(f[0])));
    float sa = 0.f, sq = 0.f;
#pragma unroll
    for (int c = 0; c < VEC; c++) {
        const float d = f[c] - pivot;
        sa += d;
        sq += d * d;
    }
    a = act ? sa : 0.f;
    q = act ? sq : 0.f;
}

// acc += the values of one stored vector
template <typename T> __device__ __forceinline__ void add_vector(float (&acc)[Elem<T>::VEC], const u32x4 &raw)
{
    float f[Elem<T>::VEC];
    Elem<T>::unpack(raw, f);
#pragma unroll
    for (int c = 0; c < Elem<T>::VEC; c++) acc[c] += f[c];
}

// A sample's extra tokens copied to its first packed rows.  xs / cs: the sample's first token row and its first
// packed row, both at this lane's vector; rec: the first packed row's record (REC).
template <typename T, bool REC>
__device__ __forceinline__ void pack_front_rows(const T *xs, T *cs, u32x4 *rec, int extra, int C, float eps, bool act,
                                                int lane)
{
    for (int e = 0; e < extra; e++) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (act) {
            raw = *reinterpret_cast<const u32x4 *>(xs + (int64_t)e * C);
            *reinterpret_cast<u32x4 *>(cs + (int64_t)e * C) = raw;
        }
        if constexpr (REC) {
            float pivot, st[2];
            lane_sums<T>(raw, act, pivot, st[0], st[1]);
            wave_sum_n<2>(st);
            u32x4 lo, hi;
            row_record(pivot, st[0], st[1], C, eps, lo, hi);
            if (lane < 2) rec[e * 2 + lane] = lane ? hi : lo;
        }
    }
}

// The 16 tokens of one 4 x 4 region -> its 16, 4 or 1 packed rows (ps = 4, 2, 1 windows a side), one wave, lane =
// 16-byte vector of a row (`act`: the lane holds one).  xp: the region's first token, cp: its first packed row, both at
// this lane's vector; rec: that row's record (REC).  fp32 sums in dy-outer / dx-inner order, one rounding.
template <typename T, bool REC>
__device__ __forceinline__ void pack_region(const T *xp, T *cp, u32x4 *rec, int ps, int W, int C, float eps, bool act,
                                            int lane)
{
    constexpr int VEC = Elem<T>::VEC;
    const u32x4 z = {0u, 0u, 0u, 0u};
    // Four token vectors in flight per lane at a time (16 registers): the kernel is meant to run beside a
    // weight-stationary Linear that leaves 48 registers a lane free on every SIMD, and only waves that fit there
    // make progress before that Linear ends.
    float acc[VEC];
    if (ps == 4) {
        // every token is its own query (0 + x, rounded: the mean of a window of one); one token row at a time
#pragma unroll 1
        for (int dy = 0; dy < 4; dy++) {
            u32x4 raw[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                raw[t] = z;
                if (act) raw[t] = *reinterpret_cast<const u32x4 *>(xp + ((int64_t)dy * W + t) * C);
            }
            float pivot[4], st[8];
#pragma unroll
            for (int t = 0; t < 4; t++) {
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] = 0.f;
                add_vector<T>(acc, raw[t]);
                const u32x4 packed = Elem<T>::pack(acc);
                if (act) *reinterpret_cast<u32x4 *>(cp + (int64_t)(4 * dy + t) * C) = packed;
                if constexpr (REC) lane_sums<T>(packed, act, pivot[t], st[2 * t], st[2 * t + 1]);
            }
            if constexpr (REC) write_records4(st, pivot[0], pivot[1], pivot[2], pivot[3], C, eps, rec + 4 * dy * 2);
        }
    } else if (ps == 2) {
        // 2 x 2 windows, one at a time: tokens (2 wy, 2 wx), (2 wy, 2 wx + 1), (2 wy + 1, 2 wx), (2 wy + 1, 2 wx + 1)
#pragma unroll 1
        for (int wy = 0; wy < 2; wy++) {
            float pivot[4] = {0.f, 0.f, 0.f, 0.f}, st[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int wx = 0; wx < 2; wx++) {
                u32x4 raw[4];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    raw[t] = z;
                    if (act)
                        raw[t] = *reinterpret_cast<const u32x4 *>(xp + ((int64_t)(2 * wy + t / 2) * W + 2 * wx + t % 2) * C);
                }
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] = 0.f;
#pragma unroll
                for (int t = 0; t < 4; t++) add_vector<T>(acc, raw[t]);
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] *= 0.25f;
                const u32x4 packed = Elem<T>::pack(acc);
                if (act) *reinterpret_cast<u32x4 *>(cp + (int64_t)(2 * wy + wx) * C) = packed;
                if constexpr (REC) lane_sums<T>(packed, act, pivot[wx], st[2 * wx], st[2 * wx + 1]);
            }
            if constexpr (REC) write_records4(st, pivot[0], pivot[1], pivot[2], pivot[3], C, eps, rec + 2 * wy * 2, 2);
        }
    } else {
        // one window over the whole region
#pragma unroll
        for (int c = 0; c < VEC; c++) acc[c] = 0.f;
#pragma unroll 1
        for (int dy = 0; dy < 4; dy++) {
            u32x4 raw[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                raw[t] = z;
                if (act) raw[t] = *reinterpret_cast<const u32x4 *>(xp + ((int64_t)dy * W + t) * C);
            }
#pragma unroll
            for (int t = 0; t < 4; t++) add_vector<T>(acc, raw[t]);
        }
#pragma unroll
        for (int c = 0; c < VEC; c++) acc[c] *= 0.0625f;
        const u32x4 packed = Elem<T>::pack(acc);
        if (act) *reinterpret_cast<u32x4 *>(cp) = packed;
        if constexpr (REC) {
            float pivot, st[2];
            lane_sums<T>(packed, act, pivot, st[0], st[1]);
            wave_sum_n<2>(st);
            u32x4 lo, hi;
            row_record(pivot, st[0], st[1], C, eps, lo, hi);
            if (lane < 2) rec[lane] = lane ? hi : lo;
        }
    }
}

}  // namespace vtdge
