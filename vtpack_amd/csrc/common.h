// Shared device/host helpers of the vtdge kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <mutex>
#include <utility>

#include "../../include/vtdge.h"

namespace vtdge {

// ---------------------------------------------------------------- errors
void set_error(const char *fmt, ...);
int check_launch(const char *what);
void note_kernel(const void *host_function);      // called just before every launch (see vtdge_last_kernel)
int compute_units();      // of the current device (256 on an MI355X)

#define VT_REQUIRE(cond, code, ...)  \
    do {                             \
        if (!(cond)) {               \
            set_error(__VA_ARGS__);  \
            return (code);           \
        }                            \
    } while (0)

// Raises a kernel's dynamic-LDS limit the first time its call site runs (once per template instantiation, safe
// when several host threads make their first call at the same time).
#define VT_RESERVE_LDS(kern, bytes, what)                                                                       \
    do {                                                                                                        \
        static std::once_flag vt_once;                                                                          \
        static hipError_t vt_err = hipSuccess;                                                                  \
        std::call_once(vt_once, [&] {                                                                           \
            vt_err = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes));             \
        });                                                                                                     \
        if (vt_err != hipSuccess) {                                                                             \
            ::vtdge::set_error("%s: cannot reserve %zu bytes of LDS", what, (size_t)(bytes));                   \
            return VTDGE_ERR_LAUNCH;                                                                            \
        }                                                                                                       \
    } while (0)

// ---------------------------------------------------------------- types
typedef uint16_t bf16_t;  // raw bfloat16 bits

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round-to-nearest-even, NaN stays NaN (quiet)
__device__ __forceinline__ bf16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

// two floats -> packed bf16 pair, round-to-nearest-even: one v_cvt_pk_bf16_f32 on gfx950
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Statistics record of a row for the Linear that layer-normalises its input on the fly (linear_ws8.hip, HAS_LN):
// 16 bf16 values, the A-side operand of one 16-deep MFMA K step.  mean = m1 + m2 + m3 and sigma = sqrt(var + eps)
// = s1 + s2 are split into bf16 parts; against the column record (-c1, -c2, -c1, -c3, -c2, -c1, b1, b1 | b2, 0, ...)
// of a column with colsum c = c1 + c2 + c3 and bias b = b1 + b2 the K step yields -mean * c + sigma * b with all
// partial products of weight 2^-24 and above (2^-16 for the bias term).  Both halves carry (s1, s2) so that every
// lane of the consumer finds sigma in its own half.
//   lo = (m1, m1, m2, m1, m2, m3, s1, s2)   hi = (s1, s2, 0, 0, 0, 0, 0, 0)
__device__ __forceinline__ void split_bf16x3(float v, uint32_t &p1, uint32_t &p2, uint32_t &p3)
{
    p1 = f32_to_bf16(v);
    const float r1 = v - bf16_to_f32((bf16_t)p1);
    p2 = f32_to_bf16(r1);
    p3 = f32_to_bf16(r1 - bf16_to_f32((bf16_t)p2));
}
__device__ __forceinline__ void ln_record(float mean, float sigma, u32x4 &lo, u32x4 &hi)
{
    uint32_t m1, m2, m3, s1, s2, s3;
    split_bf16x3(mean, m1, m2, m3);
    split_bf16x3(sigma, s1, s2, s3);
    lo.x = m1 | (m1 << 16);
    lo.y = m2 | (m1 << 16);
    lo.z = m2 | (m3 << 16);
    lo.w = s1 | (s2 << 16);
    hi.x = s1 | (s2 << 16);
    hi.y = hi.z = hi.w = 0u;
}
// the matching record of an output column: colsum of the folded weights and the folded bias
__device__ __forceinline__ void ln_column_record(float colsum, float b, u32x4 &lo, u32x4 &hi)
{
    uint32_t c1, c2, c3, b1, b2, b3;
    split_bf16x3(-colsum, c1, c2, c3);
    split_bf16x3(b, b1, b2, b3);
    lo.x = c1 | (c2 << 16);
    lo.y = c1 | (c3 << 16);
    lo.z = c2 | (c1 << 16);
    lo.w = b1 | (b1 << 16);
    hi.x = b2;
    hi.y = hi.z = hi.w = 0u;
}

// Storage-type traits: a 16-byte vector of T holds VEC elements.
template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
    static __device__ __forceinline__ void unpack(const u32x4 &r, float *f)
    {
        f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
        f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float *f)
    {
        u32x4 r;
        r.x = __float_as_uint(f[0]); r.y = __float_as_uint(f[1]);
        r.z = __float_as_uint(f[2]); r.w = __float_as_uint(f[3]);
        return r;
    }
};
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float load(const bf16_t *p) { return bf16_to_f32(*p); }
    static __device__ __forceinline__ void store(bf16_t *p, float v) { *p = f32_to_bf16(v); }
    // the value as stored: the same hardware conversion as pack() (one convert and one shift)
    static __device__ __forceinline__ float round(float v) { return bf16lo(pack_bf16x2(v, 0.f)); }
    static __device__ __forceinline__ void unpack(const u32x4 &r, float *f)
    {
        f[0] = bf16lo(r.x); f[1] = bf16hi(r.x); f[2] = bf16lo(r.y); f[3] = bf16hi(r.y);
        f[4] = bf16lo(r.z); f[5] = bf16hi(r.z); f[6] = bf16lo(r.w); f[7] = bf16hi(r.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float *f)
    {
        u32x4 r;
        r.x = pack_bf16x2(f[0], f[1]); r.y = pack_bf16x2(f[2], f[3]);
        r.z = pack_bf16x2(f[4], f[5]); r.w = pack_bf16x2(f[6], f[7]);
        return r;
    }
};

// ---------------------------------------------------------------- MFMA
// One 32-byte K-slab of a 32x32 output block: lane (r = lane%32, g = lane/32)
// supplies bytes [16g, 16g+16) of row r of each operand.
template <typename T> struct Slab;
template <> struct Slab<bf16_t> {
    static __device__ __forceinline__ void mma(const u32x4 &a, const u32x4 &b, f32x16 &c)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                    0, 0, 0);
    }
};
template <> struct Slab<float> {
    static __device__ __forceinline__ void mma(const u32x4 &a, const u32x4 &b, f32x16 &c)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    }
};

// ---------------------------------------------------------------- direct loads to LDS
// global_load_lds_dwordx4: every lane names 16 bytes of global memory; the wave's 1 KB lands at the wave-uniform
// LDS address `lptr` + lane*16 without passing through VGPRs.  Completion is tracked by vmcnt.
#define VT_GLOBAL_TO_LDS(gptr, lptr)                                                                     \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gptr),             \
                                     (__attribute__((address_space(3))) void *)(lptr), 16, 0, 0)

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding)
template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// one direct load: 64 lanes x 16 B from base + the per-lane byte offset to LDS bytes [lds_addr, lds_addr + 1024)
__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base)
                 : "memory", "m0");
}
// the same for data that is read once and not again (streamed past the caches' reuse-oriented replacement)
__device__ __forceinline__ void dma16_nt(const void *base, uint32_t off, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base)
                 : "memory", "m0");
}
// a wave-uniform pointer as the scalar register pair an address operand of the direct loads needs
__device__ __forceinline__ const void *uniform_ptr(const void *p)
{
    const uint64_t u = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)u);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(u >> 32));
    return reinterpret_cast<const void *>((uintptr_t)(((uint64_t)hi << 32) | lo));
}
// the same with a compile-time byte offset (0 .. 4095) added to the global address.  The instruction adds its
// immediate to the LDS address too, so that is lowered by as much first: lds_addr must be at least IMM.
template <int IMM> __device__ __forceinline__ void dma16_imm(const void *base, uint32_t off, uint32_t lds_addr)
{
    static_assert(IMM >= 0 && IMM < 4096, "immediate offset of a global load");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3" ::"s"(lds_addr - IMM),
                 "v"(off), "s"(base), "n"(IMM)
                 : "memory", "m0");
}
// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N-1>{}): a loop whose index is a constant expression
template <class F, int... I> __device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}
// makes a lane constant opaque at this point, so address arithmetic built on it is redone where it is used instead
// of being kept in registers for the whole kernel
__device__ __forceinline__ int fresh(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// s_waitcnt vmcnt(n) for a wave-uniform runtime n, rounded down to a multiple of 6 and to at most 42 (waiting for
// fewer operations in flight than allowed is always safe).  A balanced tree of three compares: the immediate of
// s_waitcnt cannot come from a register.
__device__ __forceinline__ void wait_vmcnt_dyn(int n)
{
    if (n >= 24) {
        if (n >= 36) {
            if (n >= 42) wait_vmcnt<42>();
            else wait_vmcnt<36>();
        } else {
            if (n >= 30) wait_vmcnt<30>();
            else wait_vmcnt<24>();
        }
    } else {
        if (n >= 12) {
            if (n >= 18) wait_vmcnt<18>();
            else wait_vmcnt<12>();
        } else {
            if (n >= 6) wait_vmcnt<6>();
            else wait_vmcnt<0>();
        }
    }
}

__device__ __forceinline__ void block_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// barrier that also publishes this wave's LDS accesses (all of them complete first) but, unlike __syncthreads(),
// leaves vector-memory operations - the prefetches - in flight
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---------------------------------------------------------------- wave ops
// Sum over the 64 lanes, returned in every lane.  DPP row shifts inside rows of 16 lanes, row broadcasts
// across rows (total in lane 63), one readlane: six short-latency VALU ops instead of six LDS permutes.
__device__ __forceinline__ float wave_sum(float v)
{
#define VT_DPP_ADD(ctrl, row_mask) \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, true))
    VT_DPP_ADD(0x111, 0xf);  // row_shr:1
    VT_DPP_ADD(0x112, 0xf);  // row_shr:2
    VT_DPP_ADD(0x114, 0xf);  // row_shr:4
    VT_DPP_ADD(0x118, 0xf);  // row_shr:8
    VT_DPP_ADD(0x142, 0xa);  // row_bcast:15
    VT_DPP_ADD(0x143, 0xc);  // row_bcast:31
#undef VT_DPP_ADD
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// The same sum for NV values at once, one step of all of them after the other: NV independent dependency chains
// instead of NV times one.
template <int NV> __device__ __forceinline__ void wave_sum_n(float (&v)[NV])
{
#define VT_DPP_STEP(ctrl, row_mask)                                                                          \
    _Pragma("unroll") for (int i = 0; i < NV; i++)                                                           \
        v[i] += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v[i]), ctrl, \
                                                                      row_mask, 0xf, true))
    VT_DPP_STEP(0x111, 0xf);
    VT_DPP_STEP(0x112, 0xf);
    VT_DPP_STEP(0x114, 0xf);
    VT_DPP_STEP(0x118, 0xf);
    VT_DPP_STEP(0x142, 0xa);
    VT_DPP_STEP(0x143, 0xc);
#undef VT_DPP_STEP
#pragma unroll
    for (int i = 0; i < NV; i++)
        v[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[i]), 63));
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// ---------------------------------------------------------------- statistics records of rows held by a wave
// Lane exchanges of the record sums below: the value of the lane whose number differs in one bit.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// v summed over the lanes that differ in bits 2..5 of the lane number (16 of them), returned in each of them
__device__ __forceinline__ float sum_over_lane_bits_2_to_5(float v)
{
    v += dpp_move<0x141>(dpp_move<0x1B>(v));      // lane ^ 4: the quad reversed, then the half row mirrored
    v += dpp_move<0x128>(v);                      // lane ^ 8: the row rotated by eight
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);        // lane ^ 16: odd rows swapped with even rows
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r32[0]) + __uint_as_float(r32[1]);     // lane ^ 32: the halves swapped
}
// Statistics record of one stored row from the sums of (x - pivot) and (x - pivot)^2 over its C values, the pivot
// being a value of the row itself (no cancellation however far the row's mean is from zero).
__device__ __forceinline__ void row_record(float pivot, float s1, float s2, int C, float eps, u32x4 &lo, u32x4 &hi)
{
    const float m = s1 / (float)C;
    const float var = fmaxf(s2 / (float)C - m * m, 0.f);
    ln_record(pivot + m, sqrtf(var + eps), lo, hi);
}
// The records of FOUR rows that a wave holds side by side (every lane a piece of each row): st[2 t], st[2 t + 1] are
// the lane's sums of (x - pivot[t]) and (x - pivot[t])^2 over its piece of row t (zero in lanes that hold nothing),
// pivot[t] wave-uniform.  The eight sums are added up over the wave so that each lane ends with the pair of ONE row:
// lanes exchange halves of what they hold with lane ^ 1 (even lanes keep rows 0 and 1, odd ones 2 and 3), then with
// lane ^ 2, and the remaining pair is summed over the other four lane bits.  Lane l then holds row
// 2 (l % 2) + (l / 2) % 2 and works out that row's record - the four records are made side by side in different
// lanes, not one after the other in all of them - and lanes 0..7 write the 128 contiguous bytes at `rec4` (the record
// of the first row; the rows are consecutive): half (l / 4) % 2 of their row.  Rows nrows .. 3 are not written.
// (The pivots come by value: behind a reference the selection below turns into a load through a computed address
// and the array into a spill.)
__device__ __forceinline__ void write_records4(const float (&st)[8], float pivot0, float pivot1, float pivot2,
                                               float pivot3, int C, float eps, u32x4 *__restrict__ rec4,
                                               int nrows = 4)
{
    const int lane = threadIdx.x & 63;
    const bool b0 = (lane & 1) != 0, b1 = (lane & 2) != 0;
    float r4[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float keep = b0 ? st[4 + i] : st[i], send = b0 ? st[i] : st[4 + i];
        r4[i] = keep + dpp_move<0xB1>(send);                 // lane ^ 1
    }
    float tot[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float keep = b1 ? r4[2 + i] : r4[i], send = b1 ? r4[i] : r4[2 + i];
        tot[i] = sum_over_lane_bits_2_to_5(keep + dpp_move<0x4E>(send));      // lane ^ 2, then the rest
    }
    const float pv = b0 ? (b1 ? pivot3 : pivot2) : (b1 ? pivot1 : pivot0);
    u32x4 lo, hi;
    row_record(pv, tot[0], tot[1], C, eps, lo, hi);
    const int row = 2 * (lane & 1) + ((lane >> 1) & 1), half = (lane >> 2) & 1;
    if (lane < 8 && row < nrows) rec4[row * 2 + half] = half ? hi : lo;
}

__device__ __forceinline__ int64_t live_rows(const int64_t *rows_dev, int64_t rows)
{
    if (rows_dev == nullptr) return rows;
    int64_t r = *rows_dev;
    return r < rows ? r : rows;
}

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace vtdge
