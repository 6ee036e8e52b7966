// Sparse attention, bf16 / head_dim 64 fast path (gfx950).
//
// Same mathematics and MFMA mapping as attention.hip (S^T = K Q^T, O^T = V^T P^T, a lane owns one query),
// restructured around what limits this operator at head_dim 64: the softmax's vector instructions (a wave issues
// one every ~5 clocks, and there are about five per score against a quarter of an MFMA clock) and the K/V staging.
//   * up to 288 keys (the 256 px models): K and V of a (sample, head) stay resident in LDS, double buffered across
//     items by direct loads; V is transposed by the LDS read itself (ds_read_b64_tr_b16); the tile loop is a
//     hand-ordered software pipeline in which the reference of the softmax rides in the MFMA accumulator;
//   * longer sequences (512 px, spatially reduced PVT stages): K/V stages of 128 keys double buffered in LDS, K by
//     direct loads, V through registers and transposed writes, online softmax in the log2 domain.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

namespace vtdge {

constexpr int AQ = 128;    // query rows per workgroup of the streaming kernel (4 waves x 32)

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
constexpr float ATT_RESCALE = 8.0f;   // log2 units a score may exceed its row's reference by before that is raised
constexpr int ATT_TBL = 512;          // items per workgroup whose first row and query count are kept in LDS

// acc + lo + hi of a packed bf16 pair in fp32 (v_dot2c_f32_bf16 against (1, 1))
__device__ __forceinline__ float bf16_pair_sum(uint32_t pair, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), __builtin_bit_cast(bf16x2, 0x3f803f80u),
                                           acc, false);
}

// ---------------------------------------------------------------------------------------------------------
// One 32-query tile against all resident keys, software-pipelined over blocks of 32 keys: while the vector ALU
// turns the scores of block kb into probabilities, the matrix pipe already multiplies K of block kb+1 with Q, and
// every fragment of K is read from LDS one block before the MFMA that consumes it.  The order of the instructions
// below is the order they are meant to issue in (pinned by scheduling barriers): a wave issues one vector
// instruction every ~5 clocks (v_exp_f32 ~12, v_cvt_pk_bf16_f32 ~8) and the softmax is what the tile waits for, so
// its instruction count is what is kept small; the MFMAs ride along.
//
// The queries are multiplied by scale * log2(e) when they are loaded, and the score MFMAs start from an
// accumulator that holds minus the row's reference m: a block's scores come out of the matrix pipe as
// s' = log2-scaled score - m, and a probability is one v_exp_f32 of that.  The reference of a row is its maximum
// over the first block; later it is only raised (and the running sums rescaled) when some score of a block exceeds
// it by more than ATT_RESCALE, which is decided before the next block's MFMAs are issued.  Any reference cancels in
// the final division, so this is the same softmax as the max-subtracted one.
struct AttnTile {
    const unsigned char *krow;      // K row `lr` of block 0 in LDS
    const unsigned char *vlane;     // this lane's source address for the transposing reads of V, block 0, d < 32
    const unsigned char *vlane_hi;  // HI: the same for d >= 32, vlane ^ 64 (key offsets are multiples of 128 bytes,
                                    // so the XOR can be taken once and every read is a base plus a constant)
    int n, lg;
};

__device__ __forceinline__ u32x4 att_read_k(const AttnTile &t, const int (&cs)[4], int kb, int sl)
{
    return *reinterpret_cast<const u32x4 *>(t.krow + kb * 32 * 128 + cs[sl]);
}
// V stays row-major in LDS ([key][d], 128-byte rows like K) and is transposed on the way to the registers:
// ds_read_b64_tr_b16 works on blocks of 16 lanes; source lane 4e + r of a block names four consecutive 16-bit
// elements, and lane i of the block receives, as its element e, column (i & 3) of source lane 4e + (i >> 2).  With
// source lane 4e + r pointing at key k0 + e, channels d0 + 4r .. d0 + 4r + 3, lane i receives keys k0 .. k0 + 3 of
// channel d0 + i: four K-elements of a row of V^T.  The first operand of O^T += V^T P^T wants, in lane (lr, lg),
// channel 32 db + lr and the eight keys the lane's own P fragment holds (16 h + 4 lg + j and 16 h + 8 + 4 lg + j,
// j < 4): two such reads, with k0 = 16 h + 4 lg (+ 8) and d0 = 32 db + 16 (block & 1).  Rows are stored with their
// 16-byte chunks XOR-ed by 2 (key & 3), so the sixteen 8-byte pieces of a block come from sixteen different bank
// groups; the XOR constant of a lane does not depend on kb, h or the +8, and db = 1 is the address XOR 64.
typedef short att_v4s __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 att_tr_read(const unsigned char *p)
{
    const att_v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) att_v4s *)(uint32_t)(uintptr_t)p);
    return __builtin_bit_cast(u32x2, r);
}
__device__ __forceinline__ const unsigned char *att_v_lane(const unsigned char *vbase, int lane)
{
    const int blk = lane >> 4, i = lane & 15;
    const int e = i >> 2, r = i & 3;                   // role of this lane as a source
    const int key = 4 * (blk >> 1) + e;                 // + 32 kb + 16 h (+ 8)
    const int chunk = (2 * (blk & 1) + (r >> 1)) ^ (2 * (key & 3));
    return vbase + key * 128 + chunk * 16 + 8 * (r & 1);
}
// HI: the tile carries the address for d >= 32 (two instructions a block less; in the resident kernel the extra
// register costs more than they do: 45 against 38 us)
template <bool HI>
__device__ __forceinline__ void att_read_v(const AttnTile &t, int kb, u32x4 (&vf)[4])
{
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int db = 0; db < 2; db++) {
            const unsigned char *p =
                HI ? (db ? t.vlane_hi : t.vlane) + (kb * 32 + 16 * h) * 128
                   : reinterpret_cast<const unsigned char *>((uintptr_t)(t.vlane + (kb * 32 + 16 * h) * 128) ^ (64u * db));
            const u32x2 lo = att_tr_read(p), hi = att_tr_read(p + 8 * 128);
            vf[2 * h + db].x = lo.x;
            vf[2 * h + db].y = lo.y;
            vf[2 * h + db].z = hi.x;
            vf[2 * h + db].w = hi.y;
        }
}
#define VT_PIN() __builtin_amdgcn_sched_barrier(0)
__device__ __forceinline__ f32x16 att_mfma(const u32x4 &a, const u32x4 &b, const f32x16 &acc)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0,
                                                   0, 0);
}
// q * f for the packed bf16 pairs of a fragment (round to nearest even)
__device__ __forceinline__ u32x4 att_scale_frag(const u32x4 &q, float f)
{
    u32x4 r;
    r.x = pack_bf16x2(bf16lo(q.x) * f, bf16hi(q.x) * f);
    r.y = pack_bf16x2(bf16lo(q.y) * f, bf16hi(q.y) * f);
    r.z = pack_bf16x2(bf16lo(q.z) * f, bf16hi(q.z) * f);
    r.w = pack_bf16x2(bf16lo(q.w) * f, bf16hi(q.w) * f);
    return r;
}
__device__ __forceinline__ float att_max16(const f32x16 &s)
{
    const float a = fmaxf(fmaxf(fmaxf(s[0], s[1]), s[2]), fmaxf(fmaxf(s[3], s[4]), s[5]));
    const float b = fmaxf(fmaxf(fmaxf(s[6], s[7]), s[8]), fmaxf(fmaxf(s[9], s[10]), s[11]));
    return fmaxf(fmaxf(a, b), fmaxf(fmaxf(fmaxf(s[12], s[13]), s[14]), s[15]));
}
// The largest of a lane's 16 scores IF one of them is positive (else some negative value): the maximum of their bit
// patterns as signed integers, which orders positive floats as floats and puts every negative one below them.  That
// is all the test against the (positive) rescaling threshold needs, and it takes eight v_max3_i32, where fmaxf() on
// values whose origin the compiler cannot see (the output of an MFMA) brings one more instruction per operand to
// quiet signalling NaNs: 14 instructions for the same decision, a quarter of the softmax's full-rate vector work.
__device__ __forceinline__ float att_max16_if_positive(const f32x16 &s)
{
    const auto bits = [&](int e) { return __float_as_int(s[e]); };
    const auto max3 = [](int a, int b, int c) { return max(max(a, b), c); };
    int a = max3(bits(0), bits(1), bits(2)), b = max3(bits(8), bits(9), bits(10));
    a = max3(a, bits(3), bits(4));
    b = max3(b, bits(11), bits(12));
    a = max3(a, bits(5), bits(6));
    b = max3(b, bits(13), bits(14));
    a = max3(a, bits(7), bits(15));
    return __int_as_float(max(a, b));
}

// One step of the pipeline: softmax of block kb (scores relative to the reference in `sc`) and O^T += V^T P^T,
// interleaved with the score MFMAs of block kb+1 (fragments in `kf` -> `sn`, when NEXT); each fragment of K is
// replaced by that of block kb+2 (when NEXT2) as soon as its MFMA has been issued.  MASK: block kb is the last
// one and runs past the keys.
// FAST: no test of the block's scores against the reference (the caller looks at the row sums once per stage).
template <bool NEXT, bool NEXT2, bool MASK, bool HI = false, bool FAST = false>
__device__ __forceinline__ void att_step(const AttnTile &t, const int (&cs)[4], int kb, f32x16 &sc, f32x16 &sn,
                                         u32x4 (&kf)[4], const u32x4 (&qf)[4], f32x16 (&o)[2], f32x16 &negm,
                                         float (&l)[2])
{
    u32x4 vf[4];
    att_read_v<HI>(t, kb, vf);
    if constexpr (MASK) {
        const int lim = t.n - kb * 32 - 4 * t.lg;
#pragma unroll
        for (int e = 0; e < 16; e++)
            if (8 * (e >> 2) + (e & 3) >= lim) sc[e] = -INFINITY;
    }
    const float mx = FAST ? 0.f : att_max16_if_positive(sc);
    if (!FAST && __builtin_amdgcn_ballot_w64(mx > ATT_RESCALE) != 0) {      // wave-uniform and rare
        const float mrow = fmaxf(mx, __shfl_xor(mx, 32, WAVE));     // both lanes of a row decide alike
        const float delta = mrow > ATT_RESCALE ? mrow : 0.f;
        const float alpha = __builtin_amdgcn_exp2f(-delta);
        l[0] *= alpha;
        l[1] *= alpha;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            o[0][e] *= alpha;
            o[1][e] *= alpha;
            sc[e] -= delta;
            negm[e] -= delta;
        }
    }
    VT_PIN();
    u32x4 pf[2];
    float p[16];
#pragma unroll
    for (int e = 0; e < 4; e++) p[e] = __builtin_amdgcn_exp2f(sc[e]);
    VT_PIN();
    if constexpr (NEXT) sn = att_mfma(kf[0], qf[0], negm);
    if constexpr (NEXT2) kf[0] = att_read_k(t, cs, kb + 2, 0);
    VT_PIN();
#pragma unroll
    for (int e = 4; e < 8; e++) p[e] = __builtin_amdgcn_exp2f(sc[e]);
    VT_PIN();
    if constexpr (NEXT) sn = att_mfma(kf[1], qf[1], sn);
    if constexpr (NEXT2) kf[1] = att_read_k(t, cs, kb + 2, 1);
    VT_PIN();
    pf[0].x = pack_bf16x2(p[0], p[1]);
    pf[0].y = pack_bf16x2(p[2], p[3]);
    pf[0].z = pack_bf16x2(p[4], p[5]);
    pf[0].w = pack_bf16x2(p[6], p[7]);
    // the row sum is taken over the rounded probabilities, the values the second MFMA multiplies with
    l[0] = bf16_pair_sum(pf[0].x, l[0]);
    l[1] = bf16_pair_sum(pf[0].y, l[1]);
    l[0] = bf16_pair_sum(pf[0].z, l[0]);
    l[1] = bf16_pair_sum(pf[0].w, l[1]);
    VT_PIN();
    o[0] = att_mfma(vf[0], pf[0], o[0]);
    VT_PIN();
#pragma unroll
    for (int e = 8; e < 12; e++) p[e] = __builtin_amdgcn_exp2f(sc[e]);
    VT_PIN();
    o[1] = att_mfma(vf[1], pf[0], o[1]);
    VT_PIN();
#pragma unroll
    for (int e = 12; e < 16; e++) p[e] = __builtin_amdgcn_exp2f(sc[e]);
    VT_PIN();
    if constexpr (NEXT) sn = att_mfma(kf[2], qf[2], sn);
    if constexpr (NEXT2) kf[2] = att_read_k(t, cs, kb + 2, 2);
    VT_PIN();
    pf[1].x = pack_bf16x2(p[8], p[9]);
    pf[1].y = pack_bf16x2(p[10], p[11]);
    pf[1].z = pack_bf16x2(p[12], p[13]);
    pf[1].w = pack_bf16x2(p[14], p[15]);
    VT_PIN();
    if constexpr (NEXT) sn = att_mfma(kf[3], qf[3], sn);
    if constexpr (NEXT2) kf[3] = att_read_k(t, cs, kb + 2, 3);
    VT_PIN();
    l[0] = bf16_pair_sum(pf[1].x, l[0]);
    l[1] = bf16_pair_sum(pf[1].y, l[1]);
    l[0] = bf16_pair_sum(pf[1].z, l[0]);
    l[1] = bf16_pair_sum(pf[1].w, l[1]);
    VT_PIN();
    o[0] = att_mfma(vf[2], pf[1], o[0]);
    o[1] = att_mfma(vf[3], pf[1], o[1]);
    VT_PIN();
}

// Block 0 of a tile: raw scores, the row's first reference, and the accumulator the later score MFMAs start from.
__device__ __forceinline__ void att_first_block(const AttnTile &t, const int (&cs)[4], int nblk, u32x4 (&kf)[4],
                                                const u32x4 (&qf)[4], f32x16 &s0, f32x16 &negm)
{
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sl = 0; sl < 4; sl++) kf[sl] = att_read_k(t, cs, 0, sl);
    s0 = att_mfma(kf[0], qf[0], zero);
    s0 = att_mfma(kf[1], qf[1], s0);
    s0 = att_mfma(kf[2], qf[2], s0);
    s0 = att_mfma(kf[3], qf[3], s0);
    if (nblk > 1) {
#pragma unroll
        for (int sl = 0; sl < 4; sl++) kf[sl] = att_read_k(t, cs, 1, sl);
    }
    if (nblk == 1 && t.n < 32) {               // a lone, partial block: its missing keys must not set the reference
        const int lim = t.n - 4 * t.lg;
#pragma unroll
        for (int e = 0; e < 16; e++)
            if (8 * (e >> 2) + (e & 3) >= lim) s0[e] = -INFINITY;
    }
    float m = att_max16(s0);
    m = fmaxf(m, __shfl_xor(m, 32, WAVE));         // key 0 always exists: m is finite
#pragma unroll
    for (int e = 0; e < 16; e++) {
        s0[e] -= m;
        negm[e] = -m;
    }
}

// All key blocks of one tile, the number of blocks known at compile time: the pipeline fully unrolled, the two
// score buffers addressed by constants.  Leaves the halves of the row sum of this lane's keys in l[0] + l[1].
template <int NBLK>
__device__ __forceinline__ void att_tile_fixed(const AttnTile &t, const int (&cs)[4], const u32x4 (&qf)[4],
                                               f32x16 (&o)[2], float &l_run)
{
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    u32x4 kf[4];
    f32x16 sbuf[2], negm;
    float l[2] = {0.f, 0.f};
    o[0] = zero;
    o[1] = zero;
    att_first_block(t, cs, NBLK, kf, qf, sbuf[0], negm);
    const bool partial = (t.n & 31) != 0;           // wave-uniform
    static_for<NBLK>([&](auto kbc) {
        constexpr int kb = decltype(kbc)::value;
        constexpr bool NEXT = kb + 1 < NBLK, NEXT2 = kb + 2 < NBLK;
        if constexpr (kb == NBLK - 1) {
            if (partial) att_step<NEXT, NEXT2, true>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
            else att_step<NEXT, NEXT2, false>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
        } else {
            att_step<NEXT, NEXT2, false>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
        }
    });
    l_run = l[0] + l[1];
}

// One stage of NB key blocks of a sequence that is streamed through LDS in stages (t addresses the stage's rows;
// t.n = keys left from the stage's first one).  `first`: the stage opens the sequence (negm is zero and the row's
// reference is taken from the stage's first block); otherwise the running reference in negm is carried on.  The
// last block is masked when t.n < 32 NB.
//
// FAST: the blocks of the stage run without the per-block test (nine vector instructions a block, a fifth of the
// softmax's).  Probabilities may then grow past 2^8 - harmless in floating point, values and sums keep their
// precision - and the stage ends with a look at the row sums instead: past ATT_FAST_LIMIT everything is scaled down
// by a power of two (exactly) and the reference raised by its exponent; a sum that is no longer below ATT_FAST_OVER
// (a score more than ~100 above everything before it inside one stage, or an overflow outright) sets `bad`, and the
// caller runs the whole tile again with the per-block test.
constexpr float ATT_FAST_LIMIT = 16777216.0f;              // 2^24
constexpr float ATT_FAST_OVER = 1.2676506e30f;             // 2^100
template <int NB, bool FAST = false>
__device__ __forceinline__ void att_stage_fixed(const AttnTile &t, const int (&cs)[4], bool first,
                                                const u32x4 (&qf)[4], f32x16 (&o)[2], f32x16 &negm, float (&l)[2],
                                                bool *bad = nullptr)
{
    u32x4 kf[4];
    f32x16 sbuf[2];
#pragma unroll
    for (int sl = 0; sl < 4; sl++) kf[sl] = att_read_k(t, cs, 0, sl);
    sbuf[0] = att_mfma(kf[0], qf[0], negm);
    sbuf[0] = att_mfma(kf[1], qf[1], sbuf[0]);
    sbuf[0] = att_mfma(kf[2], qf[2], sbuf[0]);
    sbuf[0] = att_mfma(kf[3], qf[3], sbuf[0]);
    if constexpr (NB > 1) {
#pragma unroll
        for (int sl = 0; sl < 4; sl++) kf[sl] = att_read_k(t, cs, 1, sl);
    }
    if (first) {                                     // wave-uniform
        if (NB == 1 && t.n < 32) {                   // a lone, partial block: its missing keys must not set the reference
            const int lim = t.n - 4 * t.lg;
#pragma unroll
            for (int e = 0; e < 16; e++)
                if (8 * (e >> 2) + (e & 3) >= lim) sbuf[0][e] = -INFINITY;
        }
        float m = att_max16(sbuf[0]);
        m = fmaxf(m, __shfl_xor(m, 32, WAVE));       // key 0 always exists: m is finite
#pragma unroll
        for (int e = 0; e < 16; e++) {
            sbuf[0][e] -= m;
            negm[e] = -m;
        }
    }
    const bool partial = t.n < 32 * NB;              // wave-uniform
    static_for<NB>([&](auto kbc) {
        constexpr int kb = decltype(kbc)::value;
        constexpr bool NEXT = kb + 1 < NB, NEXT2 = kb + 2 < NB;
        if constexpr (kb == NB - 1) {
            if (partial) att_step<NEXT, NEXT2, true, true, FAST>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
            else att_step<NEXT, NEXT2, false, true, FAST>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
        } else {
            att_step<NEXT, NEXT2, false, true, FAST>(t, cs, kb, sbuf[kb & 1], sbuf[(kb + 1) & 1], kf, qf, o, negm, l);
        }
    });
    if constexpr (FAST) {
        const float ls = l[0] + l[1];
        if (__builtin_amdgcn_ballot_w64(!(ls <= ATT_FAST_LIMIT)) != 0) {         // wave-uniform and rare
            const float other = __shfl_xor(ls, 32, WAVE);
            const float mrow = ls > other ? ls : other;                          // both lanes of a row decide alike
            if (__builtin_amdgcn_ballot_w64(!(ls < ATT_FAST_OVER) || !(other < ATT_FAST_OVER)) != 0) *bad = true;
            const int k = mrow > ATT_FAST_LIMIT ? __builtin_amdgcn_frexp_expf(mrow) : 0;
            const float alpha = __builtin_amdgcn_ldexpf(1.0f, -k), delta = (float)k;
            l[0] *= alpha;
            l[1] *= alpha;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                o[0][e] *= alpha;
                o[1][e] *= alpha;
                negm[e] -= delta;
            }
        }
    }
}

#undef VT_PIN

// ---------------------------------------------------------------------------------------------------------
// Short key sequences (n <= 288, e.g. 257 tokens at 256 px): one persistent workgroup of eight waves per compute
// unit walks the (sample, head) items c, c + grid, c + 2 grid, ... with two buffers in LDS, each holding the item's K
// rows and V rows (128-byte rows, 16-byte chunks XOR-swizzled).  While the first four waves multiply item i out of
// one buffer (a wave per 32-query tile; the other four join in for samples of more than 128 queries), the second
// four bring item i+1 into the other buffer by direct loads; one barrier per item.  The staging of an item (its
// 64 KB come as 128-byte pieces out of 1.5 KB token rows) thus overlaps the arithmetic of the item before it.
// Vector-memory operations retire in issue order: a wave asks for its first Q tile of the next item right after the
// prefetch and nothing inside the tile arithmetic depends on either; only a sample with more than eight query
// tiles (more than 256 queries) loads Q in between.
// One instantiation per number of 32-key blocks (1 .. 9), so that the tile pipeline is fully unrolled.
template <int NBLK>
__global__ __launch_bounds__(512, 1) void sparse_attention_bf16_d64_pipelined_kernel(
    const bf16_t *__restrict__ q, int64_t q_rs, int64_t q_hs, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, int64_t kv_bs, int64_t kv_ts, int64_t kv_hs, const int64_t *__restrict__ offsets,
    bf16_t *__restrict__ out, int64_t o_rs, int64_t o_hs, int n, float scale, int items, int h)
{
    constexpr int NW = 8;                   // waves
    constexpr int npad = NBLK * 32;         // the host picks the instantiation: NBLK = ceil(n / 32)
    constexpr int bufsz = 2 * npad * 128;   // K rows, then V rows
    extern __shared__ __attribute__((aligned(128))) unsigned char smem[];    // rows start on 128-byte boundaries

    const int tid = threadIdx.x, lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, lg = lane >> 5;
    const int64_t row_bytes = kv_ts * 2;
    const float c = scale * 1.44269504088896340736f;

    // Items of this workgroup: blockIdx.x + li * gridDim.x, li = 0, 1, ...; item -> (sample, head) with the heads of a
    // sample as neighbours, so the pieces of one token row are fetched by workgroups that run at the same time.
    // First row and query count of every item are put into a small LDS table up front (up to ATT_TBL items per
    // workgroup; beyond that they are read from `offsets` when needed), so that no step of the loop waits for them.
    struct Item {
        int64_t row0;
        int Lb, b, head;
    };
    int64_t *t_row0 = reinterpret_cast<int64_t *>(smem + 2 * bufsz);
    int *t_len = reinterpret_cast<int *>(t_row0 + ATT_TBL);
    const int grid = gridDim.x;
    if ((int)blockIdx.x >= items) return;
    const int my_items = (items - (int)blockIdx.x + grid - 1) / grid;
    const bool tabled = my_items <= ATT_TBL;
    if (tabled) {
        for (int li = tid; li < my_items; li += 512) {
            const int b = ((int)blockIdx.x + li * grid) / h;
            const int64_t r0 = offsets[b];
            t_row0[li] = r0;
            t_len[li] = (int)(offsets[b + 1] - r0);
        }
    }
    auto item_of = [&](int li, bool from_table) {
        Item r;
        const int it = (int)blockIdx.x + li * grid;
        r.b = it / h;
        r.head = it - r.b * h;
        if (from_table) {
            const int64_t r0 = t_row0[li];
            r.row0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(r0 >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)r0);
            r.Lb = __builtin_amdgcn_readfirstlane(t_len[li]);
        } else {
            r.row0 = offsets[r.b];
            r.Lb = (int)(offsets[r.b + 1] - r.row0);
        }
        return r;
    };
    auto load_q = [&](const Item &im, int rt, u32x4 (&dst)[4]) {
        const int qrow = rt * 32 + lr;
        const unsigned char *qp =
            reinterpret_cast<const unsigned char *>(q + (im.row0 + qrow) * q_rs + (int64_t)im.head * q_hs) + lg * 16;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            dst[s] = qrow < im.Lb ? *reinterpret_cast<const u32x4 *>(qp + s * 32) : z;
        }
    };
    auto scale_q = [&](u32x4 (&f)[4]) {       // scores come out of the MFMA in log2 units
#pragma unroll
        for (int s = 0; s < 4; s++) f[s] = att_scale_frag(f[s], c);
    };
    // K and V of an item by direct loads, issued by the waves w0, w0 + nw, ...: wave-load j covers rows 8j .. 8j+7 of
    // K (j < npad / 8) or of V; a lane fetches the 16-byte chunk that belongs at its position of the swizzled row.
    // Rows past the last key repeat it (their scores are masked).  Issued from assembly: the compiler would
    // otherwise wait for every direct load in flight before any later read of LDS, i.e. put the prefetch in front
    // of the arithmetic it is meant to overlap.
    // Lane constants of a wave-load: row (lane / 8) of its eight rows, chunk position lane % 8; the chunk fetched for
    // a position depends on the row through the swizzle (K: on (row / 2) % 8, i.e. on the parity of j as well; V: on
    // row % 4 only).
    const int lrow = lane >> 3, lchunk = lane & 7;
    const uint32_t lrow_off = (uint32_t)(lrow * row_bytes);
    const uint32_t koff[2] = {lrow_off + (uint32_t)((lchunk ^ (lrow >> 1)) * 16),
                              lrow_off + (uint32_t)((lchunk ^ (4 + (lrow >> 1))) * 16)};
    const uint32_t voff = lrow_off + (uint32_t)((lchunk ^ (2 * (lrow & 3))) * 16);
    auto stage_issue = [&](const Item &im, unsigned char *buf, int w0, int nw) {
        const void *kbase = uniform_ptr(k + (int64_t)im.b * kv_bs + (int64_t)im.head * kv_hs);
        const void *vbase = uniform_ptr(v + (int64_t)im.b * kv_bs + (int64_t)im.head * kv_hs);
        const uint32_t lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)buf);
        for (int j = w0; j < 2 * (npad / 8); j += nw) {
            const bool is_v = j >= npad / 8;
            const int jj = is_v ? j - npad / 8 : j;
            uint32_t off;
            if (jj * 8 + 8 <= n) {             // wave-uniform: all eight rows exist
                off = (is_v ? voff : koff[jj & 1]) + (uint32_t)(jj * 8 * row_bytes);
            } else {
                const int r = jj * 8 + lrow;
                const int chunk = lchunk ^ (is_v ? 2 * (r & 3) : (r >> 1) & 7);
                off = (uint32_t)((r < n ? r : n - 1) * row_bytes + chunk * 16);
            }
            dma16_nt(is_v ? vbase : kbase, off, lds + j * 1024);
        }
    };

    const int sw = (lr >> 1) & 7;
    int cs[4];
#pragma unroll
    for (int s = 0; s < 4; s++) cs[s] = ((2 * s + lg) ^ sw) * 16;

    Item cur = item_of(0, false);
    stage_issue(cur, smem, wid, NW);
    u32x4 qf[4], qn[4];
    load_q(cur, wid, qf);
    wait_vmcnt<0>();
    __syncthreads();
    Item nxt = cur;
    if (my_items > 1) nxt = item_of(1, tabled);

    for (int li = 0, par = 0; li < my_items; li++, par ^= 1) {
        unsigned char *buf = smem + par * bufsz;
        const bool has_next = li + 1 < my_items;
        // The second half of the waves has a tile only in samples of more than 128 queries: it issues the prefetch
        // of the next item, the first half goes straight to its tiles.  Every wave then asks for its first Q tile of
        // the next item; nothing in the tile arithmetic depends on these loads.
        if (has_next) {
            if (wid >= NW / 2) stage_issue(nxt, smem + (par ^ 1) * bufsz, wid - NW / 2, NW / 2);
            load_q(nxt, wid, qn);
        }
        const AttnTile tile = {buf + lr * 128, att_v_lane(buf + npad * 128, lane), nullptr, n, lg};
        for (int rt = wid; rt * 32 < cur.Lb; rt += NW) {
            const int qrow = rt * 32 + lr;
            if (rt != wid) {        // a ninth tile and beyond (more than 256 queries): waits behind the prefetch
                load_q(cur, rt, qf);
                wait_vmcnt<0>();    // here, so that the common path carries no pending load into the arithmetic
            }
            f32x16 o[2];
            float l_run;
            scale_q(qf);
            att_tile_fixed<NBLK>(tile, cs, qf, o, l_run);
            const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
            if (qrow < cur.Lb) attn_store(out + (cur.row0 + qrow) * o_rs + (int64_t)cur.head * o_hs, o, l_tot, lg);
        }
        cur = nxt;
        if (li + 2 < my_items) nxt = item_of(li + 2, tabled);
        // The waves that issued direct loads wait for them here (the compiler does not know of them); stores count
        // in the same queue, so a wave that has just stored a tile would wait for that too: the first half of the
        // waves, which stores in every item, has issued no direct load and needs no wait of its own - the compiler
        // places the wait for the Q loads where they are used.
        if (wid >= NW / 2) wait_vmcnt<0>();
#pragma unroll
        for (int s = 0; s < 4; s++) qf[s] = qn[s];
        // The next item's buffer is complete (its loaders have waited) and this item's buffer is free (its fragments
        // are in registers or consumed).  A plain barrier: the fence of __syncthreads() would make every wave wait
        // for its output stores as well.
        block_barrier();
    }
}

// ---------------------------------------------------------------------------------------------------------
// Longer key sequences (512 px models, spatially reduced PVT stages): a workgroup of four waves takes 128 query
// rows of one (sample, head), a wave 32 of them, and the keys and values pass through LDS in stages of 128 (four
// blocks of the tile pipeline above), double buffered: the direct loads of stage s+1 are issued before stage s is
// multiplied and waited for after it.  Two workgroups share a compute unit, out of step with each other (with
// eight waves and 256 rows per workgroup the per-stage barrier makes every SIMD wait for its slower wave:
// measured 7 % slower).  K and V rows are laid out as in the resident kernel (V transposed by the LDS read).
constexpr int ASK = 128;                            // keys per stage
constexpr int ASBUF = 2 * ASK * 128;                // one stage: K rows, then V rows

__global__ __launch_bounds__(256, 2) void sparse_attention_bf16_d64_stream_kernel(
    const bf16_t *__restrict__ q, int64_t q_rs, int64_t q_hs, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, int64_t kv_bs, int64_t kv_ts, int64_t kv_hs, const int64_t *__restrict__ offsets,
    bf16_t *__restrict__ out, int64_t o_rs, int64_t o_hs, int n, int qchunks, float scale, int items, int h)
{
    extern __shared__ __attribute__((aligned(128))) unsigned char smem[];
    // Workgroups are dealt to the eight XCDs in turn (id % 8).  The query chunks of one (sample, head) all stream the
    // same keys and values: they are given ids that land on one XCD, one after the other, so that its L2 fetches
    // them from memory once.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int item = (slot / qchunks) * 8 + xcd, qc = slot % qchunks;
    if (item >= items) return;
    const int b = item / h, head = item - b * h;
    const int64_t row0 = offsets[b];
    const int Lb = (int)(offsets[b + 1] - row0);
    if (qc * AQ >= Lb) return;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, lg = lane >> 5;
    const int qrow = qc * AQ + wid * 32 + lr;
    const bool wave_live = qc * AQ + wid * 32 < Lb;
    const bool row_live = qrow < Lb;
    const float c = scale * 1.44269504088896340736f;
    const int64_t row_bytes = kv_ts * 2;
    const void *kbase = uniform_ptr(k + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const void *vbase = uniform_ptr(v + (int64_t)b * kv_bs + (int64_t)head * kv_hs);
    const int nstage = (n + ASK - 1) / ASK;

    // stage st into buffer st & 1: wave-load j covers rows 8j .. 8j+7 of K (j < 16) or of V; this wave issues the
    // loads j = wid, wid + 4, ..., whose lane offsets and LDS addresses are worked out once.  Issued from assembly so
    // that the compiler does not wait for them before the LDS reads of the stage being multiplied.
    constexpr int NLD = 2 * (ASK / 8) / (AQ / 32);       // loads per wave and stage
    uint32_t ld_off[NLD], ld_row[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
        const int j = wid + i * (AQ / 32);
        const bool is_v = j >= ASK / 8;
        const int r = (is_v ? j - ASK / 8 : j) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ (is_v ? 2 * (r & 3) : (r >> 1) & 7);
        ld_row[i] = (uint32_t)r;
        ld_off[i] = (uint32_t)(r * row_bytes + chunk * 16);
    }
    auto issue = [&](int st) {
        const uint32_t lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(smem + (st & 1) * ASBUF + wid * 1024));
        const uint32_t stage_off = (uint32_t)(st * ASK * row_bytes);
        const bool whole = (st + 1) * ASK <= n;          // wave-uniform: no row of the stage lies past the keys
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const bool is_v = wid + i * (AQ / 32) >= ASK / 8;      // the same for every wave: AQ / 32 divides ASK / 8
            uint32_t off = ld_off[i] + stage_off;
            if (!whole) {
                const int key = st * ASK + (int)ld_row[i];
                if (key >= n) off -= (uint32_t)((key - (n - 1)) * row_bytes);        // repeat the last key
            }
            dma16(is_v ? vbase : kbase, off, lds + i * (AQ / 32) * 1024);
        }
    };
    issue(0);

    // Q fragments (second operand of S^T): bytes [32 s + 16 g, +16) of the query row, times scale * log2(e)
    u32x4 qf[4];
    {
        const unsigned char *qp =
            reinterpret_cast<const unsigned char *>(q + (row0 + qrow) * q_rs + (int64_t)head * q_hs) + lg * 16;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            qf[s] = row_live ? *reinterpret_cast<const u32x4 *>(qp + s * 32) : z;
        }
#pragma unroll
        for (int s = 0; s < 4; s++) qf[s] = att_scale_frag(qf[s], c);
    }
    const int sw = (lr >> 1) & 7;
    int cs[4];
#pragma unroll
    for (int s = 0; s < 4; s++) cs[s] = ((2 * s + lg) ^ sw) * 16;

    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16 o[2], negm;
    float l[2];
    const int nfull = n / ASK;                        // stages of four whole blocks; then at most one shorter stage
    auto stage_tile = [&](int st) {
        const unsigned char *buf = smem + (st & 1) * ASBUF;
        const unsigned char *vl = att_v_lane(buf + ASK * 128, lane);
        return AttnTile{buf + lr * 128, vl, reinterpret_cast<const unsigned char *>((uintptr_t)vl ^ 64u), n - st * ASK, lg};
    };
    // All stages of the sequence (stage 0 is on its way); FAST: see att_stage_fixed.  -> whether a row sum left
    // the range the fast form is good for.
    auto all_stages = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
        bool bad = false;
        o[0] = o[1] = negm = zero;
        l[0] = l[1] = 0.f;
        for (int st = 0; st < nfull; st++) {
            wait_vmcnt<0>();                 // this wave's loads of stage st (nothing younger is in flight)
            __syncthreads();                 // stage st is complete; the other buffer was last read in iteration st-1
            if (st + 1 < nstage) issue(st + 1);
            if (wave_live) att_stage_fixed<4, FAST>(stage_tile(st), cs, st == 0, qf, o, negm, l, &bad);
        }
        if (nfull < nstage) {                // the last, shorter stage: 1 .. 3 blocks (its own code, outside the loop)
            wait_vmcnt<0>();
            __syncthreads();
            if (wave_live) {
                const AttnTile tile = stage_tile(nfull);
                switch ((tile.n + 31) / 32) {
                case 3: att_stage_fixed<3, FAST>(tile, cs, nfull == 0, qf, o, negm, l, &bad); break;
                case 2: att_stage_fixed<2, FAST>(tile, cs, nfull == 0, qf, o, negm, l, &bad); break;
                default: att_stage_fixed<1, FAST>(tile, cs, nfull == 0, qf, o, negm, l, &bad); break;
                }
            }
        }
        return bad;
    };
    const bool bad = all_stages(std::true_type{});
    // The keys are staged for the whole workgroup, so a second pass is one for all its waves (their results come out
    // the same as before); it starts once every wave has left the buffers of the first.
    if (__syncthreads_or(bad ? 1 : 0)) {
        issue(0);
        all_stages(std::false_type{});
    }
    if (!wave_live) return;
    const float l_run = l[0] + l[1];
    const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    if (row_live) attn_store(out + (row0 + qrow) * o_rs + (int64_t)head * o_hs, o, l_tot, lg);
}

int launch_attention_bf16_d64(const void *q, int64_t q_rs, int64_t q_hs, const void *k, const void *v, int64_t kv_bs,
                              int64_t kv_ts, int64_t kv_hs, const int64_t *offsets, void *out, int64_t o_rs,
                              int64_t o_hs, int B, int h, int n, int max_rows, float scale, hipStream_t st)
{
    if (n <= 288) {
        // keys and values resident in LDS: one persistent workgroup per compute unit, two buffers of K rows + V rows
        const int npad = (n + 31) & ~31;
        const size_t lds_p = 4 * (size_t)npad * 128 + ATT_TBL * 12;       // + the item table
        const int items = B * h;
        const int cus = compute_units();
        dim3 grid_p((unsigned)(items < cus ? items : cus)), block_p(512);
#define VT_ATT_PIPE(NB)                                                                                            \
    case NB: {                                                                                                     \
        auto kern_p = sparse_attention_bf16_d64_pipelined_kernel<NB>;                                              \
        VT_RESERVE_LDS(kern_p, 160 * 1024, "sparse_attention");                                                    \
        note_kernel(reinterpret_cast<const void *>(kern_p)),                                                        \
        kern_p<<<grid_p, block_p, lds_p, st>>>((const bf16_t *)q, q_rs, q_hs, (const bf16_t *)k, (const bf16_t *)v, \
                                               kv_bs, kv_ts, kv_hs, offsets, (bf16_t *)out, o_rs, o_hs, n, scale,  \
                                               items, h);                                                          \
        return check_launch("sparse_attention");                                                                   \
    }
        switch (npad / 32) {
            VT_ATT_PIPE(1)
            VT_ATT_PIPE(2)
            VT_ATT_PIPE(3)
            VT_ATT_PIPE(4)
            VT_ATT_PIPE(5)
            VT_ATT_PIPE(6)
            VT_ATT_PIPE(7)
            VT_ATT_PIPE(8)
            VT_ATT_PIPE(9)
        }
#undef VT_ATT_PIPE
    }
    const size_t lds = 2 * (size_t)ASBUF;
    const int qchunks = (int)ceil_div(max_rows, AQ);
    auto kern = sparse_attention_bf16_d64_stream_kernel;
    VT_RESERVE_LDS(kern, lds, "sparse_attention");
    const int items = B * h;
    dim3 grid((unsigned)(ceil_div(items, 8) * 8 * qchunks)), block(AQ * 2);
    note_kernel(reinterpret_cast<const void *>(kern));
    kern<<<grid, block, lds, st>>>((const bf16_t *)q, q_rs, q_hs, (const bf16_t *)k, (const bf16_t *)v, kv_bs, kv_ts,
                                   kv_hs, offsets, (bf16_t *)out, o_rs, o_hs, n, qchunks, scale, items, h);
    return check_launch("sparse_attention");
}

}  // namespace vtdge
