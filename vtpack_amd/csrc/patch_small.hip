// Patch embedding with small patches (gfx950): Conv2d(Cin = 3, N = 64, kernel 4, stride 4) + bias, the LayerNorm of
// the embedding and the position embedding in one pass over the images - the first stage of the pyramid models
// (vtpack/models/dge/pvt_dge.py:143-176 with :312-314).
//
// A patch row is 4 pixels = 8 bytes, too short for the 16-byte direct loads of the streaming Linear, and K = 48 is
// less than one of its 128-byte slabs; through a gathered copy of the images and the generic Linear the stage took
// three launches and two more passes over the 134 MB of tokens.  Here a wave owns 16 neighbouring patches of one
// patch row: for a fixed channel and pixel row their 8-byte pieces are 128 contiguous bytes of the image.  The
// 48 x 64 weight lives in registers as eight fragments of v_mfma_f32_16x16x32_bf16 (K padded to 64 with zeros), the
// product is D = W A^T, so a lane ends with 16 of the 64 outputs of ONE patch (columns 16 cb + 4 kg + i) and the
// LayerNorm's sums need two exchanges between the four lanes of a patch.  Rounding follows the separate modules:
// convolution + bias rounded to bf16, LayerNorm (fp32, two passes) rounded, + pos rounded.
#include "common.h"

namespace vtdge {

constexpr int PS_P = 4, PS_CIN = 3, PS_N = 64, PS_K = PS_CIN * PS_P * PS_P;      // 48
constexpr int PS_TILES = 8;              // 16-patch tiles per wave

__global__ __launch_bounds__(256) void patch_small_kernel(const bf16_t *__restrict__ img, const bf16_t *__restrict__ wgt,
                                                          const bf16_t *__restrict__ bias,
                                                          const bf16_t *__restrict__ lnw, const bf16_t *__restrict__ lnb,
                                                          float eps, const bf16_t *__restrict__ pos,
                                                          bf16_t *__restrict__ out, int B, int S, int64_t tiles)
{
    const int lane = threadIdx.x & 63, t16 = lane & 15, kg = lane >> 4;
    const int G = S / PS_P, tiles_x = G / 16;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);

    // the weight: fragment (cb, ks): lane (t16, kg) holds W[16 cb + t16][32 ks + 8 kg .. + 7], zero past K = 48
    u32x4 wf[4][2];
#pragma unroll
    for (int cb = 0; cb < 4; cb++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int k0 = 32 * ks + 8 * kg;
            wf[cb][ks] = u32x4{0u, 0u, 0u, 0u};
            if (k0 < PS_K) wf[cb][ks] = *reinterpret_cast<const u32x4 *>(wgt + (16 * cb + t16) * PS_K + k0);
        }
    // per-lane vectors of the lane's 16 output columns 16 cb + 4 kg + i
    float bv[4][4], gw[4][4], gb[4][4];
#pragma unroll
    for (int cb = 0; cb < 4; cb++) {
        const int c0 = 16 * cb + 4 * kg;
        const u32x2 b2 = *reinterpret_cast<const u32x2 *>(bias + c0);
        const u32x2 w2 = *reinterpret_cast<const u32x2 *>(lnw + c0);
        const u32x2 g2 = *reinterpret_cast<const u32x2 *>(lnb + c0);
        bv[cb][0] = bf16lo(b2.x); bv[cb][1] = bf16hi(b2.x); bv[cb][2] = bf16lo(b2.y); bv[cb][3] = bf16hi(b2.y);
        gw[cb][0] = bf16lo(w2.x); gw[cb][1] = bf16hi(w2.x); gw[cb][2] = bf16lo(w2.y); gw[cb][3] = bf16hi(w2.y);
        gb[cb][0] = bf16lo(g2.x); gb[cb][1] = bf16hi(g2.x); gb[cb][2] = bf16lo(g2.y); gb[cb][3] = bf16hi(g2.y);
    }

    // A^T fragments of a tile: k = 32 ks + 8 kg + j -> channel 2 ks + kg / 2, pixel rows 2 (kg % 2) and + 1, 4 pixels
    // each; a tile past the end gives zeros
    const auto fetch = [&](int64_t tile, u32x4 (&af)[2]) {
        const int tx = (int)(tile % tiles_x);
        const int64_t rest = tile / tiles_x;
        const int y = (int)(rest % G), b = (int)(rest / G);
        const int x = tx * 16 + t16;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int c = 2 * ks + (kg >> 1);
            af[ks] = u32x4{0u, 0u, 0u, 0u};
            if (c < PS_CIN && tile < tiles) {
                const bf16_t *p = img + (((int64_t)b * PS_CIN + c) * S + (PS_P * y + 2 * (kg & 1))) * S + PS_P * x;
                const u32x2 r0 = *reinterpret_cast<const u32x2 *>(p);
                const u32x2 r1 = *reinterpret_cast<const u32x2 *>(p + S);
                af[ks] = u32x4{r0.x, r0.y, r1.x, r1.y};
            }
        }
    };
    u32x4 af[2], an[2];
    fetch(wave * PS_TILES, af);
#pragma unroll 1
    for (int tt = 0; tt < PS_TILES; tt++) {
        const int64_t tile = wave * PS_TILES + tt;
        if (tile >= tiles) return;
        if (tt + 1 < PS_TILES) fetch(tile + 1, an);              // the next tile's pixels are on their way meanwhile
        const int tx = (int)(tile % tiles_x);
        const int64_t rest = tile / tiles_x;
        const int y = (int)(rest % G), b = (int)(rest / G);
        const int x = tx * 16 + t16;                              // this lane's patch
        float v[4][4];
        float s = 0.f;
#pragma unroll
        for (int cb = 0; cb < 4; cb++) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[cb][ks]),
                                                              __builtin_bit_cast(bf16x8, af[ks]), acc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[cb][i] = Elem<bf16_t>::round(acc[i] + bv[cb][i]);       // the convolution's output as stored
                s += v[cb][i];
            }
        }
        // LayerNorm over the patch's 64 outputs: four lanes (kg = 0..3) hold 16 each
        s += __shfl_xor(s, 16, WAVE);
        s += __shfl_xor(s, 32, WAVE);
        const float mean = s / (float)PS_N;
        float q = 0.f;
#pragma unroll
        for (int cb = 0; cb < 4; cb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float d = v[cb][i] - mean;
                q += d * d;
            }
        q += __shfl_xor(q, 16, WAVE);
        q += __shfl_xor(q, 32, WAVE);
        const float rstd = 1.0f / sqrtf(q / (float)PS_N + eps);
        const int64_t row = ((int64_t)b * G + y) * G + x;
        const int64_t prow = (int64_t)y * G + x;
        // Two column blocks leave together, 16 bytes a lane: the lanes kg = 1, 3 of a patch hand their half of the
        // first block to kg = 0, 2 and take those lanes' half of the second (rows of 16 lanes swapped between the
        // two registers), so that lane kg holds columns 16 (kg % 2) + 8 (kg / 2) .. + 7 of the pair's 32 - half as many
        // store (and position-embedding load) instructions, each covering 64 contiguous bytes of a row instead of 32.
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
            u32x2 ob[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int cb = 2 * pr + h;
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) o[i] = (v[cb][i] - mean) * rstd * gw[cb][i] + gb[cb][i];
                ob[h].x = pack_bf16x2(o[0], o[1]);
                ob[h].y = pack_bf16x2(o[2], o[3]);
            }
            const auto sx = __builtin_amdgcn_permlane16_swap(ob[0].x, ob[1].x, false, false);
            const auto sy = __builtin_amdgcn_permlane16_swap(ob[0].y, ob[1].y, false, false);
            u32x4 w = {sx[0], sy[0], sx[1], sy[1]};
            const int c0 = 32 * pr + 16 * (kg & 1) + 8 * (kg >> 1);
            if (pos != nullptr) {
                float a[8], p8[8];
                Elem<bf16_t>::unpack(w, a);
                Elem<bf16_t>::unpack(*reinterpret_cast<const u32x4 *>(pos + prow * PS_N + c0), p8);
#pragma unroll
                for (int c = 0; c < 8; c++) a[c] += p8[c];
                w = Elem<bf16_t>::pack(a);
            }
            *reinterpret_cast<u32x4 *>(out + row * PS_N + c0) = w;
        }
        af[0] = an[0];
        af[1] = an[1];
    }
}

}  // namespace vtdge

using namespace vtdge;

extern "C" int vtdge_patch_embed_norm(const void *images, const void *weight, const void *bias, const void *ln_weight,
                                      const void *ln_bias, float ln_eps, const void *pos, void *out, int B, int Cin,
                                      int S, int P, int N, int dtype, void *stream)
{
    VT_REQUIRE(images && weight && bias && ln_weight && ln_bias && out, VTDGE_ERR_ARG, "patch_embed_norm: NULL operand");
    VT_REQUIRE(B > 0 && S > 0, VTDGE_ERR_ARG, "patch_embed_norm: bad sizes");
    VT_REQUIRE(dtype == VTDGE_BF16 && Cin == PS_CIN && P == PS_P && N == PS_N && S % (16 * PS_P) == 0,
               VTDGE_ERR_UNSUPPORTED,
               "patch_embed_norm: bf16, %d channels, %d x %d patches, %d outputs and an image side that is a multiple of %d "
               "(got Cin=%d P=%d N=%d S=%d)", PS_CIN, PS_P, PS_P, PS_N, 16 * PS_P, Cin, P, N, S);
    const auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    VT_REQUIRE(a16(images) && a16(weight) && a16(bias) && a16(ln_weight) && a16(ln_bias) && a16(pos) && a16(out),
               VTDGE_ERR_ARG, "patch_embed_norm: operands must be 16-byte aligned");
    const int G = S / PS_P;
    const int64_t tiles = (int64_t)B * G * (G / 16);
    const int64_t groups = ceil_div(tiles, (int64_t)4 * PS_TILES);
    VT_REQUIRE(groups < (1ll << 31), VTDGE_ERR_UNSUPPORTED, "patch_embed_norm: %lld workgroups exceed one launch",
               (long long)groups);
    note_kernel(reinterpret_cast<const void *>(patch_small_kernel));
    patch_small_kernel<<<dim3((unsigned)groups), dim3(256), 0, (hipStream_t)stream>>>(
        (const bf16_t *)images, (const bf16_t *)weight, (const bf16_t *)bias, (const bf16_t *)ln_weight,
        (const bf16_t *)ln_bias, ln_eps, (const bf16_t *)pos, (bf16_t *)out, B, S, tiles);
    return check_launch("patch_embed_norm");
}
