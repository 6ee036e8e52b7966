/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the Dynamic Grained Encoder
 * query-path operators of StevenGrove/vtpack, in plain C.
 *
 * Nothing in the shipped package may link, import or call this file; it is the
 * checker the HIP kernels are compared against (tests, the smoke check and the
 * cpu_baseline leg of the benchmark).
 *
 * Every function states the reference lines it restates (paths relative to the
 * reference checkout).  The reference ships no CPU implementation and no test
 * vectors for these operators (its extension is CUDA only), so each function is
 * pinned by independent closed forms / invariants in tests/test_oracle_pins.py:
 *
 *   dge_index_to_patch        partition-of-the-grid, ordering, L_i closed form,
 *                             hand-worked example, all-fine / all-coarse cases
 *   dge_index_to_patch_dense  closed-form enumeration per granularity
 *   dge_compress_f32          F.avg_pool2d sampled at (y0/s, x0/s)  (the
 *                             reference's own dense statement,
 *                             vtpack/layers/grained_sample.py:126-147)
 *   dge_decompress_f32        repeat/one-hot-gate dense statement
 *                             (vtpack/layers/grained_sample.py:150-177),
 *                             adjoint identity, round trips
 *   dge_attention_f32         float64 softmax(QK^T)V from library routines
 *   dge_sparse_gemm_f32       per-sample torch.bmm + cat
 *
 * Floating point: sums that the reference performs in a fixed order in fp32
 * (compress) are reproduced in that order in fp32; contractions that the
 * reference hands to cuBLAS/cuDNN (order unspecified) are accumulated in double
 * and rounded to float wherever the reference stores an fp32 intermediate.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* vtpack/layers/csrc/grained_sample/grained_sample.cu:302-345 (host: counts,
 * cumsum, batch lengths) and :146-196 (kernel: row contents).
 * patches may be NULL to obtain only the lengths / the row total.
 * Column 2 of extra-token rows is left unwritten by the reference (:169-174);
 * it is written as 0 here. */
int64_t dge_index_to_patch(const int64_t *indices, int B, int Hr, int Wr,
                           const int64_t *splits, int S, int R, int extra,
                           int64_t *patches, int64_t *lengths)
{
    int64_t row = 0;
    for (int b = 0; b < B; b++) {
        int64_t start = row;
        for (int e = 0; e < extra; e++) {
            if (patches) {
                int64_t *p = patches + 4 * row;
                p[0] = b; p[1] = -(int64_t)e - 1; p[2] = 0; p[3] = 1;
            }
            row++;
        }
        for (int ry = 0; ry < Hr; ry++) {
            for (int rx = 0; rx < Wr; rx++) {
                int64_t g = indices[((int64_t)b * Hr + ry) * Wr + rx];
                if (g < 0 || g >= S) return -1;
                int ps = (int)splits[g];
                int step = R / ps;
                for (int dy = 0; dy < ps; dy++) {
                    for (int dx = 0; dx < ps; dx++) {
                        if (patches) {
                            int64_t *p = patches + 4 * row;
                            p[0] = b;
                            p[1] = (int64_t)ry * R + dy * step;
                            p[2] = (int64_t)rx * R + dx * step;
                            p[3] = step;
                        }
                        row++;
                    }
                }
            }
        }
        if (lengths) lengths[b] = row - start;
    }
    return row;
}

/* vtpack/layers/csrc/grained_sample/grained_sample.cu:347-433: every patch at
 * every granularity, per sample: extras, then for each split all sub-patches
 * of the whole token grid in raster order.  Note the reference indexes with
 * the REGION grid size (height,width = indices.size(1,2)), i.e. a split of
 * `ps` enumerates (Hr*ps) x (Wr*ps) windows of `step` tokens. */
int64_t dge_index_to_patch_dense(int B, int Hr, int Wr, const int64_t *splits,
                                 int S, int R, int extra, int64_t *patches,
                                 int64_t *lengths)
{
    int64_t per = extra;
    for (int s = 0; s < S; s++) per += splits[s] * splits[s] * Hr * Wr;
    for (int b = 0; b < B; b++) {
        if (lengths) lengths[b] = per;
        if (!patches) continue;
        int64_t row = (int64_t)b * per;
        for (int e = 0; e < extra; e++, row++) {
            int64_t *p = patches + 4 * row;
            p[0] = b; p[1] = -(int64_t)e - 1; p[2] = 0; p[3] = 1;
        }
        for (int s = 0; s < S; s++) {
            int ps = (int)splits[s], step = R / ps;
            int64_t len = (int64_t)Hr * Wr * ps * ps;
            for (int64_t sp = 0; sp < len; sp++, row++) {
                int64_t *p = patches + 4 * row;
                p[0] = b;
                p[1] = (sp / ((int64_t)Wr * ps)) * step;
                p[2] = (sp % ((int64_t)Wr * ps)) * step;
                p[3] = step;
            }
        }
    }
    return per * B;
}

/* vtpack/layers/csrc/grained_sample/grained_sample.cu:31-69.  fp32
 * accumulation, dy outer / dx inner, then one division by size*size. */
void dge_compress_f32(const float *x, const int64_t *patches, int64_t L,
                      int N, int C, int W, int extra, float *out)
{
    for (int64_t p = 0; p < L; p++) {
        int64_t b = patches[4 * p], y0 = patches[4 * p + 1];
        int64_t x0 = patches[4 * p + 2], sz = patches[4 * p + 3];
        const float *xb = x + b * (int64_t)N * C;
        float *o = out + p * (int64_t)C;
        if (y0 < 0) {
            memcpy(o, xb + (-y0 - 1) * (int64_t)C, sizeof(float) * C);
            continue;
        }
        for (int c = 0; c < C; c++) {
            volatile float acc = 0.0f; /* volatile: no reassociation, no x87 excess */
            for (int64_t dy = 0; dy < sz; dy++)
                for (int64_t dx = 0; dx < sz; dx++)
                    acc = acc + xb[((y0 + dy) * W + x0 + dx + extra) * (int64_t)C + c];
            o[c] = acc / (float)(sz * sz);
        }
    }
}

/* vtpack/layers/csrc/grained_sample/grained_sample.cu:71-144 (both overloads).
 * out must be pre-filled by the caller with whatever "unwritten" should read
 * as (the reference allocates with at::empty; windows of a valid patch list
 * cover every token, so nothing stays unwritten). */
void dge_decompress_f32(const float *in, const int64_t *patches, int64_t L,
                        const float *ref, int N, int C, int W, int extra,
                        int add_ref, float *out)
{
    for (int64_t p = 0; p < L; p++) {
        int64_t b = patches[4 * p], y0 = patches[4 * p + 1];
        int64_t x0 = patches[4 * p + 2], sz = patches[4 * p + 3];
        const float *v = in + p * (int64_t)C;
        int64_t base = b * (int64_t)N * C;
        if (y0 < 0) {
            int64_t t = base + (-y0 - 1) * (int64_t)C;
            for (int c = 0; c < C; c++)
                out[t + c] = add_ref ? v[c] + ref[t + c] : v[c];
            continue;
        }
        for (int64_t dy = 0; dy < sz; dy++)
            for (int64_t dx = 0; dx < sz; dx++) {
                int64_t t = base + ((y0 + dy) * W + x0 + dx + extra) * (int64_t)C;
                for (int c = 0; c < C; c++)
                    out[t + c] = add_ref ? v[c] + ref[t + c] : v[c];
            }
    }
}

/* vtpack/layers/csrc/batched_sparse_gemm/batched_sparse_gemm.cu:219-305.
 * q,out [h, L, d]; k,v [h, B, n, d]; lengths [B] (sum = L).
 * scores (scale applied inside the GEMM as alpha, :272-277) and the softmax
 * result (:280-285, max-subtracted "ACCURATE" mode) are fp32 tensors in the
 * reference, so both are rounded to float here. */
int dge_attention_f32(const float *q, const float *k, const float *v,
                      const int64_t *lengths, int B, int h, int64_t L, int n,
                      int d, float scale, float *out)
{
    float *s = (float *)malloc(sizeof(float) * (size_t)n);
    if (!s) return -1;
    for (int a = 0; a < h; a++) {
        int64_t off = 0;
        for (int i = 0; i < B; i++) {
            const float *ki = k + ((int64_t)a * B + i) * n * d;
            const float *vi = v + ((int64_t)a * B + i) * n * d;
            for (int64_t r = 0; r < lengths[i]; r++) {
                const float *qr = q + ((int64_t)a * L + off + r) * d;
                float mx = -INFINITY;
                for (int j = 0; j < n; j++) {
                    double acc = 0.0;
                    for (int c = 0; c < d; c++) acc += (double)qr[c] * ki[(int64_t)j * d + c];
                    s[j] = (float)((double)scale * acc);
                    if (s[j] > mx) mx = s[j];
                }
                double den = 0.0;
                for (int j = 0; j < n; j++) den += exp((double)s[j] - mx);
                for (int j = 0; j < n; j++) s[j] = (float)(exp((double)s[j] - mx) / den);
                float *o = out + ((int64_t)a * L + off + r) * d;
                for (int c = 0; c < d; c++) {
                    double acc = 0.0;
                    for (int j = 0; j < n; j++) acc += (double)s[j] * vi[(int64_t)j * d + c];
                    o[c] = (float)acc;
                }
            }
            off += lengths[i];
        }
    }
    free(s);
    return 0;
}

/* vtpack/layers/csrc/batched_sparse_gemm/batched_sparse_gemm.cu:150-195.
 * a [h, La, ka], b [h, Lb, kb]; per sample i the slices a[:, sa:sa+la, :] and
 * b[:, sb:sb+lb, :] are optionally transposed (last two dims) and multiplied;
 * results are concatenated along dim 1.  out [h, rows_total, ncols] where
 * ncols is the same for every sample (required by the reference's cat).
 * Returns rows_total, or -1 on a shape mismatch. */
int64_t dge_sparse_gemm_f32(const float *a, const float *b,
                            const int64_t *a_lengths, const int64_t *b_lengths,
                            int B, int h, int64_t La, int ka, int64_t Lb, int kb,
                            int ta, int tb, float *out, int64_t out_rows,
                            int64_t out_cols)
{
    int64_t sa = 0, sb = 0, ro = 0;
    for (int i = 0; i < B; i++) {
        int64_t la = a_lengths[i], lb = b_lengths[i];
        int64_t m = ta ? ka : la, kk = ta ? la : ka;
        int64_t kk2 = tb ? kb : lb, nn = tb ? lb : kb;
        if (kk != kk2 || nn != out_cols) return -1;
        if (out) {
            for (int hd = 0; hd < h; hd++) {
                const float *ai = a + ((int64_t)hd * La + sa) * ka;
                const float *bi = b + ((int64_t)hd * Lb + sb) * kb;
                float *oi = out + ((int64_t)hd * out_rows + ro) * out_cols;
                for (int64_t r = 0; r < m; r++)
                    for (int64_t c = 0; c < nn; c++) {
                        double acc = 0.0;
                        for (int64_t t = 0; t < kk; t++) {
                            float av = ta ? ai[t * ka + r] : ai[r * ka + t];
                            float bv = tb ? bi[c * kb + t] : bi[t * kb + c];
                            acc += (double)av * bv;
                        }
                        oi[r * out_cols + c] = (float)acc;
                    }
            }
        }
        sa += la; sb += lb; ro += m;
    }
    return ro;
}
