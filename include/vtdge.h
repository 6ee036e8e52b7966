/*
 * vtdge -- C ABI of the MI355X (gfx950) Dynamic Grained Encoder query path.
 *
 * One entry point per operator of the reference's native module `vtpack._C`
 * (vtpack/layers/csrc/vision.cpp:9-29) that lies on the inference query path,
 * plus the dense pieces of the transformer block that sit between them
 * (LayerNorm, Linear) so a whole block runs without leaving the library.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in `_host`;
 *   - the library never allocates, frees or synchronises: the caller owns all
 *     buffers, every kernel is enqueued on `stream` (a hipStream_t, passed as
 *     void* so the header needs no HIP include) and the call returns at once;
 *   - tensors are dense row-major unless explicit element strides are given;
 *   - `dtype` selects storage AND arithmetic flavour: VTDGE_F32 = fp32 storage,
 *     fp32 arithmetic; VTDGE_BF16 = bf16 storage, fp32 accumulation, one
 *     round-to-nearest-even on store;
 *   - packed ("sparse") operands are [rows, C] matrices whose row count is only
 *     known on the device after routing.  Such calls take `rows` (a host-side
 *     upper bound: grid size, buffer capacity) and `rows_dev` (nullable device
 *     pointer to the live int64 row count; when NULL, `rows` itself is live);
 *   - return value: VTDGE_OK (0) or a negative VTDGE_ERR_*; vtdge_last_error()
 *     gives a thread-local message.  No exceptions cross the ABI.
 */
#ifndef VTDGE_H
#define VTDGE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VTDGE_OK 0
#define VTDGE_ERR_ARG (-1)         /* NULL pointer, non-positive size, bad enum     */
#define VTDGE_ERR_UNSUPPORTED (-2) /* valid request outside the built kernel family */
#define VTDGE_ERR_LAUNCH (-3)      /* hipLaunchKernel / hipGetLastError failed      */

#define VTDGE_F32 0
#define VTDGE_BF16 1

#define VTDGE_ACT_NONE 0
#define VTDGE_ACT_GELU 1 /* exact erf GELU (torch.nn.GELU default) */

#define VTDGE_MAX_SPLITS 8

int vtdge_version(void);
const char *vtdge_last_error(void);
/* The demangled name of the kernel that the calling thread's latest launch was (the last one, for an entry point
 * that launches several), as a profiler lists it; "" before the first launch.  For measurement tools. */
const char *vtdge_last_kernel(void);

/* Router: region mean of the spatial tokens, Linear(C -> S), argmax.
 * Replaces DynamicRouter.forward + argmax (vtpack/layers/dge.py:145-150, :75).
 *   x       [B, extra + H*W, C]      weight [S, C]      bias [S]
 *   gate    [B, H/R, W/R, S] in `dtype` (nullable)      indices int64 [B, H/R, W/R]
 * The mean is taken over the R x R window in dy-outer / dx-inner order in fp32;
 * with VTDGE_BF16 the pooled value and the logits are rounded to bf16 as the
 * reference's modules would, and the argmax (lowest index wins a tie) is taken
 * on the rounded logits. */
int vtdge_router(const void *x, const void *weight, const void *bias, void *gate, int64_t *indices,
                 int B, int H, int W, int C, int extra, int R, int S, int dtype, void *stream);

/* The router and the block's first LayerNorm in one pass over x: gate / indices as vtdge_router, plus
 *   ln_out [B, extra + H*W, C] = LayerNorm(x) * ln_weight + ln_bias   (every token, the extra ones included).
 * Replaces DynamicRouter.forward + argmax (vtpack/layers/dge.py:145-150, :75) together with norm1 applied to
 * all tokens (vtpack/models/dge/deit_dge.py:127); both results are bit-identical to vtdge_router and
 * vtdge_layernorm.  R must be 4 or 2 and a row must fit one 16-byte vector per lane (C <= 512 in bf16, 256 in
 * fp32); VTDGE_ERR_UNSUPPORTED otherwise. */
int vtdge_router_layernorm(const void *x, const void *weight, const void *bias, void *gate, int64_t *indices,
                           const void *ln_weight, const void *ln_bias, float ln_eps, void *ln_out, int B, int H,
                           int W, int C, int extra, int R, int S, int dtype, void *stream);

/* Gate indices -> packed query descriptors.
 * Replaces grained_sample_index_to_patch
 * (vtpack/layers/csrc/grained_sample/grained_sample.cu:302-345, kernel :146-196).
 *   indices int64 [B, Hr, Wr]   splits int64 [S] (device, as in the reference)
 *   patches int64 [capacity_rows, 4] rows = [sample, y0, x0, size]; extra-token
 *           rows are [sample, -(e+1), 0, 1] (the reference leaves column 2 of
 *           those rows unwritten; 0 is written here).  Nullable: lengths only.
 *   offsets int64 [B+1] exclusive prefix of lengths (offsets[B] = total rows L)
 *   lengths int64 [B]   (the reference returns these on the host; copying them
 *           is the caller's business so that the fused path needs no sync)
 * Rows past `capacity_rows` are never written.  Gate indices outside [0,S) are
 * clamped (the reference reads out of bounds). */
int vtdge_index_to_patch(const int64_t *indices, const int64_t *splits, int B, int Hr, int Wr, int S,
                         int R, int extra, int64_t *patches, int64_t capacity_rows, int64_t *offsets,
                         int64_t *lengths, void *stream);

/* Every patch of every granularity (exported by the reference, unused by its
 * models).  Replaces grained_sample_index_to_patch_dense (grained_sample.cu:347-433).
 *   patches int64 [B * per_sample, 4], per_sample = extra + Hr*Wr*sum(splits^2)
 *   splits_host: HOST pointer (the reference copies it to the host too, :401). */
int vtdge_index_to_patch_dense(const int64_t *splits_host, int B, int Hr, int Wr, int S, int R, int extra,
                               int64_t *patches, void *stream);

/* Grained sampling ("compress"): one packed query row per patch = mean of its
 * size x size token window (fp32 accumulation, dy outer / dx inner, one divide),
 * or a copy of the extra token.
 * Replaces grained_sample_compress (grained_sample.cu:198-239, kernel :31-69).
 *   x [B, N, C]   patches [rows, 4]   out [rows, C]
 * Optional fused LayerNorm of the (rounded) output row, as the block applies
 * norm1 to the compressed queries (vtpack/models/dge/deit_dge.py:127):
 *   ln_out [rows, C] nullable; ln_weight, ln_bias [C]. */
int vtdge_compress(const void *x, const int64_t *patches, const int64_t *rows_dev, int64_t rows,
                   void *out, void *ln_out, const void *ln_weight, const void *ln_bias, float ln_eps,
                   int B, int N, int C, int W, int extra, int dtype, void *stream);

/* Scatter back ("decompress"): every token covered by a patch receives
 *   out[b,t,:] = (in[row,:] - sub[row,:]) + ref[b,t,:]
 * with `sub` and `ref` each optional (NULL = term absent).
 * Replaces grained_sample_decompress, both overloads (grained_sample.cu:241-300,
 * kernels :71-144; ref == NULL is is_add_ref = false) and, with `sub`, the
 * subtraction in DynamicGrainedEncoder.decompress (vtpack/layers/dge.py:88).
 * In bf16 the difference is rounded to bf16 before the add, as the reference's
 * separate elementwise op would.  Tokens no patch covers are left untouched. */
int vtdge_decompress(const void *in, const void *sub, const int64_t *patches, const int64_t *rows_dev,
                     int64_t rows, const void *ref, void *out, int B, int N, int C, int W, int extra,
                     int dtype, void *stream);

/* The same scatter with `ref` present, plus the LayerNorm of every token written:
 *   out[b,t,:] = (in[row,:] - sub[row,:]) + ref[b,t,:],   ln_out[b,t,:] = LayerNorm(out[b,t,:])
 * i.e. the last step of one block (vtpack/layers/dge.py:87-112) together with the first LayerNorm of the next
 * (norm1 at vtpack/models/dge/deit_dge.py:127), which would read the same tokens back.  The statistics are taken
 * from the values as stored in `out`.  Rows of at most 64 16-byte vectors (C <= 512 in bf16, 256 in fp32). */
int vtdge_decompress_layernorm(const void *in, const void *sub, const int64_t *patches, const int64_t *rows_dev,
                               int64_t rows, const void *ref, void *out, void *ln_out, const void *ln_weight,
                               const void *ln_bias, float ln_eps, int B, int N, int C, int W, int extra, int dtype,
                               void *stream);

/* Scatter back by region, and the NEXT block's router on the tokens just written:
 *   out[b,t,:] = (in[row,:] - sub[row,:]) + ref[b,t,:]        (as vtdge_decompress with `sub` and `ref`; sub nullable)
 *   next_gate [B, H/R, W/R, S2], next_indices int64 [B, H/R, W/R] = vtdge_router(out, next_weight, next_bias)
 * i.e. the last step of one block (vtpack/layers/dge.py:87-112) together with DynamicRouter.forward + argmax of the
 * block that follows (vtpack/layers/dge.py:145-150, :75), which would read the same tokens back.  The packed rows
 * are found from this block's gate indices `cur_indices` [B, H/R, W/R] (S splits in `splits`, as given to
 * vtdge_index_to_patch) and `offsets` [B+1] instead of the patch list.  Both results are bit-identical to the two
 * separate calls.  next_weight == NULL (with next_bias, next_indices) leaves the router out.  R must be 4 and every
 * split size must divide it; VTDGE_ERR_UNSUPPORTED for another R.
 * out_records (nullable) [B * (extra + H*W), 16] bf16: the statistics record of every row of `out` as stored (mean
 * and sqrt(var + records_eps), see vtdge_layernorm_stats), for the next block's norm1 -> kv through
 * vtdge_linear_layernorm; one-pass fp32 sums about a value of the row itself.  bf16 rows of 264 to 512 channels.
 * next_counts (nullable; needs the next router) uint8 [B * H/R * W/R]: the number of queries the next block takes
 * from every region, next_splits[next_indices]^2 with next_splits int64 [S2] on the device: what
 * vtdge_compress_regions adds up to place a region's queries.
 * region_rows (nullable) int32 [B * H/R * W/R] with cur_counts uint8 of the same length: the first packed row and the
 * query count of every region of THIS block as vtdge_compress_regions left them; the kernel then takes a region's
 * place from them instead of adding it up from cur_indices and offsets. */
int vtdge_decompress_router(const void *in, const void *sub, const int64_t *cur_indices, const int64_t *splits,
                            const int64_t *offsets, const void *ref, void *out, const void *next_weight,
                            const void *next_bias, void *next_gate, int64_t *next_indices, void *out_records,
                            float records_eps, const int64_t *next_splits, uint8_t *next_counts,
                            const int32_t *region_rows, const uint8_t *cur_counts, int B, int H, int W, int C,
                            int extra, int R, int S, int S2, int dtype, void *stream);

/* vtdge_decompress_router that goes on to pack the NEXT block's queries from the tokens it has just written: the
 * scatter-back of one block (vtpack/layers/dge.py:87-112), the next block's router (:145-150, :75) and the next
 * block's index->patch + compress (:76-79) in one launch, i.e. vtdge_decompress_router followed by
 * vtdge_compress_regions without a second pass over the tokens.  All outputs are bit-identical to those two calls.
 *   next_comp [capacity_rows, C], next_comp_records [capacity_rows, 16] bf16 with next_records_eps,
 *   next_patches (nullable) [capacity_rows, 4], next_offsets [B+1], next_region_rows (nullable) int32 [regions]:
 *   as vtdge_compress_regions writes comp, records, patches, offsets and region_rows (lengths are the differences
 *   of the offsets and are not written)
 *   workspace: vtdge_decompress_router_compress_workspace(B, H, W, R) bytes of device memory, 8-byte aligned, all
 *   zero when the kernel starts (clear_workspace != 0: the call clears it first with a small fill kernel; a caller
 *   that keeps one slice per block can clear them all at once instead).  The workgroups hand the running number of
 *   queries along through it (one 64-bit word each); word 0 is raised to 1 if a workgroup gave up waiting for the
 *   ones before it, in which case rows are missing from next_comp and next_offsets[B] exceeds capacity_rows.
 * bf16 rows of 264 to 512 channels, R = 4, splits out of {1, 2, 4}, the regions a multiple of 4 up to 65536, the
 * next router with its splits and count bytes, out_records present; VTDGE_ERR_UNSUPPORTED otherwise. */
int64_t vtdge_decompress_router_compress_workspace(int B, int H, int W, int R);
int vtdge_decompress_router_compress(const void *in, const void *sub, const int64_t *cur_indices,
                                     const int64_t *splits, const int64_t *offsets, const void *ref, void *out,
                                     const void *next_weight, const void *next_bias, void *next_gate,
                                     int64_t *next_indices, void *out_records, float records_eps,
                                     const int64_t *next_splits, uint8_t *next_counts, const int32_t *region_rows,
                                     const uint8_t *cur_counts, void *next_comp, void *next_comp_records,
                                     float next_records_eps, int64_t *next_patches, int64_t capacity_rows,
                                     int64_t *next_offsets, int32_t *next_region_rows, void *workspace,
                                     int64_t workspace_bytes, int clear_workspace, int B, int H, int W, int C,
                                     int extra, int R, int S, int S2, int dtype, void *stream);

/* vtdge_decompress_router_compress for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc); it has no counterpart in the reference.  The arguments are
 * those of vtdge_decompress_router_compress without the workspace: the status words live in an array inside the
 * library's device image (128 KB on every GPU the library runs on, held until the process ends), cleared by a small
 * fill kernel on `stream` before the kernel runs.  The call allocates and frees nothing.  At most 65536 regions
 * (VTDGE_ERR_UNSUPPORTED beyond).  All calls on one GPU share the array: calls that overlap on one GPU (two streams,
 * two threads) race - run them in turn.  The first call on a GPU looks the array's address up
 * (hipGetSymbolAddress) and should therefore come before any stream capture.  A kernel that gave up shows as
 * next_offsets[B] > capacity_rows, as in vtdge_decompress_router_compress. */
int vtdge_decompress_router_compress_static(const void *in, const void *sub, const int64_t *cur_indices,
                                            const int64_t *splits, const int64_t *offsets, const void *ref,
                                            void *out, const void *next_weight, const void *next_bias,
                                            void *next_gate, int64_t *next_indices, void *out_records,
                                            float records_eps, const int64_t *next_splits, uint8_t *next_counts,
                                            const int32_t *region_rows, const uint8_t *cur_counts, void *next_comp,
                                            void *next_comp_records, float next_records_eps, int64_t *next_patches,
                                            int64_t capacity_rows, int64_t *next_offsets, int32_t *next_region_rows,
                                            int B, int H, int W, int C, int extra, int R, int S, int S2, int dtype,
                                            void *stream);

/* The router of a model's FIRST block together with the statistics records of all its tokens (no scatter-back
 * precedes it that could leave them): vtdge_router and vtdge_layernorm_stats in one pass over x, i.e.
 * DynamicRouter.forward + argmax (vtpack/layers/dge.py:145-150, :75) and the statistics half of norm1
 * (vtpack/models/dge/deit_dge.py:127).  gate / indices are bit-identical to vtdge_router's; the records are one-pass
 * fp32 sums about a value of the row itself, as vtdge_decompress_router writes them.
 *   x [B, extra + H*W, C]   records [B * (extra + H*W), 16] bf16   counts (nullable) as in vtdge_decompress_router,
 *   from `splits` int64 [S] on the device
 *   front_rows (nullable) [extra, C]: rows that are first stored as tokens 0 .. extra-1 of EVERY sample of x - the
 *   class (and distillation) token plus its position embedding, which the reference concatenates in front of the
 *   patch tokens (deit_dge.py:270-277) and which do not depend on the sample.
 *   clear_words (nullable) with n_clear_words: 64-bit words the launch sets to zero on the way - the workspaces of
 *   the vtdge_decompress_router_compress calls that follow it on the stream, so that a forward needs no fill kernel.
 * bf16 rows of 264 to 512 channels, R = 4. */
int vtdge_router_stats(void *x, const void *front_rows, const void *weight, const void *bias, void *gate,
                       int64_t *indices, void *records, float records_eps, const int64_t *splits, uint8_t *counts,
                       void *clear_words, int64_t n_clear_words, int B, int H, int W, int C, int extra, int R, int S,
                       int dtype, void *stream);

/* Gate indices -> packed queries in one step, by region: vtdge_index_to_patch and vtdge_compress together, i.e.
 * grained_sample_index_to_patch followed by grained_sample_compress
 * (vtpack/layers/csrc/grained_sample/grained_sample.cu:302-345 with :146-196, and :198-239 with :31-69) as
 * DynamicGrainedEncoder.compress calls them (vtpack/layers/dge.py:76-79), without the descriptor list in between: a
 * region's packed rows are consecutive, so the kernel places them from the query counts of the regions before it.
 *   x [B, extra + H*W, C]   indices int64 [B, H/R, W/R]   splits int64 [S] (device)
 *   counts  nullable uint8 [B * H/R * W/R, padded to a multiple of 16 bytes]: splits[indices]^2 per region, as
 *           vtdge_decompress_router leaves them; without it the kernel works the counts out from `indices`
 *   comp    [capacity_rows, C]: the packed queries, bit for bit those of vtdge_compress
 *   records nullable [capacity_rows, 16] bf16: the statistics record of every row of comp as stored (mean and
 *           sqrt(var + records_eps), see vtdge_layernorm_stats) for a vtdge_linear_layernorm that takes comp next
 *           (norm1 -> q, vtpack/models/dge/deit_dge.py:127 with :72); bf16 only
 *   patches (nullable), offsets [B+1], lengths [B]: as vtdge_index_to_patch writes them
 *   region_rows (nullable) int32 [B * H/R * W/R]: the first packed row of every region, for vtdge_decompress_router
 * The caller guarantees capacity_rows >= the number of queries (B * (extra + H*W) always is).  R must be 4 with splits
 * out of {1, 2, 4}, a row one 16-byte vector per lane (C <= 512 in bf16, 256 in fp32), at most 65536 regions and
 * 64 extra tokens; VTDGE_ERR_UNSUPPORTED otherwise. */
int vtdge_compress_regions(const void *x, const int64_t *indices, const int64_t *splits, const uint8_t *counts,
                           void *comp, void *records, float records_eps, int64_t *patches, int64_t capacity_rows,
                           int64_t *offsets, int64_t *lengths, int32_t *region_rows, int B, int H, int W, int C,
                           int extra, int R, int S, int dtype, void *stream);

/* The patch embedding of a pyramid model's first stage in one pass over the images: Conv2d(Cin, N, kernel P, stride P)
 * + bias, the embedding's LayerNorm and `+ pos_embed` (vtpack/models/dge/pvt_dge.py:143-176 with :312-314), each
 * rounded to the storage type as the separate modules would round.
 *   images [B, Cin, S, S]   weight [N, Cin*P*P] (the convolution's weight, flattened)   bias, ln_weight, ln_bias [N]
 *   pos (nullable) [(S/P)^2, N]   out [B * (S/P)^2, N]
 * bf16, Cin = 3, P = 4, N = 64, S a multiple of 64; VTDGE_ERR_UNSUPPORTED otherwise (the caller then gathers the patches
 * and uses vtdge_linear, vtdge_layernorm_add). */
int vtdge_patch_embed_norm(const void *images, const void *weight, const void *bias, const void *ln_weight,
                           const void *ln_bias, float ln_eps, const void *pos, void *out, int B, int Cin, int S, int P,
                           int N, int dtype, void *stream);

/* vtdge_layernorm followed by the addition of a periodic set of rows: out[r] = LayerNorm(x[r]) + add[r mod add_rows],
 * the LayerNorm's result rounded to the storage type before the addition as the two modules would.  Stands in for a
 * patch embedding's norm followed by `x + pos_embed` (vtpack/models/dge/pvt_dge.py:176 with :312-314; add =
 * pos_embed [H*W, C], rows = B * H*W). */
int vtdge_layernorm_add(const void *x, const void *weight, const void *bias, const void *add, int64_t add_rows,
                        void *out, int64_t rows, int C, float eps, int dtype, void *stream);

/* Row-wise LayerNorm over the last dimension (biased variance, fp32 statistics).
 * Stands in for nn.LayerNorm(eps=1e-6) at vtpack/models/dge/deit_dge.py:127-128. */
int vtdge_layernorm(const void *x, const void *weight, const void *bias, void *out, const int64_t *rows_dev,
                    int64_t rows, int C, float eps, int dtype, void *stream);
/* The same for input rows that lie in groups: row r is x + (r / x_group_rows) * x_group_stride + (r % x_group_rows) * C
 * (elements); out [rows, C] is dense.  The final norm of a model only on the rows the classifier reads - the class
 * (and distillation) tokens, the first rows of every sample (vtpack/models/dge/deit_dge.py:283-285 with :288-299) -
 * without a gathered copy of them: x_group_rows = extra, x_group_stride = N * C. */
int vtdge_layernorm_rows(const void *x, int64_t x_group_stride, int x_group_rows, const void *weight, const void *bias,
                         void *out, int64_t rows, int C, float eps, int dtype, void *stream);

/* Packed-M Linear: out[m, n] = act(sum_k A[m,k] * W[n,k] + bias[n]) + residual[m,n].
 * The M dimension is the packed query set of all samples (weights are shared),
 * which is what the reference's q / proj / fc1 / fc2 nn.Linear calls compute on
 * [L, C] (vtpack/models/dge/deit_dge.py:72,96,38-44) and kv on [B*N, C] (:73).
 *   A [rows, K] leading dim lda      W [N, K] dense      bias [N] nullable
 *   residual [rows, N] leading dim ldr, nullable         out [rows, N] leading dim ldo
 * MFMA kernels; K must be a multiple of 16 bytes worth of elements (4 fp32 / 8 bf16).  Rows of K that are a
 * multiple of 128 bytes (and 16-byte aligned operands) take the direct-to-LDS persistent kernel. */
int vtdge_linear(const void *A, int64_t lda, const void *W, const void *bias, const void *residual,
                 int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev, int64_t rows, int N, int K,
                 int act, int dtype, void *stream);

/* The same Linear with a packed copy of W beside it.  The weight-stationary kernels keep a strip of W in registers
 * for the life of a workgroup; from a copy laid out in the order of those registers they fill them with contiguous
 * loads (half the start-up time of a launch).  The weights of an nn.Linear (vtpack/models/dge/deit_dge.py:70-74,
 * :38-44) do not change between calls at inference, so a caller packs them once:
 *   vtdge_linear_packed_size  *bytes = size of the packed copy of W [N, K], or 0 when no kernel for this shape uses
 *                             one (pass packed = NULL then)
 *   vtdge_linear_prepack      fills `packed` (16-byte aligned, *bytes long) from W; VTDGE_ERR_UNSUPPORTED when the
 *                             size is 0
 *   vtdge_linear_prepacked    vtdge_linear with `packed` (nullable; must have been made from this W).  W itself is
 *                             still required: the kernels chosen for few rows read it.
 * Results are bit-identical with and without the packed copy. */
int vtdge_linear_packed_size(int N, int K, int dtype, int64_t *bytes);
int vtdge_linear_prepack(const void *W, int N, int K, int dtype, void *packed, void *stream);
int vtdge_linear_prepacked(const void *A, int64_t lda, const void *W, const void *packed, const void *bias,
                           const void *residual, int64_t ldr, void *out, int64_t ldo, const int64_t *rows_dev,
                           int64_t rows, int N, int K, int act, int dtype, void *stream);

/* Patch embedding, position embedding included: the stride-P P x P convolution of the reference's PatchEmbed
 * (nn.Conv2d, vtpack/models/dge/deit_dge.py:141-155) as a Linear over the patches, read straight from the images
 * (no unfolded copy), with the addition of the position table (x = x + pos_embed, deit_dge.py:277) in its epilogue:
 *   images [B, Cin, S, S]   weight [C, Cin * P * P] (the convolution's weight, flattened)   bias [C]
 *   pos_embed [extra + G*G, C], G = S / P   tokens [B, extra + G*G, C]
 *   tokens[b, extra + gy*G + gx, :] = conv(images)[b, :, gy, gx] + bias + pos_embed[extra + gy*G + gx, :]
 * in fp32 with one rounding; rows 0 .. extra-1 of every sample (class / distillation tokens) are left untouched.
 * A patch row must be 16, 32, 64 or 128 bytes (P = 16: both types) and all operands 16-byte aligned, else
 * VTDGE_ERR_UNSUPPORTED. */
int vtdge_patch_embed(const void *images, const void *weight, const void *bias, const void *pos_embed, void *tokens,
                      int B, int Cin, int S, int P, int C, int extra, int dtype, void *stream);

/* A stride-P P x P convolution over a channels-last token grid, as a Linear over the P x P blocks of tokens read
 * straight from the grid (no gathered copy): the spatial reduction in front of the key/value projection
 * (nn.Conv2d(dim, dim, sr_ratio, sr_ratio), vtpack/models/dge/pvt_dge.py:62, :81-83) and the patch embedding of the
 * later stages (nn.Conv2d(in_chans, embed_dim, patch_size, patch_size), pvt_dge.py:164, :175), whose input here stays
 * [B, H*W, C] tokens instead of going back to [B, C, H, W]:
 *   tokens [B, H*W, C]   weight [N, P*P*C], the convolution's weight in (kh, kw, c) order   bias [N]
 *   out [B*(H/P)*(W/P), N]:  out[(b, gy, gx), :] = sum over (dy, dx, c) of
 *        tokens[b, (gy*P + dy)*W + gx*P + dx, c] * weight[:, (dy*P + dx)*C + c]  + bias,   fp32 sums, one rounding.
 * C values must fill whole 128-byte pieces (C % 64 == 0 for bf16, % 32 for fp32), H and W be multiples of P and all
 * operands 16-byte aligned, else VTDGE_ERR_UNSUPPORTED. */
int vtdge_patch_linear(const void *tokens, const void *weight, const void *bias, void *out, int B, int H, int W, int C,
                       int P, int N, int dtype, void *stream);

/* LayerNorm folded into the Linear that consumes it: out = act(LayerNorm(A) W^T + bias) computed from the raw rows
 * of A, so that nn.LayerNorm followed by nn.Linear (norm1 -> kv and norm2 -> fc1,
 * vtpack/models/dge/deit_dge.py:127-128 with :73 and :38-44) costs no pass over the rows of its own:
 *     LayerNorm(a) W^T + bias = rstd * (a W'^T - mean * colsum(W') + sigma * b'),
 *     W' = W * ln_weight (rounded to the storage type),  b' = bias + W ln_bias,  sigma = 1 / rstd = sqrt(var + eps).
 *   vtdge_layernorm_stats   records [rows, 16] bf16 (32 bytes a row): mean and sigma of every row of x [rows, C],
 *                           each split into bf16 parts in the operand order of the matrix instruction (two-pass
 *                           fp32 statistics, as vtdge_layernorm).  Other kernels that produce the rows can write
 *                           the same records (see vtdge_decompress_router, vtdge_linear_stats).
 *   vtdge_layernorm_fold    once per weight: W_folded [N, K] = W', col_records [N, 16] bf16 = -colsum(W') and b'
 *                           in the matching order.  bias is nullable.
 *   vtdge_linear_layernorm  the Linear: A [rows, K] raw rows with their row_records, W_folded (and optionally its
 *                           packed copy from vtdge_linear_prepack), col_records.  Weight-stationary kernel only:
 *                           bf16, K = 384, N a multiple of 384 up to 3072, rows >= 2048 (capacity; the live count
 *                           may be anything), else VTDGE_ERR_UNSUPPORTED.
 * Against vtdge_layernorm followed by vtdge_linear the result differs by the rounding of W' instead of that of
 * LayerNorm(a) to bf16: the same order of magnitude, not the same bits. */
/* vtdge_linear (no activation) that also writes the statistics records of its output rows, for a
 * vtdge_linear_layernorm that takes `out` next: proj + residual followed by norm2 -> fc1
 * (vtpack/models/dge/deit_dge.py:96, :128, :38-44).  The records are computed from the fp32 sums before their rounding
 * to bf16.  Weight-stationary kernel with one column group only: bf16, K = 384, N = 384, rows >= 2048. */
int vtdge_linear_stats(const void *A, int64_t lda, const void *W, const void *packed, const void *bias,
                       const void *residual, int64_t ldr, void *out, int64_t ldo, void *out_records,
                       float records_eps, const int64_t *rows_dev, int64_t rows, int N, int K, int dtype,
                       void *stream);
int vtdge_layernorm_stats(const void *x, void *records, const int64_t *rows_dev, int64_t rows, int C, float eps,
                          int dtype, void *stream);
int vtdge_layernorm_fold(const void *W, const void *bias, const void *ln_weight, const void *ln_bias, int N, int K,
                         int dtype, void *W_folded, void *col_records, void *stream);
int vtdge_linear_layernorm(const void *A, int64_t lda, const void *row_records, const void *W_folded,
                           const void *packed, const void *col_records, void *out, int64_t ldo,
                           const int64_t *rows_dev, int64_t rows, int N, int K, int act, int dtype, void *stream);

/* Two vtdge_linear_layernorm calls without activation as ONE launch: norm1 -> kv on all tokens and norm1 -> q on the
 * packed queries (vtpack/models/dge/deit_dge.py:127 with :73 and :72), which the reference issues one after the
 * other.  The workgroups are dealt out between the two in proportion to their live rows (read on the device), so
 * the smaller one no longer runs a few tiles per workgroup behind the fixed cost of a launch of its own.  Operands
 * with suffix 0 and 1 as in vtdge_linear_layernorm, same K; results are bit-identical to the two separate calls. */
int vtdge_linear_layernorm_pair(const void *A0, int64_t lda0, const void *row_records0, const void *W_folded0,
                                const void *packed0, const void *col_records0, void *out0, int64_t ldo0,
                                const int64_t *rows_dev0, int64_t rows0, int N0, const void *A1, int64_t lda1,
                                const void *row_records1, const void *W_folded1, const void *packed1,
                                const void *col_records1, void *out1, int64_t ldo1, const int64_t *rows_dev1,
                                int64_t rows1, int N1, int K, int dtype, void *stream);

/* Sparse attention of packed queries against each sample's full K/V:
 *   out[rows of sample i, head a] = softmax(scale * Q_i,a K_i,a^T) V_i,a
 * Replaces batched_sparse_attention_forward
 * (vtpack/layers/csrc/batched_sparse_gemm/batched_sparse_gemm.cu:219-305).
 * All operands are addressed through element strides so that both the
 * reference's contiguous [h, L, d] / [h, B, n, d] tensors and the un-permuted
 * outputs of the q / kv Linears ([L, h*d] and [B, n, 2, h, d]) can be passed:
 *   q(row, a, c)   = q[row*q_row_stride + a*q_head_stride + c]
 *   k(i, t, a, c)  = k[i*kv_batch_stride + t*kv_tok_stride + a*kv_head_stride + c]  (same for v)
 *   out(row, a, c) = out[row*o_row_stride + a*o_head_stride + c]
 *   offsets int64 [B+1] (device) exclusive prefix of the per-sample query counts
 *   max_rows_per_sample: host upper bound of any sample's query count (grid size)
 * head_dim d must be 64 or 32. */
int vtdge_sparse_attention(const void *q, int64_t q_row_stride, int64_t q_head_stride, const void *k,
                           const void *v, int64_t kv_batch_stride, int64_t kv_tok_stride,
                           int64_t kv_head_stride, const int64_t *offsets, void *out, int64_t o_row_stride,
                           int64_t o_head_stride, int B, int h, int d, int n, int max_rows_per_sample,
                           float scale, int dtype, void *stream);

/* Per-sample variable-length batched matmul over heads.
 * Replaces batched_sparse_gemm_forward and batched_sparse_gemm_v2_forward
 * (batched_sparse_gemm.cu:150-195, :83-148):
 *   a [h, La, ka], b [h, Lb, kb]; sample i uses rows a_offsets[i]..a_offsets[i+1]
 *   of a and b_offsets[i]..b_offsets[i+1] of b, each optionally transposed in its
 *   last two dims; out [h, out_rows, out_cols] is the concatenation along dim 1.
 *   a_offsets, b_offsets int64 [B+1] on the device.
 *   max_m: host upper bound of any sample's output row count (grid size). */
int vtdge_batched_sparse_gemm(const void *a, const void *b, const int64_t *a_offsets, const int64_t *b_offsets,
                              void *out, int B, int h, int64_t La, int ka, int64_t Lb, int kb, int trans_a,
                              int trans_b, int64_t out_rows, int64_t out_cols, int64_t max_m, int dtype,
                              void *stream);

#ifdef __cplusplus
}
#endif
#endif /* VTDGE_H */
