/*
 * lookupffn_hip.h -- C ABI of the MI355X (gfx950) LookupFFN kernel library.
 *
 * One shared library (liblookupffn_hip.so), plain C linkage, raw device
 * pointers, sizes as int64_t, a hipStream_t passed as void*.  No C++ types and
 * no torch types cross this boundary.  The entry points are what the reference's
 * three pybind modules bind for this path (paths relative to the reference
 * checkout, PL/ = src/roberta/models/prenorm_lookup/):
 *
 *   fast_hadamard_transform_kernel  PL/bh4/fast_hadamard_transform/extension/torch_extension.cpp:30-32
 *   gather_add                      PL/gather/cuda/extension/torch_extension.cpp:91-96
 *   ccs_cpu                         PL/compute_code_score/torch_extension.cc:45
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer to a contiguous row-major array that the
 *     caller owns.  The library allocates nothing, frees nothing and keeps no
 *     results between calls (it remembers, per device, which kernels were granted
 *     large LDS sizes and where its one static scratch array lives).
 *   - Forward outputs are fully overwritten (no zero-initialisation needed).
 *     Only lffn_scatter_add_f32 / _f16 accumulate into their output.
 *   - Calls are asynchronous on `stream` (NULL = the legacy default stream) and
 *     may be issued from any host thread.
 *   - Return value: LFFN_OK, or a negative LFFN_ERR_* code.  Nothing throws or
 *     aborts.  lffn_error_string() names a code.
 *   - Indices are never trusted: a row index outside [0, source_size) is clamped
 *     into range inside the kernels, so a bad index gives a wrong value, not a
 *     memory fault.
 */
#ifndef LOOKUPFFN_HIP_H
#define LOOKUPFFN_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LFFN_OK               0
#define LFFN_ERR_BAD_ARG     -1   /* null pointer, negative size, misaligned pointer */
#define LFFN_ERR_UNSUPPORTED -2   /* a shape outside what the kernels are built for */
#define LFFN_ERR_LAUNCH      -3   /* hipGetLastError() after the launch was not hipSuccess */
#define LFFN_ERR_SCRATCH     -4   /* an entry point that allocates nothing: the shape exceeds its static scratch */

#define LFFN_ABI_VERSION 7

/* ABI version of the loaded library (LFFN_ABI_VERSION at build time). */
int lffn_version(void);

/* Static, human-readable name of a return code. */
const char *lffn_error_string(int code);

/* ---------------------------------------------------------------- projection */

/*
 * out[b,:] = in[b,:] . H_D, unnormalised Sylvester (natural) order, fp32.
 * in, out: [B, D]; D a power of two, 4 <= D <= 1024.  in == out is allowed.
 * Replaces fast_hadamard_transform (fast_hadamard_transform/extension/cuda_launch.cu:56-78,
 * kernel cuda_kernel.cu:219-257); the transform is its own transpose, so the
 * same call is the backward (fast_hadamard_transform/kernel.py:47-54).
 */
int lffn_fht_f32(const float *in, float *out, int64_t B, int64_t D, void *stream);

/*
 * The same transform on rows stored as IEEE half (f16) or bfloat16 (bf16), raw 16-bit
 * patterns: values are widened on load, all butterflies run in fp32, the result is
 * rounded to nearest even once on the store.  in == out is allowed; 8-byte alignment.
 * Takes the place of fast_hadamard_transform_dim512_fp16 / _dim1024_fp16
 * (fast_hadamard_transform/extension/cuda_launch.cu:12-54, kernels cuda_kernel.cu:19-216),
 * which exist for D = 512 and 1024 only and round in half precision after every stage.
 */
int lffn_fht_f16(const uint16_t *in, uint16_t *out, int64_t B, int64_t D, void *stream);
int lffn_fht_bf16(const uint16_t *in, uint16_t *out, int64_t B, int64_t D, void *stream);

/*
 * BH4 mixing with block size 1 (a diagonal scale before every transform):
 *   for r < R:  y = pad(x);  for j < J:  y = FHT(diag[r,j,:] * y);  out[b, r*D:(r+1)*D] = y
 * x: [B, H] with H <= D (zero-padded on load, PL/lookup.py:32-34); diag: [R, J, D];
 * out: [B, R*D].  Replaces bh4_cuda (PL/bh4/kernel.py:23-36) for weight
 * [R, J, D, 1, 1], where the einsum "bni,noi->bno" (":32") is an element-wise product.
 */
int lffn_bh4_diag_f32(const float *x, const float *diag, float *out,
                      int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, void *stream);

/*
 * Backward of lffn_project_hash_f32 (block size 1, 8-bit codes) in one kernel: from x, the
 * diagonals, the z the forward kept and the gradient of the scores, the gradients of x, of the
 * diagonals and of the projection bias.  The forward stages are recomputed in registers; the
 * transform is its own transpose.
 * x: [B, H], H % 4 == 0; diag: [R, J, D], J <= 4, 256 <= D <= 1024; z: [B, T*8]; g_score: [B, T];
 * g_x: [R, B, H], one slab per repeat (the caller adds them; R == 1 needs nothing);
 * part_diag: [num_partials, R, J, D] and part_bias: [num_partials, R*D]: one partial sum per
 * workgroup, fully written; the caller adds them over the first axis (grad bias = the first
 * T*8 columns).  num_partials is the number of workgroups per repeat, 1..65535 (512 is a good
 * value on 256 compute units).  The code has no gradient.
 * Replaces what autograd records for BH4._forward + compute_code_score_torch
 * (PL/lookup.py:29-39, PL/bh4/kernel.py:23-36, PL/compute_code_score/kernel.py:47-53).
 */
int lffn_project_hash_bwd_f32(const float *x, const float *diag, const float *z, const float *g_score,
                              float *g_x, float *part_diag, float *part_bias, int64_t B, int64_t H,
                              int64_t D, int64_t R, int64_t J, int64_t T, int64_t num_partials,
                              float decay, float residual, void *stream);

/*
 * lffn_ln_project_hash_bwd_f32: the same for the forward with LayerNorm inside
 * (lffn_ln_project_hash_f32 with z kept): h = LayerNorm(x; ln_weight, ln_bias, ln_eps) is formed on
 * load as in that forward, and g_h [R, B, H] is the gradient w.r.t. h, which
 * lffn_layer_norm_bwd_f32 takes on to x and the LayerNorm parameters (it adds the R slabs itself).
 * Replaces what autograd records for self.LayerNorm's output feeding BH4._forward +
 * compute_code_score_torch (PL/lookup.py:99,29-39): the normalised activations are never stored.
 */
int lffn_ln_project_hash_bwd_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                 const float *diag, const float *z, const float *g_score, float *g_h,
                                 float *part_diag, float *part_bias, int64_t B, int64_t H, int64_t D, int64_t R,
                                 int64_t J, int64_t T, int64_t num_partials, float decay, float residual,
                                 void *stream);

/*
 * BH4 mixing with 64 x 64 blocks, all stages of a repeat in one kernel:
 *   for r < R:  y = pad(x);  for j < J:  y = FHT(blockdiag(w[r,j]) y);  out[b, r*D:(r+1)*D] = y
 * x: [B, H], H <= D, H % 4 == 0 (zero-padded on load, PL/lookup.py:32-34);
 * out: [B, R*D]; D = 64 * num_block a power of two, 64 <= D <= 1024; block_size must be 64.
 * The 64-point part of every transform is applied to the weights beforehand:
 * lffn_bh4_fold_f32 turns w [R, J, num_block, 64, 64] (PL/lookup.py:22) into
 * w_folded (same size, caller-allocated, must not alias w; each 64 x 64 block
 * is stored in the order the product kernel's lanes fetch it:
 * [o/16][(i%16)/4][i/16][o%16][i%4] for output o, input i), which
 * lffn_bh4_block_f32 takes.  Fold again whenever w changes.  The products run on
 * the fp32 matrix cores; results agree with "product, then transform" to fp32
 * rounding, not bit for bit.
 * Replaces bh4_cuda (PL/bh4/kernel.py:23-36): the einsum "bni,noi->bno" (":32")
 * and hadamard (":34") of every stage.
 */
int lffn_bh4_fold_f32(const float *w, float *w_folded, int64_t R, int64_t J, int64_t num_block,
                      int64_t block_size, void *stream);
int lffn_bh4_block_f32(const float *x, const float *w_folded, float *out, int64_t B, int64_t H,
                       int64_t D, int64_t R, int64_t J, int64_t block_size, void *stream);

/*
 * The whole hashing front end of the layer for 64 x 64 blocks and 8-bit codes, one kernel:
 * (LayerNorm ->) zero-pad -> BH4 as lffn_bh4_block_f32 -> z = decay*y + residual*pad(h) + bias
 * -> code and score of every 8 columns of z[:, :T*8].  ln_weight == NULL: no LayerNorm
 * (h = x), else h = LayerNorm(x; ln_weight, ln_bias, ln_eps) over the H columns.
 * x: [B, H], H % 4 == 0; w_folded from lffn_bh4_fold_f32; proj_bias: [T*8] or NULL;
 * codes: [B, T] int32; scores: [B, T]; T*8 <= R*D.  Neither y nor z is written.
 * Replaces self.LayerNorm (PL/lookup.py:99), BH4._forward (PL/lookup.py:29-39) and
 * compute_code_score (PL/compute_code_score/kernel.py:22-55) for block_size == 64.
 */
int lffn_ln_bh4_block_hash_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                               const float *w_folded, const float *proj_bias, int32_t *codes, float *scores,
                               int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                               int64_t block_size, float decay, float residual, void *stream);

/*
 * Training form of the 64 x 64-block front end and its backward.
 *
 * lffn_bh4_block_hash_train_f32: as lffn_ln_bh4_block_hash_f32 without LayerNorm, and keeping
 * what the backward needs: z [B, T*8] and stage_inputs [R, J-1, B, D], the input of stages
 * 1 .. J-1 (the input of stage 0 is pad(x)).
 *
 * lffn_bh4_fold_mode_f32: the 64-point transform down the output index of num_blocks 64 x 64
 * blocks, written in one of three orders: mode 0 = what the forward kernels fetch (as
 * lffn_bh4_fold_f32), mode 1 = what lffn_bh4_block_bwd_f32 fetches (transposed blocks),
 * mode 2 = natural [o][i] order (applied to a gradient w.r.t. the folded weights it gives the
 * gradient w.r.t. the weights).
 *
 * lffn_bh4_block_bwd_f32: from g_z [B, T*8] (the gradient of z, e.g. from
 * lffn_code_score_bwd_f32) and the mode-1 folded weights: g_x [R, B, H], one slab per repeat
 * (the caller adds them), and stage_grads [R, J, B, D], the gradient in front of each stage's
 * block product after the cross-block part of the transform.  The gradient w.r.t. the folded
 * weights of block n of stage (r, j) is  sum_b stage_grads[r,j,b,64n+o] * input[r,j,b,64n+i];
 * the caller forms it (a batched product over the tokens) and applies mode 2.
 * Replaces what autograd records for bh4_cuda with block_size == 64 (PL/bh4/kernel.py:23-36)
 * and the mix of BH4._forward (PL/lookup.py:36-37).
 *
 * lffn_ln_bh4_block_hash_train_f32: the same with the layer's LayerNorm (PL/lookup.py:99) run on the
 * token tile as it is loaded, as in lffn_ln_bh4_block_hash_f32; row_stats [B, 2] receives every row's
 * mean and 1/sigma.  The normalised rows are not stored: lffn_ln_bh4_block_wgrad_f32 forms them again
 * from x and row_stats (the same operations in the same order), and g_x of lffn_bh4_block_bwd_f32 is
 * then the gradient w.r.t. the LayerNorm output, which lffn_layer_norm_bwd_f32 takes back to x.
 */
int lffn_ln_bh4_block_hash_train_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                     const float *w_folded, const float *proj_bias, int32_t *codes, float *scores,
                                     float *z, float *stage_inputs, float *row_stats, int64_t B, int64_t H,
                                     int64_t D, int64_t R, int64_t J, int64_t T, int64_t block_size, float decay,
                                     float residual, void *stream);
int lffn_bh4_block_hash_train_f32(const float *x, const float *w_folded, const float *proj_bias,
                                  int32_t *codes, float *scores, float *z, float *stage_inputs,
                                  int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                  int64_t block_size, float decay, float residual, void *stream);
int lffn_bh4_fold_mode_f32(const float *w, float *out, int64_t num_blocks, int64_t block_size,
                           int32_t mode, void *stream);
int lffn_bh4_block_bwd_f32(const float *g_z, const float *w_folded_t, float *g_x, float *stage_grads,
                           int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                           int64_t block_size, float decay, float residual, void *stream);

/*
 * Column sums of the per-workgroup partial sums that lffn_layer_norm_bwd_f32 and
 * lffn_project_hash_bwd_f32 leave to the caller, two arrays in one launch:
 *   out_a[c] = sum_p parts_a[p][c]  (c < n_a),   out_b[c] = sum_p parts_b[p][c]  (c < n_b),
 * p < num_partials, in a fixed order (reproducible).  n_a, n_b multiples of 4 (n_b == 0: one array).
 * chunks > 1 splits the rows into that many consecutive chunks of ceil(num_partials / chunks) rows and
 * writes one row of sums per chunk (out_a: [chunks, n_a], out_b: [chunks, n_b]; no chunk may be
 * empty): a first pass over a long array (the bias gradient g.sum(0) over all tokens), whose
 * result a second call with chunks == 1 finishes.
 * Replaces the column reductions autograd runs for the weight and bias gradients of
 * torch.nn.LayerNorm (PL/lookup.py:99), of BH4's diagonal weights and bias (PL/lookup.py:29-39) and
 * of the layer's output bias (PL/lookup.py:108).
 */
int lffn_sum_partials_f32(const float *parts_a, float *out_a, int64_t n_a, const float *parts_b, float *out_b,
                          int64_t n_b, int64_t num_partials, int64_t chunks, void *stream);

/*
 * Backward of the layer's LayerNorm (torch.nn.LayerNorm over the last dimension, PL/lookup.py:84,99)
 * in one kernel; mean and 1/sigma are recomputed from x.
 *   g = sum_r g_y[r];  g_x = rstd * (g*w - mean(g*w) - x^ * mean(g*w*x^));  g_w = sum_b g*x^;  g_b = sum_b g
 * x: [B, H]; ln_weight: [H] or null (no affine); g_y: [R, B, H] (R >= 1 gradients that are added up:
 * the repeats of the projection); g_x: [B, H]; part_weight, part_bias: [num_partials, H], one
 * partial sum per workgroup, to be added up by the caller, or both null.  H % 4 == 0, H <= 1024.
 * Replaces what autograd records for the LayerNorm of PL/lookup.py:99.
 */
int lffn_layer_norm_bwd_f32(const float *x, const float *ln_weight, float ln_eps, const float *g_y, float *g_x,
                            float *part_weight, float *part_bias, int64_t B, int64_t H, int64_t R,
                            int64_t num_partials, void *stream);

/*
 * lffn_layer_norm_bwd_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the partial sums go to a buffer
 * the library itself holds (a static device array of 4 MiB: 2 x 512 partials x 1024 columns of fp32,
 * present on every GPU the library runs on for the life of the process) and the column sums are
 * finished here, so the caller passes only inputs and outputs:
 *   g_x [B, H] as lffn_layer_norm_bwd_f32;  g_weight [H] = sum_b g * x^;  g_bias [H] = sum_b g
 * with min(512, max(1, ceil(B / 4))) partials, added up by lffn_sum_partials_f32 (chunks = 1): the
 * results are bit-identical to those two calls with that many partials.  No hipMalloc, hipFree or
 * other allocating call is made.  Rows wider than the buffer is sized for (H > 1024) return
 * LFFN_ERR_SCRATCH, whatever B, before anything is launched.  The first call on a device looks up the
 * buffer's device address (hipGetSymbolAddress, once per device): a caller that captures HIP graphs makes
 * one call per device outside any capture first (an empty batch, B = 0, is enough).  The buffer keeps the last call's contents; every call overwrites all it reads, so
 * nothing needs clearing.  All calls on one GPU share the one buffer: calls that overlap on a GPU
 * (two streams, two threads) race.  ln_weight may be null (no affine; g_weight is still written).
 * No counterpart in the reference (it has no entry point of this kind; the operator is the LayerNorm
 * backward autograd records for PL/lookup.py:99).
 */
int lffn_layer_norm_bwd_noalloc_f32(const float *x, const float *ln_weight, float ln_eps, const float *g_y,
                                    float *g_x, float *g_weight, float *g_bias, int64_t B, int64_t H, int64_t R,
                                    void *stream);

/*
 * The whole layer in one launch, for small batches without gradient (PL/lookup.py:99-108):
 *   out[b, :] = sum_t score[b,t] * tables[t, code[b,t], :] + out_bias (+ residual_in[b, :])
 * with (code, score) the 8-bit hash of 0.7 * BH4(LayerNorm(x)) + 0.3 * tile(LayerNorm(x)) +
 * proj_bias as lffn_ln_project_hash_f32 computes it (same kernel body: the codes and scores
 * are bit-identical), kept in LDS instead of written out.  One wavefront per token; each
 * token reads its own T rows from memory, so from a few hundred tokens on the two-kernel
 * form (lffn_ln_project_hash_f32 + lffn_lookup_gather_f32), which shares table slices
 * through LDS, is the faster one.
 * ln_weight/ln_bias: [H], both null for no LayerNorm; diag: [R, J, D]; proj_bias: [T*8] or
 * null; tables: [T, S, Do] with S >= 256; out_bias: [Do] or null; residual_in: [B, Do] or
 * null; out: [B, Do].  D in {256, 512, 1024}, T <= 512, Do % 4 == 0.
 * Replaces, in one call, LookupFFN.forward's LayerNorm, hash and gather (PL/lookup.py:99-108,
 * 120-130) for the diagonal BH4 projection (PL/lookup.py:29-39 with block_size 1).
 */
int lffn_lookup_ffn_fused_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                              const float *diag, const float *proj_bias, const float *tables,
                              const float *out_bias, const float *residual_in, float *out, int64_t B, int64_t H,
                              int64_t D, int64_t R, int64_t J, int64_t T, int64_t S, int64_t Do, float decay,
                              float residual, void *stream);

/*
 * The same call with the layer's parameters and sizes in a block the caller fills once per parameter set
 * (plain data: the library keeps no pointer to it after the call returns).  For callers whose per-call cost
 * matters at small batches: through a foreign-function interface every argument is converted on every call,
 * and at 256 tokens the kernel takes 7 microseconds.  Same checks, same kernel, same results.
 */
typedef struct lffn_fused_layer {
    const float *ln_weight, *ln_bias;       /* [H], both NULL for no LayerNorm */
    const float *diag;                      /* [R, J, D] */
    const float *proj_bias;                 /* [T*8] or NULL */
    const float *tables;                    /* [T, S, Do] */
    const float *out_bias;                  /* [Do] or NULL */
    int64_t H, D, R, J, T, S, Do;
    float ln_eps, decay, residual;
} lffn_fused_layer;
int lffn_lookup_ffn_fused_layer_f32(const lffn_fused_layer *layer, const float *x, const float *residual_in,
                                    float *out, int64_t B, void *stream);

/*
 * Weight gradient of the BH4 module with 64 x 64 blocks, all stages in one launch, in the
 * folded basis: for stage s = r * J + j and block n
 *   g_folded[s][n][o][i] += sum_b stage_grads[s][b][64n + o] * u_s[b][64n + i]
 * stage_grads: [R*J, B, D] as lffn_bh4_block_bwd_f32 writes it; u_s is x [B, H] (zero from
 * column H on) for j = 0, else stage_inputs[r][j-1] of lffn_bh4_block_hash_train_f32
 * ([R, J-1, B, D], may be null when J = 1); g_folded: [R*J, D/64, 64, 64], natural order,
 * accumulated into with atomics (zero it first for a plain result).
 * lffn_bh4_fold_mode_f32(mode 2) turns the sum into the gradient of the weights.  Replaces
 * the einsum "bno,bni->noi" autograd records for PL/bh4/kernel.py:32.
 */
int lffn_bh4_block_wgrad_f32(const float *stage_grads, const float *x, const float *stage_inputs, float *g_folded,
                             int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t block_size, void *stream);
/* The same with u_s = LayerNorm(x) for j = 0, formed on load from x, ln_weight, ln_bias [H] and the row_stats
 * [B, 2] lffn_ln_bh4_block_hash_train_f32 kept (PL/lookup.py:99 in front of PL/bh4/kernel.py:32). */
int lffn_ln_bh4_block_wgrad_f32(const float *stage_grads, const float *x, const float *ln_weight, const float *ln_bias,
                                const float *row_stats, const float *stage_inputs, float *g_folded, int64_t B,
                                int64_t H, int64_t D, int64_t R, int64_t J, int64_t block_size, void *stream);

/*
 * The tail of the BH4 module and the hash in one pass, for any block size:
 *   z[b, c] = decay * y[b, c] + residual * pad(x)[b, c % D] + bias[c],  c < T*k
 *   (code, score)[b, t] = code and score of z[b, t*k : (t+1)*k]   (as lffn_code_score_f32)
 * y: [B, ldy], the output of bh4 (ldy = R*D >= T*k); x: [B, H], H <= D, the projection's
 * input before zero padding; bias: [T*k] or NULL; codes: [B, T] int32; scores: [B, T].
 * z is not written.  Replaces the mix, slice and bias of BH4._forward (PL/lookup.py:36-37)
 * together with compute_code_score (PL/compute_code_score/kernel.py:22-55).
 */
int lffn_mix_code_score_f32(const float *y, const float *x, const float *bias, int32_t *codes,
                            float *scores, int64_t B, int64_t T, int64_t k, int64_t H, int64_t D,
                            int64_t ldy, float decay, float residual, void *stream);

/*
 * The whole hashing front-end of the layer in one pass over x, for block size 1
 * and 8-bit codes (PL/lookup.py:29-39,64-77 + PL/compute_code_score/kernel.py:43-55):
 *   y      = bh4_diag(x)                                   (as above)
 *   z      = decay * y + residual * tile(pad(x), R)        (PL/lookup.py:36)
 *   z      = z[:, :T*8] + proj_bias                        (PL/lookup.py:37)
 *   code   = sum_d (z[b,t,d] > 0) << (7-d)   int32         (compute_code_score/kernel.py:32-34,47-48)
 *   score  = sum_d |z| / prod_d (1 + exp(-2|z|))           (compute_code_score/kernel.py:51-53)
 * x: [B, H]; diag: [R, J, D]; proj_bias: [T*8] or NULL; z_out: [B, T*8] or NULL
 * (written only when non-NULL: the backward of the score needs it);
 * codes: [B, T] int32; scores: [B, T].  Requires T*8 <= R*D and D >= 8.
 * `residual` is passed separately from `decay` so that the caller decides how
 * 1 - decay is rounded (torch rounds the python double to fp32).
 */
int lffn_project_hash_f32(const float *x, const float *diag, const float *proj_bias,
                          float *z_out, int32_t *codes, float *scores,
                          int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                          float decay, float residual, void *stream);

/*
 * lffn_project_hash_f32 with the layer's LayerNorm (PL/lookup.py:84,99) applied to
 * each row of x on load: h = (x - mean) / sqrt(var + eps) * ln_weight + ln_bias over
 * the H valid columns (biased variance), then exactly as above on h.
 * ln_weight, ln_bias: [H].  Replaces nn.LayerNorm + BH4._forward + Hashing.forward +
 * compute_code_score_torch (PL/lookup.py:29-39,64-77,99) for block size 1, 8-bit codes.
 * The LayerNorm sums are formed in a different order than torch's kernel, so h (and
 * with it z) agrees with torch to rounding, not bit for bit.
 */
int lffn_ln_project_hash_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                             const float *diag, const float *proj_bias,
                             float *z_out, int32_t *codes, float *scores,
                             int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                             float decay, float residual, void *stream);

/*
 * The layer's inference path at many tokens without the [B, T] codes and scores in between: the
 * projection kernel writes the record stream that the four-lanes-per-token gather reads (the form
 * lffn_lookup_gather_ws_f32 packs for itself), and the gather runs from it.  Three calls:
 *
 * lffn_lookup_gather_records_plan: host-side query.  When this form is the one to use for a shape
 * (fp32 rows, S = 256, an even number of tables, enough tokens: the conditions under which
 * lffn_lookup_gather_workspace_bytes asks for a record stream, without the cost of the packing kernel)
 * it sets *tokens_per_workgroup (a multiple of 16 up to 2048: the tokens are spread evenly over the
 * workgroups of a slice), *record_stride (12-byte record slots per table pair: whole workgroups' worth,
 * a multiple of 16, fewer than B + 2048) and *bytes (the size of the stream: 6 * T * record_stride);
 * otherwise all three are 0 and the caller uses the other entry points.
 *
 * lffn_ln_project_hash_records_f32: lffn_ln_project_hash_f32 (ln_weight and ln_bias both NULL: no
 * LayerNorm, as lffn_project_hash_f32) with its codes and scores written as records for a gather of
 * tokens_per_workgroup tokens per workgroup (the plan's): 16-byte aligned device memory of `bytes`,
 * record_stride records of three words per table pair k:
 *   word 0: score of the pair's first table, word 1: score of its second, word 2: row of the first |
 *   row of the second << 8, where token b takes the tables in the order (2k, 2k+1) when bit 1 of b is
 *   clear and (2k+1, 2k) when it is set (the order its lanes read them in the gather kernel);
 *   a pair's records are kept in the order the gather's wavefronts copy them, which depends on
 *   tokens_per_workgroup: writer and reader must be given the same value.
 * Records of tokens from B up to record_stride are left as they are: the gather ignores them.  T even,
 * D >= 16.  The layout is private to these entry points: write it with these calls only.
 *
 * lffn_lookup_gather_records_f32: out[b,:] = residual[b,:] + bias + sum_t score[b,t] * tables[t, code[b,t], :]
 * from such a stream, with the tokens_per_workgroup it was written for and a record_stride of at least the
 * plan's (a multiple of 4).  Results are bit-identical to lffn_lookup_gather_ws_f32's for the same shape.
 * bias and residual may be NULL.
 *
 * lffn_lookup_gather_records_plan_rows / lffn_lookup_gather_records_rows: the same two calls for any
 * row format (row_format 0 fp32, 1 bfloat16, 2 half; tables typed accordingly).  16-bit rows run 1024
 * tokens per workgroup over 64-column slices, fp32 sums.  The records do not depend on the row format.
 *
 * Replaces the same reference code as lffn_ln_project_hash_f32 followed by lffn_lookup_gather_f32
 * (PL/lookup.py:29-39,64-77,99 and 120-130,108); with half rows, the gather of
 * PL/gather/cuda/extension/gather_kernel_fp16.cu:6-62 (fp32 sums instead of its half sums).
 */
int lffn_lookup_gather_records_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t *tokens_per_workgroup,
                                    int64_t *record_stride, int64_t *bytes);
int lffn_ln_project_hash_records_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                     const float *diag, const float *proj_bias, uint32_t *records,
                                     int64_t record_stride, int32_t tokens_per_workgroup, int64_t B, int64_t H,
                                     int64_t D, int64_t R, int64_t J, int64_t T, float decay, float residual,
                                     void *stream);
/* lffn_ln_bh4_block_hash_f32 (below) with its codes and scores written as records in the same way. */
int lffn_ln_bh4_block_hash_records_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                       const float *w_folded, const float *proj_bias, uint32_t *records,
                                       int64_t record_stride, int32_t tokens_per_workgroup, int64_t B, int64_t H,
                                       int64_t D, int64_t R, int64_t J, int64_t T, int64_t block_size, float decay,
                                       float residual, void *stream);
int lffn_lookup_gather_records_f32(const uint32_t *records, int64_t record_stride, const float *tables,
                                   const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                   int64_t S, int64_t Do, int32_t tokens_per_workgroup, void *stream);
int lffn_lookup_gather_records_plan_rows(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format,
                                         int32_t *tokens_per_workgroup, int64_t *record_stride, int64_t *bytes);
int lffn_lookup_gather_records_rows(const uint32_t *records, int64_t record_stride, const void *tables,
                                    const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                    int64_t S, int64_t Do, int32_t row_format, int32_t tokens_per_workgroup,
                                    void *stream);

/* ---------------------------------------------------------------- code + score */

/*
 * Per (token, table) n < N = B*T, over k consecutive values of z (1 <= k <= 24):
 *   codes[n]  = sum_d (z[n,d] > 0) << (k-1-d)      (MSB first, strict >)
 *   scores[n] = sum_d |z[n,d]| / prod_d (1 + exp(-2 |z[n,d]|))   (d ascending)
 * Replaces ccs_cpu.compute_code_score (PL/compute_code_score/torch_extension.cc:14-42)
 * and the eight torch ops of compute_code_score_torch (PL/compute_code_score/kernel.py:43-55).
 */
int lffn_code_score_f32(const float *z, int32_t *codes, float *scores,
                        int64_t N, int64_t k, void *stream);

/*
 * g_z[n,j] = g_score[n] * d score[n] / d z[n,j]
 *          = g_score[n] * sgn(z_j) * (1 + S * 2 e_j / (1 + e_j)) / P,
 *   e_j = exp(-2|z_j|), S = sum|z|, P = prod(1 + e).   sgn(0) = 0 as in torch.
 * The reference leaves this to autograd over PL/compute_code_score/kernel.py:51-53
 * (its ComputeCodeScore.backward raises NotImplementedError, kernel.py:63-65).
 */
int lffn_code_score_bwd_f32(const float *z, const float *g_score, float *g_z,
                            int64_t N, int64_t k, void *stream);

/* ---------------------------------------------------------------- gather-add */

/*
 * out[b,:] = sum_i w[b,i] * src[idx[b,i],:], fp32 accumulation, i ascending.
 * idx: [B, I] int32; src: [source_size, Dv]; w: [B, I]; out: [B, Dv]; Dv % 64 == 0.
 * Replaces gather_add.weighted_vector_gather_add_fp32
 * (PL/gather/cuda/extension/gather_fp32.cu:6-36, kernel gather_kernel_fp32.cu:3-47).
 */
int lffn_gather_add_f32(const int32_t *idx, const float *src, const float *w, float *out,
                        int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream);

/*
 * Same with rows stored as bfloat16 (raw 16-bit patterns) and fp32 weights,
 * accumulation and output.  Takes the place of the reference's fp16 variant
 * (gather_fp16.cu:9-39), which stores and accumulates in fp16.
 */
int lffn_gather_add_bf16(const int32_t *idx, const uint16_t *src, const float *w, float *out,
                         int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream);

/*
 * The same with half rows (IEEE binary16), fp32 sums.  Replaces
 * gather_add.weighted_vector_gather_add_fp16 (PL/gather/cuda/extension/gather_kernel_fp16.cu:6-62),
 * which multiplies and accumulates in half (__hfma2, :56-57): the results here are the fp32 sums of
 * the same products, i.e. closer to the exact sum than the reference's, not bit-identical to it.
 */
int lffn_gather_add_f16(const int32_t *idx, const uint16_t *src, const float *w, float *out,
                        int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream);

/*
 * The gather as LookupFFN.gather issues it (PL/lookup.py:120-130): one index per
 * table, idx[b,t] = code[b,t] + t*S folded in, optional bias (PL/lookup.py:108):
 *   out[b,:] = bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
 * code: [B, T] int32; score: [B, T]; tables: [T, S, Do]; bias: [Do] or NULL;
 * out: [B, Do].  S a power of two, Do % 64 == 0.  Table-major: a slice of each
 * table is staged in LDS and consumed by a block of tokens.
 */
int lffn_lookup_gather_f32(const int32_t *code, const float *score, const float *tables,
                           const float *bias, float *out,
                           int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);

/* bfloat16 tables, fp32 accumulate; otherwise as lffn_lookup_gather_f32. */
int lffn_lookup_gather_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                            const float *bias, float *out,
                            int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);

/*
 * lffn_lookup_gather_{f32,bf16} with a residual added to the result:
 *   out[b,:] = residual[b,:] + bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
 * residual: [B, Do] fp32 or NULL; it may be the output buffer itself (every element is read
 * and then written by the same lane).  Replaces, in addition, the residual add of the
 * encoder layer around the FFN, "self.dropout(self.FFN(x)) + x" (PL/layer.py:77), where
 * dropout is the identity (eval mode or p == 0).
 */
int lffn_lookup_gather_residual_f32(const int32_t *code, const float *score, const float *tables,
                                    const float *bias, const float *residual, float *out,
                                    int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);
int lffn_lookup_gather_residual_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                     const float *bias, const float *residual, float *out,
                                     int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);

/*
 * The same gather with a caller-provided workspace, which two forms use:
 *  - many tokens, S = 256, an even number of tables (16384 tokens at the RoBERTa-base tables): the
 *    four-lanes-per-token kernel (fp32, bfloat16 and half rows; 128-byte column slices = 32 fp32 or
 *    64 16-bit columns).  A small kernel first packs the (code, score) pairs
 *    into a stream of 12-byte records in the workspace (6 bytes per (token, table)), one row of
 *    records per table pair, which the gather kernel copies into LDS a pair ahead; the gather
 *    kernel walks 128-byte column slices, two tables per LDS buffer, 1024 to 2048 tokens per
 *    workgroup.  Within a table pair a token adds the two rows in an order that depends on its
 *    index (bit 1), so results equal lffn_lookup_gather_f32's up to the association of the fp32
 *    sums; they are reproducible from run to run;
 *  - a few thousand tokens: too few (token tile, column slice) units to fill the chip at the tile
 *    sizes that make staging tables in LDS pay.  Several workgroups then share a unit, each adding
 *    a range of the tables into its own partial output in the workspace, and a second kernel adds
 *    the partials, in table order, with bias and residual (reproducible, and equal to the one-part
 *    kernel's up to the association of the fp32 sums).
 * lffn_lookup_gather_workspace_bytes sets *bytes to the workspace that pays for a shape, or to 0
 * when the plain entry points are as fast (very few tokens); row_format is 0 (fp32 rows), 1
 * (bfloat16) or 2 (half).  With a null or too small workspace the _ws entry points behave exactly
 * like lffn_lookup_gather_residual_* (half rows: the token-major kernel).  lffn_lookup_gather_ws_plan
 * reports which kernel the _ws entry points run for a shape and a workspace size: the return value
 * is the tokens per workgroup (0: token-major) and *form (may be NULL) receives 0 (token-major), 1 or
 * 2 (tables per LDS buffer, as lffn_lookup_gather_plan), 3 (four lanes per token, record stream in
 * the workspace) or 4 (table split, partial outputs in the workspace); a batch taken in pieces
 * reports the form of a piece.  Pure host functions.
 * lffn_lookup_gather_ws_f16: half rows (the row format of the reference's reduced-precision gather,
 * gather_kernel_fp16.cu:6-62, with fp32 sums instead of its half sums): form 3 or token-major.  The workspace is scratch: 16-byte
 * aligned device memory, contents undefined afterwards; calls that share one must be ordered on
 * the stream.  residual may be null.
 * Same replacement as lffn_lookup_gather_f32 (PL/lookup.py:120-130, 108).
 */
int lffn_lookup_gather_workspace_bytes(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format, int64_t *bytes);
int lffn_lookup_gather_ws_f32(const int32_t *code, const float *score, const float *tables, const float *bias,
                              const float *residual, float *out, void *workspace, int64_t workspace_bytes,
                              int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);
int lffn_lookup_gather_ws_bf16(const int32_t *code, const float *score, const uint16_t *tables, const float *bias,
                               const float *residual, float *out, void *workspace, int64_t workspace_bytes,
                               int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);
int lffn_lookup_gather_ws_f16(const int32_t *code, const float *score, const uint16_t *tables, const float *bias,
                              const float *residual, float *out, void *workspace, int64_t workspace_bytes,
                              int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);
int lffn_lookup_gather_ws_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format,
                               int64_t workspace_bytes, int32_t *form);

/*
 * Which kernel lffn_lookup_gather_{f32,bf16} runs for a shape.  Returns the number
 * of tokens whose accumulators one workgroup keeps in registers while it walks the
 * tables through LDS, or 0 when the token-major kernel is used (small batches,
 * S > 256); *tables_per_buffer (may be NULL) receives 0 (token-major), 1 (256-byte
 * column slices, one table per LDS buffer) or 2 (128-byte slices, two tables per
 * buffer).  The workspace entry points may run forms this function does not report
 * (3, the four-lanes-per-token kernel, and the table split): lffn_lookup_gather_ws_plan
 * reports those.  Pure host function, no GPU work; negative on bad arguments.
 * No counterpart in the reference (its gather has one kernel, gather_fp32.cu:6-36).
 */
int lffn_lookup_gather_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t bf16,
                            int32_t *tables_per_buffer);

/*
 * lffn_lookup_gather_{f32,bf16} with the kernel named by the caller instead of
 * chosen by lffn_lookup_gather_plan (for tuning, and so that every built kernel
 * can be tested on any shape): tables_per_buffer 0, 1 or 2 as reported by the plan
 * function; tokens_per_workgroup a multiple of 64 (one table per buffer: 256, 512,
 * 832, 1024; bf16 256, 512) or of 128 (two tables per buffer: 512, 1024, 1664, 2048;
 * bf16 512, 1024), ignored for 0.  LFFN_ERR_UNSUPPORTED if that kernel is not built or
 * the shape does not meet its conditions (S <= 256, Do a multiple of the slice width).
 * lffn_lookup_gather_ws_planned_f32 also takes residual and a workspace and with them
 * form 3, the four-lanes-per-token kernel (tokens_per_workgroup any multiple of 16
 * from 784 to 2048: a workgroup takes its tokens in passes of 256, 4 to 8 of them, and
 * wavefronts whose share of the last pass lies beyond the tile leave it out; S = 256, T
 * even, Do a multiple of 32; the workspace must hold the record stream, 6 * T * (B + 2048)
 * bytes, or the call is refused with LFFN_ERR_UNSUPPORTED).
 * lffn_lookup_gather_ws_planned_rows is the same for any row format (row_format 0 fp32,
 * 1 bfloat16, 2 half; tables typed accordingly): 16-bit rows take form 3 with 784 to 1024
 * tokens per workgroup and Do a multiple of 64; half rows take forms 0 and 3 only.
 * No counterpart in the reference.
 */
int lffn_lookup_gather_planned_f32(const int32_t *code, const float *score, const float *tables,
                                   const float *bias, float *out,
                                   int64_t B, int64_t T, int64_t S, int64_t Do,
                                   int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream);
int lffn_lookup_gather_ws_planned_f32(const int32_t *code, const float *score, const float *tables,
                                      const float *bias, const float *residual, float *out, void *workspace,
                                      int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                      int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream);
int lffn_lookup_gather_planned_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                    const float *bias, float *out,
                                    int64_t B, int64_t T, int64_t S, int64_t Do,
                                    int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream);
int lffn_lookup_gather_ws_planned_rows(const int32_t *code, const float *score, const void *tables,
                                       const float *bias, const float *residual, float *out, void *workspace,
                                       int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                       int32_t row_format, int32_t tables_per_buffer, int32_t tokens_per_workgroup,
                                       void *stream);

/*
 * out[b,i] = <g[b,:], src[idx[b,i],:]>   (gradient w.r.t. the weights).
 * g: [B, Dv]; src: [source_size, Dv]; out: [B, I].
 * Replaces gather_add.indexed_inner_product_fp32 (gather_fp32.cu:69-98,
 * kernel gather_kernel_fp32.cu:94-157).
 */
int lffn_indexed_inner_product_f32(const int32_t *idx, const float *g, const float *src, float *out,
                                   int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream);

/*
 * out[idx[b,i],:] += w[b,i] * g[b,:]     (gradient w.r.t. the table rows).
 * g: [B, Dv]; w: [B, I]; out: [out_size, Dv], ACCUMULATED INTO: zero it first
 * for a plain gradient (the reference pre-zeroes it in Python,
 * PL/gather/cuda/kernel.py:162).  fp32 atomics: the order of additions, and so the
 * last bits of the result, vary from run to run, as in the reference
 * (gather_kernel_fp32.cu:88).
 * Replaces gather_add.weighted_vector_scatter_add_fp32 (gather_fp32.cu:38-67).
 */
int lffn_scatter_add_f32(const int32_t *idx, const float *g, const float *w, float *out,
                         int64_t B, int64_t I, int64_t out_size, int64_t Dv, void *stream);

/*
 * The two backward operators with half (IEEE binary16) inputs, the rest of the reference's
 * reduced-precision trio beside lffn_gather_add_f16:
 *   lffn_indexed_inner_product_f16: g [B, Dv] and src [source_size, Dv] half, out [B, I] fp32: every
 *     product exact, the sum fp32.  Replaces gather_add.indexed_inner_product_fp16
 *     (PL/gather/cuda/extension/gather_kernel_fp16.cu:121-184), which rounds each product to half
 *     (__hmul, :165) before its fp32 sum and the result to half (:181).
 *   lffn_scatter_add_f16: g [B, Dv] half, w [B, I] fp32, out [out_size, Dv] fp32, ACCUMULATED INTO
 *     with fp32 atomics.  Replaces gather_add.weighted_vector_scatter_add_fp16 (:64-119), which
 *     multiplies and accumulates in half (__hmul2 and a half2 atomicAdd, :112-115).
 * The caller rounds the fp32 results to half where it wants the reference's dtypes; they are the
 * fp32 sums of the exact products, closer to the exact result than the reference's, not
 * bit-identical to it.
 */
int lffn_indexed_inner_product_f16(const int32_t *idx, const uint16_t *g, const uint16_t *src, float *out,
                                   int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream);
int lffn_scatter_add_f16(const int32_t *idx, const uint16_t *g, const float *w, float *out,
                         int64_t B, int64_t I, int64_t out_size, int64_t Dv, void *stream);

/*
 * The scatter-add as the layer's backward issues it: table-local codes, the
 * gradient of the whole [T, S, Do] table array in one call,
 *   grad_tables[t, s, :] (+)= sum_{b : (code[b,t] & (S-1)) == s} score[b,t] * g[b,:]
 * code: [B, T] int32; score: [B, T]; g: [B, Do]; grad_tables: [T, S, Do].
 * accumulate == 0: grad_tables is overwritten (it needs no zero-fill); otherwise
 * added to.  For S <= 256 the sums are formed in LDS (no global atomics); the
 * order of additions is still free, as with the reference's atomics.
 * Replaces WeightedVectorGatherAdd.backward's weighted_vector_scatter_add call
 * (PL/gather/cuda/kernel.py:200) together with the index offset of PL/lookup.py:126.
 */
int lffn_lookup_scatter_f32(const int32_t *code, const float *score, const float *g, float *grad_tables,
                            int64_t B, int64_t T, int64_t S, int64_t Do, int32_t accumulate, void *stream);

/*
 * The same sums without atomics on the accumulators, through a caller-provided workspace:
 * the inputs are transposed / copied slice-major, each table's tokens are sorted by code
 * (stable counting sort, (token, score) pairs, buckets padded to multiples of eight), and a
 * last kernel walks the sorted lists and adds the rows of g in registers; rows of
 * grad_tables are written with plain stores and the order of additions is fixed (token order
 * inside a code), so results are reproducible from run to run, unlike the reference's
 * atomics.  Tokens are taken 16384 at a time (the workspace is sized for one such chunk).
 * About twice as fast as lffn_lookup_scatter_f32 at 16384 tokens x 128 tables x 768
 * columns; slower below about 4e8 multiply-adds (B * T * Do).
 * lffn_lookup_scatter_workspace_bytes sets *bytes to the workspace this form needs for a
 * shape, or to 0 when the form does not cover it (S > 512, Do % 32 != 0, B == 0 or T == 0):
 * lffn_lookup_scatter_f32 covers those.  workspace: device memory, 16-byte aligned, at
 * least that many bytes; its contents are scratch.  Same replacement as
 * lffn_lookup_scatter_f32 (PL/gather/cuda/kernel.py:200, PL/lookup.py:126).
 */
int lffn_lookup_scatter_workspace_bytes(int64_t B, int64_t T, int64_t S, int64_t Do, int64_t *bytes);
int lffn_lookup_scatter_sorted_f32(const int32_t *code, const float *score, const float *g, float *grad_tables,
                                   void *workspace, int64_t workspace_bytes, int64_t B, int64_t T, int64_t S,
                                   int64_t Do, int32_t accumulate, void *stream);

/*
 * Both gradients of the layer's gather in one call, sharing one workspace (the size
 * lffn_lookup_scatter_workspace_bytes reports; the call is refused where that is 0):
 *   grad_score[b, t]     = < g[b, :], tables[t, code[b,t] & (S-1), :] >                       overwritten
 *   grad_tables[t, s, :] = sum over the tokens b with code[b,t] = s of score[b,t] * g[b, :]   overwritten,
 *                                                                     or added to when accumulate != 0
 * i.e. lffn_lookup_inner_f32 and lffn_lookup_scatter_sorted_f32 with their common work done once: per
 * chunk of 16384 tokens one kernel transposes code and score and copies g slice-major, and the
 * score-gradient kernel and the sorted scatter both read that copy (for the score gradient, a token
 * tile's slice of g is then contiguous instead of one 128-byte line per row).  Results are bit-identical
 * to the two separate calls.  grad_score or grad_tables may be NULL (that gradient is not computed; tables
 * is needed for the former only, score for the latter only).  Do % 64 == 0, S <= 512.
 * Replaces WeightedVectorGatherAdd.backward (PL/gather/cuda/kernel.py:190-202: indexed_inner_product +
 * weighted_vector_scatter_add, kernels gather_kernel_fp32.cu:49-157) with the index offset of
 * PL/lookup.py:126.
 */
int lffn_lookup_backward_f32(const int32_t *code, const float *score, const float *g, const float *tables,
                             float *grad_score, float *grad_tables, void *workspace, int64_t workspace_bytes,
                             int64_t B, int64_t T, int64_t S, int64_t Do, int32_t accumulate, void *stream);

/*
 * The indexed inner product as the layer's backward issues it: table-local codes,
 *   grad_score[b, t] = < g[b, :], tables[t, code[b,t] & (S-1), :] >
 * code: [B, T] int32; g: [B, Do]; tables: [T, S, Do] fp32; grad_score: [B, T],
 * overwritten (it needs no zero-fill).  For S <= 256 the table slices are staged
 * in LDS.  At the layer's shapes (S = 256, T even, Do a multiple of 32, a few thousand
 * tokens or more) every (token, table) sum has one owner that walks the column slices
 * itself: no atomics, a fixed order of additions, results bit-identical from run to
 * run.  The other shapes (S < 256, odd T, small batches) combine the partial sums of
 * the 64-column slices of a row with global atomics, in no fixed order (as the partial
 * sums of the reference's kernel are, PL/gather/cuda/extension/gather_kernel_fp32.cu:141).
 * Replaces WeightedVectorGatherAdd.backward's indexed_inner_product call
 * (PL/gather/cuda/kernel.py:199) together with the index offset of PL/lookup.py:126.
 */
int lffn_lookup_inner_f32(const int32_t *code, const float *g, const float *tables, float *grad_score,
                          int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LOOKUPFFN_HIP_H */
