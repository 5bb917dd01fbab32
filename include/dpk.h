/*
 * dpk.h - C ABI of libdpsgd_hip.so: the DP-SGD hot path (per-sample gradients,
 * ghost-clipping per-sample norms, clip + accumulate + Gaussian noise) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions shared by every entry point
 *   - Plain C: pointers, sizes, scalars. No C++ or torch types cross the boundary.
 *   - Every pointer is a DEVICE pointer unless its comment says "host".
 *   - All tensors are dense, row-major, batch first; float tensors are 16-byte
 *     aligned (bf16 too), id tensors are int64 and 8-byte aligned.
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *     null stream) and the call returns without waiting for it.
 *   - The library never allocates or frees device memory: the caller passes
 *     outputs and, where an entry point needs scratch, a workspace whose size
 *     the matching dpk_*_workspace_bytes() query returns.
 *   - Return value: DPK_OK (0) or a negative DPK_E_* code; dpk_last_error()
 *     then holds a message for the calling thread. Nothing is launched when an
 *     argument check fails. n == 0 returns DPK_OK without launching.
 *   - `scale` multiplies the backprops on the fly. The reference multiplies the
 *     backprops tensor by the batch size for a mean-reduced loss in a pass of
 *     its own (opacus/grad_sample/grad_sample_module.py:402-406); pass 1.0f for
 *     a sum-reduced loss.
 *   - Reductions use a fixed order: the same inputs give the same bits.
 */
#ifndef DPK_H
#define DPK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* dpk_stream_t;

enum dpk_status {
  DPK_OK = 0,
  DPK_E_SHAPE = -1,     /* a size is negative, zero where it may not be, or too large */
  DPK_E_DTYPE = -2,     /* dtype code not supported by this entry point */
  DPK_E_ALIGN = -3,     /* pointer not aligned as the conventions above require */
  DPK_E_LAUNCH = -4,    /* the HIP runtime refused the launch */
  DPK_E_WORKSPACE = -5, /* workspace missing or smaller than the query says */
  DPK_E_ARG = -6        /* NULL where a pointer is required, or a bad flag */
};

enum dpk_dtype { DPK_F32 = 0, DPK_BF16 = 1 };

/* Two entry points choose between two kernels by cost. The caller may name the one it wants
 * instead (tests drive both on one shape); every other caller passes the AUTO value. The
 * library reads no environment variable and keeps no setting between calls. */
enum dpk_linear_tile { DPK_TILE_AUTO = 0, DPK_TILE_128 = 128, DPK_TILE_256 = 256 };
enum dpk_ghost_route { DPK_ROUTE_AUTO = 0, DPK_ROUTE_GRAM = 1, DPK_ROUTE_DIRECT = 2 };

#define DPK_MULTI_MAX 48 /* tensors per call of the *_multi entry points */

/* ABI revision; bumped when a signature changes. */
int dpk_abi_version(void);
/* Message of the last failing call on this host thread ("" if none). */
const char* dpk_last_error(void);
/* Number of compute units of the current device (host query, cached per device). */
int dpk_device_cus(void);

/* ------------------------------------------------------------------------- *
 * Per-sample gradients of nn.Linear
 * replaces opacus/grad_sample/linear.py:29-51 (compute_linear_grad_sample)
 * ------------------------------------------------------------------------- */

/* gs[n,i,j] = scale * sum_t b[n,t,i] * a[n,t,j]          (linear.py:47)
 * b: [n,T,out], a: [n,T,in] of `in_dtype`; gs: [n,out,in] of `gs_dtype`.
 * sumsq (nullable, float[n]) receives sum_ij gs[n,i,j]^2 of the values as
 * written (fp32 accumulators before any down-cast), so that the optimizer's
 * norm pass (optimizers/optimizer.py:444-446) need not re-read gs.
 * T == 1 takes a store-bound outer-product kernel; T > 1 an MFMA kernel.
 * gs may be NULL when sumsq is given: only the squared norms are formed then
 * (the gradient tiles never leave the registers).
 * tile: DPK_TILE_AUTO, or the block tile of the bf16 T > 1 kernel for shapes that kernel
 * takes (ignored by the others).
 * ws is needed only when sumsq != NULL. */
size_t dpk_linear_gs_workspace_bytes(int64_t n, int64_t T, int64_t out, int64_t in);
int dpk_linear_gs(const void* b, const void* a, int in_dtype, void* gs, int gs_dtype,
                  float* sumsq, int64_t n, int64_t T, int64_t out, int64_t in, float scale,
                  int tile, void* ws, size_t ws_bytes, dpk_stream_t stream);

/* out[i,j] = scale * sum_s coef[s] * sum_t b[s,t,i] * a[s,t,j]
 * The clip-weighted sum of a Linear layer's per-sample gradients from the activations and
 * backprops of one backward pass: what the reference's second backward pass of
 * sum_s coef[s] * loss[s] leaves in weight.grad (utils/fast_gradient_clipping_utils.py:193-201,
 * DPTensorFastGradientClipping.backward), without that pass and without a weighted copy of
 * either operand. b: [n,T,out], a: [n,T,in] of `in_dtype`; coef: float[n] (non-negative);
 * out: [out,in] of `out_dtype`.
 * bf16 operands with T % 32 == 0, out and in multiples of 8 above 64, n % pieces == 0 and
 * 16-byte aligned tensors: one bf16 MFMA contraction over samples and positions at once, the
 * accumulators rescaled by coef[s-1]/coef[s] where sample s begins, so no per-sample product is
 * stored anywhere. No rescaling multiplies by more than 2^40: a coefficient below 2^-40 of the
 * one before it (an exact zero) counts as that fraction of it, one below 1e-30 as 1e-30.
 * pieces > 1 cuts the samples into that many runs (more blocks for a layer with few output
 * tiles) whose fp32 sums go through the workspace and are added by a second kernel.
 * fp32 operands with T % 16 == 0, out and in multiples of 4 (in of 8 for a bf16 result) above 64:
 * the same on the fp32 MFMA with operands loaded straight into LDS.
 * Everything else (any T, any feature sizes, any alignment): the fp32 MFMA contraction over all
 * n*T rows with the rows of b multiplied by their coefficients on the way into LDS (bf16 rows
 * are widened first); pieces are then runs of rows.
 * ws: dpk_linear_weighted_sum_workspace_bytes bytes, 256-byte aligned. */
size_t dpk_linear_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t out_features, int64_t in_features,
                                               int in_dtype, int pieces);
int dpk_linear_weighted_sum(const void* b, const void* a, int in_dtype, const float* coef, void* out,
                            int out_dtype, int64_t n, int64_t T, int64_t out_features,
                            int64_t in_features, float scale, int pieces, void* ws, size_t ws_bytes,
                            dpk_stream_t stream);

/* dpk_linear_weighted_sum for several layers in one call: the block tiles of all layers are
 * one pool of work, so the GPU stays full across layers whose own tile count is not a
 * multiple of what it holds at once (C5: 29 layers, 37 launches -> one). A pool with too few
 * tiles to fill the GPU (a two-layer MLP) has every layer's samples cut into 2, 4 or 8 pieces
 * (dividing every n), whose fp32 sums go to the workspace and are added by one more launch;
 * dpk_linear_weighted_sum_multi_workspace_bytes says how much the same table will need (0: one
 * piece). ws must be 256-byte aligned. Per-layer requirements as above, all results of
 * `out_dtype`. `layers` is a host array of any length (32 layers per launch). */
typedef struct dpk_wsum_layer {
  const void* b;     /* [n,T,out] bf16 */
  const void* a;     /* [n,T,in] bf16 */
  const float* coef; /* [n] */
  void* out_sum;     /* [out,in] */
  int64_t n, T, out, in;
  float scale;
} dpk_wsum_layer;
size_t dpk_linear_weighted_sum_multi_workspace_bytes(const dpk_wsum_layer* layers /*host*/, int count);
int dpk_linear_weighted_sum_multi(const dpk_wsum_layer* layers /*host*/, int count, int in_dtype, int out_dtype,
                                  void* ws, size_t ws_bytes, dpk_stream_t stream);

/* gs_bias[n,k] = scale * sum_t b[n,t,k]                   (linear.py:50)
 * sumsq (nullable, float[n]) receives sum_k gs_bias[n,k]^2 of the values as stored, for
 * the optimizer's norm pass (optimizers/optimizer.py:444-446). */
int dpk_linear_bias_gs(const void* b, int in_dtype, void* gs_bias, int gs_dtype, float* sumsq,
                       int64_t n, int64_t T, int64_t out, float scale, dpk_stream_t stream);

/* out[k] = scale * sum_s coef[s] * sum_t b[s,t,k]: the clip-weighted sum of the per-sample bias
 * gradients (linear.py:50), what the second backward pass leaves in bias.grad
 * (utils/fast_gradient_clipping_utils.py:193-201). One pass over b in 256 chunks of rows whose
 * fp32 sums are added in a fixed order. b: [n,T,out] of `in_dtype`; out: [out] of `out_dtype`.
 * ws: dpk_linear_bias_weighted_sum_workspace_bytes bytes, 256-byte aligned. */
size_t dpk_linear_bias_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t out);
int dpk_linear_bias_weighted_sum(const void* b, int in_dtype, const float* coef, void* out_sum, int out_dtype,
                                 int64_t n, int64_t T, int64_t out, float scale, void* ws, size_t ws_bytes,
                                 dpk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Ghost-clipping per-sample norms of nn.Linear
 * replaces opacus/grad_sample/linear.py:54-93 (compute_linear_norm_sample)
 * ------------------------------------------------------------------------- */

/* norm_w[n] = sqrt(max(0, sum_{t,t'} (b_t.b_t')(a_t.a_t')))   (linear.py:83-89)
 * norm_b[n] = sqrt(max(0, sum_{t,t'} b_t.b_t'))              (linear.py:91-92)
 * For T == 1 these are the closed forms of linear.py:71-79.
 * Either output may be NULL (parameter without requires_grad). Outputs are
 * fp32 whatever `dtype` the inputs have. The T x T Gram matrices are never
 * written to memory: matching tiles of b b^T and a a^T are formed in MFMA
 * accumulators, multiplied and reduced in registers. A layer thin enough that
 * T * in * out is below the work of the two Grams has the tiles of
 * sum_t b_t a_t^T formed and squared instead (never stored either); the
 * results agree to rounding. route: DPK_ROUTE_AUTO (by cost), or the route to
 * take. The workspace query covers either route. ws must be 256-byte aligned. */
size_t dpk_linear_ghost_norm_workspace_bytes(int64_t n, int64_t T, int64_t out, int64_t in);
int dpk_linear_ghost_norm(const void* b, const void* a, int dtype, float* norm_w, float* norm_b,
                          int64_t n, int64_t T, int64_t out, int64_t in, float scale, int route,
                          void* ws, size_t ws_bytes, dpk_stream_t stream);

/* The ghost norms of several Linear layers in one call: all layers of a backward pass, say,
 * once their backprops exist (linear.py:54-93 for each of them). One layer's launch is a few
 * hundred tile pairs, which leaves the device's last round of blocks mostly empty; pooled, the
 * tile pairs of all layers fill the rounds, longest first. Layers share the batch size n and
 * the dtype; each has its own T, sizes, outputs (either may be NULL) and scale. A layer the
 * pooled kernel does not take (T == 1, a thin layer, odd feature sizes) is served as by
 * dpk_linear_ghost_norm inside the same call. Results equal dpk_linear_ghost_norm's to
 * rounding. `layers` is a host array of at most DPK_GHOST_MULTI_MAX entries; ws 256-byte aligned. */
#define DPK_GHOST_MULTI_MAX 256
typedef struct dpk_ghost_layer {
  const void* b;  /* [n,T,out] */
  const void* a;  /* [n,T,in] */
  float* norm_w;  /* [n] or NULL */
  float* norm_b;  /* [n] or NULL */
  int64_t T, out, in;
  float scale;
} dpk_ghost_layer;
size_t dpk_linear_ghost_norm_multi_workspace_bytes(const dpk_ghost_layer* layers /*host*/, int count, int64_t n);
int dpk_linear_ghost_norm_multi(const dpk_ghost_layer* layers /*host*/, int count, int dtype, int64_t n,
                                void* ws, size_t ws_bytes, dpk_stream_t stream);

/* dpk_linear_ghost_norm for callers that cannot allocate device memory or pass a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. It has no counterpart in the reference. Same arguments, results and kernels;
 * the partial sums go to a buffer of DPK_STATIC_SCRATCH_BYTES that is part of the library's
 * device image (every GPU the library runs on holds it until the process ends). The call
 * allocates and frees nothing; the first call on a device looks up the buffer's address.
 * Shapes whose dpk_linear_ghost_norm_workspace_bytes() exceeds the buffer are refused with
 * DPK_E_SHAPE before anything is launched. All calls on one GPU share the one buffer:
 * calls that may overlap in time on a GPU (different streams, different host threads)
 * race on it and must be serialised by the caller. */
#define DPK_STATIC_SCRATCH_BYTES (8u << 20)
int dpk_linear_ghost_norm_static(const void* b, const void* a, int dtype, float* norm_w,
                                 float* norm_b, int64_t n, int64_t T, int64_t out, int64_t in,
                                 float scale, int route, dpk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Per-sample gradients of nn.Conv2d (nn.Conv1d as a height-one image) and nn.Conv3d
 * replaces opacus/grad_sample/conv.py:28-119 (compute_conv_grad_sample, the
 * Conv2d branch) together with opacus/utils/tensor_utils.py:116-172 (unfold2d)
 * ------------------------------------------------------------------------- */

/* gs[n,o,c,kh,kw] = scale * sum_{oh,ow} b[n,o,oh,ow] *
 *        xpad[n, g(o)*C/groups + c, oh*sh + kh*dh, ow*sw + kw*dw]
 * x: [n,C,H,W], b: [n,O,OH,OW] (OH, OW follow from the geometry exactly as
 * unfold2d computes H_effective/W_effective), gs: [n,O,C/groups,KH,KW].
 * The unfolded activation matrix is never materialised. Padding is given per
 * side so that padding="same" (asymmetric, tensor_utils.py:128-134) is
 * expressible. sumsq as for dpk_linear_gs; gs may be NULL when sumsq is given (norms only:
 * the gradient tiles are formed and squared, never stored).
 * Workspace: block sums for sumsq and, for a layer with few and long blocks (few kernel
 * elements, many output positions: a network's first convolution), room for the pieces
 * into which the contraction over the output positions is then cut. Q = OH * OW (times OD)
 * tells the query how long that contraction is; Q = 0 asks for the block sums only, and a
 * call that finds no room for the pieces runs unsplit. */
size_t dpk_conv2d_gs_workspace_bytes(int64_t n, int64_t C, int64_t O, int64_t KH, int64_t KW,
                                     int64_t groups, int64_t Q);
int dpk_conv2d_gs(const void* x, const void* b, int in_dtype, void* gs, int gs_dtype, float* sumsq,
                  int64_t n, int64_t C, int64_t H, int64_t W, int64_t O, int64_t KH, int64_t KW,
                  int64_t sh, int64_t sw, int64_t ph_lo, int64_t ph_hi, int64_t pw_lo,
                  int64_t pw_hi, int64_t dh, int64_t dw, int64_t groups, float scale, void* ws,
                  size_t ws_bytes, dpk_stream_t stream);

/* The same for nn.Conv3d (conv.py:89-96 with unfold3d, tensor_utils.py:175-279):
 * x: [n,C,D,H,W], b: [n,O,OD,OH,OW], gs: [n,O,C/groups,KD,KH,KW]. kernel, stride,
 * pad_lo, pad_hi, dilation: host arrays of three values in (depth, height, width) order. */
size_t dpk_conv3d_gs_workspace_bytes(int64_t n, int64_t C, int64_t O, int64_t KD, int64_t KH,
                                     int64_t KW, int64_t groups, int64_t Q);
int dpk_conv3d_gs(const void* x, const void* b, int in_dtype, void* gs, int gs_dtype, float* sumsq,
                  int64_t n, int64_t C, int64_t D, int64_t H, int64_t W, int64_t O,
                  const int64_t* kernel /*host*/, const int64_t* stride /*host*/,
                  const int64_t* pad_lo /*host*/, const int64_t* pad_hi /*host*/,
                  const int64_t* dilation /*host*/, int64_t groups, float scale, void* ws,
                  size_t ws_bytes, dpk_stream_t stream);

/* gs_bias[n,o] = scale * sum_q b[n,o,q]                    (conv.py:117)
 * b: [n,O,q]. sumsq as for dpk_linear_bias_gs. */
int dpk_conv_bias_gs(const void* b, int in_dtype, void* gs_bias, int gs_dtype, float* sumsq,
                     int64_t n, int64_t O, int64_t q, float scale, dpk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * nn.Embedding
 * replaces opacus/grad_sample/embedding.py:25-64 (compute_embedding_grad_sample)
 * and opacus/grad_sample/embedding_norm_sample.py:27-151
 * ------------------------------------------------------------------------- */

/* The integer stage of embedding_norm_sample.py:116-129, bit-exact:
 * the (row, id) pairs of ids[n,T] made unique in sorted order.
 *   inverse[n*T]      position of pair (row(t), ids[t]) in the sorted unique list
 *   unique_pairs[U,2] the list itself (only the first U rows are written)
 *   n_unique[1]       U
 * ids need not lie in any range here. */
/* One workspace layout serves the three entry points below; pass D = 0 when only
 * dpk_embedding_unique_pairs is called. The workspace must be 256-byte aligned. */
size_t dpk_embedding_workspace_bytes(int64_t n, int64_t T, int64_t D);
int dpk_embedding_unique_pairs(const int64_t* ids, int64_t n, int64_t T, int64_t* inverse,
                               int64_t* unique_pairs, int64_t* n_unique, void* ws,
                               size_t ws_bytes, dpk_stream_t stream);

/* gs[n,v,:] = scale * sum_{t : ids[n,t]==v} b[n,t,:]        (embedding.py:48-61)
 * gs: [n,V,D] of gs_dtype, fully written (rows no id names are zero).
 * An id outside [0,V) contributes nothing and nothing is written for it. status
 * (nullable, device int32[1], the caller's): set to 1 when such an id is met and
 * never cleared by the library, so that one flag can collect over many calls and
 * be read back whenever the caller next waits for the stream anyway. */
int dpk_embedding_gs(const int64_t* ids, const void* b, int in_dtype, void* gs, int gs_dtype,
                     int64_t n, int64_t T, int64_t V, int64_t D, float scale, int32_t* status,
                     void* ws, size_t ws_bytes, dpk_stream_t stream);

/* out[v,:] = scale * sum_n coef[n] * sum_{t : ids[n,t]==v} b[n,t,:]
 * The clip-weighted sum of an Embedding table's per-sample gradients (embedding.py:48-61), what
 * the reference's second backward pass of sum_n coef[n] * loss[n] leaves in weight.grad
 * (utils/fast_gradient_clipping_utils.py:193-201), without a weighted copy of the backprops.
 * Equal ids are linked across the whole batch, every list is summed in fp32 in position order
 * (each row times its sample's coefficient) and every row of the table is written once: no
 * atomics, the same bits on every run. out: [V,D] of `out_dtype` (the input's type or fp32),
 * 16-byte aligned, fully written. ids outside [0,V) and `status` as for dpk_embedding_gs.
 * ws: dpk_embedding_weighted_sum_workspace_bytes bytes, 256-byte aligned. */
size_t dpk_embedding_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t D);
int dpk_embedding_weighted_sum(const int64_t* ids, const void* b, int in_dtype, const float* coef, void* out,
                               int out_dtype, int64_t n, int64_t T, int64_t V, int64_t D, float scale,
                               int32_t* status, void* ws, size_t ws_bytes, dpk_stream_t stream);

/* nn.EmbeddingBag (embedding.py:67-94): bag i = index[offsets[i] : offsets[i+1]] (the
 * last one runs to L); gs[i, index[j], :] = scale * b[i,:] for every j of bag i, divided
 * by the bag length when `mean` != 0. An index that occurs several times in a bag still
 * receives b[i,:] once, as the reference's indexed "+=" leaves it. gs: [bags,V,D], fully
 * written, 16-byte aligned. Nothing is written for an index outside [0,V). status as for
 * dpk_embedding_gs; it is also raised for offsets that are not ascending in [0,L] (the
 * result is then unspecified but every access stays inside the tensors). */
int dpk_embedding_bag_gs(const int64_t* index, const int64_t* offsets, const void* b, int in_dtype,
                         void* gs, int gs_dtype, int64_t bags, int64_t L, int64_t V, int64_t D,
                         int mean, float scale, int32_t* status, dpk_stream_t stream);

/* norm[n] = sqrt(sum_{v} || scale * sum_{t : ids[n,t]==v} b[n,t,:] ||^2)
 * (embedding_norm_sample.py:131-150). fp32 output. */
int dpk_embedding_ghost_norm(const int64_t* ids, const void* b, int dtype, float* norm, int64_t n,
                             int64_t T, int64_t D, float scale, void* ws, size_t ws_bytes,
                             dpk_stream_t stream);

/* An embedding table that is also the weight of the output projection (tied input and
 * output embeddings). The reference refuses tied parameters under ghost clipping
 * (opacus/grad_sample/grad_sample_module_fast_gradient_clipping.py:172-179); the materialising
 * path handles them by adding the two layers' gradients (grad_sample_module.py:58-59), and
 * this entry point supplies what the norm of that sum needs beyond the two layers' own ghost
 * norms:  |G_emb + G_head|^2 = |G_emb|^2 + |G_head|^2 + 2 cross,
 *   cross[n] = scale * sum_t < e[n,t,:] , sum_t2 g[n,t2,ids[n,t]] * a[n,t2,:] >.
 * ids: int64 [n,T]; e: [n,T,D] backprops of the embedding output (`emb_dtype`); a: [n,T2,D]
 * inputs and g: [n,T2,V] output backprops of the projection (`head_dtype`); cross: float[n].
 * An id outside [0,V) contributes nothing. Workspace 256-byte aligned. */
size_t dpk_tied_embedding_cross_workspace_bytes(int64_t n, int64_t T, int64_t T2, int64_t D,
                                                int head_dtype);
int dpk_tied_embedding_cross(const int64_t* ids, const void* e, int emb_dtype, const void* a,
                             const void* g, int head_dtype, float* cross, int64_t n, int64_t T,
                             int64_t T2, int64_t D, int64_t V, float scale, void* ws,
                             size_t ws_bytes, dpk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Normalisation layers with an affine weight
 * replaces opacus/grad_sample/group_norm.py:26-47, rms_norm.py:27-47,
 * layer_norm.py:27-52 and instance_norm.py:30-56
 * ------------------------------------------------------------------------- */

/* gs_w[n,c] = scale * sum_s group_norm(x)[n,c,s] * b[n,c,s]   (group_norm.py:43-44)
 * gs_b[n,c] = scale * sum_s b[n,c,s]                          (group_norm.py:46)
 * x, b: [n,C,S]; normalisation without affine over each (n, group). Either
 * output may be NULL. sumsq_w[n] / sumsq_b[n] (float, may be NULL): the per-sample
 * sums of squares of gs_w / gs_b. */
int dpk_group_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, void* gs_b,
                      int gs_dtype, float* sumsq_w, float* sumsq_b, int64_t n, int64_t C,
                      int64_t S, int64_t groups, float eps, float scale, dpk_stream_t stream);

/* gs_w[n,d] = scale * sum_t x[n,t,d] * rsqrt(mean_d x[n,t,:]^2 + eps) * b[n,t,d]
 * (rms_norm.py:44-47). x, b: [n,T,D], D = number of normalised elements.
 * sumsq[n] (float, may be NULL) = sum_d gs_w[n,d]^2, for the optimizer's norm pass. */
size_t dpk_rms_norm_gs_workspace_bytes(int64_t n, int64_t T, int64_t D);
int dpk_rms_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, int gs_dtype,
                    float* sumsq, int64_t n, int64_t T, int64_t D, float eps, float scale,
                    void* ws, size_t ws_bytes, dpk_stream_t stream);

/* gs_w[n,d] = scale * sum_t layer_norm(x)[n,t,d] * b[n,t,d]   (layer_norm.py:41-47)
 * gs_b[n,d] = scale * sum_t b[n,t,d]                          (layer_norm.py:49)
 * x, b: [n,T,D], D = number of normalised elements (the product of
 * normalized_shape), T = everything between the batch and those dimensions.
 * Normalisation without affine: (x - mean) * rsqrt(var + eps), biased variance.
 * Either output may be NULL. sumsq_w[n] / sumsq_b[n] (float, may be NULL): the
 * per-sample sums of squares of gs_w / gs_b. (InstanceNorm, instance_norm.py:50-55,
 * is dpk_group_norm_gs with groups == C.) */
size_t dpk_layer_norm_gs_workspace_bytes(int64_t n, int64_t T, int64_t D);
int dpk_layer_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, void* gs_b,
                      int gs_dtype, float* sumsq_w, float* sumsq_b, int64_t n, int64_t T,
                      int64_t D, float eps, float scale, void* ws, size_t ws_bytes,
                      dpk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * DPOptimizer.clip_and_accumulate, add_noise, scale_grad
 * replaces opacus/optimizers/optimizer.py:432-504
 * ------------------------------------------------------------------------- */

/* sumsq[n] = sum_p gs[n,p]^2                                (optimizer.py:444-446)
 * gs: [n,P]. */
size_t dpk_sumsq_rows_workspace_bytes(int64_t n, int64_t P);
int dpk_sumsq_rows(const void* gs, int dtype, int64_t n, int64_t P, float* sumsq, void* ws,
                   size_t ws_bytes, dpk_stream_t stream);

/* norm[n] = sqrt(sum_k sumsq[k,n]); clip[n] = min(1, C / (norm[n] + 1e-6))
 * (optimizer.py:452-455; grad_sample_module_fast_gradient_clipping.py:137-150)
 * sumsq: [K,n] squared per-parameter norms. With `is_norm` != 0 the input
 * holds norms instead of squared norms (the ghost path stores norms).
 * norm (nullable) and clip (nullable) are float[n]. */
int dpk_clip_factor(const float* sumsq, int64_t K, int64_t n, int is_norm, float max_grad_norm,
                    float* norm, float* clip, dpk_stream_t stream);

/* summed[p] (+)= sum_n clip[n] * gs[n,p]                    (optimizer.py:464-473)
 * gs: [n,P] of gs_dtype; summed: [P] of out_dtype; `accumulate` != 0 adds to
 * what summed holds (optimizer.py:470-471), else overwrites. The n x P tensor
 * is read exactly once. */
int dpk_clip_accumulate(const void* gs, int gs_dtype, const float* clip, void* summed,
                        int out_dtype, int64_t n, int64_t P, int accumulate, dpk_stream_t stream);

/* The same two passes over up to DPK_MULTI_MAX parameters in one launch each:
 * the per-parameter Python loop of optimizer.py:457-475 folded into the grid.
 * Host arrays of K device pointers / sizes. All tensors share n and dtypes.
 * dpk_sumsq_rows_multi writes sumsq[k*n + i]. */
size_t dpk_sumsq_rows_multi_workspace_bytes(int64_t n, const int64_t* P /*host*/, int64_t K);
int dpk_sumsq_rows_multi(const void* const* gs /*host*/, const int64_t* P /*host*/, int64_t K,
                         int dtype, int64_t n, float* sumsq, void* ws, size_t ws_bytes,
                         dpk_stream_t stream);
int dpk_clip_accumulate_multi(const void* const* gs /*host*/, void* const* summed /*host*/,
                              const int64_t* P /*host*/, int64_t K, int gs_dtype, int out_dtype,
                              const float* clip, int64_t n, int accumulate, dpk_stream_t stream);

/* Per-layer clipping (opacus/optimizers/perlayeroptimizer.py:58-76): every parameter k
 * has its own bound. clip[k*n + i] = min(1, C[k] / (sqrt(sumsq[k*n + i]) + 1e-6))
 * (with `is_norm` != 0 the input holds norms), max_grad_norms: host array of K floats,
 * K <= DPK_MULTI_MAX. dpk_clip_accumulate_per_layer is dpk_clip_accumulate_multi with
 * tensor k weighted by row k of that [K,n] factor table. */
int dpk_clip_factor_per_layer(const float* sumsq, int64_t K, int64_t n, int is_norm,
                              const float* max_grad_norms /*host*/, float* clip, dpk_stream_t stream);
int dpk_clip_accumulate_per_layer(const void* const* gs /*host*/, void* const* summed /*host*/,
                                  const int64_t* P /*host*/, int64_t K, int gs_dtype, int out_dtype,
                                  const float* clip /*[K,n]*/, int64_t n, int accumulate,
                                  dpk_stream_t stream);

/* grad[p] = (summed[p] + std * z[p]) / denom,  z ~ N(0,1)   (optimizer.py:485-504)
 * Folds _generate_noise (optimizer.py:104-169), the add (:491) and scale_grad's
 * division (:502-504) into one pass. std == 0 adds exact zeros and draws
 * nothing (optimizer.py:139-140). z comes from Philox4x32-10 keyed by `seed`
 * with counter (element index / 4, offset); `draws` = 1, or 4 for the
 * reference's secure mode (sum of four normals halved, optimizer.py:150-160).
 * A call consumes `draws` units of offset. grad may alias summed. */
int dpk_add_noise(const void* summed, int in_dtype, void* grad, int out_dtype, int64_t P,
                  float std, float denom, uint64_t seed, uint64_t offset, int draws,
                  dpk_stream_t stream);

/* The same for up to DPK_MULTI_MAX parameters in one launch (the Python loop of
 * optimizer.py:482-493 folded into the grid). Host arrays of K device pointers and
 * sizes; all tensors share the dtypes. The tensors draw from ONE Philox stream laid
 * end to end: element i of tensor k uses counter (sum_{j<k} ceil(P[j]/4) + i/4, offset).
 * The call consumes `draws` units of offset in total. */
int dpk_add_noise_multi(const void* const* summed /*host*/, void* const* grad /*host*/,
                        const int64_t* P /*host*/, int64_t K, int in_dtype, int out_dtype, float std,
                        float denom, uint64_t seed, uint64_t offset, int draws, dpk_stream_t stream);

/* The whole DPOptimizer step of a small model in one launch: clip factors
 * min(1, C / (sqrt(sum_k sumsq[k][i]) + 1e-6)) (optimizer.py:444-455), the clip-weighted sum over
 * the batch (:456-475), the noise and the division (:477-504). Replaces the loop of
 * DPOptimizer.clip_and_accumulate + add_noise + scale_grad for K <= DPK_MULTI_MAX parameters of
 * 64 <= n <= 1024 samples. gs[k]: [n, P[k]] of `gs_dtype`; sumsq[k]: float[n], the squared norms of
 * the rows of gs[k] (the samplers leave them); grad[k] (written) and summed[k] (nullable; the clipped
 * sum before the noise) of `out_dtype`. Host arrays of K device pointers and sizes. Every block
 * recomputes the n factors; sums, factors and noise are bit-identical to dpk_clip_factor on the
 * stacked squared norms, dpk_clip_accumulate_multi in its small-tensor shape and
 * dpk_add_noise_multi with the same (std, denom, seed, offset, draws), in that order. */
int dpk_clip_noise_step(const void* const* gs /*host*/, const float* const* sumsq /*host*/, void* const* grad /*host*/,
                        void* const* summed /*host, nullable*/, const int64_t* P /*host*/, int64_t K, int gs_dtype,
                        int out_dtype, int64_t n, float max_grad_norm, float std, float denom, uint64_t seed,
                        uint64_t offset, int draws, dpk_stream_t stream);

/* out[p] = std * z[p]: the bare generator, for statistical tests. */
int dpk_fill_normal(float* out, int64_t P, float std, uint64_t seed, uint64_t offset,
                    dpk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DPK_H */
