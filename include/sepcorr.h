/*
 * sepcorr.h - C ABI of libsepcorr.so: memory-saving separation of the 4D correlation volume
 * for AMD gfx950 (MI355X).  The 4D volume S[b,i,j,u,v] = <f1[b,i,j,:], f2[b,u,v,:]> is formed tile
 * by tile in registers with fp32 MFMA and reduced on the fly; it is never written to memory.
 *
 * Every entry point replaces one function of the reference's native module `MemorySaver`
 * (libs/MemorySaver/src/MemorySaver_cuda.cpp:105-112) with plain pointers and sizes in place of
 * at::Tensor.  Conventions shared by all of them:
 *
 *  - All pointers are DEVICE pointers on the current HIP device.  Inputs are borrowed and never
 *    written; outputs are fully overwritten (no pre-initialisation needed, unlike the reference
 *    kernels which accumulate into buffers the host pre-fills, MemorySaver_kernel_forward.cu:916-927).
 *  - All tensors are contiguous fp32 except the argmax tensors (int32):
 *      f1      (B, H1, W1, C)   image-1 features at pyramid level 0, pre-scaled by the caller
 *      f2      (B, H2, W2, C)   image-2 features at pyramid level k
 *      *_u     (B, H1, W1, ch, H2)   keeps u (fmap2 row), was reduced over v (fmap2 column)
 *      *_v     (B, H1, W1, ch, W2)   keeps v, was reduced over u
 *    ch = 2 (max, avg) for the max/avg tensors, 1 for argmax, K for the attention tensors.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls are asynchronous:
 *    they enqueue kernels and return.
 *  - Return value: 0 on success, a negative SEPCORR_E* code otherwise; sepcorr_last_error() then
 *    returns a message for the calling thread.  Nothing is launched when a check fails.
 *  - Limits of this build: 1 <= W2 <= 2048, 1 <= C <= 1024, 1 <= K <= 8, all sizes >= 1 and small
 *    enough that every tensor has fewer than 2^31 elements.
 *  - Backward entry points need scratch memory: query sepcorr_backward_workspace_bytes() and pass a
 *    device buffer of at least that size (256-byte aligned).  Its contents on entry are ignored.
 *  - Forward entry points take scratch memory optionally (sepcorr_forward_workspace_bytes(), 256-byte aligned,
 *    contents on entry ignored; NULL is allowed).  With it the sweep is dealt out to the chip in pieces smaller
 *    than a 32-pixel tile where whole tiles would leave compute units idle (e.g. 440 tiles on 256 units); results
 *    are deterministic either way and differ from each other only in the rounding of the sums over u.
 */
#ifndef SEPCORR_H
#define SEPCORR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SEPCORR_OK 0
#define SEPCORR_EINVAL (-1)   /* null pointer, non-positive or unsupported size */
#define SEPCORR_ELAUNCH (-2)  /* HIP reported an error at launch */
#define SEPCORR_EWORKSPACE (-3) /* workspace missing or too small */

/* Message describing the last failure on this thread ("" if none). */
const char *sepcorr_last_error(void);

/* ABI version of this library (bumped on incompatible change). */
int sepcorr_abi_version(void);

/*
 * Measurement aid; no counterpart in the reference.  While enabled, every kernel launched by this
 * library is bracketed by HIP events on its launch stream.  sepcorr_profile_collect() waits for the
 * recorded kernels, writes up to `cap` durations (milliseconds, launch order) to `ms` and the kernel
 * labels joined by '\n' to `names`, forgets them, and returns how many it wrote.
 */
int sepcorr_profile_enable(int on);
int sepcorr_profile_collect(char *names, size_t names_cap, float *ms, int cap);

/*
 * Arithmetic of the contractions of the forward sweeps (max/avg, max/argmax/avg, compression forward and the
 * attention-gradient pass of the compression backward) and of d_f1; no counterpart in the reference.
 *   SEPCORR_CONTRACT_FP32    fp32 MFMA (the initial choice).
 *   SEPCORR_CONTRACT_BF16X3  every fp32 operand is written exactly as the sum of three bf16 numbers and the
 *                            product taken as the six largest of the nine plane products, with bf16 MFMA
 *                            accumulating in fp32.  What is dropped is below 2^-24 of each product, so results
 *                            agree with the fp32 contraction to its own rounding error; argmax may differ
 *                            where two maxima are that close.  Used where C == 256 and a row of fmap2 has at
 *                            most 256 columns, silently fp32 elsewhere.  Takes its scratch memory (about
 *                            B*H2*W2*1536 bytes of planes; for d_f1 also ceil(W2/32) partial copies of d_f1 and
 *                            the transposed weights) from the stream's memory pool (hipMallocAsync) for the
 *                            duration of each call.
 * The setting is process-wide and read when a call is enqueued.  Returns the previous mode; an unknown mode
 * changes nothing.  SEPCORR_BF16X3=1 in the environment makes BF16X3 the initial choice.
 */
#define SEPCORR_CONTRACT_FP32 0
#define SEPCORR_CONTRACT_BF16X3 1
int sepcorr_set_contraction(int mode);

/*
 * How sepcorr_max_argmax_avg_backward (and its _static variant) computes the two feature gradients; no counterpart
 * in the reference, whose kernel visits every (pixel, position) pair.
 *   SEPCORR_MAXAVG_AUTO    by gathers where the sizes allow and that is the faster way on MI355X: fmap2 has at
 *                          least 12 positions per line (H2*W2 >= 12*(H2+W2)), or at least 8 and B*N1 >= 16384;
 *                          dense otherwise (the initial choice).
 *   SEPCORR_MAXAVG_DENSE   recompute the correlation tile by tile on fp32 MFMA and multiply by the gradient it
 *                          implies: 4*N1*N2*C flops per gradient.
 *   SEPCORR_MAXAVG_GATHER  the gradient of a maximum selects one feature row, the gradient of an average multiplies
 *                          a line mean: B*N1*(H2+W2) rows of C floats fetched per gradient plus two small products.
 *                          Needs C % 4 == 0 and C <= 256; other sizes take the dense path silently.
 * Both give the same gradients up to fp32 rounding, and each is reproducible from run to run.  The setting is
 * process-wide and read when a call is enqueued.  Returns the previous mode; an unknown mode changes nothing.
 */
#define SEPCORR_MAXAVG_AUTO 0
#define SEPCORR_MAXAVG_DENSE 1
#define SEPCORR_MAXAVG_GATHER 2
int sepcorr_set_max_avg_backward(int mode);

/*
 * Replaces MemorySaver.max_avg_forward (MemorySaver_cuda.cpp:10-21 -> max_avg_cuda_forward,
 * MemorySaver_kernel_forward.cu:901-949).
 *   out_u[b,i,j,0,u] = max_v S   out_u[b,i,j,1,u] = (sum_v S) / W2      (B,H1,W1,2,H2)
 *   out_v[b,i,j,0,v] = max_u S   out_v[b,i,j,1,v] = (sum_u S) / H2      (B,H1,W1,2,W2)
 */
int sepcorr_max_avg_forward(const float *f1, const float *f2, float *out_u, float *out_v,
                            int B, int H1, int W1, int H2, int W2, int C,
                            void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes a forward entry point can make use of for these sizes (K = 2 for the max/avg entry points); 0 when
 * whole tiles already fill the chip. */
size_t sepcorr_forward_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C, int K);

/*
 * Replaces MemorySaver.max_argmax_avg_forward (MemorySaver_cuda.cpp:23-34 ->
 * MemorySaver_kernel_forward.cu:962-1016).  As above plus
 *   argmax_u[b,i,j,0,u] = the v attaining max_v S,  argmax_v[b,i,j,0,v] = the u attaining max_u S,
 * lowest index on exact ties (MemorySaver_kernel_forward.cu:498-507).
 */
int sepcorr_max_argmax_avg_forward(const float *f1, const float *f2, float *out_u, float *out_v,
                                   int32_t *argmax_u, int32_t *argmax_v,
                                   int B, int H1, int W1, int H2, int W2, int C,
                                   void *workspace, size_t workspace_bytes, void *stream);

/*
 * Replaces MemorySaver.compression_forward (MemorySaver_cuda.cpp:36-53 ->
 * MemorySaver_kernel_forward.cu:1029-1074), for any K (the reference kernel is fixed to K=2).
 *   comp_u[b,i,j,k,u] = sum_v S * a_u[b,i,j,k,v]      a_u (B,H1,W1,K,W2) -> comp_u (B,H1,W1,K,H2)
 *   comp_v[b,i,j,k,v] = sum_u S * a_v[b,i,j,k,u]      a_v (B,H1,W1,K,H2) -> comp_v (B,H1,W1,K,W2)
 * Weights are used as given (the caller applies the softmax, core/corr.py:441-442).
 */
int sepcorr_compression_forward(const float *f1, const float *f2, const float *a_u, const float *a_v,
                                float *comp_u, float *comp_v,
                                int B, int H1, int W1, int H2, int W2, int C, int K,
                                void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes needed by any of the three backward entry points for these sizes (0 is possible). */
size_t sepcorr_backward_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C);

/*
 * Replaces MemorySaver.max_argmax_avg_backward (MemorySaver_cuda.cpp:55-78 ->
 * MemorySaver_kernel_max_avg_argmax_backward.cu:1198-1221).  With
 *   G = g_u[..,0,u]*[v==argmax_u[..,u]] + g_u[..,1,u]/W2 + g_v[..,0,v]*[u==argmax_v[..,v]] + g_v[..,1,v]/H2
 *   d_f1[b,i,j,:] = sum_{u,v} G f2[b,u,v,:]     d_f2[b,u,v,:] = sum_{i,j} G f1[b,i,j,:]
 * d_f2 is accumulated by the owner of each (u,v) in a fixed order: no atomics, run-to-run identical
 * (the reference uses atomicAdd, MemorySaver_kernel_max_avg_argmax_backward.cu:305-310).
 * Argmax entries are data: a value outside its axis selects nothing.
 */
int sepcorr_max_argmax_avg_backward(const float *f1, const float *f2,
                                    const int32_t *argmax_u, const int32_t *argmax_v,
                                    const float *grad_u, const float *grad_v,
                                    float *d_f1, float *d_f2,
                                    int B, int H1, int W1, int H2, int W2, int C,
                                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same computation and results as sepcorr_max_argmax_avg_backward, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The scratch memory is an array of SEPCORR_STATIC_SCRATCH_BYTES bytes inside the
 * library's device image (one copy per GPU, held until the process ends) instead of a workspace argument; the
 * call allocates nothing, creates no streams or events and runs all its kernels on `stream`.
 *   - It always contracts in fp32: results are bit-equal to the workspace variant's under SEPCORR_CONTRACT_FP32 (the
 *     default); with sepcorr_set_contraction(SEPCORR_CONTRACT_BF16X3) the workspace variant's dense d_f1 takes the
 *     bf16-plane kernels (which allocate stream-ordered memory) and the two agree to rounding only.
 *   - Sizes that need more scratch than SEPCORR_STATIC_SCRATCH_BYTES are refused with SEPCORR_EWORKSPACE; use the
 *     workspace variant for them.  (Any size whose sepcorr_backward_workspace_bytes() fits is accepted; that figure
 *     also covers the other backward entry points, so somewhat larger sizes fit as well.)
 *   - All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 *     threads) race and give undefined results.  Calls on one stream are ordered and safe.  The array's contents
 *     between calls are unspecified; every call overwrites what it reads.
 */
#define SEPCORR_STATIC_SCRATCH_BYTES (64u << 20)
int sepcorr_max_argmax_avg_backward_static(const float *f1, const float *f2,
                                           const int32_t *argmax_u, const int32_t *argmax_v,
                                           const float *grad_u, const float *grad_v,
                                           float *d_f1, float *d_f2,
                                           int B, int H1, int W1, int H2, int W2, int C, void *stream);

/*
 * Replaces MemorySaver.compression_backward (MemorySaver_cuda.cpp:80-103 ->
 * MemorySaver_kernel_compression_backward.cu:651-666).  With
 *   G = sum_k a_u[..,k,v]*g_cu[..,k,u] + a_v[..,k,u]*g_cv[..,k,v]
 *   d_f1 = sum_{u,v} G f2      d_f2 = sum_{i,j} G f1
 *   d_a_u[b,i,j,k,v] = sum_u S * g_cu[b,i,j,k,u]      d_a_v[b,i,j,k,u] = sum_v S * g_cv[b,i,j,k,v]
 * d_f1 and d_f2 may both be NULL: then only d_a_u and d_a_v are computed (one sweep; workspace as for a forward
 * entry point: optional, sepcorr_forward_workspace_bytes(..., K)).
 */
int sepcorr_compression_backward(const float *f1, const float *f2, const float *a_u, const float *a_v,
                                 const float *g_cu, const float *g_cv,
                                 float *d_f1, float *d_f2, float *d_a_u, float *d_a_v,
                                 int B, int H1, int W1, int H2, int W2, int C, int K,
                                 void *workspace, size_t workspace_bytes, void *stream);

/*
 * Attention compression straight from the logits.  The caller's
 *   a_u = attention1(sep_u).softmax(dim=2) ...; ComputeSelfCompressionFunction.apply(fmap1, fmap2, a_u, a_v)
 * (core/corr.py:437-448, libs/MemorySaver/functions/MemorySaver.py:107-177) with the softmax moved inside the operator:
 *   logits_u (B,H1,W1,K,W2), logits_v (B,H1,W1,K,H2)   what the attention modules return, in the operator's layout
 *   comp_u, comp_v                                     as sepcorr_compression_forward with a = softmax over the last axis
 *   stats_u, stats_v (B,H1,W1,K,2)                     per row (max, sum of exp(z - max)): written here (one pass over
 *                                                      the logits) unless stats_given != 0, in which case they are read
 *                                                      (sepcorr_attention_logits_forward supplies them for free)
 * The weights exp(z - max) / sum are formed where the sweep loads them; no tensor of softmax outputs exists.
 * workspace: as for sepcorr_compression_forward (optional).
 */
int sepcorr_compression_forward_from_logits(const float *f1, const float *f2,
                                            const float *logits_u, const float *logits_v,
                                            float *comp_u, float *comp_v, float *stats_u, float *stats_v, int stats_given,
                                            int B, int H1, int W1, int H2, int W2, int C, int K,
                                            void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes of the call below: without (with_features = 0) or with the feature gradients. */
size_t sepcorr_compression_backward_from_logits_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C, int K,
                                                                int with_features);

/*
 * Gradients of the above: what torch autograd computes through ComputeSelfCompressionFunction.backward
 * (libs/MemorySaver/functions/MemorySaver.py:139-177) and the softmax in front of it (core/corr.py:441-442).
 * Inputs are those of the forward call, its outputs comp_u, comp_v and statistics, and the upstream gradients
 * g_cu (B,H1,W1,K,H2), g_cv (B,H1,W1,K,W2).  With a = softmax(z) and d_a as in sepcorr_compression_backward,
 *   d_logits_u[..,k,v] = a_u (d_a_u - sum_v a_u d_a_u),   d_logits_v[..,k,u] = a_v (d_a_v - sum_u a_v d_a_v);
 * the row sums are taken as sum_u g_cu comp_u and sum_v g_cv comp_v (the same numbers), so the gradients leave the
 * weight-gradient sweep finished: no tensor d_a and no softmax-backward pass exist.
 * d_f1, d_f2 as in sepcorr_compression_backward; both may be NULL (then only the logit gradients are computed).
 */
int sepcorr_compression_backward_from_logits(const float *f1, const float *f2,
                                             const float *logits_u, const float *logits_v,
                                             const float *stats_u, const float *stats_v,
                                             const float *comp_u, const float *comp_v,
                                             const float *g_cu, const float *g_cv,
                                             float *d_f1, float *d_f2, float *d_logits_u, float *d_logits_v,
                                             int B, int H1, int W1, int H2, int W2, int C, int K,
                                             void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same operators for several pyramid levels of fmap2 in one call: level l is (B,h2[l],w2[l],C), all pointer tables
 * and the size tables are host arrays of nlev <= 4 entries, outputs per level as in the single-level calls.  Replaces
 * the loop over levels of the caller (core/corr.py:416-457): one launch covers all levels given (their work is dealt
 * out together and the image-1 tile is shared) when every w2[l] is at most 128 and fills 1, 2 or 4 chunks of 32
 * columns, C is a multiple of 32 and scratch is given; other shapes run level by level inside the call.
 *   workspace: sepcorr_forward_levels_workspace_bytes(...) bytes, 256-byte aligned; optional (NULL) for the two forward
 *   calls, required for the backward call.  The statistics of the logits are inputs here (the attention producer
 *   supplies them); the backward call returns the logit gradients only (feature gradients: sepcorr_fused_backward or
 *   sepcorr_compression_backward_from_logits per level).
 */
size_t sepcorr_forward_levels_workspace_bytes(const int *h2, const int *w2, int nlev, int B, int H1, int W1, int C, int K);
int sepcorr_max_argmax_avg_forward_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2, int nlev,
                                          float *const *out_u, float *const *out_v,
                                          int32_t *const *argmax_u, int32_t *const *argmax_v,
                                          int B, int H1, int W1, int C,
                                          void *workspace, size_t workspace_bytes, void *stream);
int sepcorr_compression_forward_from_logits_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                                                   int nlev, const float *const *logits_u, const float *const *logits_v,
                                                   const float *const *stats_u, const float *const *stats_v,
                                                   float *const *comp_u, float *const *comp_v,
                                                   int B, int H1, int W1, int C, int K,
                                                   void *workspace, size_t workspace_bytes, void *stream);
int sepcorr_compression_backward_from_logits_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                                                    int nlev, const float *const *logits_u, const float *const *logits_v,
                                                    const float *const *stats_u, const float *const *stats_v,
                                                    const float *const *comp_u, const float *const *comp_v,
                                                    const float *const *g_cu, const float *const *g_cv,
                                                    float *const *d_logits_u, float *const *d_logits_v,
                                                    int B, int H1, int W1, int C, int K,
                                                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * Row softmax helper of the two calls above for callers that need the weights themselves: for nrows rows of L logits,
 * stats (nrows,2) = (max, sum of exp) is computed (stats_given == 0) or read, and, when a is not NULL,
 * a = exp(z - max) / sum is written.  No counterpart in the reference (torch's softmax stands there, core/corr.py:441).
 */
int sepcorr_softmax_rows(const float *logits, float *stats, int stats_given, float *a, long nrows, int L, void *stream);

/*
 * Feature gradients of both operators of one pyramid level in one pass; no counterpart in the reference,
 * whose two backward functions (MemorySaver_cuda.cpp:55-103) each contract their own dL/dS.  With G the sum
 * of the two expressions given above for sepcorr_max_argmax_avg_backward and sepcorr_compression_backward,
 *   d_f1 = sum_{u,v} G f2      d_f2 = sum_{i,j} G f1
 * i.e. the sum of the d_f1 (d_f2) the two calls would return, from 2 sweeps over the volume instead of 4.
 * For callers that have the complete gradient of the max/avg outputs before they need feature gradients
 * (in core/corr.py:437-448 it arrives through d_a_u/d_a_v and the attention weights' producer).
 */
int sepcorr_fused_backward(const float *f1, const float *f2,
                           const int32_t *argmax_u, const int32_t *argmax_v,
                           const float *grad_u, const float *grad_v,
                           const float *a_u, const float *a_v, const float *g_cu, const float *g_cv,
                           float *d_f1, float *d_f2,
                           int B, int H1, int W1, int H2, int W2, int C, int K,
                           void *workspace, size_t workspace_bytes, void *stream);
/* The same, but d_f1 is added to what the buffer holds: fmap1 is shared by all pyramid levels (core/corr.py:419),
 * so its gradient is the sum over the levels' calls; d_f2 (one tensor per level) is written as above. */
int sepcorr_fused_backward_add(const float *f1, const float *f2,
                               const int32_t *argmax_u, const int32_t *argmax_v,
                               const float *grad_u, const float *grad_v,
                               const float *a_u, const float *a_v, const float *g_cu, const float *g_cv,
                               float *d_f1, float *d_f2,
                               int B, int H1, int W1, int H2, int W2, int C, int K,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * Attention-weight producer in the operator's layout.  Replaces, for one of the two volumes, the caller's
 *   a = attention(sep.permute(0,3,4,1,2)).softmax(dim=2).permute(0,3,4,1,2).contiguous()
 * (core/corr.py:428-429, 437-446) where `attention` is the reference's torch.nn.Conv3d(2, K, 3, padding=1)
 * (core/sepflow.py:59-60):
 *   sep    (B,H1,W1,2,L)   the max/avg output of sepcorr_max_*_forward (either one)
 *   weight (K,2,3,3,3)     Conv3d weight; kernel axes are (L, H1, W1)        bias (K) or NULL
 *   a      (B,H1,W1,K,L)   softmax over L of the convolution: the weights sepcorr_compression_forward takes
 */
int sepcorr_attention_forward(const float *sep, const float *weight, const float *bias, float *a,
                              int B, int H1, int W1, int L, int K, void *stream);

/*
 * The same producer stopping at the logits: logits (B,H1,W1,K,L) = Conv3d(sep) in the operator's layout, and, when
 * stats is not NULL, stats (B,H1,W1,K,2) = per row (max, sum of exp(z - max)), which the kernel has at hand.  Feeds
 * sepcorr_compression_forward_from_logits (core/corr.py:437-448 with the softmax moved into the operator).
 */
int sepcorr_attention_logits_forward(const float *sep, const float *weight, const float *bias, float *logits, float *stats,
                                     int B, int H1, int W1, int L, int K, void *stream);

/* Its gradients from the gradient of the logits (no softmax in between): d_sep, d_weight, d_bias (or NULL) as
 * sepcorr_attention_backward; scratch: sepcorr_attention_logits_workspace_bytes. */
size_t sepcorr_attention_logits_workspace_bytes(int B, int H1, int W1, int L, int K);
int sepcorr_attention_logits_backward(const float *sep, const float *weight, const float *d_logits,
                                      float *d_sep, float *d_weight, float *d_bias,
                                      int B, int H1, int W1, int L, int K,
                                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * The two calls above for several pyramid levels of one attention module in one set of launches (the module is
 * applied to the max/avg volume of every level, core/corr.py:416-446): host arrays of nlev (1 to 4) device pointers
 * and row lengths L[l]; weight, bias, B, H1, W1, K are shared.  The backward call returns d_weight and d_bias summed
 * over the levels and, when d_sep_init is not NULL, d_sep[l] = d_sep_init[l] + (gradient through the convolution):
 * the gradient that reaches the max/avg volume directly, added in the same pass.
 */
int sepcorr_attention_logits_forward_levels(const float *const *sep, const float *weight, const float *bias,
                                            float *const *logits, float *const *stats, const int *L, int nlev,
                                            int B, int H1, int W1, int K, void *stream);
size_t sepcorr_attention_logits_levels_workspace_bytes(const int *L, int nlev, int B, int H1, int W1, int K);
int sepcorr_attention_logits_backward_levels(const float *const *sep, const float *weight, const float *const *d_logits,
                                             const float *const *d_sep_init, float *const *d_sep, float *d_weight,
                                             float *d_bias, const int *L, int nlev, int B, int H1, int W1, int K,
                                             void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes needed by sepcorr_attention_backward. */
size_t sepcorr_attention_workspace_bytes(int B, int H1, int W1, int L, int K);

/*
 * Gradients of the above (what torch autograd computes through softmax and Conv3d in the reference,
 * core/corr.py:437-446): given grad_a = dLoss/da and the saved output a,
 *   d_sep (B,H1,W1,2,L), d_weight (K,2,3,3,3), d_bias (K) or NULL.
 * Sums run in a fixed order: results are run-to-run identical.
 */
int sepcorr_attention_backward(const float *sep, const float *weight, const float *a, const float *grad_a,
                               float *d_sep, float *d_weight, float *d_bias,
                               int B, int H1, int W1, int L, int K,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * Assembly of a module-level volume from operator-level outputs.  Writes channels [c0, c0+ch) of
 * dst (B,CT,L0,H1,W1) from src (B,H1,W1,ch,Li):
 *   dst[b,c0+c,l0,i,j] = linear interpolation (align_corners=True) of src[b,i,j,c,:] at l0 * (Li-1)/(L0-1).
 * Replaces, per level and per operator output, the caller's permute(0,3,4,1,2), torch.cat over channels,
 * F.interpolate(..., [L0,h1,w1], mode='trilinear', align_corners=True) and the torch.cat over levels
 * (core/corr.py:428-429, 451-475); H1 and W1 keep their size there, so only L is interpolated.
 * Limits: Li and L0 up to about 500 (one LDS tile), B*ch < 65536.
 */
int sepcorr_assemble_forward(const float *src, float *dst, int B, int H1, int W1, int ch, int Li,
                             int CT, int c0, int L0, void *stream);

/* Adjoint of the above: grad_src (B,H1,W1,ch,Li), fully overwritten, from grad_dst (B,CT,L0,H1,W1). */
int sepcorr_assemble_backward(const float *grad_dst, float *grad_src, int B, int H1, int W1, int ch, int Li,
                              int CT, int c0, int L0, void *stream);

/*
 * The same for up to 8 sources in one launch: source n (B,H1,W1,ch[n],Li[n]) fills the channels after those of the
 * sources before it (the first starts at channel 0); ch, Li and the pointer tables are host arrays of nsrc entries.
 * One launch per module-level volume instead of one per level and operator output.
 */
int sepcorr_assemble_forward_multi(const float *const *srcs, const int *ch, const int *Li, int nsrc, float *dst,
                                   int B, int H1, int W1, int CT, int L0, void *stream);
int sepcorr_assemble_backward_multi(const float *grad_dst, float *const *grad_srcs, const int *ch, const int *Li,
                                    int nsrc, int B, int H1, int W1, int CT, int L0, void *stream);

/*
 * The caller's preparation of a feature map for the operator, in one pass: the block keeps fmap1 and fmap2 as
 * (B,C,H,W), pools fmap2 level after level with F.avg_pool2d(fmap2, 2, stride=2) (core/corr.py:376-382) and hands every
 * level over as permute(0,2,3,1).contiguous(), fmap1 also divided by sqrt(C) (core/corr.py:419-422).
 *   fmap     (B,C,H,W)
 *   levels   host array of nlev device pointers: level l in (B, H >> l, W >> l, C); level 0 = the permuted map
 *            divided by `divisor` (sqrt(C) for fmap1 with nlev = 1; 1 for fmap2), level l = 2x2 average pooling of
 *            level l - 1 (sizes round down), fully overwritten
 * Limits: 1 to 4 levels, none of them empty; B * ceil(C / 32) < 65536.
 */
int sepcorr_feature_pyramid_forward(const float *fmap, float *const *levels, int B, int C, int H, int W, int nlev,
                                    float divisor, void *stream);
/* Adjoint of the above: grad_fmap (B,C,H,W), fully overwritten, from the gradients of all levels (same layouts). */
int sepcorr_feature_pyramid_backward(const float *const *grad_levels, float *grad_fmap, int B, int C, int H, int W,
                                     int nlev, float divisor, void *stream);

/*
 * Windowed bilinear lookup of the correlation pyramid without the 4D volume: what the caller's
 * corr_fn(coords) returns on the stored-volume path (CorrBlock.__call__, core/corr.py:193-248), for the block
 * that never stores the volume (AlternateCorrBlockSepflow.__call__, core/corr.py:479-510, which raises
 * NotImplementedError in the reference: its native part, RAFT's alt_cuda_corr.forward, is not in the tree).
 *   f1         (B,H1,W1,C)       unscaled NHWC fmap1 (core/corr.py:500)
 *   f2_levels  host array of L device pointers; level l is the pooled NHWC fmap2 (B,h2[l],w2[l],C)
 *              (core/corr.py:377-382, 501); h2, w2 are host arrays of L ints
 *   coords     (B,2,H1,W1)       channel 0 = x (fmap2 column), channel 1 = y (fmap2 row), level-0 pixels;
 *                                level l samples at coords / 2^l (core/corr.py:219, 503)
 *   out        (B, L*n*n, H1, W1), n = 2*radius+1, fully overwritten:
 *              out[b, l*n*n + a*n + c, i, j] = scale * bilinear(S_l[b,i,j,:,:])(x/2^l + a - radius, y/2^l + c - radius)
 *              with S_l = <f1[b,i,j,:], f2_l[b,u,v,:]>, corners outside the level counting as zero
 *              (grid_sample with align_corners=True, core/utils/utils.py:110-118); the x offset runs with the
 *              first window index as in the reference (core/corr.py:213-226).  scale = 1/sqrt(C) reproduces
 *              core/corr.py:282, 509.
 * Limits: C <= 1024, L <= 8, radius 1..8.
 */
int sepcorr_lookup_forward(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                           const float *coords, float *out, int B, int H1, int W1, int C, int L, int radius,
                           float scale, void *stream);

/* Scratch bytes needed by sepcorr_lookup_backward (h2, w2: host arrays of L level sizes). 0 for invalid sizes. */
size_t sepcorr_lookup_backward_workspace_bytes(const int *h2, const int *w2, int B, int H1, int W1, int C, int L,
                                               int radius);

/*
 * Gradients of sepcorr_lookup_forward with respect to the feature maps: what torch autograd computes through
 * bilinear_sampler and the stored pyramid on the reference's 4D path (core/corr.py:193-248, 19-38) and what
 * alt_cuda_corr.backward would supply to the draft at core/corr.py:494-509.  coords receive no gradient (the flow
 * iterations detach them, core/sepflow.py:194).
 *   grad_out     (B, L*n*n, H1, W1)
 *   d_f1         (B,H1,W1,C)                      fully overwritten
 *   d_f2_levels  host array of L device pointers; level l (B,h2[l],w2[l],C), fully overwritten: the gradient of that
 *                level's pooled fmap2 (the caller's avg_pool2d chain carries it on to fmap2)
 * No atomics; sums run in a fixed order: results are run-to-run identical.  workspace: 256-byte aligned device memory
 * of at least sepcorr_lookup_backward_workspace_bytes(...) bytes.
 */
int sepcorr_lookup_backward(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                            const float *coords, const float *grad_out, float *d_f1, float *const *d_f2_levels,
                            int B, int H1, int W1, int C, int L, int radius, float scale,
                            void *workspace, size_t workspace_bytes, void *stream);

/*
 * Lookup in one of the two separated 3D volumes: the reference's CorrBlock1D (core/corr.py:513-624), per volume.
 *   corr    (B,dim,L,H1,W1)   a volume in the layout AlternateCorrBlockSepflow.separate returns (corr1: L = W2, corr2: L = H2)
 *   coords  (B,2,H1,W1)       coord_channel 0 (x) addresses corr1, 1 (y) corr2 (core/corr.py:573, 598)
 *   out     (B, levels*dim*n, H1, W1), n = 2*radius+1, fully overwritten:
 *           out[b, l*dim*n + d*n + k, i, j] = linear sample of level l of corr[b,d,:,i,j] at coords/2^l + k - radius,
 *           level l = l-fold average pooling by two along L (core/corr.py:546-550), zero outside the level
 *           (grid_sample, align_corners=True, core/corr.py:553-560).  The pyramid is formed on the fly, not stored.
 *   clamp_unit != 0 clamps the sampling positions to [-1, 1] first, as the reference does for its first volume
 *           (core/corr.py:593); pass 1 for corr1 and 0 for corr2 to reproduce it.
 * Limits: 8 levels, radius <= 16, L >> (levels-1) >= 1.
 */
int sepcorr_lookup1d_forward(const float *corr, const float *coords, float *out, int B, int dim, int L, int H1, int W1,
                             int coord_channel, int clamp_unit, int levels, int radius, void *stream);

/* Adjoint of the above with respect to corr: d_corr (B,dim,L,H1,W1), fully overwritten, from grad_out.  Every
 * (b,d,i,j) column is owned by one thread: no atomics, fixed summation order.  coords get no gradient here. */
int sepcorr_lookup1d_backward(const float *coords, const float *grad_out, float *d_corr, int B, int dim, int L, int H1,
                              int W1, int coord_channel, int clamp_unit, int levels, int radius, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SEPCORR_H */
