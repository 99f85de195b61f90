/*
 * monet_hip.h - C ABI of libmonet_hip.so, the gfx950 (MI355X) kernels behind
 * the low-memory operator library (the lm_ops op classes).
 *
 * Conventions shared by every entry point
 *   - Every pointer is a raw DEVICE pointer into memory owned by the caller
 *     (inputs, outputs and workspaces).  The library never allocates, frees or
 *     caches device memory and keeps no mutable global state, so it is
 *     re-entrant; the caller's allocator sees every byte that is used.  (One
 *     exception, marked as such: mn_bn_bwd_from_y_static_f32 works in a
 *     fixed device array inside the library.)
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and
 *     no entry point synchronises with the host.
 *   - Return value: MN_OK (0) or one of the MN_E* codes below.  Nothing throws
 *     or exits across the boundary.  mn_status_string() names a code.
 *   - Tensors are dense, row-major (NCHW for 4-D), fp32 unless the name says
 *     otherwise.  "In place" is allowed exactly where a comment says so.
 *
 * Each declaration cites the function of the reference implementation
 * (utsaslab/MONeT, paths relative to its root) whose role it takes over.
 */
#ifndef MONET_HIP_H
#define MONET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MN_OK 0
#define MN_EINVAL 1       /* null pointer, negative size, misaligned operand, ws too small */
#define MN_EUNSUPPORTED 2 /* shape / variant / dtype this build has no kernel for */
#define MN_ELAUNCH 3      /* hipGetLastError() reported a failed launch */
#define MN_ELIMIT 4       /* the call needs more than a fixed limit of the entry point allows */

typedef void* mn_stream_t;

/* ABI version of this header; bumped on any signature change. */
int mn_abi_version(void);
const char* mn_status_string(int status);
/* Optional.  Does now, for the CURRENT device, what a few entry points would
 * otherwise do on their first call there and what is not a stream operation:
 * looks up the address of the fixed workspace of mn_bn_bwd_from_y_static_f32
 * and raises the LDS limit of the one-kernel Winograd convolution.  A caller
 * that captures HIP graphs calls it once per device before the first capture
 * (or makes one call of those entry points outside capture); everyone else may
 * ignore it.  Idempotent, thread-safe; MN_ELAUNCH if a lookup fails.  No
 * counterpart in the reference. */
int mn_init(void);

/* ------------------------------------------------------------------ pack --
 * 1-bit pack: n bytes (each 0 or 1) -> (n+7)/8 bytes, first element in bit 7
 * of byte 0, tail bits zero.  Replaces pack / pack_ (monet/lm_ops/pack.cpp:72-98,
 * kernel monet/lm_ops/pack.cu:22-31). */
int mn_pack_bits(const uint8_t* bools, uint8_t* packed, size_t n, mn_stream_t stream);
/* Inverse: writes n bytes of 0/1.  Replaces unpack (pack.cpp:99-111, pack.cu:32-40). */
int mn_unpack_bits(const uint8_t* packed, uint8_t* bools, size_t n, mn_stream_t stream);
/* r[i] = bit(i) * v[i]; r may alias v.  Replaces unpack_multiply
 * (pack.cpp:112-131, pack.cu:41-50). */
int mn_unpack_bits_mul_f32(const uint8_t* packed, const float* v, float* r, size_t n,
                           mn_stream_t stream);
/* 4-bit pack: n bytes (each < 16) -> (n+1)/2 bytes, element 2j in the high
 * nibble of byte j, 2j+1 in the low nibble, tail nibble zero.  Replaces
 * pack_two (pack.cpp:38-54, pack.cu:3-12). */
int mn_pack_nibbles(const uint8_t* u, uint8_t* packed, size_t n, mn_stream_t stream);
/* Inverse: writes n bytes.  Replaces unpack_two (pack.cpp:55-70, pack.cu:13-21). */
int mn_unpack_nibbles(const uint8_t* packed, uint8_t* u, size_t n, mn_stream_t stream);

/* ------------------------------------------------------------------ relu --
 * Fused y = max(x, 0) (NaN propagates) and mask = pack(x > 0) in one pass.
 * y may alias x (in-place ReLU); y may be NULL to produce the mask only.
 * Replaces the clamp_min + (x > 0) + pack sequence of BinaryActReLU.forward /
 * .intermediate (monet/lm_ops/relu.py:100-107). */
int mn_relu_fwd_mask_f32(const float* x, float* y, uint8_t* mask, size_t n, mn_stream_t stream);
/* dx[i] = bit(i) ? grad[i] : grad[i] * 0 (so NaN/inf and the sign of zero
 * behave like the multiply in the reference).  dx may alias grad.  Replaces
 * unpack + in-place multiply of BinaryActReLU.backward (relu.py:109-118). */
int mn_relu_bwd_mask_f32(const float* grad, const uint8_t* mask, float* dx, size_t n,
                         mn_stream_t stream);
/* dx[i] = ref[i] > threshold ? grad[i] : 0 with ref the stored ReLU input or
 * output.  dx may alias grad.  Replaces relu_backward / threshold_kernel
 * (monet/lm_ops/lrrelu.cpp:11-20, lrrelu.cu:4-15). */
int mn_relu_bwd_ref_f32(const float* grad, const float* ref, float threshold, float* dx, size_t n,
                        mn_stream_t stream);

/* --------------------------------------------------------------- maxpool --
 * Geometry of a 2-D max pool over an NCHW tensor.  PH/PW are the output sizes
 * (mn_pool_out_size gives them). */
typedef struct mn_pool2d {
  int32_t N, C, H, W;
  int32_t kH, kW, sH, sW, pH, pW, dH, dW;
  int32_t PH, PW;
} mn_pool2d;

/* Output extent along one axis; the rule of pooling_output_shape
 * (monet/lm_ops/maxpool.cpp:54-75).  Returns -1 on invalid arguments. */
int64_t mn_pool_out_size(int64_t in, int64_t k, int64_t pad, int64_t stride, int64_t dil,
                         int ceil_mode);
/* y = max over each window; idx4 = the window-relative argmax ch*kW+cw (rows
 * and columns counted from the unclipped window origin, first maximum in
 * row-major order wins, a NaN always wins) packed two per byte like
 * mn_pack_nibbles over the flat NCHW output order.  Needs kH*kW <= 16.
 * Replaces max_pool2d_with_indices_cuda + pack_two of
 * IndicesActMaxPool2D.forward (monet/lm_ops/pool.py:43-53,
 * maxpool.cpp:369-405, kernel maxpool.cu:26-72). */
int mn_maxpool_fwd_idx_f32(const mn_pool2d* g, const float* x, float* y, uint8_t* idx4,
                           mn_stream_t stream);
/* dx[n,c,h,w] = sum of dy over the windows that cover (h,w) and whose stored
 * index names it (window rows outer, columns inner).  Writes every element of
 * dx, so dx needs no clearing.  Replaces unpack_two + zeros +
 * max_pool2d_with_indices_backward_out_cuda of IndicesActMaxPool2D.backward
 * (pool.py:55-69, maxpool.cpp:407-435, kernel maxpool.cu:81-131). */
int mn_maxpool_bwd_idx_f32(const mn_pool2d* g, const float* dy, const uint8_t* idx4, float* dx,
                           mn_stream_t stream);

/* ------------------------------------------------------------- batchnorm --
 * All BN entry points view the tensor as [N, C, HW] and reduce over N and HW.
 * Bytes of caller-provided workspace the BN entry points need for a tensor of
 * this shape (cross-workgroup partial sums). */
size_t mn_bn_ws_bytes(int64_t N, int64_t C, int64_t HW);
/* Training forward: batch mean / biased variance per channel, y = (x - mean) *
 * invstd * gamma + beta, running_mean/var updated in place with `momentum`
 * (unbiased variance), save_mean / save_invstd written.  gamma / beta may be
 * NULL (1 / 0); running_* may be NULL.  y may alias x.  Replaces do_forward
 * -> cudnn_batch_norm (monet/lm_ops/lrbn.cpp:21-41). */
int mn_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                        float* running_var, float* y, float* save_mean, float* save_invstd,
                        int64_t N, int64_t C, int64_t HW, double momentum, double eps, void* ws,
                        size_t ws_bytes, mn_stream_t stream);
/* Recompute forward from saved statistics: y = (x - mean) * invstd * gamma +
 * beta.  y may alias x.  Takes the role of the F.batch_norm call in
 * InputActBatchNorm.forward when params are set (monet/lm_ops/bn.py:32-34). */
int mn_bn_fwd_apply_f32(const float* x, const float* mean, const float* invstd, const float* gamma,
                        const float* beta, float* y, int64_t N, int64_t C, int64_t HW,
                        mn_stream_t stream);
/* Backward from the INPUT x: dgamma = sum dy*xhat, dbeta = sum dy,
 * dx = (dy - xhat*dgamma/M - dbeta/M) * invstd * gamma, xhat = (x-mean)*invstd.
 * dx may alias dy.  Replaces do_cudnn_backward -> cudnn_batch_norm_backward
 * (monet/lm_ops/lrbn.cpp:43-70). */
int mn_bn_bwd_from_x_f32(const float* dy, const float* x, const float* gamma, const float* mean,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream);
/* Backward from the OUTPUT y (the input is never read): gsum = sum dy,
 * dot = sum dy*(y-beta); dbeta = gsum, dgamma = dot/gamma,
 * dx = (dy - (y-beta)*dot/(M*gamma^2) - gsum/M) * invstd * gamma.  Undefined
 * for gamma == 0, like the reference.  dx may alias dy.  Replaces
 * output_activated_bn_backward (monet/lm_ops/lrbn.cpp:154-172, kernel
 * batch_norm_backward_kernel1 monet/lm_ops/lrbn.cu:138-209). */
int mn_bn_bwd_from_y_f32(const float* dy, const float* y, const float* gamma, const float* beta,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream);
/* The statistics-then-apply entry points above may run as ONE launch in which a
 * workgroup waits (bounded) for the other workgroups of its channel.  If such a
 * wait ever gives up (the device ran fewer workgroups at once than the launch
 * relies on), every result derived from the missing totals is NaN and an error
 * word in the workspace is raised; each launch clears the word first.
 * mn_bn_ws_status waits for `stream`, reads the word left by the LAST launch
 * that used `ws` for a tensor of this shape and returns MN_ELAUNCH if it is
 * raised; ws == NULL (ws_bytes ignored) asks about the library's own array,
 * i.e. about the last mn_bn_bwd_from_y_static_f32 call on this device.  The reference's kernel (one block per channel, lrbn.cu:212-235)
 * has no cross-block wait and so no counterpart of this call. */
int mn_bn_ws_status(const void* ws, size_t ws_bytes, int64_t N, int64_t C, int64_t HW,
                    mn_stream_t stream);
/* The same question for callers that free a workspace right after the call: a
 * wait that gives up also raises one word per device, which stays raised.
 * host_word == NULL: waits for `stream`, returns MN_ELAUNCH if any BatchNorm
 * launch on the current device gave up a wait since the last such call, and
 * clears the word.  host_word != NULL (pinned host memory): only enqueues a
 * copy of the word to *host_word on `stream` and returns at once; the caller
 * reads it when the stream has passed that point (non-zero = raised) and makes
 * the synchronous call to clear it.  No counterpart in the reference. */
int mn_bn_wait_status(uint32_t* host_word, mn_stream_t stream);
/* mn_bn_bwd_from_y_f32 with its launch parameters given explicitly (0 = the
 * default): `spin_limit` polls before a wait gives up, at most
 * `max_workgroups` persistent workgroups, pieces of `channel_group`
 * neighbouring channels handed out interleaved, `cache_hints` = 4 | 1 (loads
 * non-temporal) | 2 (stores non-temporal).  For diagnosis and for testing
 * the error path above from the host; no counterpart in the reference. */
int mn_bn_bwd_from_y_f32_limits(const float* dy, const float* y, const float* gamma,
                                const float* beta, const float* invstd, float* dx, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW, void* ws,
                                size_t ws_bytes, uint32_t spin_limit, uint32_t max_workgroups,
                                uint32_t channel_group, uint32_t cache_hints, mn_stream_t stream);

/* mn_bn_bwd_from_y_f32 for callers that cannot allocate device memory or hand
 * over a workspace (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the cross-workgroup partial sums live in a
 * fixed array of MN_BN_STATIC_WS_BYTES inside the library instead of a caller
 * workspace, and the call allocates nothing.  Same kernels, same results bit
 * for bit.  Shapes whose workspace (mn_bn_ws_bytes) exceeds the array are
 * refused with MN_ELIMIT.  Every GPU holds one copy of the array for the life
 * of the process and every call on that GPU uses it: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream do not.  No
 * counterpart in the reference. */
#define MN_BN_STATIC_WS_BYTES (4u << 20)
int mn_bn_bwd_from_y_static_f32(const float* dy, const float* y, const float* gamma,
                                const float* beta, const float* invstd, float* dx, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW,
                                mn_stream_t stream);

/* --------------------------------------------------------------- softmax --
 * The tensor is viewed as [outer, dim, inner]; softmax runs over `dim`.
 * Replaces softmax_forward (monet/lm_ops/softmax.cpp:11-15). */
int mn_softmax_fwd_f32(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner,
                       mn_stream_t stream);
/* dx = dy*y - y * sum_dim(dy*y), without materialising dy*y.  dx may alias dy.
 * Replaces softmax_backward1 (monet/lm_ops/softmax.cpp:17-33). */
int mn_softmax_bwd_f32(const float* dy, const float* y, float* dx, int64_t outer, int64_t dim,
                       int64_t inner, mn_stream_t stream);
/* Fused backward of mean-reduced softmax cross-entropy over [outer, dim,
 * inner] logits with int64 labels [outer, inner]:
 * dlogits = (softmax(logits) - onehot(label)) * scale.  The reference applies
 * the loss outside its operator library with the stock nn.CrossEntropyLoss
 * (examples/imagenet.py:199,327); this is the fused kernel for that step. */
int mn_xent_bwd_f32(const float* logits, const int64_t* labels, float* dlogits, int64_t outer,
                    int64_t dim, int64_t inner, float scale, mn_stream_t stream);

/* y = max(a + alpha*b, 0) and, if mask != NULL, the packed 1-bit mask of
 * (a + alpha*b > 0) in the format of mn_pack_bits: the residual add and the
 * ReLU behind it in one pass.  y may alias a.  No counterpart in the reference
 * (it runs AddIP, monet/lm_ops/funcs.py:41-59, then a ReLU operator); the
 * backward of the pair is mn_relu_bwd_mask_f32 / mn_relu_bwd_ref_f32 on y. */
int mn_add_relu_fwd_f32(const float* a, const float* b, float alpha, float* y, uint8_t* mask,
                        size_t n, mn_stream_t stream);

/* BatchNorm fused with the ReLU that follows it (no counterpart in the
 * reference, whose executor runs them as two operators, monet/lm_ops/bn.py and
 * relu.py; fusing saves one read and one write of the activation in each
 * direction and needs no mask, because the backward recomputes the sign of the
 * pre-activation from the stored INPUT).
 *   forward (training):   y = max(BN(x), 0), statistics as mn_bn_fwd_train_f32
 *   forward (saved stats): y = max((x-mean)*invstd*gamma + beta, 0)
 *   backward: dy is the gradient of the ReLU OUTPUT; g = dy where
 *             (x-mean)*invstd*gamma + beta > 0, else 0; then as
 *             mn_bn_bwd_from_x_f32 with g in place of dy.  dx may alias dy. */
int mn_bn_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                             float* running_mean, float* running_var, float* y, float* save_mean,
                             float* save_invstd, int64_t N, int64_t C, int64_t HW, double momentum,
                             double eps, void* ws, size_t ws_bytes, mn_stream_t stream);
int mn_bn_relu_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                             const float* gamma, const float* beta, float* y, int64_t N, int64_t C,
                             int64_t HW, mn_stream_t stream);
int mn_bn_relu_bwd_from_x_f32(const float* dy, const float* x, const float* gamma,
                              const float* beta, const float* mean, const float* invstd, float* dx,
                              float* dgamma, float* dbeta, int64_t N, int64_t C, int64_t HW,
                              void* ws, size_t ws_bytes, mn_stream_t stream);

/* The end of a residual block as ONE forward operator (no counterpart in the
 * reference, which runs F.batch_norm, bn.py:12-54, then `out += identity`,
 * funcs.py:34-59, then a ReLU, relu.py: five passes over the activation where
 * this kernel makes three):
 *   forward (training):    y = max(BN(x) + alpha * added, 0), statistics of x as
 *                          mn_bn_fwd_train_f32
 *   forward (saved stats): y = max((x-mean)*invstd*gamma + beta + alpha * added, 0)
 * `added` has the shape of x.  y may alias `added` or x.
 *   backward: g = dy where y > 0, else 0 (the ReLU backward from the stored
 *             output, relu.py:31-52); dadded = alpha * g; (dx, dgamma, dbeta) as
 *             mn_bn_bwd_from_x_f32 with g in place of dy.  One pass: reads dy,
 *             x, y once, writes dx and dadded once (channels short enough for
 *             one workgroup run as two launches instead).  dadded may alias dy. */
int mn_bn_add_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                                 float* running_mean, float* running_var, const float* added,
                                 double alpha, float* y, float* save_mean, float* save_invstd,
                                 int64_t N, int64_t C, int64_t HW, double momentum, double eps,
                                 void* ws, size_t ws_bytes, mn_stream_t stream);
int mn_bn_add_relu_bwd_f32(const float* dy, const float* x, const float* y, const float* gamma,
                           const float* mean, const float* invstd, double alpha, float* dx,
                           float* dadded, float* dgamma, float* dbeta, int64_t N, int64_t C,
                           int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream);
/* The same operator keeping a 1-bit mask of y > 0 (format of mn_pack_bits_u8 /
 * mn_relu_fwd_mask_f32: (N*C*HW + 7) / 8 bytes over the flat tensor, first
 * element in bit 7) instead of relying on y in the backward: the forward writes
 * the mask from the registers that hold y (planes of a multiple of 8 elements;
 * other shapes pack y in a second launch), the backward reads dy, x and the
 * mask and writes dx and dadded: 4 + 1/32 passes instead of 5. */
int mn_bn_add_relu_mask_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                                      float* running_mean, float* running_var, const float* added,
                                      double alpha, float* y, uint8_t* mask, float* save_mean,
                                      float* save_invstd, int64_t N, int64_t C, int64_t HW,
                                      double momentum, double eps, void* ws, size_t ws_bytes,
                                      mn_stream_t stream);
int mn_bn_add_relu_mask_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                                      const float* gamma, const float* beta, const float* added,
                                      double alpha, float* y, uint8_t* mask, int64_t N, int64_t C,
                                      int64_t HW, mn_stream_t stream);
int mn_bn_add_relu_mask_bwd_f32(const float* dy, const float* x, const uint8_t* mask,
                                const float* gamma, const float* mean, const float* invstd,
                                double alpha, float* dx, float* dadded, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW, void* ws,
                                size_t ws_bytes, mn_stream_t stream);
int mn_bn_add_relu_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                                 const float* gamma, const float* beta, const float* added,
                                 double alpha, float* y, int64_t N, int64_t C, int64_t HW,
                                 mn_stream_t stream);

/* ----------------------------------------------------------- convolution --
 * 2-D convolution over NCHW tensors, weights [K, C, R, S], groups == 1.
 * P/Q are the output sizes: floor((H + 2*pH - dH*(R-1) - 1) / sH) + 1. */
typedef struct mn_conv2d {
  int32_t N, C, H, W;
  int32_t K, R, S;
  int32_t sH, sW, pH, pW, dH, dW;
  int32_t P, Q;
  int32_t groups;
} mn_conv2d;

#define MN_CONV_FWD 0
#define MN_CONV_BWD_DATA 1
#define MN_CONV_BWD_WEIGHT 2
#define MN_F32 0 /* fp32 NCHW tensors, weights [K,C,R,S], fp32 matrix-core arithmetic */
/* bf16 tensors in channels-last order - activations [N,H,W,C], weights
 * [K,R,S,C], outputs [N,P,Q,K], bias bf16 - multiplied on the bf16 matrix
 * cores with fp32 accumulation and rounded once (to nearest even) on output.
 * Needs channel counts that are multiples of 32 on the reduction side
 * (forward: C; backward-data: K) and multiples of 64 for backward-weight (C and
 * K); otherwise MN_EUNSUPPORTED.  Two variants per direction, further ones
 * are fp32 only.  Forward and backward-data: variant 0 reads the weight rows
 * where they lie (forward: no workspace; backward-data: the transposed
 * weights, K*C*R*S*2 bytes), variant 1 a copy packed in fragment order in
 * the workspace (rows padded to 32: one contiguous KB per fragment), which
 * the multiplying wavefronts load straight into registers.  Backward-weight:
 * fp32 split partials in the workspace, added in a fixed order; variant 1 is
 * the large-tile kernel (both channel counts multiples of 128, at least 4096
 * output positions; other shapes run variant 0's kernel), twice as fast at
 * the ResNet-50 layer3 shape - ask mn_conv_ws_bytes for either.  The
 * reference has no reduced-precision path; this dtype serves the bf16
 * configuration of the layer3 benchmark. */
#define MN_BF16 1

/* Number of kernel variants ("algorithms") per direction; variant 0 always
 * runs and needs no workspace.  Takes the role of n_fwd_algos / n_bwd_ip_algos
 * / n_bwd_wt_algos (monet/lm_ops/conv.cpp:728-730); the variants are this
 * library's own memory / speed tiers, not cuDNN's algorithm list
 * (conv.cpp:21-46):
 *   forward          0 implicit GEMM, weights read in place, no workspace
 *                    1 same with the weights repacked [tap][c][k] (k padded
 *                      to a multiple of 128) into the workspace, so operand
 *                      tiles load as full 16-byte vectors; channel counts
 *                      that are not a multiple of 16 run it like variant 0,
 *                      except the 3 -> 64 channel 7x7 / stride 2 / padding 3
 *                      stem, which runs a kernel of its own (workspace: the
 *                      transposed weights, 148 x 64 floats).
 *                      Launches with few, long workgroups split the reduction
 *                      in TWO and add the slices with atomics into a cleared
 *                      output: 0 + a + b and 0 + b + a round identically, so
 *                      the forward gives the same bits on every run (a
 *                      recomputed forward must reproduce masks and indices)
 *                    2 Winograd F(2x2, 3x3) for 3x3 filters with stride 1 and
 *                      dilation 1 over a multiple of 16 input channels
 *                      (MN_EUNSUPPORTED otherwise, and for MN_BF16): 2.25 times
 *                      fewer multiplications, paid for with a workspace of 16
 *                      floats per 2x2 output tile and channel, input and output
 *                      side, capped at 512 MB: a larger problem runs in slices
 *                      of tiles through the same buffers (the role of the
 *                      reference's WINOGRAD_NONFUSED slot,
 *                      monet/lm_ops/conv.cpp:21-27, :314-324)
 *                    3 the same algorithm in one kernel: source patches and
 *                      weights are transformed on the way into LDS and the 16
 *                      products of a block of 64 outputs x 64 tiles stay in
 *                      registers until the output transform, so the only
 *                      workspace is the transformed weights (16 * C *
 *                      pad128(K) floats; the role of the reference's fused
 *                      WINOGRAD slot).  Same shapes as variant 2, tensors
 *                      below 2 GB (MN_EUNSUPPORTED otherwise, and on a device
 *                      that does not grant a workgroup 80 KB of LDS); faster
 *                      than variant 2 where channels are few and planes large
 *                    4 fp32 on the bf16 matrix cores: every fp32 operand is cut
 *                      into three bf16 slices (x = x0 + x1 + x2, the remainders
 *                      exact) and the six slice products down to 2^-16 of the
 *                      full product are accumulated in fp32, which keeps fp32
 *                      accuracy (measured 1e-7..5e-7 of the output's scale,
 *                      like the fp32 matrix instruction) at 3/8 of its matrix
 *                      time.  1x1 filters, stride 1, no padding, H*W a
 *                      multiple of 4, C a multiple of 16, tensors below 2 GB
 *                      (MN_EUNSUPPORTED otherwise, and for MN_BF16).
 *                      Workspace: the three slices of the weights, rows padded
 *                      to 256 (3 * pad256(K) * C * 2 bytes).  Non-finite inputs
 *                      give NaN.  Takes the place of the reference's slots
 *                      that trade workspace for time on shapes Winograd cannot
 *                      take (monet/lm_ops/conv.cpp:21-46)
 *   backward-data    0 implicit GEMM reading the weights through strides
 *                    1 same with the weights repacked [tap][k][c] (c padded
 *                      to a multiple of 128) into the workspace; may split
 *                      the reduction up to 8 ways and add the slices with
 *                      atomics (last bits can differ from run to run; variant
 *                      0 never does)
 *                    2 Winograd F(2x2, 3x3), as for the forward (the filter
 *                      rotated by 180 degrees, channel roles swapped)
 *                    3 the one-kernel Winograd form, as for the forward
 *                    4 three bf16 slices per operand, as for the forward (K
 *                      a multiple of 16; the weights are transposed as they
 *                      are split)
 *   backward-weight  0 split reduction combined with atomics into a cleared dw
 *                    1 split reduction through per-split partials in the
 *                      workspace, then a fixed-order sum (reproducible); the
 *                      3 -> 64 channel 7x7 / 2 stem runs a kernel of its own
 *                      (workspace: one 64 x 148 partial result per workgroup)
 *                    2 Winograd (the transposed form of F(2x2, 3x3): the 16
 *                      transform-domain products reduced over the 2x2 output
 *                      tiles): 3x3, stride 1, dilation 1, C a multiple of 4,
 *                      fp32; workspace of 16 floats per tile and channel for
 *                      dy and x (capped at 512 MB: more tiles are taken in
 *                      passes added in order) plus the partial results;
 *                      reproducible
 *                    3 the same algorithm in one kernel: both transforms are
 *                      applied on the way into LDS, no transformed tensors in
 *                      memory; padding 1, even height, W a multiple of 4,
 *                      K and C multiples of 64; workspace: the partial
 *                      results of at most one range of tile rows per CU
 *                      (16 * ranges * K * C floats, and ranges * K for the
 *                      bias gradient, which the same kernel sums from the
 *                      tiles it stages); reproducible.  The
 *                      faster form below 256 channels and on large planes */
int mn_conv_n_variants(int direction);
/* The same per dtype: the list above for MN_F32; 2 for MN_BF16 (see MN_BF16);
 * 0 for an unknown dtype.  The reference is fp32 only and has no counterpart. */
int mn_conv_n_variants_for(int direction, int dtype);
/* Workspace bytes a (direction, variant, dtype) needs for this geometry
 * (role of the cudnnGet*WorkspaceSize queries at conv.cpp:314-324). */
int mn_conv_ws_bytes(const mn_conv2d* g, int direction, int variant, int dtype, size_t* bytes);
/* y = conv(x, w) (+ bias[k] if bias != NULL).  Replaces cudnn_convolution
 * (monet/lm_ops/conv.cpp:389-400, raw call :299-340) plus the bias add of
 * conv.py:284-285.  MN_EUNSUPPORTED for a variant that cannot run the shape. */
int mn_conv_fwd(const mn_conv2d* g, const void* x, const void* w, const void* bias, void* y,
                void* ws, size_t ws_bytes, int variant, int dtype, mn_stream_t stream);
/* dx = gradient w.r.t. the input; writes every element of dx.  Replaces
 * cudnn_convolution_backward_input (conv.cpp:503-515, raw call :409-449). */
int mn_conv_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                     size_t ws_bytes, int variant, int dtype, mn_stream_t stream);
/* dx += gradient w.r.t. the input (fp32 only): the same kernels with an
 * accumulating epilogue, for a caller that would otherwise add the result to
 * a gradient it already holds (a residual join).  cuDNN offers this as beta = 1
 * in cudnnConvolutionBackwardData; the reference always passes beta = 0
 * (conv.cpp:409-449) and adds afterwards (monet/schedule.py:295-301). */
int mn_conv_bwd_data_accumulate(const mn_conv2d* g, const void* dy, const void* w, void* dx,
                                void* ws, size_t ws_bytes, int variant, int dtype,
                                mn_stream_t stream);
/* dw = gradient w.r.t. the weights; writes every element of dw.  Replaces
 * cudnn_convolution_backward_weight (conv.cpp:676-688, raw call :550-591). */
int mn_conv_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* ws,
                       size_t ws_bytes, int variant, int dtype, mn_stream_t stream);
/* The same, and db[k] = sum over (n, p, q) of dy[n,k,p,q] (fp32, K elements)
 * from the dy tiles the weight-gradient kernel fetches anyway: no separate
 * pass over dy.  fp32 only (MN_EUNSUPPORTED for MN_BF16).  The reference
 * computes the bias gradient with a separate reduction, grad.sum([0,2,3])
 * (monet/lm_ops/conv.py:314).  Variant 1 stays reproducible run to run
 * (per-split partial sums in the workspace, added in a fixed order). */
int mn_conv_bwd_weight_bias(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* db,
                            void* ws, size_t ws_bytes, int variant, int dtype,
                            mn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MONET_HIP_H */
