/*
 * fitre_hip.h -- C-ABI of the MI355X (gfx950) device layer.
 *
 * This is the whole boundary between the C host code and the HIP kernels:
 * plain pointers and sizes, no C++ or framework types.  It replaces the
 * reference's device/cuda_environment.[ch], device/cuda_utils.[ch],
 * device/handles.h, device/query.c, and every cuBLAS call and __global__
 * kernel reached from cnnForward / cnnBackward.
 *
 * Conventions
 *   - every function returns 0 on success and a non-zero FITRE_E_* code on
 *     failure; fitre_hip_last_error() then describes the failure;
 *   - all tensor pointers are device pointers; work is queued on the layer's
 *     own stream and is NOT complete on return unless stated -- call
 *     fitre_hip_sync() before reading results on the host;
 *   - activations are [C][N][A][B] reals, B fastest (the reference's
 *     column-major (N*H*W) x C matrix with A = image column, B = image row);
 *   - "ws" arguments are caller-provided device workspaces of at least the
 *     number of bytes the matching *_workspace() function returns.
 */
#ifndef FITRE_HIP_H
#define FITRE_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FITRE_OK            0
#define FITRE_E_DEVICE      1 /* a HIP runtime call failed */
#define FITRE_E_ARGUMENT    2 /* null pointer, non-positive size, inconsistent shape */
#define FITRE_E_UNSUPPORTED 3 /* activation / pooling code or shape the kernels do not cover */
#define FITRE_E_WORKSPACE   4 /* workspace smaller than required */

/* ---------------- environment (device/cuda_environment.c:29-77, device/query.c:7-49) ---------------- */
int fitre_hip_init(int device);
int fitre_hip_shutdown(void);
int fitre_hip_sync(void);
const char *fitre_hip_last_error(void);
/* compute units, wavefront size, max threads per block, total and free bytes; name may be NULL */
int fitre_hip_device_info(int *computeUnits, int *waveSize, int *maxThreadsPerBlock, size_t *totalBytes,
                          size_t *freeBytes, char *name, int nameLen);
/* the hipStream_t of the selected lane, as an opaque pointer */
void *fitre_hip_stream(void);
/* The layer owns four streams ("lanes" 0..3, all at default priority).  Every call queues its work on the
 * selected lane (0 after init).  A caller that has independent chains of work may put them on different
 * lanes and order them with fitre_hip_lane_wait(waiter, signaller): work queued on `waiter` after the
 * call starts only when everything queued on `signaller` before the call has finished.  The backward
 * pass uses lanes 0 and 1, the KFAC inverse passes all four.  fitre_hip_sync() waits for every lane.  While per-launch accounting is on (fitre_hip_profile_enable)
 * lane selection is ignored and everything runs on lane 0, so that launch durations are unshared.
 * No counterpart in the reference, which runs on the null stream and synchronises after every launch. */
int fitre_hip_lane_select(int lane);
/* on = 0: every later fitre_hip_lane_select() picks lane 0 (strictly serial execution, e.g. under a
 * kernel tracer whose per-kernel durations should not overlap); on = 1 (the default) restores lanes. */
int fitre_hip_lanes_enable(int on);
int fitre_hip_lane_wait(int waiter, int signaller);
/* The 3 x 3 weight gradients (fitre_hip_conv_weight_grad and its relatives on maps up to 32 cells wide) are cut into
 * workgroups for `eighths` eighths of the compute units (4 to 8; 8, the default: all of them), so that the rest of the
 * chip stays free for whatever the caller runs beside them on another lane.  The setting changes how a reduction is
 * split, hence the last bits of a result: a caller that wants the same bits with and without lanes keeps it the same
 * in both.  cnnBackward sets it per layer from the network (include/fitre_cnn.h) and restores 8.  No counterpart in
 * the reference (one stream). */
int fitre_hip_weight_grad_share(int eighths);

/* ---------------- memory (device/cuda_utils.c; device/cuda_utils.h:15-26) ---------------- */
int fitre_hip_malloc(void **ptr, size_t bytes);
int fitre_hip_free(void *ptr);
int fitre_hip_malloc_host(void **ptr, size_t bytes); /* pinned */
int fitre_hip_free_host(void *ptr);
int fitre_hip_memset(void *ptr, int value, size_t bytes);          /* stream-ordered */
int fitre_hip_copy_h2d(void *dev, const void *host, size_t bytes); /* complete on return */
int fitre_hip_copy_d2h(void *host, const void *dev, size_t bytes); /* complete on return */
int fitre_hip_copy_d2d(void *dst, const void *src, size_t bytes);  /* stream-ordered */

/* ---------------- timing ---------------- */
/* Events on the layer's stream. */
int fitre_hip_event_create(void **event);
int fitre_hip_event_destroy(void *event);
int fitre_hip_event_record(void *event);
int fitre_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for stop */

/* Per-kernel-class accounting: while enabled, every launch is bracketed by
 * events on the stream and attributed to one FITRE_KC_* class together with
 * its algorithmic work (flops for GEMM classes, bytes for the others). */
enum fitre_kernel_class {
	FITRE_KC_CONV_DW = 0,
	FITRE_KC_CONV_DX = 1,
	FITRE_KC_CONV_FWD = 2,
	FITRE_KC_FC_GEMM = 3,
	FITRE_KC_SPLITK_REDUCE = 4,
	FITRE_KC_BN_BWD = 5,
	FITRE_KC_BN_FWD = 6,
	FITRE_KC_POOL_BWD = 7,
	FITRE_KC_POOL_FWD = 8,
	FITRE_KC_ACT_BWD = 9,
	FITRE_KC_ACT_FWD = 10,
	FITRE_KC_BIAS_GRAD = 11,
	FITRE_KC_SOFTMAX = 12,
	FITRE_KC_PERMUTE = 13,
	FITRE_KC_BLAS1 = 14,
	FITRE_KC_POOL_ACT_BWD = 15,
	FITRE_KC_KFAC_FACTOR = 16,
	FITRE_KC_SPD_INVERSE = 17,
	FITRE_KC_COUNT = 18
};
int fitre_hip_profile_enable(int on); /* on=1 clears the counters and starts; on=0 stops */
/* launches, summed milliseconds and summed algorithmic work of one class (syncs first) */
int fitre_hip_profile_read(int kernelClass, long *launches, double *milliseconds, double *work);
/* The MFMA classes run one of several tile instantiations of the same kernel template; tile selects
 * one: 0 = not tiled, 1 = 64x64, 2 = 64x128, 3 = 128x64, 4 = 128x128, 5 = 96x128 (channel rows x contiguous columns);
 * 6 and 7 are the 3x3 convolution kernels that leave out the arithmetic on the padding: 6 = the dense per-image form
 * on 2x2 maps, 7 = the cell form on 4x4 maps, 8 = the cell form of the weight gradient on 8x8 maps (their work is
 * still counted as the nine-tap 2*M*K*Cout); 9 = the weight gradient of a wide linear layer at a batch of at most 64
 * (the whole reduction in registers). */
#define FITRE_TILE_VARIANTS 10
int fitre_hip_profile_read_tile(int kernelClass, int tile, long *launches, double *milliseconds, double *work);
/* The accounted launches one by one, in issue order since the last fitre_hip_profile_enable(1) (at most 65 536
 * are kept): class, tile variant, duration and algorithmic work of launch `index` < *count. */
int fitre_hip_profile_launch_count(long *count);
int fitre_hip_profile_read_launch(long index, int *kernelClass, int *tile, double *milliseconds, double *work);

/* ---------------- level-1 helpers (the cublasD* calls of the solvers and of
 * functions/cnn_gradient.cu:54-56, functions/softmax_loss.cu:243) ---------------- */
int fitre_hip_axpy(int n, float alpha, const float *x, float *y);         /* y += alpha x */
int fitre_hip_scal(int n, float alpha, float *x);                         /* x *= alpha */
int fitre_hip_copy(int n, const float *x, float *y);                      /* y = x */
/* dst[c*ldd + r] = src[c*lds + r], r < rows, c < cols: cudaMemcpy2D device-to-device as the reference
 * uses it (solvers/kfac_inverses.cu:596-600, kfac_natural_gradient.cu:107-111), widths in elements.
 * Leading dimensions below `rows` are allowed (ld 1 with rows 1 walks a strided vector). */
int fitre_hip_copy_2d(float *dst, long ldd, const float *src, long lds, int rows, int cols);
/* C(m x n) = alpha * op(A) + beta * op(B), column-major, with the argument meaning of cublasDgeam as the
 * reference's solvers use it to transpose (solvers/kfac_natural_gradient.cu:166-170: OP_T, OP_N, beta = 0, B = NULL).
 * transA / transB: 0 = N, 1 = T.  A null operand needs a zero coefficient; C may alias an untransposed operand
 * that has the same leading dimension. */
int fitre_hip_geam(int transA, int transB, int m, int n, float alpha, const float *A, int lda, float beta, const float *B,
                   int ldb, float *C, int ldc);
int fitre_hip_dot(int n, const float *x, const float *y, float *result);  /* host result, complete on return */
int fitre_hip_nrm2(int n, const float *x, float *result);                 /* host result */
int fitre_hip_asum(int n, const float *x, float *result);                 /* host result */
int fitre_hip_norm_inf(int n, const float *x, float *result);             /* device/reduce.cu:110-153 kerNormInf */
int fitre_hip_sum(int n, const float *x, float *result);                  /* utilities/reduce.cu:32-84 */

/* ---------------- elementwise helpers ---------------- */
/* Output heads of the fully connected models (functions/eval_gradient.cu:231-555).
 * column_softmax: x[:, c] = exp(x[:, c]) / sum_r exp(x[r, c]) in place, column-major rows x cols, no
 * maximum shift (kerNNApplyExp + Dgemv column sums + kerNNComputeSoftmax, eval_gradient.cu:162-193).
 * output_terms: out[i] = f(y[i], z[i]) with
 *   SCALED_DIFFERENCE   scale*(y - z)                     kerNNComputeLayerError, dev_layer_error.cu:4-11
 *   SQUARED_DIFFERENCE  (y - z)^2                         kerNNComputeLogLikelihoodLinear / kerNNComputeModelError
 *   LOGISTIC_LL         z*(y - [z>=0]) - log(1 + exp(z - 2 z [z>=0]))   (z = logit) dev_loglikelihood.cu:22-41
 *   SOFTMAX_LL          y*log(z)                          dev_loglikelihood.cu:4-11 */
#define FITRE_TERM_SCALED_DIFFERENCE  0
#define FITRE_TERM_SQUARED_DIFFERENCE 1
#define FITRE_TERM_LOGISTIC_LL        2
#define FITRE_TERM_SOFTMAX_LL         3
int fitre_hip_column_softmax(float *x, int rows, int cols);
int fitre_hip_output_terms(int kind, const float *y, const float *z, long n, float scale, float *out);

/* Seeded generator replacing the cuRAND handle of device/gen_random.cu:25-52: a counter-based
 * stream (splitmix64 of seed and position; restated in the test oracle), uniform in (0, 1] resp.
 * standard normal (Box-Muller on consecutive pairs).  Each call continues the stream;
 * fitre_hip_random_seed() restarts it.  Default seed 1234 (gen_random.cu:36). */
int fitre_hip_random_seed(unsigned long long seed);
int fitre_hip_random_uniform(float *out, long n);
int fitre_hip_random_normal(float *out, long n);
int fitre_hip_fill(float *x, long n, float value);                        /* dev_initializations.cu:7-14, dev_activations.cu:89-95 */
int fitre_hip_hadamard(const float *x, float *y, long n);                 /* y *= x                  dev_hadamard.cu:4-10 */
int fitre_hip_hadamard2(const float *m1, const float *m2, const float *m3, const float *m4, long n,
                        float *out);                                      /* out = m1*m2 + m3*m4     dev_hadamard.cu:12-20 */
int fitre_hip_elem_inv_scale(const float *x, const float *y, float eps, long n, float *out);
                                                                          /* out = x/(sqrt(y)+eps)   dev_elem_scale.cu */
int fitre_hip_elem_sqr(const float *x, long n, float *out);               /* out = x*x               dev_elem_sqr.cu */
int fitre_hip_elem_sqr_decay(const float *x, const float *y, float decay, long n, float *out);
                                                                          /* out = decay*x+(1-decay)*y*y  dev_elem_sqr_decay.cu */
int fitre_hip_mat_mat_scale(const float *x, const float *y, long n, float *out); /* out = x*y        dev_mat_mat_scale.cu */
int fitre_hip_mat_row_vec_scale(const float *x, int rows, int cols, const float *y, float *out);
                                                                          /* out[i] = x[i]*y[i/rows] dev_mat_vec_scale.cu */
int fitre_hip_add_column(float *mat, int rows, int cols, const float *vec); /* mat[:,c] += vec; column-major  dev_mat_vec_addition.cu:6-17 */
int fitre_hip_add_channel_bias(float *x, int channels, long perChannel, const float *bias); /* eval_convolution.cu:26-34 */

/* ---------------- activations (codes of ACTIVATION_FUNCTIONS / CNN_ACTIVATION_FUNCTIONS) ---------------- */
/* out = f(in); in == out allowed.  dev_activations.cu:8-95, swish.cu:14-23 */
int fitre_hip_activation_forward(int actFun, const float *in, float *out, long n);
/* out = delta * f'(.) ; z_in = activation input, z_out = activation output; out == delta allowed.
 * swish.cu:34-43, dev_layer_error.cu:13-48; ReLU uses z_out > 0. */
int fitre_hip_activation_backward(int actFun, const float *delta, const float *z_in, const float *z_out,
                                  float *out, long n);

/* ---------------- pooling on [C][N][A][B] (functions/dev_pool.cu) ---------------- */
/* poolType: 0 max, 1 average.  inA/inB = input extent along A/B; window origin k*stride - padding. */
int fitre_hip_pool_forward(int poolType, const float *in, int channels, int samples, int inA, int inB,
                           int ksize, int stride, int padding, int outA, int outB, float *out);
/* Max pool: delta at the first maximum in memory order (strict >), zero elsewhere; overlapping
 * windows add.  Average pool: delta / ksize^2 spread over the window.  dev_pool.cu:269-298,346-398 */
int fitre_hip_pool_backward(int poolType, const float *delta, const float *z_in, int channels, int samples,
                            int inA, int inB, int ksize, int stride, int padding, int outA, int outB,
                            float *out);
/* argmax offset inside each A x B map for every pooled cell (int32, layout of the pooled tensor) */
int fitre_hip_max_pool_argmax(const float *z_in, int channels, int samples, int inA, int inB, int ksize,
                              int stride, int padding, int outA, int outB, int *index);
/* Fused max/avg/no pool backward + activation backward: writes dxPool (pool-backward result) and
 * dxAct = dxPool * f'(.).  poolType 2 = no pooling (delta has the input extent). */
int fitre_hip_pool_act_backward(int poolType, int actFun, const float *delta, const float *z_in,
                                const float *z_act, int channels, int samples, int inA, int inB,
                                int ksize, int stride, int padding, int outA, int outB, float *dxPool,
                                float *dxAct);

/* ---------------- batch normalisation, non-affine, per channel over N*A*B (functions/dev_batch_norm.cu) ---------------- */
size_t fitre_hip_batch_norm_workspace(int channels, long perChannel);
/* train != 0: batch mean / biased variance, running = momentum*running + (1-momentum)*batch,
 * zhat = (x-mean)/sqrt(var+eps); train == 0: normalise with the running statistics.  :263-393 */
int fitre_hip_batch_norm_forward(const float *in, int channels, long perChannel, float *zhat, float *mean,
                                 float *variance, float *runningMean, float *runningVariance,
                                 float epsilon, float momentum, int train, void *ws, size_t wsBytes);
/* fitre_hip_batch_norm_forward, fitre_hip_activation_forward of its zhat and fitre_hip_pool_forward of that, as the
 * forward pass runs them for a convolution layer (functions/cnn_forward.cu:124-205): after the statistics, ONE pass
 * reads the convolution output and writes zhat, the activation output and the pooled output (the three passes read
 * four tensors for the same results; the values are the same bit for bit).  zhat NULL: a layer without batch norm, `in`
 * goes into the activation as it is (the statistics pointers are not used).  poolType NO_POOL: poolOut and the
 * window arguments are not used.  Fused for no pooling and for 2x2 / stride 2 max pooling (A even, B a multiple of 4,
 * 16-byte-aligned tensors); every other case runs the separate passes.  Workspace (with batch norm):
 * fitre_hip_batch_norm_workspace(channels, samples * inA * inB). */
int fitre_hip_bn_act_pool_forward(const float *in, int channels, int samples, int inA, int inB, float *zhat, float *mean,
                                  float *variance, float *runningMean, float *runningVariance, float epsilon,
                                  float momentum, int train, int actFun, float *actOut, int poolType, int ksize,
                                  int stride, int padding, int outA, int outB, float *poolOut, void *ws, size_t wsBytes);
/* out = (m*delta - sum(delta) - zhat*sum(delta*zhat)) / (m*sqrt(eps+var)), m = perChannel.  :550-621.
 * biasGrad (may be NULL) receives the per-channel sum of out. */
int fitre_hip_batch_norm_backward(const float *delta, const float *zhat, const float *variance,
                                  int channels, long perChannel, float epsilon, float *out,
                                  float *biasGrad, void *ws, size_t wsBytes);
/* The same step for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-(channel, segment) partial sums live in a file-scope device array of FITRE_HIP_STATIC_SCRATCH_BYTES that
 * every GPU the library runs on holds until the process ends; the call makes no hipMalloc / hipFree and no
 * allocating library call.  Shapes whose partial sums (fitre_hip_batch_norm_workspace) exceed the array are
 * rejected with FITRE_E_WORKSPACE.  All calls on one GPU share that GPU's array: calls that overlap on one GPU
 * (two lanes, two host threads) race; calls queued on one lane do not.  Results are bit-identical to
 * fitre_hip_batch_norm_backward on the same inputs. */
#define FITRE_HIP_STATIC_SCRATCH_BYTES (1 << 20)
int fitre_hip_batch_norm_backward_static(const float *delta, const float *zhat, const float *variance,
                                         int channels, long perChannel, float epsilon, float *out,
                                         float *biasGrad);

/* fitre_hip_pool_act_backward followed by fitre_hip_batch_norm_backward of its dxAct, as the backward pass
 * runs them for a layer with batch norm (functions/cnn_backward.cu:586-660): the pool/activation pass leaves the
 * batch-norm sums behind, so the batch-norm step moves 12 bytes per element instead of 20.  zhat is the
 * activation input (the batch-norm output).  z_act may be NULL when actFun is ReLU: the activation output is
 * then taken as max(zhat, 0), bit-identical to what the forward pass stored.  Fused for no pooling and for
 * 2x2 / stride 2 max pooling on 16-byte-aligned tensors; every other case runs the two separate passes.
 * delta may be given as deltaSplits > 1 slabs deltaStride floats apart whose sum, in slab order, is the
 * gradient (the view fitre_hip_conv_input_grad_split leaves; the unfused fallback sums them into the first
 * slab); deltaSplits = 1 for a plain tensor.
 * Workspace: fitre_hip_batch_norm_workspace(channels, samples * inA * inB). */
int fitre_hip_pool_act_bn_backward(int poolType, int actFun, float *delta, int deltaSplits, long deltaStride,
                                   const float *zhat, const float *z_act, const float *variance, int channels,
                                   int samples, int inA, int inB, int ksize, int stride, int padding, int outA,
                                   int outB, float epsilon, float *dxPool, float *dxAct, float *dxBn,
                                   float *biasGrad, void *ws, size_t wsBytes);

/* ---------------- mini-batch selection and augmentation ---------------- */
/* tgt column j = src column indices[j], columns of `rows` values (kerExtractColumns,
 * device/extract_columns.cu:8-20).  indices is a device array. */
int fitre_hip_extract_columns(float *tgt, const float *src, const int *indices, int rows, int columns);
/* The layer-0 input in one pass: out[c][n][col][row] (height = rows, fastest) gathered from `sampled`,
 * which is [samples][channels][cells] when sampleMajor (reshapeMatrix of solvers/kfac_da.cu:37) or already
 * channel-major; cropUniforms (2*samples device values in (0, 1], row shifts then column shifts, or NULL):
 * shift by trunc(100 u) mod (2 padding + 1) - padding, cells from outside read `fill`
 * (augmentation/dev_crop.cu:10-58); flipUniforms (samples values or NULL): below 0.5 the image is mirrored
 * along the width axis (dev_flip.cu:68-104; the crop applies to the unflipped image, as in the reference's
 * order); mean/stdv (HOST arrays of `channels` values, or NULL): x = (x / scale - mean[c]) / stdv[c]
 * (dev_normalize.cu:12-36), applied to filled cells too.  In place only for the normalisation alone. */
int fitre_hip_augment_batch(const float *sampled, int sampleMajor, int samples, int channels, int height,
                            int width, const float *cropUniforms, int padding, float fill,
                            const float *flipUniforms, const float *mean, const float *stdv, float scale,
                            float *out);
/* the two kernels of randomCrop on their own (dev_crop.cu:52-58 and 10-50, channel-major images) */
int fitre_hip_crop_shifts(const float *uniforms, int count, int padding, int *shifts);
int fitre_hip_shift_images(const float *in, int samples, int channels, int height, int width,
                           const int *shiftRow, const int *shiftCol, float fill, float *out);

/* ---------------- reductions ---------------- */
/* out[c] = sum of the perChannel contiguous values of channel c (conv bias gradient,
 * functions/cnn_backward.cu:662-689). */
size_t fitre_hip_channel_sum_workspace(int channels, long perChannel);
int fitre_hip_channel_sum(const float *x, int channels, long perChannel, float *out, void *ws,
                          size_t wsBytes);
/* out[r] = sum over columns of a column-major rows x cols matrix (FC bias gradient, :212-224). */
int fitre_hip_row_sum(const float *mat, int rows, int cols, float *out);

/* ---------------- softmax cross entropy (functions/softmax_loss.cu:17-79,141-245) ---------------- */
/* logits/probs/errors: classes x rows, class fastest; target: 1-based class ids as float.
 * probs = softmax + 1e-10; errors = (probs - onehot)/rows; *lossHost = mean(-log probs[target]),
 * written to host memory, complete on return.  errors may be NULL. */
int fitre_hip_softmax_cross_entropy(const float *logits, const float *target, int rows, int classes,
                                    float *probs, float *errors, float *lossHost);
/* errors = (probs - onehot)/rows only (computeCrossEntropyError, :231-245) */
int fitre_hip_cross_entropy_error(const float *probs, const float *target, int rows, int classes,
                                  float *errors);
/* hits[r] = 1 if the first class of largest probability equals the 1-based label target[r], else 0
 * (ker_compute_accuracy, functions/cnn_accuracy.cu:15-37: strict '<' scan starting from probability 0). */
int fitre_hip_accuracy_hits(const float *probs, const float *target, int rows, int classes, float *hits);
/* out[r] = 1-based class drawn from row r of probs by inverting the cumulative sum at uniforms[r]
 * (ker_compute_dist_classes, functions/dev_dist_errors.cu:12-35; classes + 1 when rounding keeps the
 * cumulative sum below the draw). */
int fitre_hip_multinomial_classes(const float *probs, const float *uniforms, int samples, int classes, float *out);

/* ---------------- layout changes at the conv <-> FC boundary ---------------- */
/* [right][left][chunk] -> [left][right][chunk]   (dev_backprop_convolution.cu:140-168) */
int fitre_hip_reshape(const float *in, int right, int left, int chunk, float *out);
/* [C][N][a*B+b] -> [N][C][b*A+a]  (reshape + ker_transpose, cnn_forward.cu:238-261); in != out */
int fitre_hip_conv_to_fc(const float *in, int channels, int samples, int extA, int extB, float *out);
/* [N][C][b*A+a] -> [C][N][a*B+b]  (cnn_backward.cu:310-326); in != out */
int fitre_hip_fc_to_conv(const float *in, int channels, int samples, int extA, int extB, float *out);

/* ---------------- fp32-MFMA contractions ---------------- */
/* Convolution geometry shared by the three convolution entry points. */
typedef struct fitre_conv_shape {
	int samples;      /* N */
	int inChannels;   /* Cin */
	int outChannels;  /* Cout */
	int inA, inB;     /* input extent along A (image column) and B (image row) */
	int outA, outB;   /* output extent */
	int ksize, stride, padding;
} fitre_conv_shape;

/* y[Cout][N][outA][outB] = conv(x[Cin][N][inA][inB], w[Cout][Cin][k][k]) + bias (bias may be NULL).
 * Replaces im2col + GEMM + bias of functions/eval_convolution.cu:110-121. */
size_t fitre_hip_conv_forward_workspace(const fitre_conv_shape *s);
int fitre_hip_conv_forward(const fitre_conv_shape *s, const float *x, const float *w, const float *bias,
                           float *y, void *ws, size_t wsBytes);
/* dW[Cout][Cin*k*k] = sum over (n,a,b) of patch(x) * delta.  Replaces im2col + GEMM of
 * functions/cnn_backward.cu:771-783. */
size_t fitre_hip_conv_weight_grad_workspace(const fitre_conv_shape *s);
/* Whether cnnBackward should put this shape's weight gradient on its second lane, beside the chain of input gradients:
 * 1 for every shape by now.  (Weight gradients on the general tile engine used to stay in line -- AlexNet batch 64 then
 * took 3.27 ms with them on the second lane against 3.08 in line; since the chain's bandwidth kernels find room and
 * priority beside a matrix kernel it is 2.69 against 2.83 ms the other way round.) */
int fitre_hip_conv_weight_grad_runs_beside(const fitre_conv_shape *s);
int fitre_hip_conv_weight_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW,
                               void *ws, size_t wsBytes);
/* The same with the bias gradient db[Cout] = sum of delta over samples and positions (functions/cnn_backward.cu:
 * 662-689), for layers without batch norm: one pass over delta where the layer has few channels, else
 * fitre_hip_channel_sum followed by fitre_hip_conv_weight_grad.  db may be NULL (then this is
 * fitre_hip_conv_weight_grad). */
/* Layers with very few channels (LeNet's) leave their weight gradient as per-workgroup blocks that a second, short launch
 * adds up.  fitre_hip_thin_reduce_defer(1): from now on that second launch is held back (up to four layers; a fifth
 * flushes first) and fitre_hip_thin_reduce_flush() -- or fitre_hip_thin_reduce_defer(0) -- makes them all in ONE launch
 * on the lane selected then: the same sums in the same order.  While a layer's reduction is held back its workspace must
 * stay untouched and its dW / db are not yet written: give every such call a workspace of its own.  Layers of other
 * shapes are not affected.  No counterpart in the reference. */
/* fitre_hip_thin_reduce_bytes: 0 for a shape whose weight gradient has no such second launch, else the bytes at the
 * head of its workspace that must stay untouched while it is held back. */
size_t fitre_hip_thin_reduce_bytes(const fitre_conv_shape *s);
int fitre_hip_thin_reduce_defer(int on);
int fitre_hip_thin_reduce_flush(void);
size_t fitre_hip_conv_weight_bias_grad_workspace(const fitre_conv_shape *s);
int fitre_hip_conv_weight_bias_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW,
                                    float *db, void *ws, size_t wsBytes);
/* dx[Cin][N][inA][inB] = transposed convolution of delta with w; stride must be 1.  Replaces
 * functions/dev_backprop_convolution.cu:173-247. */
size_t fitre_hip_conv_input_grad_workspace(const fitre_conv_shape *s);
int fitre_hip_conv_input_grad(const fitre_conv_shape *s, const float *delta, const float *w, float *dx,
                              void *ws, size_t wsBytes);
/* The same, taken on through the layer below where that ends in an activation and a 2 x 2 / stride 2 max pool without
 * padding (its maps are 2 inA x 2 inB): dx as above, dxPool (may be NULL) and dxAct as fitre_hip_pool_act_backward(MAX_POOL,
 * actFun, dx, z_in, z_act, Cin, N, 2 inA, 2 inB, 2, 2, 0, inA, inB, dxPool, dxAct) leaves them, the same bits.  One
 * launch where fitre_hip_conv_input_grad_folds_pool says 1 (few channels, inB even) and the tensors are 16-byte aligned,
 * else the two steps one after the other.  functions/cnn_backward.cu:560-640 runs the pool and activation steps of a
 * layer as launches of their own behind the convolution step of the layer above. */
int fitre_hip_conv_input_grad_folds_pool(const fitre_conv_shape *s);
int fitre_hip_conv_input_grad_pool_act(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, int actFun,
                                       const float *z_in, const float *z_act, float *dxPool, float *dxAct, void *ws,
                                       size_t wsBytes);
/* Sums of two products of one shape in one launch, for the R operator of the Hessian-vector product
 * (functions/cnn_hv_forward.cu, cnn_hv_backward.cu: every convolution there is a sum of two):
 *   forward_pair:      y  = conv(x1, w1) + conv(x2, w2) + bias
 *   input_grad_pair:   dx = dX(delta1, w1) + dX(delta2, w2)
 *   weight_grad_pair:  dW = dW(x1, delta1) + dW(x2, delta2)
 * The reduction simply runs over the first pair and then over the second: one set of accumulators, one epilogue, one
 * reduction of split partials, no temporary and no addition pass.  3x3 / stride 1 / padding 1 shapes that the
 * specialised kernels take only (kind 0 forward, 1 input gradient, 2 weight gradient): ask _pair_supported first;
 * the _pair_workspace of an unsupported shape is 0. */
int fitre_hip_conv_pair_supported(const fitre_conv_shape *s, int kind);
size_t fitre_hip_conv_pair_workspace(const fitre_conv_shape *s, int kind);
int fitre_hip_conv_forward_pair(const fitre_conv_shape *s, const float *x1, const float *w1, const float *x2,
                                const float *w2, const float *bias, float *y, void *ws, size_t wsBytes);
int fitre_hip_conv_input_grad_pair(const fitre_conv_shape *s, const float *delta1, const float *w1,
                                   const float *delta2, const float *w2, float *dx, void *ws, size_t wsBytes);
int fitre_hip_conv_weight_grad_pair(const fitre_conv_shape *s, const float *x1, const float *delta1, const float *x2,
                                    const float *delta2, float *dW, void *ws, size_t wsBytes);
/* The same product, but when its reduction is split over workgroups the partial results are left unsummed
 * for the consumer to add up while it reads them (fitre_hip_pool_act_bn_backward takes such a view): one
 * launch and one pass over dx less.  view->base points at view->splits slabs of Cin*N*inA*inB floats,
 * view->stride floats apart, inside ws (which must then stay untouched until the consumer has run); the
 * gradient is their sum in slab order.  An unsplit product writes dx as usual and reports splits = 1,
 * base = dx. */
typedef struct fitre_split_view {
	float *base;
	int splits;
	long stride;
} fitre_split_view;
int fitre_hip_conv_input_grad_split(const fitre_conv_shape *s, const float *delta, const float *w, float *dx,
                                    void *ws, size_t wsBytes, fitre_split_view *view);
/* Some shapes multiply by a rearranged copy of the weights (3x3 windows on 2 x 2 maps: the dense per-image form
 * of the convolution, 16/36 of the multiply-adds of the nine-tap form).  The copy depends on the weights only, so
 * a caller can have it made ahead of the chain that needs it, on another lane:
 *   _prepared_bytes  size of the copy, 0 when the shape has none;
 *   _prepare         builds it (stream-ordered);
 *   _split_prepared  fitre_hip_conv_input_grad_split reading it (prepared == NULL: built inside, in ws).
 * No counterpart in the reference, whose weights are reordered per call (dev_backprop_convolution.cu:140-156). */
size_t fitre_hip_conv_input_grad_prepared_bytes(const fitre_conv_shape *s);
int fitre_hip_conv_input_grad_prepare(const fitre_conv_shape *s, const float *w, void *prepared, size_t preparedBytes);
int fitre_hip_conv_input_grad_split_prepared(const fitre_conv_shape *s, const float *delta, const float *w,
                                             const void *prepared, float *dx, void *ws, size_t wsBytes,
                                             fitre_split_view *view);

/* Column-major GEMM C(MxN) = alpha*op(A)*op(B) + beta*C with the argument meaning of cublasDgemm
 * (transA/transB: 0 = N, 1 = T).  Used for the FC layers (eval_gradient.cu:63-67,
 * cnn_backward.cu:189-197,250-254) and the KFAC factor products (kfac_inverses.cu:531-536,808-813).
 * bias (may be NULL) is added to every column (length M) after the product when beta == 0. */
size_t fitre_hip_gemm_workspace(int M, int N, int K);
int fitre_hip_gemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                   const float *B, int ldb, float beta, float *C, int ldc, const float *bias, void *ws,
                   size_t wsBytes);

/* Backward products of one fully connected layer, W out x in column-major, delta out x n, one launch each
 * where the layer is small (fitre_hip_linear_is_small), the plain sequence of steps otherwise.
 *   input gradient (functions/cnn_backward.cu:250-254 followed by the activation step of the layer below,
 *   :100-172): result(in x n) = f'(.) .* (W' * delta) with f = actBelow read from zPre / zPost (in x n each; the
 *   pointers a call of fitre_hip_activation_backward would take), no derivative for CNN_ACT_NONE / ACT_LINEAR / a
 *   negative code.  extA, extB > 0: the rows are whole extA x extB maps of a convolution layer and the result is
 *   stored in its layout [channel][sample][a][b] (the permutation of fitre_hip_fc_to_conv); `staging` (in x n
 *   floats, may be NULL for a small layer) then holds the unpermuted product of a large layer.  deltaCopy (may be
 *   NULL): delta is also copied there (the snapshot of functions/cnn_backward.cu:238-240, for a layer whose delta the
 *   caller did not produce itself).
 *   weight gradient (:189-197 and the bias gradient :216-224): dW(out x in) = delta * zin', db(out) = delta * 1
 *   (db may be NULL).
 * ws / wsBytes: fitre_hip_gemm_workspace(in, n, out) for the input gradient, fitre_hip_linear_weight_grad_workspace for
 * the weight gradient (a small layer at a large batch cuts the batch into ranges and adds their partial results in a
 * second launch); unused for small layers. */
int fitre_hip_linear_is_small(int in, int out, int n);
size_t fitre_hip_linear_weight_grad_workspace(int in, int out, int n);
int fitre_hip_linear_input_grad(int in, int out, int n, const float *W, const float *delta, int actBelow,
                                const float *zPre, const float *zPost, int extA, int extB, float *result,
                                float *staging, void *ws, size_t wsBytes, float *deltaCopy);
int fitre_hip_linear_weight_grad(int in, int out, int n, const float *delta, const float *zin, float *dW, float *db,
                                 void *ws, size_t wsBytes);

/* The backward products of a whole tail of small fully connected layers (layers[0] the lowest) in two launches (three
 * when the batch is above 512): every layer's delta (after its activation derivative) into its slot, dW = delta * zin',
 * db = delta * 1, and the lowest layer's input gradient W' * delta into `features` -- in a convolution layer's layout
 * [channel][sample][a][b] when extA, extB > 0 (the permutation of fitre_hip_fc_to_conv), in x n otherwise.  The same
 * bits as the per-layer entry points above give for layers this small (functions/cnn_backward.cu:100-254 for every
 * layer of the tail): every sum runs in the same order.  delta: at the top layer's output (out x n), before that
 * layer's activation derivative.  _fits: at most four layers of at most 1024 units, each of them small in the sense
 * of fitre_hip_linear_is_small (or, above 512 samples, within the ranged weight gradient's limits), the layers above the
 * lowest together within 16384 floats of LDS (the sum of in * (out + 1)).  Workspace:
 * fitre_hip_fc_tail_workspace bytes (only read above 512 samples; ws may be NULL otherwise). */
typedef struct fitre_fc_tail_layer {
	int in, out;
	int act;                   /* activation of this layer (CNN_ACT_NONE / ACT_LINEAR / negative: none) */
	const float *W;            /* out x in, column-major */
	const float *zPre, *zPost; /* its output before / after the activation, out x n (unused without an activation) */
	const float *zin;          /* its input, in x n */
	float *slot;               /* receives delta, out x n */
	float *dW, *db;            /* out x in, out (db may be NULL) */
} fitre_fc_tail_layer;
int fitre_hip_fc_tail_fits(int layers, const fitre_fc_tail_layer *l, int n);
size_t fitre_hip_fc_tail_workspace(int layers, const fitre_fc_tail_layer *l, int n);
int fitre_hip_fc_tail_backward(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA, int extB,
                               float *features, void *ws, size_t wsBytes);
/* The same where the lowest layer reads the output of a 2 x 2 / stride 2 max pool (no padding) behind an activation:
 * features as above, then dxPool (may be NULL) and dxAct as fitre_hip_pool_act_backward(MAX_POOL, actFun, features, z_in,
 * z_act, C, n, 2 extA, 2 extB, 2, 2, 0, extA, extB, dxPool, dxAct) leaves them, the same bits, from the launch that
 * writes features when the four tensors are 8-byte aligned.  extA, extB > 0. */
int fitre_hip_fc_tail_backward_pool_act(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA,
                                        int extB, float *features, int actFun, const float *z_in, const float *z_act,
                                        float *dxPool, float *dxAct, void *ws, size_t wsBytes);

/* ---- Kronecker factors of the KFAC curvature approximation --------------------------------------
 * Each factor is a dense symmetric matrix, written in full (row-major == column-major).  The
 * products are symmetric, so only the tiles on and above the diagonal are computed.
 *
 * Convolution, input side (solvers/kfac_inverses.cu:489-540): A = P^T P / samples with
 * P = [ im2col(x) / (outA*outB) , 1 ], order Cin*k*k (+1 with bias); patch column order
 * (c, ta, tb) as in the weight layout.  With the workspace the _workspace call asks for, the transposed
 * patch matrix (Cin*k*k rows of samples*outA*outB values) is written there first and the product runs on
 * it; with a 256-byte aligned workspace that only covers the split-K partials, or a smaller one, both
 * operands gather their elements from x instead (slower, no extra memory). */
size_t fitre_hip_kfac_conv_input_factor_workspace(const fitre_conv_shape *s, int withBias);
int fitre_hip_kfac_conv_input_factor(const fitre_conv_shape *s, const float *x, int withBias, float *factor,
                                     void *ws, size_t wsBytes);
/* Workspace of the three factors below: order = matrix order, reduce = length of the sum
 * (positions = samples*outA*outB for a convolution, samples for a fully connected layer). */
size_t fitre_hip_kfac_gram_workspace(int order, long reduce);
/* Convolution, output side (kfac_inverses.cu:806-816): G = D^T D * (samples*outA*outB), D = delta
 * [Cout][samples*outA*outB] seen as positions x Cout; order Cout. */
int fitre_hip_kfac_conv_output_factor(const fitre_conv_shape *s, const float *delta, float *factor, void *ws,
                                      size_t wsBytes);
/* Fully connected, input side (kfac_inverses.cu:596-625): A = Z Z^T / samples, Z = [ z ; 1 ] with z
 * column-major in x samples; order in (+1 with bias).  Workspace: fitre_hip_kfac_gram_workspace(in, samples). */
int fitre_hip_kfac_fc_input_factor(const float *z, int in, int samples, int withBias, float *factor, void *ws,
                                   size_t wsBytes);
/* Fully connected, output side (kfac_inverses.cu:838-852): G = D D^T * samples, D = delta column-major
 * out x samples; order out. */
int fitre_hip_kfac_fc_output_factor(const float *delta, int out, int samples, float *factor, void *ws,
                                    size_t wsBytes);

/* ---- R-operator (Hessian-vector product) pieces --------------------------------------------------
 * out = rdelta * f'(.) + delta * f''(.) * rz_in, the directional derivative of delta * f'(.) when
 * delta moves by rdelta and the activation's input by rz_in (second derivatives of
 * functions/swish.cu:45-56, dev_activations.cu; z_in / z_out as in fitre_hip_activation_backward). */
int fitre_hip_activation_rop_backward(int actFun, const float *rdelta, const float *delta, const float *z_in,
                                      const float *z_out, const float *rz_in, float *out, long n);
/* Max pool: out = values at the arg-max positions of z_act (ker_rop_max_pool_layer, functions/dev_pool.cu:123-174);
 * average pool: the average of values (z_act unused). */
int fitre_hip_pool_forward_routed(int poolType, const float *values, const float *z_act, int channels, int samples,
                                  int inA, int inB, int ksize, int stride, int padding, int outA, int outB, float *out);
/* The R operator's forward sweep through what follows a convolution with batch norm (functions/cnn_hv_forward.cu:120-222):
 * R{bn out} = the batch-norm backward formula applied to rx (fitre_hip_batch_norm_backward), R{act out} = R{bn out} * f'(.)
 * (fitre_hip_activation_backward) and, through a max pool, the value at the arg-max of the activation output
 * (fitre_hip_pool_forward_routed) -- after the sums, ONE pass that reads rx and zhat and writes all three (the same results as
 * the three passes).  z_act may be NULL when actFun is ReLU (the activation output is then max(zhat, 0)) and the shape is
 * fused: no pooling or 2x2 / stride 2 max pooling, A even, B a multiple of 4, 16-byte-aligned tensors; every other case
 * runs the three passes and needs z_act.  Workspace: fitre_hip_batch_norm_workspace(channels, samples * inA * inB). */
int fitre_hip_bn_act_pool_rop_forward(const float *rx, const float *zhat, const float *z_act, const float *variance,
                                      int channels, int samples, int inA, int inB, float epsilon, int actFun, float *rbn,
                                      float *ract, int poolType, int ksize, int stride, int padding, int outA, int outB,
                                      float *rpool, void *ws, size_t wsBytes);
/* Directional derivative of batch-norm backward (computeROpBatchNormBackward, functions/dev_batch_norm.cu:787-960):
 * with s = sqrt(var + eps) and <.> the per-channel mean,
 *   out = (rdelta_x - <rdelta_x> - rzhat <delta_x zhat> - zhat (<rdelta_x zhat> + <delta_x rzhat>)) / s - delta_c <zhat rx> / s
 * delta_x / delta_c: gradient at the batch-norm output / input, rx / rzhat: R{.} of its input / output.
 * The directional derivative of batch-norm FORWARD is fitre_hip_batch_norm_backward applied to rx.
 * Workspace: fitre_hip_batch_norm_workspace(channels, perChannel). */
int fitre_hip_batch_norm_rop_backward(const float *rdelta_x, const float *delta_x, const float *zhat, const float *rzhat,
                                      const float *rx, const float *delta_c, const float *variance, int channels,
                                      long perChannel, float epsilon, float *out, void *ws, size_t wsBytes);
/* The backward sweep's R-steps between a layer's pooled R{delta} and R{delta at the convolution output}
 * (functions/cnn_hv_backward.cu:328-754): fitre_hip_pool_backward of rdelta (routing by the arg-max of z_act),
 * fitre_hip_activation_rop_backward (delta = the gradient at the activation output, zhat = the activation input, rzhat =
 * its directional derivative) into rdeltaX, and fitre_hip_batch_norm_rop_backward of that into out -- as TWO launches
 * where the shape allows: one pass routes, applies the activation's R-step and leaves the five sums, the second applies
 * the batch-norm formula.  Fused for no pooling and 2x2 / stride 2 max pooling (A even, B a multiple of 4, 16-byte-aligned
 * tensors); z_act may then be NULL for ReLU, and rdeltaAct (the routed R{delta}, only written by the separate passes) may
 * be NULL.  Every other case runs the three calls.  Workspace: fitre_hip_batch_norm_workspace(channels, samples * inA * inB),
 * at least channels * segments * 64 bytes. */
int fitre_hip_pool_act_bn_rop_backward(int poolType, int actFun, const float *rdelta, const float *delta, const float *zhat,
                                       const float *z_act, const float *rzhat, const float *delta_x, const float *rx,
                                       const float *delta_c, const float *variance, int channels, int samples, int inA,
                                       int inB, int ksize, int stride, int padding, int outA, int outB, float epsilon,
                                       float *rdeltaAct, float *rdeltaX, float *out, void *ws, size_t wsBytes);
/* The R-operator over a fully connected model (functions/eval_hessian_vec.cu):
 * fc_rop_backward: out = f'(z) rdz + rx g(z) dx, the directional derivative of dx = f'(z) dz written with dx
 *   itself (eval_backprop_hessian, functions/dev_hessian_helpers.cu:7-15: logistic, g = 1 - 2 z; tanh here too,
 *   g = -2 z; linear: out = rdz); rx == NULL leaves the second term out (eval_gauss_newton_backprop, :17-26).
 * column_softmax_rop: out = p . rx - p sum(p . rx) per column of the rows x cols matrices
 *   (functions/eval_hessian_vec.cu:219-262). */
int fitre_hip_fc_rop_backward(int actFun, const float *z, const float *rdz, const float *rx, const float *dx, float *out, long n);
int fitre_hip_column_softmax_rop(const float *probs, const float *rx, int rows, int cols, float *out);
/* rError = p_i (rz_i - sum_j p_j rz_j) / rows (computeROpCrossEntropyError_simple, functions/softmax_loss.cu:251-300) */
int fitre_hip_cross_entropy_rop_error(const float *rz, const float *probs, int rows, int classes, float *rError);

/* inverse = (matrix + shift*I)^-1 for a symmetric positive definite matrix of order n (column-major ==
 * row-major, full storage in and out): blocked Cholesky, inverse of the factor, symmetric product.
 * Replaces computeMatrixInverseCusolver (solvers/kfac_inverses.cu:133-186: identity right-hand side,
 * ker_add_regularization with lambda + dampGamma, cusolverDnDpotrf, cusolverDnDpotrs).
 * ws: 256-byte aligned, at least fitre_hip_spd_inverse_workspace(n) bytes.  info (host pointer, may be
 * NULL): receives 0, or the 1-based index of the first non-positive pivot -- the call then also fails
 * with FITRE_E_ARGUMENT, as the reference exits on devInfo != 0; with info == NULL the call does not wait
 * for the device and a failed factorization shows as NaNs in the result. */
size_t fitre_hip_spd_inverse_workspace(int n);
int fitre_hip_spd_inverse(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes,
                          int *info);
/* The same inverse queued on the selected lane without waiting for it: pivotInfo is a DEVICE int that holds
 * 0 or the index of the first non-positive pivot once the lane has drained.  Lets independent inverses run
 * side by side on different lanes (each with its own matrix, result and workspace). */
int fitre_hip_spd_inverse_queued(const float *matrix, int n, float shift, float *inverse, void *ws,
                                 size_t wsBytes, int *pivotInfo);
/* `batch` (1..16) matrices of ONE order inverted side by side by one chain of launches, every launch covering
 * all of them (the KFAC factors of consecutive layers of equal width): matrix b is at
 * matrix + b*matrixStride, its inverse goes to inverse + b*inverseStride (strides in floats, at least n*n), its
 * workspace is (char *)ws + b*wsStrideBytes (a multiple of 256, at least fitre_hip_spd_inverse_workspace(n) =
 * wsBytes), its pivot report pivotInfo[b] (device ints).  An inverse is a chain of several hundred small dependent
 * launches; a batch pays for the chain once. */
int fitre_hip_spd_inverse_batched_queued(int batch, const float *matrix, long matrixStride, int n, float shift,
                                         float *inverse, long inverseStride, void *ws, size_t wsBytes,
                                         long wsStrideBytes, int *pivotInfo);

/* ---- float64 products and the float64 inverse -------------------------------------------------------
 * The reference's KFAC leg is double throughout (real = double, core/datadefs.h:5): cublasDgemm for the factors and the
 * natural gradient (solvers/kfac_inverses.cu:531-536,808-813, solvers/kfac_natural_gradient.cu:36-241), cusolverDnDpotrf /
 * Dpotrs for the inverses (solvers/kfac_inverses.cu:133-186).  These entry points do that arithmetic in float64 on the
 * matrix pipes, on operands that stay in the caller's float arrays.
 *
 * fitre_matrix: element (r, c) of a matrix of floats (FITRE_MAT_F32) or doubles (FITRE_MAT_F64) at
 * data[r * rowStride + c * colStride]; FITRE_MAT_SYM_PAIR is a symmetric matrix of order rowStride kept as a pair of
 * floats per element in ONE dense float array, column-major with leading dimension colStride: the value rounded to float
 * on and above the diagonal, value - rounded value below it -- 48 significant bits in the room of a float matrix.  The
 * diagonal has no word below it for its remainder: the word of element (k + 1, k) ((n - 1, 0) for the last k) keeps
 * the upper 16 bits of its own remainder and, in its lower 16 bits, the upper 16 bits of the remainder of diagonal element
 * k, so that both have 32 significant bits (orders below 3: the diagonal stays at float precision).  The upper triangle
 * alone is the matrix in floats.  onesRow / onesCol (floats only, -1 for none): a row / column that is not in memory and
 * reads as onesValue (the bias row of a KFAC input factor). */
enum { FITRE_MAT_F32 = 0, FITRE_MAT_F64 = 1, FITRE_MAT_SYM_PAIR = 2 };
typedef struct fitre_matrix {
	const void *data;
	long rowStride, colStride;
	int kind;
	long onesRow, onesCol;
	double onesValue;
} fitre_matrix;
/* flags: the product is symmetric (M == N; only the tiles on and above the diagonal are computed and mirrored);
 * A(i, k) is zero for k > i (A_LOWER) / for k < i (A_UPPER); B(k, j) is zero for k < j (B_LOWER) / for k > j (B_UPPER):
 * the reduction skips those ranges. */
#define FITRE_GEMM_SYMMETRIC 1
#define FITRE_GEMM_A_LOWER 2
#define FITRE_GEMM_A_UPPER 4
#define FITRE_GEMM_B_LOWER 8
#define FITRE_GEMM_B_UPPER 16
/* C(M x N) = alpha * A(M x K) * B(K x N) + beta * C, plus diagAdd on the diagonal; C->data is written (any kind; a
 * float-pair result needs FITRE_GEMM_SYMMETRIC and beta = 0).  ws: 256-byte aligned, fitre_hip_gemm_f64_workspace bytes. */
size_t fitre_hip_gemm_f64_workspace(long M, long N, long K, int flags);
int fitre_hip_gemm_f64(long M, long N, long K, double alpha, const fitre_matrix *A, const fitre_matrix *B, double beta,
                       const fitre_matrix *C, double diagAdd, int flags, void *ws, size_t wsBytes);
/* C = alpha * A * B + addScale * add, add a matrix of doubles (no beta term, no flags). */
int fitre_hip_gemm_f64_add(long M, long N, long K, double alpha, const fitre_matrix *A, const fitre_matrix *B, double addScale,
                           const fitre_matrix *add, const fitre_matrix *C, void *ws, size_t wsBytes);
/* inverse = matrix^-1 for a symmetric positive definite matrix of n x n doubles (dense, destroyed): Cholesky factor and
 * its inverse by halving, then X^T X, all in float64; the result is stored dense with leading dimension n as
 * inverseKind.  Queued on the selected lane; pivotInfo (device int) holds 0 or the 1-based index of the first
 * non-positive pivot once the lane has drained.  ws: 256-byte aligned, fitre_hip_spd_inverse_f64_workspace(n) bytes. */
size_t fitre_hip_spd_inverse_f64_workspace(int n);
int fitre_hip_spd_inverse_f64_queued(double *matrix, int n, void *inverse, int inverseKind, void *ws, size_t wsBytes,
                                     int *pivotInfo);
/* The operand of an input-side factor itself, for a factor kept in low-rank form (kfac_path.c): rows[r][m], row r
 * contiguous over the samples*outA*outB positions, r = the patch index (c, ta, tb), plus (withBias) a last row that is
 * outA*outB everywhere: A = rows rows^T / ((outA*outB)^2 samples).  Fully connected: rows = [ z ; 1 ], (in + 1) x samples
 * column-major, A = rows rows^T / samples. */
int fitre_hip_kfac_conv_input_rows(const fitre_conv_shape *s, const float *x, int withBias, float *rows);
int fitre_hip_kfac_fc_input_rows(const float *z, int in, int samples, int withBias, float *rows);
/* The first four 32-bit words of `count` (at most 40) device arrays, gathered into out (device, 4 * count words);
 * count (at most 16) words written to the head of a device array.  Stream-ordered. */
int fitre_hip_gather_headers(const void *const *arrays, int count, void *out);
int fitre_hip_write_header(void *dst, const unsigned int *words, int count);
/* out (n x n doubles, leading dimension ldOut, both triangles) = the symmetric matrix that the float pair `pairs` (order n,
 * leading dimension ld, FITRE_MAT_SYM_PAIR) stands for.  A product that reads a large float-pair operand many times is
 * faster on the decoded copy (coalesced reads, the large tile); no counterpart in the reference. */
int fitre_hip_pair_to_f64(const float *pairs, long ld, int n, double *out, long ldOut);
/* out(n x n doubles) = matrix(n x n floats) + shift * I */
int fitre_hip_widen_shift(const float *matrix, int n, double shift, double *out);
/* The four Kronecker factors above accumulated in float64 and written as n x n doubles, with `shift` (the damping) added
 * on the diagonal.  Workspaces: fitre_hip_kfac_conv_input_factor_f64_workspace (the transposed patch matrix and the
 * split partials) resp. fitre_hip_gemm_f64_workspace(order, order, reduce, FITRE_GEMM_SYMMETRIC). */
size_t fitre_hip_kfac_conv_input_factor_f64_workspace(const fitre_conv_shape *s, int withBias);
int fitre_hip_kfac_conv_input_factor_f64(const fitre_conv_shape *s, const float *x, int withBias, double shift,
                                         double *factor, void *ws, size_t wsBytes);
int fitre_hip_kfac_conv_output_factor_f64(const fitre_conv_shape *s, const float *delta, double shift, double *factor,
                                          void *ws, size_t wsBytes);
int fitre_hip_kfac_fc_input_factor_f64(const float *z, int in, int samples, int withBias, double shift, double *factor,
                                       void *ws, size_t wsBytes);
int fitre_hip_kfac_fc_output_factor_f64(const float *delta, int out, int samples, double shift, double *factor, void *ws,
                                        size_t wsBytes);

#ifdef __cplusplus
}
#endif
#endif
