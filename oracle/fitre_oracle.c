/*
 * fitre_oracle.c -- CPU restatement of the reference's CNN forward/backward
 * path.  TEST INFRASTRUCTURE ONLY: it is the checker the HIP kernels are
 * compared with, and the timed CPU baseline of the benchmark.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Built twice from this one file: real = double (the parity oracle) and
 * real = float (the CPU baseline), see oracle/Makefile.
 *
 * Each function cites the reference lines it follows.  It keeps the
 * reference's data flow on purpose -- materialised patch matrices, BLAS-style
 * GEMM calls with the reference's own argument lists, one pass per kernel --
 * so that it can be audited against the reference line by line, and so that
 * it shares no structure with the implicit-GEMM kernels it checks.
 *
 * Deliberate departures from the reference (each is a reference defect; the
 * HIP path makes the same choice):
 *   D1  ReLU / ELU backward multiply by the true derivative; the reference
 *       leaves delta unchanged (functions/cnn_backward.cu:561-565).
 *   D2  pooling windows start at k*stride - padding; the reference's
 *       (k-1)*stride + ksize - 2*padding (functions/dev_pool.cu:94-95) equals
 *       it only when ksize = stride + padding.
 *   D3  average-pool backward is the adjoint of the forward for any window;
 *       the reference's kernel is valid only for ksize = stride, no padding,
 *       extent divisible by ksize (functions/dev_pool.cu:269-298), where the
 *       two agree.
 *   D4  the FC<->conv boundary transpose uses row*width + col; the
 *       reference's row*height + col (functions/dev_transpose.cu:26-28) is
 *       the same for square maps, the only ones it is run on.
 *   D5  ReLU / ELU are applied on fully connected layers; the reference
 *       prints "not implemented" and leaves the values unchanged
 *       (functions/eval_gradient.cu:205-211).
 *   D6  when the last convolution layer has no pooling stage, its activation
 *       output has been rewritten in place into the fully connected layout by
 *       the forward pass (functions/cnn_forward.cu:238-261); the backward pass
 *       then recomputes that layer's activation output from its input instead
 *       of reading the permuted buffer as the reference does
 *       (functions/cnn_backward.cu:574-580).  No shipped network of the
 *       reference ends in an unpooled layer.
 *
 * Parity pins (tests/test_oracle_*.py): the stored batch-norm known answer
 * pytorch/testing/my.out:9; brute-force direct convolution and its adjoint
 * identities; float64 autograd of the textbook layers; a Taylor remainder
 * test of the whole gradient (utilities/cnn_derivative_test.cu:197-199);
 * the logged LeNet parameter offsets; the Kronecker factors against unfold
 * patches and numpy Gram products; the inverse against scipy's Cholesky
 * solver; the natural gradient against a Kronecker-product solve; the fully
 * connected model family against autograd of each head's loss, its Hessian
 * and Gauss-Newton products against float64 double backward resp. autograd's
 * jvp / vjp around the head's Hessian (tests/test_fc_model.py); the CNN
 * Hessian-vector product against float64 double backward, its symmetry and
 * the second-order Taylor remainder; the input pipeline against numpy
 * pad/slice, flip, transposes and the closed-form normalisation.
 * No function here is "parity unpinned".
 */
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fitre_nn.h"

#ifdef FITRE_REAL_DOUBLE
#define REAL_MAX DBL_MAX
#else
#define REAL_MAX FLT_MAX
#endif

#define OP_N 0
#define OP_T 1

/* ------------------------------------------------------------------ */
/* BLAS-shaped helpers (column-major), standing in for the cuBLAS calls */
/* ------------------------------------------------------------------ */

/* C(MxN) = alpha * op(A)(MxK) * op(B)(KxN) + beta * C, column-major, as cublasDgemm. */
void oracle_gemm(int transA, int transB, int M, int N, int K, real alpha, const real *A, int lda,
                 const real *B, int ldb, real beta, real *C, int ldc)
{
#pragma omp parallel for schedule(static)
	for (int j = 0; j < N; j++) {
		real *c = C + (size_t)j * ldc;
		if (beta == 0) {
			for (int i = 0; i < M; i++) c[i] = 0;
		} else if (beta != 1) {
			for (int i = 0; i < M; i++) c[i] *= beta;
		}
		if (transA == OP_N) {
			for (int k = 0; k < K; k++) {
				real b = alpha * (transB == OP_N ? B[(size_t)j * ldb + k] : B[(size_t)k * ldb + j]);
				const real *a = A + (size_t)k * lda;
#pragma omp simd
				for (int i = 0; i < M; i++) c[i] += a[i] * b;
			}
		} else {
			for (int i = 0; i < M; i++) {
				const real *a = A + (size_t)i * lda;
				real s = 0;
				if (transB == OP_N) {
					const real *b = B + (size_t)j * ldb;
#pragma omp simd reduction(+ : s)
					for (int k = 0; k < K; k++) s += a[k] * b[k];
				} else {
					for (int k = 0; k < K; k++) s += a[k] * B[(size_t)k * ldb + j];
				}
				c[i] += alpha * s;
			}
		}
	}
}

/* y = alpha * op(A) x + beta * y, as cublasDgemv (A is MxN column-major). */
static void oracle_gemv(int trans, int M, int N, real alpha, const real *A, int lda, const real *x,
                        real beta, real *y)
{
	if (trans == OP_N)
		oracle_gemm(OP_N, OP_N, M, 1, N, alpha, A, lda, x, N, beta, y, M);
	else
		oracle_gemm(OP_T, OP_N, N, 1, M, alpha, A, lda, x, M, beta, y, N);
}

/* ------------------------------------------------------------------ */
/* patch matrices                                                      */
/* ------------------------------------------------------------------ */

/* functions/dev_image.cu:12-51 (ker_im2col) with the launch of :114-141.
 * data_im is [C][N][width][height] (height fastest); data_col is the
 * (N*Hc*Wc) x (C*k*k) column-major patch matrix, column index
 * c*k*k + j*k + i with j the window column and i the window row. */
void oracle_im2col(const real *data_im, int samples, int channels, int height, int width, int ksize,
                   int pad, int stride, real *data_col)
{
	int height_col = (height + 2 * pad - ksize) / stride + 1;
	int width_col = (width + 2 * pad - ksize) / stride + 1;
	size_t plane = (size_t)height_col * width_col * samples;
#pragma omp parallel for collapse(2) schedule(static)
	for (int channel_in = 0; channel_in < channels; channel_in++) {
		for (int n = 0; n < samples; n++) {
			for (int w_out = 0; w_out < width_col; w_out++) {
				for (int h_out = 0; h_out < height_col; h_out++) {
					int h_in = h_out * stride - pad;
					int w_in = w_out * stride - pad;
					real *col = data_col + (size_t)channel_in * ksize * ksize * plane +
					            (size_t)n * height_col * width_col + (size_t)w_out * height_col + h_out;
					const real *im = data_im + ((size_t)channel_in * samples + n) * height * width;
					for (int j = 0; j < ksize; j++) {
						for (int i = 0; i < ksize; i++) {
							int h = h_in + i, w = w_in + j;
							*col = (h >= 0 && w >= 0 && h < height && w < width)
							           ? im[(size_t)w * height + h]
							           : 0;
							col += plane;
						}
					}
				}
			}
		}
	}
}

/* functions/dev_backprop_convolution.cu:60-96 (kerBackPropConvolutionBatchHelper):
 * patch matrix of delta for the input gradient, (N*H*W) x (dChannels*fH*fW),
 * window walked from (col+pad, row+pad) downwards. */
static void oracle_delta_cols(const real *delta, int dHeight, int dWidth, int dChannels, int fHeight,
                              int fWidth, real *img, int height, int width, int padding, int samples)
{
	size_t plane = (size_t)height * width * samples;
#pragma omp parallel for collapse(2) schedule(static)
	for (int chId = 0; chId < dChannels; chId++) {
		for (int imgId = 0; imgId < samples; imgId++) {
			for (int myCol = 0; myCol < width; myCol++) {
				for (int myRow = 0; myRow < height; myRow++) {
					size_t imgOffset = (size_t)chId * fHeight * fWidth * plane +
					                   (size_t)imgId * height * width + (size_t)myCol * height + myRow;
					size_t deltaOffset =
					    (size_t)chId * samples * dHeight * dWidth + (size_t)imgId * dHeight * dWidth;
					for (int c = myCol + padding; c > myCol + padding - fWidth; c--) {
						for (int r = myRow + padding; r > myRow + padding - fHeight; r--) {
							int ok = (c < dWidth) && (c >= 0) && (r >= 0) && (r < dHeight);
							img[imgOffset] = ok ? delta[deltaOffset + (size_t)c * dHeight + r] : 0;
							imgOffset += plane;
						}
					}
				}
			}
		}
	}
}

/* functions/dev_backprop_convolution.cu:140-168 (kerReshapeMatrix / reshapeMatrix):
 * [right][left][chunk] -> [left][right][chunk]. */
void oracle_reshape(const real *input, int rightChannels, int leftChannels, int chunk, real *output)
{
	for (int nId = 0; nId < rightChannels; nId++)
		for (int cId = 0; cId < leftChannels; cId++)
			for (int t = 0; t < chunk; t++)
				output[(size_t)cId * chunk * rightChannels + (size_t)nId * chunk + t] =
				    input[((size_t)nId * leftChannels + cId) * chunk + t];
}

/* functions/dev_transpose.cu:8-30 (ker_transpose): every height x width map,
 * stored column-major, is rewritten row-major (departure D4). */
void oracle_transpose(const real *input, int maps, int height, int width, real *output)
{
	for (int m = 0; m < maps; m++)
		for (int col = 0; col < width; col++)
			for (int row = 0; row < height; row++)
				output[(size_t)m * height * width + (size_t)row * width + col] =
				    input[(size_t)m * height * width + (size_t)col * height + row];
}

/* functions/dev_transpose.cu:36-58 (ker_transpose_rc): row-major -> column-major. */
void oracle_transpose_rc(const real *input, int maps, int height, int width, real *output)
{
	for (int m = 0; m < maps; m++)
		for (int row = 0; row < height; row++)
			for (int col = 0; col < width; col++)
				output[(size_t)m * height * width + (size_t)col * height + row] =
				    input[(size_t)m * height * width + (size_t)row * width + col];
}

/* ------------------------------------------------------------------ */
/* activations                                                         */
/* ------------------------------------------------------------------ */

/* Forward activations in place: functions/dev_activations.cu:8-95,
 * functions/swish.cu:14-23; switch of functions/eval_convolution.cu:172-205
 * and functions/eval_gradient.cu:141-229.  Returns -1 for an unknown code. */
int oracle_activation_forward(int actFun, real *x, size_t n)
{
	switch (actFun) {
	case CNN_ACT_RELU:
		for (size_t i = 0; i < n; i++)
			if (x[i] < 0) x[i] = 0;
		break;
	case CNN_ACT_SOFTPLUS:
		for (size_t i = 0; i < n; i++)
			if (x[i] < 20) x[i] = log(1 + exp(x[i]));
		break;
	case CNN_ACT_ELU:
		for (size_t i = 0; i < n; i++)
			if (x[i] < 0) x[i] = 1.0 * (exp(x[i]) - 1);
		break;
	case CNN_ACT_SWISH:
		for (size_t i = 0; i < n; i++) x[i] = x[i] / (1 + exp(-x[i]));
		break;
	case ACT_LOGISTIC:
		for (size_t i = 0; i < n; i++) x[i] = 1. / (1. + exp(-x[i]));
		break;
	case ACT_TANH:
		for (size_t i = 0; i < n; i++) x[i] = tanh(x[i]);
		break;
	case ACT_LINEAR:
	case CNN_ACT_NONE:
		break;
	default:
		return -1;
	}
	return 0;
}

/* delta *= f'(.) : functions/swish.cu:34-43, functions/dev_layer_error.cu:13-48,
 * switches of functions/cnn_backward.cu:120-175 and :523-592.  z_in is the
 * activation's input, z_out its output.  ReLU/ELU: departure D1. */
int oracle_activation_backward(int actFun, real *delta, const real *z_in, const real *z_out, size_t n)
{
	switch (actFun) {
	case ACT_LOGISTIC:
		for (size_t i = 0; i < n; i++) delta[i] = delta[i] * z_out[i] * (1.0 - z_out[i]);
		break;
	case ACT_TANH:
		for (size_t i = 0; i < n; i++) delta[i] *= (1.0 + z_out[i]) * (1.0 - z_out[i]);
		break;
	case CNN_ACT_SOFTPLUS:
		for (size_t i = 0; i < n; i++) delta[i] *= 1. / (1. + exp(-z_in[i]));
		break;
	case CNN_ACT_SWISH:
		for (size_t i = 0; i < n; i++) {
			real t = 1. / (1. + exp(-z_in[i]));
			delta[i] *= (z_out[i] + t * (1. - z_out[i]));
		}
		break;
	case CNN_ACT_RELU:
		for (size_t i = 0; i < n; i++)
			if (!(z_out[i] > 0)) delta[i] = 0;
		break;
	case CNN_ACT_ELU:
		for (size_t i = 0; i < n; i++)
			if (z_out[i] < 0) delta[i] *= (z_out[i] + 1.0);
		break;
	case ACT_LINEAR:
	case CNN_ACT_NONE:
		break;
	default:
		return -1;
	}
	return 0;
}

/* ------------------------------------------------------------------ */
/* pooling                                                             */
/* ------------------------------------------------------------------ */

/* functions/dev_pool.cu:79-121 (ker_max_pool_layer), window origin per D2. */
void oracle_max_pool_forward(const real *input, int samples, int channels, int height, int width,
                             int ksize, int stride, int padding, int p_height, int p_width, real *output)
{
#pragma omp parallel for collapse(2) schedule(static)
	for (int ch = 0; ch < channels; ch++) {
		for (int idx = 0; idx < samples; idx++) {
			const real *in = input + ((size_t)ch * samples + idx) * height * width;
			real *out = output + ((size_t)ch * samples + idx) * p_height * p_width;
			for (int l = 0; l < p_width; l++) {
				for (int k = 0; k < p_height; k++) {
					int i = k * stride - padding, j = l * stride - padding;
					real val = -REAL_MAX;
					for (int r = 0; r < ksize; r++) {
						for (int c = 0; c < ksize; c++) {
							int frow = i + r, fcol = j + c;
							if (frow < 0 || fcol < 0 || frow >= height || fcol >= width) continue;
							real t = in[frow + (size_t)fcol * height];
							if (t > val) val = t;
						}
					}
					out[(size_t)l * p_height + k] = val;
				}
			}
		}
	}
}

/* functions/dev_pool.cu:41-77 (ker_avg_pool_layer): sum of the in-range cells / ksize^2. */
void oracle_avg_pool_forward(const real *input, int samples, int channels, int height, int width,
                             int ksize, int stride, int padding, int p_height, int p_width, real *output)
{
	for (int ch = 0; ch < channels; ch++) {
		for (int idx = 0; idx < samples; idx++) {
			const real *in = input + ((size_t)ch * samples + idx) * height * width;
			real *out = output + ((size_t)ch * samples + idx) * p_height * p_width;
			for (int l = 0; l < p_width; l++) {
				for (int k = 0; k < p_height; k++) {
					int i = k * stride - padding, j = l * stride - padding;
					real val = 0;
					for (int r = 0; r < ksize; r++) {
						for (int c = 0; c < ksize; c++) {
							int frow = i + r, fcol = j + c;
							if (frow < 0 || fcol < 0 || frow >= height || fcol >= width) continue;
							val += in[frow + (size_t)fcol * height];
						}
					}
					out[(size_t)l * p_height + k] = val / (ksize * ksize);
				}
			}
		}
	}
}

/* Position (offset inside one height x width map) selected by the reference's
 * backward scan, functions/dev_pool.cu:374-391: window columns outer, rows
 * inner, strict '>' -- i.e. the first maximum in memory order. */
static int argmax_in_window(const real *in, int height, int width, int ksize, int i, int j)
{
	int best = INT_MAX;
	real maxVal = -REAL_MAX;
	for (int c = 0; c < ksize; c++) {
		for (int r = 0; r < ksize; r++) {
			int fcol = j + c, frow = i + r;
			if (fcol < 0 || fcol >= width || frow < 0 || frow >= height) continue;
			int tid = frow + fcol * height;
			if (in[tid] > maxVal) {
				maxVal = in[tid];
				best = tid;
			}
		}
	}
	return best;
}

/* argmax offsets for every pooled cell, same layout as the pooled tensor. */
void oracle_max_pool_argmax(const real *z_in, int samples, int channels, int height, int width,
                            int ksize, int stride, int padding, int p_height, int p_width, int *index)
{
	for (int ch = 0; ch < channels; ch++)
		for (int idx = 0; idx < samples; idx++)
			for (int l = 0; l < p_width; l++)
				for (int k = 0; k < p_height; k++)
					index[((size_t)ch * samples + idx) * p_height * p_width + (size_t)l * p_height + k] =
					    argmax_in_window(z_in + ((size_t)ch * samples + idx) * height * width, height,
					                     width, ksize, k * stride - padding, l * stride - padding);
}

/* functions/dev_pool.cu:346-398 + :474-497 (memset, then add delta at the argmax). */
void oracle_max_pool_backward(const real *delta, const real *z_in, int channels, int height, int width,
                              int ksize, int stride, int padding, int p_height, int p_width, int samples,
                              real *output)
{
	memset(output, 0, sizeof(real) * (size_t)height * width * channels * samples);
#pragma omp parallel for collapse(2) schedule(static)
	for (int ch = 0; ch < channels; ch++) {
		for (int idx = 0; idx < samples; idx++) {
			const real *in = z_in + ((size_t)ch * samples + idx) * height * width;
			real *out = output + ((size_t)ch * samples + idx) * height * width;
			const real *d = delta + ((size_t)ch * samples + idx) * p_height * p_width;
			for (int l = 0; l < p_width; l++) {
				for (int k = 0; k < p_height; k++) {
					int t = argmax_in_window(in, height, width, ksize, k * stride - padding,
					                         l * stride - padding);
					if (t != INT_MAX) out[t] += d[(size_t)l * p_height + k];
				}
			}
		}
	}
}

/* functions/cnn_backward.cu:465-481 (scale by 1/ksize^2) + functions/dev_pool.cu:269-298
 * (spread over the window), written as the adjoint of the forward (D3). */
void oracle_avg_pool_backward(const real *delta, int channels, int height, int width, int ksize,
                              int stride, int padding, int p_height, int p_width, int samples,
                              real *output)
{
	memset(output, 0, sizeof(real) * (size_t)height * width * channels * samples);
	real scale = 1. / (ksize * ksize);
	for (int ch = 0; ch < channels; ch++) {
		for (int idx = 0; idx < samples; idx++) {
			real *out = output + ((size_t)ch * samples + idx) * height * width;
			const real *d = delta + ((size_t)ch * samples + idx) * p_height * p_width;
			for (int l = 0; l < p_width; l++) {
				for (int k = 0; k < p_height; k++) {
					int i = k * stride - padding, j = l * stride - padding;
					for (int c = 0; c < ksize; c++) {
						for (int r = 0; r < ksize; r++) {
							int fcol = j + c, frow = i + r;
							if (fcol < 0 || fcol >= width || frow < 0 || frow >= height) continue;
							out[frow + (size_t)fcol * height] += scale * d[(size_t)l * p_height + k];
						}
					}
				}
			}
		}
	}
}

/* ------------------------------------------------------------------ */
/* batch normalisation (spatial, non-affine)                           */
/* ------------------------------------------------------------------ */

/* functions/dev_batch_norm.cu:263-315 (mean, biased variance, running
 * statistics), :27-38 (z-hat), :331-393 (train / evaluation switch).
 * output holds rows*channels reals followed by the four per-channel vectors
 * at the given offsets (relative to output). */
void oracle_batch_norm_forward(const real *input, int height, int width, int channels, int samples,
                               real *output, int meansOffset, int variancesOffset, real epsilon,
                               int forTesting, real momentum, int runningMeansOffset,
                               int runningVariancesOffset)
{
	size_t rows = (size_t)height * width * samples;
	real *batch_mean = output + meansOffset;
	real *batch_variance = output + variancesOffset;
	real *dataset_mean = output + runningMeansOffset;
	real *dataset_variance = output + runningVariancesOffset;

	if (forTesting == MODEL_TRAIN) {
		for (int c = 0; c < channels; c++) {
			const real *x = input + (size_t)c * rows;
			real s = 0;
			for (size_t i = 0; i < rows; i++) s += x[i];
			batch_mean[c] = s * (1. / (real)rows);
			real v = 0;
			for (size_t i = 0; i < rows; i++) {
				real t = x[i] - batch_mean[c];
				v += t * t;
			}
			batch_variance[c] = v * (1. / (real)rows);
			dataset_mean[c] = momentum * dataset_mean[c] + (1. - momentum) * batch_mean[c];
			dataset_variance[c] = momentum * dataset_variance[c] + (1. - momentum) * batch_variance[c];
		}
	}
	const real *mu = (forTesting == MODEL_TRAIN) ? batch_mean : dataset_mean;
	const real *var = (forTesting == MODEL_TRAIN) ? batch_variance : dataset_variance;
	for (int c = 0; c < channels; c++)
		for (size_t i = 0; i < rows; i++)
			output[(size_t)c * rows + i] = (input[(size_t)c * rows + i] - mu[c]) / sqrt(var[c] + epsilon);
}

/* functions/dev_batch_norm.cu:550-621 with the helper :398-466 and the kernel
 * :132-150: out = (m*delta - sum(delta) - zhat * sum(delta*zhat)) / (m*sqrt(eps+var)). */
void oracle_batch_norm_backward(const real *delta, int height, int width, int channels, int samples,
                                const real *variance, real *output, const real *zout, real epsilon)
{
	size_t rows = (size_t)height * width * samples;
#pragma omp parallel for schedule(static)
	for (int c = 0; c < channels; c++) {
		const real *d = delta + (size_t)c * rows;
		const real *zh = zout + (size_t)c * rows;
		real *o = output + (size_t)c * rows;
		real sum1 = 0, sum2 = 0;
		for (size_t i = 0; i < rows; i++) {
			sum1 += d[i];
			sum2 += d[i] * zh[i];
		}
		real m = (real)rows;
		for (size_t i = 0; i < rows; i++)
			o[i] = (m * d[i] - sum1 - sum2 * zh[i]) / (m * sqrt(epsilon + variance[c]));
	}
}

/* ------------------------------------------------------------------ */
/* softmax cross entropy                                               */
/* ------------------------------------------------------------------ */

/* functions/softmax_loss.cu:17-79 + :141-213: probs (class fastest), mean
 * negative log-likelihood.  maxdot starts at 0 and 1e-10 is added to every
 * probability, as in the reference.  target holds 1-based class ids. */
real oracle_softmax_loss(const real *input, const real *target, int rows, int num_classes, real *probs)
{
	real total = 0;
	for (int r = 0; r < rows; r++) {
		real maxdot = 0;
		for (int i = 0; i < num_classes; i++)
			if (maxdot < input[i + (size_t)r * num_classes]) maxdot = input[i + (size_t)r * num_classes];
		real s = 0;
		for (int i = 0; i < num_classes; i++) {
			probs[i + (size_t)r * num_classes] = exp(input[i + (size_t)r * num_classes] - maxdot);
			s += probs[i + (size_t)r * num_classes];
		}
		for (int i = 0; i < num_classes; i++)
			probs[i + (size_t)r * num_classes] = probs[i + (size_t)r * num_classes] / s + 1e-10;
		real ind = 0;
		for (int i = 0; i < num_classes; i++)
			if ((int)target[r] == (i + 1)) ind = -log(probs[i + (size_t)r * num_classes]);
		total += ind;
	}
	return total / rows;
}

/* functions/softmax_loss.cu:215-245: errors = (probs - onehot) / rows. */
void oracle_cross_entropy_error(const real *probs, int rows, int numclasses, const real *target,
                                real *errors)
{
	real alpha = 1. / (real)rows;
	for (int r = 0; r < rows; r++)
		for (int c = 0; c < numclasses; c++) {
			real v = probs[c + (size_t)r * numclasses];
			if ((real)(c + 1) == target[r]) v -= 1.;
			errors[c + (size_t)r * numclasses] = v * alpha;
		}
}

/* ------------------------------------------------------------------ */
/* layers                                                              */
/* ------------------------------------------------------------------ */

/* functions/eval_convolution.cu:52-267 (applyConvolutionLayer): patch matrix,
 * GEMM (:115-119), bias (:26-34), batch norm (:132-161), activation
 * (:172-205), pooling (:215-219).  devScratch >= M*K reals. */
int oracle_conv_layer_forward(const real *input, int samples, int in_channels, int height, int width,
                              int ksize, int pad, int stride, int col_height, int col_width,
                              const real *weights, const real *bias, real *output, int out_channels,
                              int actFun, int pkSize, int pkStride, int pkPad, int poolFun,
                              int poolOutHeight, int poolOutWidth, int performBatchNorm, real epsilon,
                              int activationOffset, int poolOffset, int batchNormOffset, int meansOffset,
                              int variancesOffset, real *devScratch, int forTesting,
                              int runningMeansOffset, int runningVariancesOffset)
{
	real *imgCols = devScratch;
	real *imgColWtOut = output;
	real *actOut = output + activationOffset;
	size_t M = (size_t)samples * col_height * col_width;
	int K = ksize * ksize * in_channels;

	oracle_im2col(input, samples, in_channels, height, width, ksize, pad, stride, imgCols);
	oracle_gemm(OP_N, OP_N, (int)M, out_channels, K, 1, imgCols, (int)M, weights, K, 0, imgColWtOut, (int)M);
	if (bias)
		for (int c = 0; c < out_channels; c++)
			for (size_t i = 0; i < M; i++) imgColWtOut[(size_t)c * M + i] += bias[c];

	if (performBatchNorm != PERFORM_NO_BATCH_NORM) {
		real *batchOut = output + batchNormOffset;
		oracle_batch_norm_forward(imgColWtOut, col_height, col_width, out_channels, samples, batchOut,
		                          meansOffset, variancesOffset, epsilon, forTesting, BATCH_NORM_MOMENTUM,
		                          runningMeansOffset, runningVariancesOffset);
		memcpy(actOut, batchOut, sizeof(real) * M * out_channels);
	} else {
		memcpy(actOut, imgColWtOut, sizeof(real) * M * out_channels);
	}
	if (oracle_activation_forward(actFun, actOut, M * out_channels)) return -1;

	if (poolFun == MAX_POOL)
		oracle_max_pool_forward(actOut, samples, out_channels, col_height, col_width, pkSize, pkStride,
		                        pkPad, poolOutHeight, poolOutWidth, output + poolOffset);
	else if (poolFun == AVG_POOL)
		oracle_avg_pool_forward(actOut, samples, out_channels, col_height, col_width, pkSize, pkStride,
		                        pkPad, poolOutHeight, poolOutWidth, output + poolOffset);
	else if (poolFun != NO_POOL)
		return -1;
	return 0;
}

/* functions/eval_gradient.cu:29-229 (applyLayerActivation): W z + b, saved
 * pre-activation copy behind the output, activation in place. */
int oracle_fc_layer_forward(int actFunction, const real *W, int wRows, int wCols, const real *b,
                            const real *z, int zRows, int zCols, real *output)
{
	oracle_gemm(OP_N, OP_N, wRows, zCols, wCols, 1, W, wRows, z, zRows, 0, output, wRows);
	if (b)
		for (int n = 0; n < zCols; n++)
			for (int r = 0; r < wRows; r++) output[(size_t)n * wRows + r] += b[r];
	memcpy(output + (size_t)wRows * zCols, output, sizeof(real) * (size_t)wRows * zCols);
	return oracle_activation_forward(actFunction, output, (size_t)wRows * zCols);
}

/* functions/cnn_backward.cu:771-783: dW = im2col(X)^T * delta (K x Cout, ld K). */
void oracle_conv_weight_gradient(const real *input, const real *delta, int samples, int in_channels,
                                 int height, int width, int ksize, int pad, int stride,
                                 int out_channels, real *dW, real *devScratch)
{
	int col_h = (height + 2 * pad - ksize) / stride + 1;
	int col_w = (width + 2 * pad - ksize) / stride + 1;
	int M = col_h * col_w * samples, K = ksize * ksize * in_channels;
	oracle_im2col(input, samples, in_channels, height, width, ksize, pad, stride, devScratch);
	oracle_gemm(OP_T, OP_N, K, out_channels, M, 1, devScratch, M, delta, M, 0, dW, K);
}

/* functions/dev_backprop_convolution.cu:173-247 (backpropConvolution):
 * delta patch matrix, weight reorder [Cout][Cin][k*k]->[Cin][Cout][k*k], GEMM. */
void oracle_conv_input_gradient(const real *delta, int dHeight, int dWidth, int dChannels,
                                const real *filter, int fHeight, int fWidth, int height, int width,
                                int padding, int channels, int samples, real *delta_1, real *devPtr)
{
	real *imgCols = devPtr;
	real *reordered = imgCols + (size_t)samples * height * width * fHeight * fWidth * dChannels;
	oracle_delta_cols(delta, dHeight, dWidth, dChannels, fHeight, fWidth, imgCols, height, width,
	                  padding, samples);
	oracle_reshape(filter, dChannels, channels, fHeight * fWidth, reordered);
	int M = samples * height * width, R = fHeight * fWidth * dChannels;
	oracle_gemm(OP_N, OP_N, M, channels, R, 1, imgCols, M, reordered, R, 0, delta_1, M);
}

/* ------------------------------------------------------------------ */
/* KFAC Kronecker factors (the products only; inverses are not restated) */
/* ------------------------------------------------------------------ */

/* solvers/kfac_inverses.cu:489-540 (computeOmegaZ, convolution layers): patch matrix scaled by
 * 1/(outHeight*outWidth), a column of ones when the model has a bias, Z^T Z, then 1/samples.
 * factor is zCols x zCols column-major (symmetric); devScratch holds zRows*zCols reals. */
void oracle_kfac_conv_input_factor(const real *input, int samples, int in_channels, int height, int width,
                                   int ksize, int pad, int stride, int bias, real *factor, real *devScratch)
{
	int col_h = (height + 2 * pad - ksize) / stride + 1;
	int col_w = (width + 2 * pad - ksize) / stride + 1;
	int zRows = samples * col_h * col_w;
	int zCols = in_channels * ksize * ksize + (bias ? 1 : 0);
	real *expanded = devScratch;
	oracle_im2col(input, samples, in_channels, height, width, ksize, pad, stride, expanded);
	real alpha = (real)1 / (real)(col_h * col_w);
	size_t scaled = (size_t)zRows * (bias ? zCols - 1 : zCols);
	for (size_t i = 0; i < scaled; i++) expanded[i] *= alpha;
	if (bias)
		for (int i = 0; i < zRows; i++) expanded[(size_t)zRows * (zCols - 1) + i] = 1;
	oracle_gemm(OP_T, OP_N, zCols, zCols, zRows, 1, expanded, zRows, expanded, zRows, 0, factor, zCols);
	alpha = (real)1 / (real)samples;
	for (size_t i = 0; i < (size_t)zCols * zCols; i++) factor[i] *= alpha;
}

/* solvers/kfac_inverses.cu:782-816 (computeLambdaDelta, convolution layers): delta is
 * (samples*outHeight*outWidth) x outChannels column-major; G = delta^T delta scaled by the row count. */
void oracle_kfac_conv_output_factor(const real *delta, int samples, int out_height, int out_width,
                                    int out_channels, real *factor)
{
	int rows = samples * out_height * out_width;
	oracle_gemm(OP_T, OP_N, out_channels, out_channels, rows, 1, delta, rows, delta, rows, 0, factor, out_channels);
	real alpha = (real)out_height * (real)out_width * (real)samples;
	for (size_t i = 0; i < (size_t)out_channels * out_channels; i++) factor[i] *= alpha;
}

/* solvers/kfac_inverses.cu:596-625 (computeOmegaZ, linear layers): z is in x samples column-major,
 * a row of ones is appended when the model has a bias; A = Z (Z/samples)^T.
 * devScratch holds 2*zRows*samples reals. */
void oracle_kfac_fc_input_factor(const real *z, int in, int samples, int bias, real *factor, real *devScratch)
{
	int zRows = in + (bias ? 1 : 0);
	real *zMatrix = devScratch, *scaledZ = devScratch + (size_t)zRows * samples;
	for (int n = 0; n < samples; n++) {
		for (int r = 0; r < in; r++) zMatrix[(size_t)n * zRows + r] = z[(size_t)n * in + r];
		if (bias) zMatrix[(size_t)n * zRows + in] = 1;
	}
	real alpha = (real)1 / (real)samples;
	for (size_t i = 0; i < (size_t)zRows * samples; i++) scaledZ[i] = zMatrix[i] * alpha;
	oracle_gemm(OP_N, OP_T, zRows, zRows, samples, 1, zMatrix, zRows, scaledZ, zRows, 0, factor, zRows);
}

/* solvers/kfac_inverses.cu:838-852 (computeLambdaDelta, linear layers): delta is out x samples
 * column-major; G = delta delta^T scaled by samples. */
void oracle_kfac_fc_output_factor(const real *delta, int out, int samples, real *factor)
{
	oracle_gemm(OP_N, OP_T, out, out, samples, 1, delta, out, delta, out, 0, factor, out);
	for (size_t i = 0; i < (size_t)out * out; i++) factor[i] *= (real)samples;
}

/* solvers/kfac_inverses.cu:133-186 (computeMatrixInverseCusolver): identity right-hand side, copy of
 * the matrix with lambda + dampGamma added to the diagonal, Cholesky factorization of the lower
 * triangle (what cusolverDnDpotrf computes: A = L L^T, column by column) and the two triangular
 * solves of cusolverDnDpotrs for every column of the identity.  matrix and inverse are n x n
 * column-major; devScratch holds n*n reals.  Returns 0, or the 1-based index of the first
 * non-positive pivot (cusolver's devInfo), in which case inverse is not meaningful. */
int oracle_matrix_inverse(const real *matrix, real *inverse, int n, real lambda, real dampGamma, real *devScratch)
{
	real *L = devScratch;
	for (size_t i = 0; i < (size_t)n * n; i++) inverse[i] = 0;
	for (int i = 0; i < n; i++) inverse[(size_t)i * n + i] = 1;
	memcpy(L, matrix, sizeof(real) * (size_t)n * n);
	for (int i = 0; i < n; i++) L[(size_t)i * n + i] += lambda + dampGamma;
	for (int j = 0; j < n; j++) {
		real d = L[(size_t)j * n + j];
		for (int k = 0; k < j; k++) d -= L[(size_t)k * n + j] * L[(size_t)k * n + j];
		if (!(d > 0)) return j + 1;
		d = (real)sqrt((double)d);
		L[(size_t)j * n + j] = d;
#pragma omp parallel for schedule(static)
		for (int i = j + 1; i < n; i++) {
			real v = L[(size_t)j * n + i];
			for (int k = 0; k < j; k++) v -= L[(size_t)k * n + i] * L[(size_t)k * n + j];
			L[(size_t)j * n + i] = v / d;
		}
	}
#pragma omp parallel for schedule(static)
	for (int c = 0; c < n; c++) {
		real *x = inverse + (size_t)c * n;
		for (int i = 0; i < n; i++) { /* L y = e_c */
			real v = x[i];
			for (int k = 0; k < i; k++) v -= L[(size_t)k * n + i] * x[k];
			x[i] = v / L[(size_t)i * n + i];
		}
		for (int i = n - 1; i >= 0; i--) { /* L^T x = y */
			real v = x[i];
			for (int k = i + 1; k < n; k++) v -= L[(size_t)i * n + k] * x[k];
			x[i] = v / L[(size_t)i * n + i];
		}
	}
	return 0;
}

/* solvers/kfac_natural_gradient.cu:36-241 (computeNaturalGradient): per convolution layer wb = the
 * (K+1) x Cout matrix [filter ; bias], result = Lambda * wb', nGrad = result * Omega (Cout x (K+1),
 * leading dimension Cout), then the weight part transposed back with the bias column left where the
 * flat layout keeps the bias; per linear layer Lambda * [W | b] * Omega in place.  devScratch holds
 * three of the largest (K+1) x Cout matrices. */
void oracle_natural_gradient(const CNN_MODEL *model, const int *omegaZOffsets, const int *lambdaGOffsets,
                             const real *omegaPtr, const real *lambdaPtr, const real *vec, real *nGradient,
                             real *devScratch)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets;
	for (int c = 0; c < model->cLayers; c++) {
		const CONV_LAYER *convLayer = &model->convLayer[c];
		int outChannels = convLayer->outChannels, K = convLayer->inChannels * convLayer->kSize * convLayer->kSize;
		int cols = K + ((model->bias == 0) ? 0 : 1);
		const real *omegaZ = omegaPtr + omegaZOffsets[c], *lambdaG = lambdaPtr + lambdaGOffsets[c];
		const real *vComponent = vec + wOffsets[c];
		real *nGradComponent = nGradient + wOffsets[c];
		real *wb = devScratch, *nextDevPtr = wb + (size_t)outChannels * cols;
		for (int o = 0; o < outChannels; o++) {
			for (int k = 0; k < K; k++) wb[(size_t)o * cols + k] = vComponent[(size_t)o * K + k];
			if (model->bias != 0) wb[(size_t)o * cols + cols - 1] = vec[bOffsets[c] + o];
		}
		oracle_gemm(OP_N, OP_T, outChannels, cols, outChannels, 1, lambdaG, outChannels, wb, cols, 0, nextDevPtr,
		            outChannels);
		oracle_gemm(OP_N, OP_N, outChannels, cols, cols, 1, nextDevPtr, outChannels, omegaZ, cols, 0, nGradComponent,
		            outChannels);
		/* cublasDgeam(OP_T): K x Cout <- (Cout x K)' of the weight part, then copied back */
		for (int o = 0; o < outChannels; o++)
			for (int k = 0; k < K; k++) nextDevPtr[(size_t)o * K + k] = nGradComponent[(size_t)k * outChannels + o];
		memcpy(nGradComponent, nextDevPtr, sizeof(real) * (size_t)outChannels * K);
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *ll = &model->fcLayer[l];
		int at = model->cLayers + l, cols = ll->in + ((model->bias == 0) ? 0 : 1);
		const real *omegaZ = omegaPtr + omegaZOffsets[at], *lambdaG = lambdaPtr + lambdaGOffsets[at];
		real *nextDevPtr = devScratch;
		oracle_gemm(OP_N, OP_N, ll->out, cols, ll->out, 1, lambdaG, ll->out, vec + wOffsets[at], ll->out, 0, nextDevPtr,
		            ll->out);
		oracle_gemm(OP_N, OP_N, ll->out, cols, cols, 1, nextDevPtr, ll->out, omegaZ, cols, 0, nGradient + wOffsets[at],
		            ll->out);
	}
}

/* functions/cnn_accuracy.cu:15-59 (ker_compute_accuracy + computeAccuracy): hits counted with the
 * strict '<' scan from probability 0; returns the percentage, *hitsOut the count. */
real oracle_compute_accuracy(const real *probs, const real *target, int rows, int numClasses, real *hitsOut)
{
	real hits = 0;
	for (int idx = 0; idx < rows; idx++) {
		real maxProb = 0;
		int myClass = 0;
		for (int c = 0; c < numClasses; c++) {
			if (maxProb < probs[(size_t)idx * numClasses + c]) {
				maxProb = probs[(size_t)idx * numClasses + c];
				myClass = c;
			}
		}
		if ((real)(myClass + 1) == target[idx]) hits += 1;
	}
	if (hitsOut) *hitsOut = hits;
	return (hits * 100) / (real)rows;
}

/* functions/dev_dist_errors.cu:12-35 (ker_compute_dist_classes): inverse-CDF draw of one 1-based
 * class per sample from the uniform numbers distProbs. */
void oracle_multinomial_classes(const real *probs, int samples, int numClasses, const real *distProbs, real *distClasses)
{
	for (int idx = 0; idx < samples; idx++) {
		real c = 0;
		distClasses[idx] = -1;
		for (int i = 0; i < numClasses; i++) {
			c += probs[(size_t)idx * numClasses + i];
			if (c >= distProbs[idx]) {
				distClasses[idx] = i + 1;
				i += (numClasses + 1);
			}
		}
		if (distClasses[idx] == -1) distClasses[idx] = numClasses + 1;
	}
}

/* The seeded stream that stands in for cuRAND (device/gen_random.cu:25-52): element g is the
 * splitmix64 hash of seed + (g+1)*golden, its top 24 bits + 1 scaled to (0, 1].  Integer arithmetic:
 * every implementation of it must agree bit for bit. */
void oracle_uniform_stream(unsigned long long seed, unsigned long long first, long n, float *out)
{
	for (long i = 0; i < n; i++) {
		unsigned long long z = seed + (first + (unsigned long long)i + 1ull) * 0x9E3779B97F4A7C15ull;
		z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
		z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
		z = z ^ (z >> 31);
		out[i] = (float)((z >> 40) + 1ull) * (1.0f / 16777216.0f);
	}
}

/* ------------------------------------------------------------------ */
/* fully connected model family (functions/eval_gradient.cu)           */
/* ------------------------------------------------------------------ */

/* functions/eval_gradient.cu:29-229 (applyLayerActivation) without the copy of W z + b behind the
 * output (that copy belongs to the CNN path; for the last layer of an NN_MODEL it lies past zSize).
 * ACT_SOFTMAX: exp, column sums, division -- no maximum shift (:162-193). */
static int oracle_nn_layer(int actFunction, const real *W, int wRows, int wCols, const real *b, const real *z,
                           int zCols, real *output)
{
	oracle_gemm(OP_N, OP_N, wRows, zCols, wCols, 1, W, wRows, z, wCols, 0, output, wRows);
	if (b != NULL)
		for (int n = 0; n < zCols; n++)
			for (int r = 0; r < wRows; r++) output[(size_t)n * wRows + r] += b[r];
	if (actFunction == ACT_SOFTMAX) {
		for (int n = 0; n < zCols; n++) {
			real sum = 0;
			for (int r = 0; r < wRows; r++) {
				output[(size_t)n * wRows + r] = exp(output[(size_t)n * wRows + r]);
				sum += output[(size_t)n * wRows + r];
			}
			for (int r = 0; r < wRows; r++) output[(size_t)n * wRows + r] /= sum;
		}
		return 0;
	}
	if (actFunction == ACT_NONE) return 0;
	return oracle_activation_forward(actFunction, output, (size_t)wRows * zCols);
}

/* functions/eval_gradient.cu:275-555 (nnForwardPass) on explicit data: dataset is features x numCols,
 * target outSize x numColsTarget.  Fills z (at zOffsets) and errTerm, returns the log-likelihood
 * figure (-(1/numColsTarget) * sum of the head's terms, dev_loglikelihood.cu:4-41) and *modelError. */
real oracle_nn_forward(const NN_MODEL *model, const real *weights, const real *dataset, const real *target,
                       int numCols, int numColsTarget, const int *zOffsets, real *z, real *errTerm,
                       real *modelError, real *devScratch)
{
	const int numLayers = model->numLayers;
	const int *layerSizes = model->layerSizes;
	for (int i = 0; i < numLayers; i++) {
		const real *in = (i == 0) ? dataset : z + zOffsets[i];
		if (oracle_nn_layer(model->actFuns[i], weights + model->wOffsets[i], layerSizes[i + 1], layerSizes[i],
		                    weights + model->bOffsets[i], in, numCols, z + zOffsets[i + 1]) != 0)
			return (real)NAN;
	}
	const real *out = z + zOffsets[numLayers];
	size_t numElements = (size_t)layerSizes[numLayers] * numColsTarget;
	real logLikelihood = 0;
	int head = model->actFuns[numLayers - 1];
	if (head == ACT_LINEAR) {
		for (size_t i = 0; i < numElements; i++) logLikelihood += pow(target[i] - out[i], 2.0);
		for (size_t i = 0; i < numElements; i++) errTerm[i] = 2.0 * (target[i] - out[i]);
	} else if (head == ACT_LOGISTIC) {
		real *xi = devScratch;
		const real *in = (numLayers == 1) ? dataset : z + zOffsets[numLayers - 1];
		oracle_nn_layer(ACT_LINEAR, weights + model->wOffsets[numLayers - 1], layerSizes[numLayers],
		                layerSizes[numLayers - 1], weights + model->bOffsets[numLayers - 1], in, numCols, xi);
		for (size_t i = 0; i < numElements; i++) {
			real lx = xi[i], lxx = (lx >= 0) ? 1 : 0;
			logLikelihood += lx * (target[i] - lxx) - log(1 + exp(lx - 2.0 * lx * lxx));
		}
		for (size_t i = 0; i < numElements; i++) errTerm[i] = 1.0 * (target[i] - out[i]);
	} else if (head == ACT_SOFTMAX) {
		for (size_t i = 0; i < numElements; i++) logLikelihood += target[i] * log(out[i]);
		for (size_t i = 0; i < numElements; i++) errTerm[i] = 1.0 * (target[i] - out[i]);
	}
	logLikelihood *= -1.0 / (real)numColsTarget;
	*modelError = 0;
	if (model->type == MODEL_TYPE_MSE) {
		real e = 0;
		for (size_t i = 0; i < numElements; i++) e += pow(target[i] - out[i], 2.0);
		*modelError = e / (real)numColsTarget;
	}
	return logLikelihood;
}

/* functions/eval_gradient.cu:561-914 (computeGradient): forward pass, then per layer from the top
 * db = sum(err, 2), dW = err * z_i', dx_i = err, err = W_i' * err with the logistic / tanh derivative
 * of the layer below (dev_layer_error.cu:13-29), and the final scale -1/n.  The first layer's weight
 * gradient reads the data set (:704).  errScratch holds max layer size x n reals. */
real oracle_nn_gradient(const NN_MODEL *model, const real *weights, const real *dataset, const real *target, int n,
                        const int *zOffsets, const int *rZOffsets, real *z, real *dx, real *gradient,
                        real *modelError, real *errScratch, real *devScratch)
{
	const int numLayers = model->numLayers;
	const int *layerSizes = model->layerSizes;
	real *errorTerm = errScratch;
	real ll = oracle_nn_forward(model, weights, dataset, target, n, n, zOffsets, z, errorTerm, modelError, devScratch);
	real *next = devScratch;
	for (int i = numLayers - 1; i >= 0; i--) {
		int out = layerSizes[i + 1], in = layerSizes[i];
		size_t count = (size_t)out * n;
		if (i < numLayers - 1) {
			const real *xi = z + zOffsets[i + 1];
			if (model->actFuns[i] == ACT_LOGISTIC) {
				for (size_t k = 0; k < count; k++) errorTerm[k] = errorTerm[k] * xi[k] * (1.0 - xi[k]);
			} else if (model->actFuns[i] == ACT_TANH) {
				for (size_t k = 0; k < count; k++) errorTerm[k] *= (1.0 + xi[k]) * (1.0 - xi[k]);
			} else if (model->actFuns[i] != ACT_LINEAR) {
				return (real)NAN;
			}
		}
		for (int r = 0; r < out; r++) {
			real sum = 0;
			for (int c = 0; c < n; c++) sum += errorTerm[(size_t)c * out + r];
			gradient[model->bOffsets[i] + r] = sum;
		}
		const real *zin = (i == 0) ? dataset : z + zOffsets[i];
		oracle_gemm(OP_N, OP_T, out, in, n, 1, errorTerm, out, zin, in, 0, gradient + model->wOffsets[i], out);
		memcpy(dx + rZOffsets[i], errorTerm, sizeof(real) * count);
		if (i > 0) {
			oracle_gemm(OP_T, OP_N, in, n, out, 1, weights + model->wOffsets[i], out, dx + rZOffsets[i], out, 0, next, in);
			memcpy(errorTerm, next, sizeof(real) * (size_t)in * n);
		}
	}
	for (int i = 0; i < model->pSize; i++) gradient[i] *= -(1.0 / (real)n);
	return ll;
}

/* functions/eval_hessian_vec.cu:20-545 (hessianVec, gaussNewton == 0) and
 * functions/eval_gauss_newton_hessian_vec.cu:21-361 (gaussNewtonHessianVec, gaussNewton == 1): the R-operator
 * over an NN_MODEL, given z and dx of oracle_nn_gradient at the same weights and data.
 *   forward   Rx_{i+1} = VW_i z_i + Vb_i + W_i Rz_i,  Rz_{i+1} = f'(.) Rx_{i+1}; softmax: z.rx - z sum(z.rx)
 *   head      Rdx_L = -Rz_{L+1}   (logistic and softmax heads; the linear head is refused there, NAN here)
 *   backward  RdW_i = Rdx_i z_i' [+ dx_i Rz_i'],  Rdb_i = sum(Rdx_i, 2),  Rdz_i = [VW_i' dx_i +] W_i' Rdx_i,
 *             Rdx_{i-1} = f'(z_i) Rdz_i [+ Rx_i (1 - 2 z_i) dx_{i-1}]   (dev_hessian_helpers.cu:7-26)
 *   result    -(1/n) [RdW, Rdb]
 * The bracketed terms are the second-order ones; the Gauss-Newton variant drops them EXCEPT VW' dx of the
 * top layer (eval_gauss_newton_hessian_vec.cu:262-275 keeps it); topLayerTerm = 0 drops that one too, which
 * is the textbook Gauss-Newton product and exists here so that tests can pin both.  Hidden tanh layers: the
 * reference leaves Rdx unset in the backward sweep (:418-420); the derivative is restated here
 * (f' = 1 - z^2, f'' dz = -2 z dx). */
int oracle_nn_hessian_vec(const NN_MODEL *model, const real *weights, const real *vec, const real *dataset, int n,
                          const int *zOffsets, const int *rZOffsets, const real *z, const real *dx, int gaussNewton,
                          int topLayerTerm, real *result)
{
	const int L = model->numLayers;
	const int *ls = model->layerSizes, *wOff = model->wOffsets, *bOff = model->bOffsets;
	const int head = model->actFuns[L - 1];
	if (head != ACT_LOGISTIC && head != ACT_SOFTMAX) return -1;
	size_t zTotal = 0, widest = 0;
	for (int i = 0; i <= L; i++) {
		size_t end = (size_t)zOffsets[i] + (size_t)ls[i] * n;
		if (end > zTotal) zTotal = end;
		if ((size_t)ls[i] > widest) widest = ls[i];
	}
	real *Rz = (real *)calloc(zTotal, sizeof(real)), *Rx = (real *)calloc(zTotal, sizeof(real));
	real *Rdz = (real *)calloc(zTotal, sizeof(real));
	real *Rdx = (real *)calloc(widest * n, sizeof(real));
	int rc = 0;
	for (int i = 0; i < L && rc == 0; i++) {
		const int out = ls[i + 1], in = ls[i];
		const real *zin = (i == 0) ? dataset : z + zOffsets[i];
		real *rxi = Rx + zOffsets[i + 1], *rzi = Rz + zOffsets[i + 1];
		const real *zo = z + zOffsets[i + 1];
		oracle_gemm(OP_N, OP_N, out, n, in, 1, vec + wOff[i], out, zin, in, 0, rxi, out);
		for (int c = 0; c < n; c++)
			for (int r = 0; r < out; r++) rxi[(size_t)c * out + r] += vec[bOff[i] + r];
		if (i > 0) oracle_gemm(OP_N, OP_N, out, n, in, 1, weights + wOff[i], out, Rz + zOffsets[i], in, 1, rxi, out);
		const size_t count = (size_t)out * n;
		switch (model->actFuns[i]) {
		case ACT_LOGISTIC:
			for (size_t k = 0; k < count; k++) rzi[k] = rxi[k] * zo[k] * (1.0 - zo[k]);
			break;
		case ACT_TANH:
			for (size_t k = 0; k < count; k++) rzi[k] = rxi[k] * (1.0 + zo[k]) * (1.0 - zo[k]);
			break;
		case ACT_LINEAR:
			memcpy(rzi, rxi, sizeof(real) * count);
			break;
		case ACT_SOFTMAX:
			for (int c = 0; c < n; c++) {
				real sum = 0;
				for (int r = 0; r < out; r++) sum += zo[(size_t)c * out + r] * rxi[(size_t)c * out + r];
				for (int r = 0; r < out; r++) {
					const size_t k = (size_t)c * out + r;
					rzi[k] = zo[k] * rxi[k] - zo[k] * sum;
				}
			}
			break;
		default: rc = -1;
		}
	}
	for (int i = L - 1; i >= 0 && rc == 0; i--) {
		const int out = ls[i + 1], in = ls[i];
		const size_t count = (size_t)out * n;
		const real *dxi = dx + rZOffsets[i];
		const real *zin = (i == 0) ? dataset : z + zOffsets[i];
		if (i == L - 1) {
			for (size_t k = 0; k < count; k++) Rdx[k] = -Rz[zOffsets[L] + k];
		} else {
			const real *zo = z + zOffsets[i + 1], *rdz = Rdz + zOffsets[i + 1], *rx = Rx + zOffsets[i + 1];
			const int second = !gaussNewton;
			switch (model->actFuns[i]) {
			case ACT_LOGISTIC:
				for (size_t k = 0; k < count; k++)
					Rdx[k] = (1.0 - zo[k]) * zo[k] * rdz[k] + (second ? rx[k] * (1.0 - 2 * zo[k]) * dxi[k] : 0);
				break;
			case ACT_TANH:
				for (size_t k = 0; k < count; k++)
					Rdx[k] = (1.0 + zo[k]) * (1.0 - zo[k]) * rdz[k] + (second ? rx[k] * (-2.0 * zo[k]) * dxi[k] : 0);
				break;
			case ACT_LINEAR:
				memcpy(Rdx, rdz, sizeof(real) * count);
				break;
			default: rc = -1;
			}
			if (rc) break;
		}
		oracle_gemm(OP_N, OP_T, out, in, n, 1, Rdx, out, zin, in, 0, result + wOff[i], out);
		if (!gaussNewton && i > 0)
			oracle_gemm(OP_N, OP_T, out, in, n, 1, dxi, out, Rz + zOffsets[i], in, 1, result + wOff[i], out);
		for (int r = 0; r < out; r++) {
			real sum = 0;
			for (int c = 0; c < n; c++) sum += Rdx[(size_t)c * out + r];
			result[bOff[i] + r] = sum;
		}
		if (i > 0) {
			real *rdzi = Rdz + zOffsets[i];
			oracle_gemm(OP_T, OP_N, in, n, out, 1, weights + wOff[i], out, Rdx, out, 0, rdzi, in);
			const int vwTerm = !gaussNewton || (i == L - 1 && topLayerTerm);
			if (vwTerm) oracle_gemm(OP_T, OP_N, in, n, out, 1, vec + wOff[i], out, dxi, out, 1, rdzi, in);
		}
	}
	for (int k = 0; k < model->pSize && rc == 0; k++) result[k] *= -(1.0 / (real)n);
	free(Rz), free(Rx), free(Rdz), free(Rdx);
	return rc;
}

/* ------------------------------------------------------------------ */
/* whole model                                                         */
/* ------------------------------------------------------------------ */

static size_t max_patch_reals(const CNN_MODEL *model, int batch)
{
	size_t best = 0;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		const POOL_LAYER *p = &model->poolLayer[i];
		size_t kk = (size_t)c->kSize * c->kSize;
		size_t fwd = (size_t)p->height * p->width * batch * c->inChannels * kk;
		size_t bwd = (size_t)c->height * c->width * batch * c->outChannels * kk +
		             (size_t)c->outChannels * c->inChannels * kk;
		if (fwd > best) best = fwd;
		if (bwd > best) best = bwd;
	}
	return best + 16;
}

/* functions/cnn_forward.cu:49-383 (cnnForward).  x is the batch
 * [C][N][W][H]; y the 1-based labels; returns the mean NLL, or NAN on an
 * unknown activation / pool code. */
real oracle_cnn_forward(const CNN_MODEL *model, const real *weights, const real *x, const real *y,
                        int numClasses, real *z, real *probs, real *errors, int curBatchSize,
                        int forTesting)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	int nc = model->cLayers;
	real *scratch = (real *)malloc(sizeof(real) * max_patch_reals(model, curBatchSize));
	if (!scratch) return NAN;

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *cv = &model->convLayer[l];
		const POOL_LAYER *pl = &model->poolLayer[l];
		const real *in = (l == 0) ? x : z + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		int rc = oracle_conv_layer_forward(
		    in, curBatchSize, cv->inChannels, cv->height, cv->width, cv->kSize, cv->padding, cv->stride,
		    cv->outHeight, cv->outWidth, weights + wOffsets[l],
		    (model->bias == 0) ? NULL : weights + bOffsets[l], z + zOffsets[l + 1], cv->outChannels,
		    model->actFuns[l], pl->pSize, pl->stride, pl->padding, pl->type, pl->outHeight, pl->outWidth,
		    cv->batchNorm, BATCH_NORM_EPSILON, cv->activationOffset, cv->poolOffset, cv->batchNormOffset,
		    cv->meansOffset, cv->variancesOffset, scratch, forTesting, cv->runningMeansOffset,
		    cv->runningVariancesOffset);
		if (rc) {
			free(scratch);
			return NAN;
		}
	}

	/* [C][N][w*H+h] -> [N][C][h*W+w], in place (cnn_forward.cu:238-261) */
	const CONV_LAYER *c = &model->convLayer[nc - 1];
	const POOL_LAYER *p = &model->poolLayer[nc - 1];
	int fh = (p->type != NO_POOL) ? p->outHeight : c->outHeight;
	int fw = (p->type != NO_POOL) ? p->outWidth : c->outWidth;
	real *feat = z + zOffsets[nc] + c->outputOffset;
	size_t featCount = (size_t)fh * fw * curBatchSize * c->outChannels;
	oracle_reshape(feat, c->outChannels, curBatchSize, fh * fw, scratch);
	oracle_transpose(scratch, c->outChannels * curBatchSize, fh, fw, feat);
	(void)featCount;

	int outputOffset = c->outputOffset;
	for (int l = 0; l < model->lLayers; l++) {
		if (l != 0) outputOffset = 0;
		const FC_LAYER *f = &model->fcLayer[l];
		if (oracle_fc_layer_forward(f->actFun, weights + wOffsets[l + nc], f->out, f->in,
		                            (model->bias == 0) ? NULL : weights + bOffsets[l + nc],
		                            z + zOffsets[l + nc] + outputOffset, f->in, curBatchSize,
		                            z + zOffsets[l + 1 + nc])) {
			free(scratch);
			return NAN;
		}
	}
	const real *logits = (model->lLayers == 0) ? z + zOffsets[nc] + c->outputOffset
	                                           : z + zOffsets[model->lLayers + nc];
	real loss = oracle_softmax_loss(logits, y, curBatchSize, numClasses, probs);
	oracle_cross_entropy_error(probs, curBatchSize, numClasses, y, errors);
	free(scratch);
	return loss;
}

/* functions/cnn_backward.cu:76-857 (cnnBackward).  delta holds the loss
 * errors on entry; delta and delta_new are clobbered.  Returns 0, or -1 on an
 * unknown activation / pool code (where the reference exits). */
int oracle_cnn_backward(const CNN_MODEL *model, const real *weights, const real *x, const real *z,
                        real *gradient, real *dx, real *delta, real *delta_new, int batchSize)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	int n = batchSize, cLayers = model->cLayers;
	real *scratch = (real *)malloc(sizeof(real) * max_patch_reals(model, batchSize));
	if (!scratch) return -1;
	const CONV_LAYER *cLayer = &model->convLayer[cLayers - 1];
	const POOL_LAYER *pLayer = &model->poolLayer[cLayers - 1];
	real *temp;

	for (int f = model->lLayers - 1; f >= 0; f--) {
		FC_LAYER l = model->fcLayer[f];
		const real *zl = z + zOffsets[f + cLayers + 1];
		if (oracle_activation_backward(l.actFun, delta, zl + l.offset, zl, (size_t)l.out * n)) {
			free(scratch);
			return -1;
		}
		/* dW = delta * z' (:189-197) */
		oracle_gemm(OP_N, OP_T, l.out, l.in, n, 1, delta, l.out,
		            z + zOffsets[f + cLayers] + ((f == 0) ? cLayer->outputOffset : 0), l.in, 0,
		            gradient + wOffsets[f + cLayers], l.out);
		if (model->bias != 0) {
			/* db = delta * 1 (:212-224) */
			for (int i = 0; i < n; i++) scratch[i] = 1;
			oracle_gemv(OP_N, l.out, n, 1, delta, l.out, scratch, 0, gradient + bOffsets[f + cLayers]);
		}
		memcpy(dx + zOffsets[f + cLayers + 1], delta, sizeof(real) * (size_t)l.out * n);
		/* delta = W' * delta (:250-254) */
		oracle_gemm(OP_T, OP_N, l.in, n, l.out, 1, weights + wOffsets[f + cLayers], l.out, delta, l.out, 0,
		            delta_new, l.in);
		temp = delta_new;
		delta_new = delta;
		delta = temp;
	}

	/* [N][C][h*W+w] -> [C][N][w*H+h] (:310-326) */
	{
		int fh = (pLayer->type != NO_POOL) ? pLayer->outHeight : cLayer->outHeight;
		int fw = (pLayer->type != NO_POOL) ? pLayer->outWidth : cLayer->outWidth;
		oracle_reshape(delta, n, cLayer->outChannels, fh * fw, scratch);
		oracle_transpose_rc(scratch, cLayer->outChannels * n, fh, fw, delta);
	}

	for (int c = cLayers - 1; c >= 0; c--) {
		CONV_LAYER l = model->convLayer[c];
		POOL_LAYER p = model->poolLayer[c];
		const real *slab = z + zOffsets[c + 1];
		size_t actCount = (size_t)n * l.activationVolumn;

		switch (p.type) {
		case MAX_POOL:
			oracle_max_pool_backward(delta, slab + l.activationOffset, l.outChannels, p.height, p.width,
			                         p.pSize, p.stride, p.padding, p.outHeight, p.outWidth, n, delta_new);
			break;
		case AVG_POOL:
			oracle_avg_pool_backward(delta, l.outChannels, p.height, p.width, p.pSize, p.stride,
			                         p.padding, p.outHeight, p.outWidth, n, delta_new);
			break;
		case NO_POOL:
			memcpy(delta_new, delta, sizeof(real) * actCount);
			break;
		default:
			free(scratch);
			return -1;
		}
		memcpy(dx + zOffsets[c + 1], delta_new, sizeof(real) * actCount);

		const real *actIn = (l.batchNorm != PERFORM_NO_BATCH_NORM) ? slab + l.batchNormOffset : slab;
		const real *actOut = slab + l.activationOffset;
		if (c == cLayers - 1 && p.type == NO_POOL) {
			/* departure D6: the stored activation output is in the FC layout */
			memcpy(scratch, actIn, sizeof(real) * actCount);
			if (oracle_activation_forward(model->actFuns[c], scratch, actCount)) {
				free(scratch);
				return -1;
			}
			actOut = scratch;
		}
		if (oracle_activation_backward(model->actFuns[c], delta_new, actIn, actOut, actCount)) {
			free(scratch);
			return -1;
		}
		memcpy(dx + zOffsets[c + 1] + l.activationOffset, delta_new, sizeof(real) * actCount);

		if (l.batchNorm != PERFORM_NO_BATCH_NORM) {
			oracle_batch_norm_backward(delta_new, l.outHeight, l.outWidth, l.outChannels, n,
			                           slab + l.batchNormOffset + l.variancesOffset, delta,
			                           slab + l.batchNormOffset, BATCH_NORM_EPSILON);
			memcpy(dx + zOffsets[c + 1] + l.batchNormOffset, delta, sizeof(real) * actCount);
			memcpy(delta_new, delta, sizeof(real) * actCount);
		}

		int M = p.height * p.width * n;
		if (model->bias != 0) {
			/* db = 1' * delta (:662-689) */
			for (int i = 0; i < M; i++) scratch[i] = 1;
			oracle_gemm(OP_N, OP_N, 1, l.outChannels, M, 1, scratch, 1, delta_new, M, 0,
			            gradient + bOffsets[c], 1);
		}

		const real *dataset = (c == 0) ? x : z + zOffsets[c] + model->convLayer[c - 1].outputOffset;
		oracle_conv_weight_gradient(dataset, delta_new, n, l.inChannels, l.height, l.width, l.kSize,
		                            l.padding, l.stride, l.outChannels, gradient + wOffsets[c], scratch);
		if (c != 0)
			oracle_conv_input_gradient(delta_new, p.height, p.width, l.outChannels,
			                           weights + wOffsets[c], l.kSize, l.kSize, l.height, l.width,
			                           l.padding, l.inChannels, n, delta, scratch);
	}
	free(scratch);
	return 0;
}

/* functions/cnn_gradient.cu:13-64 (computeCNNGradient): forward, backward,
 * gradient += weightDecay * weights.  Returns the loss. */
real oracle_cnn_gradient(const CNN_MODEL *model, const real *weights, const real *x, const real *y,
                         int numClasses, real *z, real *dx, real *probs, real *lossFuncErrors,
                         real *gradient, int curBatchSize, real weightDecay)
{
	real loss = oracle_cnn_forward(model, weights, x, y, numClasses, z, probs, lossFuncErrors,
	                               curBatchSize, MODEL_TRAIN);
	size_t dsz = (size_t)model->maxDeltaSize;
	real *errors = (real *)calloc(2 * dsz, sizeof(real));
	if (!errors) return NAN;
	memcpy(errors, lossFuncErrors, sizeof(real) * (size_t)numClasses * curBatchSize);
	if (oracle_cnn_backward(model, weights, x, z, gradient, dx, errors, errors + dsz, curBatchSize))
		loss = NAN;
	for (int i = 0; i < model->pSize; i++) gradient[i] += weightDecay * weights[i];
	free(errors);
	return loss;
}


/* ------------------------------------------------------------------ */
/* Hessian-vector product (R-operator forward and backward passes)     */
/* ------------------------------------------------------------------ */
/*
 * Restatement of functions/cnn_hessian_vec.cu:18-122 (cnnHv), cnn_hv_forward.cu:53-222
 * (cnnROpForward), cnn_hv_backward.cu:70-912 (cnnROpBackward), rop_fc_layer.cu:34-133
 * (applyROpLayerActivation), eval_convolution.cu:285-... (applyROpConvolutionLayer),
 * dev_pool.cu:123-221 (applyROpPoolLayer), dev_batch_norm.cu:637-960 (batch-norm R-op) and
 * softmax_loss.cu:251-300 (computeROpCrossEntropyError_simple): R{.} is the directional derivative
 * along `vector` in weight space; the forward pass carries R{z} through every layer, the backward
 * pass carries R{delta} and emits R{gradient} = H * vector.
 * Departures from the reference code, all of them defects there: every layer uses its own
 * activation (the reference passes actFuns[0] for all, cnn_hv_forward.cu:125), the batch-norm R-op
 * indexes variances by channel (dev_batch_norm.cu:181 indexes by element), the swish second
 * derivative is evaluated per element (swish.cu:47 multiplies the index), and D1-D6 of the
 * gradient path apply unchanged.
 */

/* out = rdelta * f'(.) + delta * f''(.) * rz_in: the R-operator of delta * f'(.)
 * (first derivatives as in oracle_activation_backward; second derivatives: logistic a(1-a)(1-2a),
 * tanh -2a(1-a^2), softplus s(1-s), swish s(1-s)(2 + x(1-2s)), ELU e^x below zero, ReLU 0). */
int oracle_activation_rop_backward(int actFun, const real *rdelta, const real *delta, const real *z_in,
                                   const real *z_out, const real *rz_in, real *out, size_t n)
{
	for (size_t i = 0; i < n; i++) {
		real f1, f2;
		switch (actFun) {
		case ACT_LOGISTIC: {
			real a = z_out[i];
			f1 = a * (1.0 - a), f2 = a * (1.0 - a) * (1.0 - 2.0 * a);
			break;
		}
		case ACT_TANH: {
			real a = z_out[i];
			f1 = (1.0 + a) * (1.0 - a), f2 = -2.0 * a * (1.0 + a) * (1.0 - a);
			break;
		}
		case CNN_ACT_SOFTPLUS: {
			real s = 1. / (1. + exp(-z_in[i]));
			f1 = s, f2 = s * (1. - s);
			break;
		}
		case CNN_ACT_SWISH: {
			real x = z_in[i], s = 1. / (1. + exp(-x));
			f1 = z_out[i] + s * (1. - z_out[i]);
			f2 = s * (1. - s) * (2. + x * (1. - 2. * s));
			break;
		}
		case CNN_ACT_RELU:
			f1 = (z_out[i] > 0) ? 1 : 0, f2 = 0;
			break;
		case CNN_ACT_ELU:
			f1 = (z_out[i] < 0) ? z_out[i] + 1.0 : 1, f2 = (z_out[i] < 0) ? z_out[i] + 1.0 : 0;
			break;
		case ACT_LINEAR:
		case CNN_ACT_NONE:
			f1 = 1, f2 = 0;
			break;
		default:
			return -1;
		}
		out[i] = rdelta[i] * f1 + delta[i] * f2 * rz_in[i];
	}
	return 0;
}

/* dev_pool.cu:123-174 (ker_rop_max_pool_layer): R{max pool} picks R{z} where z has its maximum
 * (first maximum in memory order, as the pooling itself). */
void oracle_max_pool_forward_routed(const real *values, const real *z_act, int samples, int channels, int height,
                                    int width, int ksize, int stride, int padding, int p_height, int p_width,
                                    real *output)
{
	size_t maps = (size_t)samples * channels;
	for (size_t m = 0; m < maps; m++) {
		const real *in = z_act + m * height * width, *val = values + m * height * width;
		real *out = output + m * p_height * p_width;
		for (int pw = 0; pw < p_width; pw++)
			for (int ph = 0; ph < p_height; ph++) {
				int idx = argmax_in_window(in, height, width, ksize, ph * stride - padding, pw * stride - padding);
				out[ph + pw * p_height] = (idx == INT_MAX) ? 0 : val[idx];
			}
	}
}

/* R-operator of the batch-norm backward formula (dev_batch_norm.cu:787-960), per channel with
 * s = sqrt(var + eps), m elements, <.> the mean over the channel:
 *   R{dc} = ( R{dx} - <R{dx}> - R{zhat} <dx zhat> - zhat ( <R{dx} zhat> + <dx R{zhat}> ) ) / s
 *           - dc <zhat R{x}> / s
 * dx = gradient at the batch-norm output, dc = at its input, x the input itself. */
void oracle_batch_norm_rop_backward(const real *rdelta_x, const real *delta_x, const real *zhat, const real *rzhat,
                                    const real *rx, const real *delta_c, const real *variance, int height, int width,
                                    int channels, int samples, real epsilon, real *output)
{
	size_t rows = (size_t)height * width * samples;
#pragma omp parallel for schedule(static)
	for (int c = 0; c < channels; c++) {
		size_t o = (size_t)c * rows;
		real a = 0, b = 0, cc = 0, d = 0, e = 0;
		for (size_t i = 0; i < rows; i++) {
			a += rdelta_x[o + i];
			b += delta_x[o + i] * zhat[o + i];
			cc += rdelta_x[o + i] * zhat[o + i];
			d += delta_x[o + i] * rzhat[o + i];
			e += zhat[o + i] * rx[o + i];
		}
		real m = (real)rows, s = sqrt(variance[c] + epsilon);
		a /= m, b /= m, cc /= m, d /= m, e /= m;
		for (size_t i = 0; i < rows; i++)
			output[o + i] = (rdelta_x[o + i] - a - rzhat[o + i] * b - zhat[o + i] * (cc + d)) / s - delta_c[o + i] * e / s;
	}
}

/* softmax_loss.cu:251-300: R{(p - y)/rows} = p_i (R{z_i} - sum_j p_j R{z_j}) / rows. */
void oracle_cross_entropy_rop_error(const real *rz, const real *probs, int rows, int numclasses, real *rError)
{
	for (int idx = 0; idx < rows; idx++) {
		real s = 0;
		for (int j = 0; j < numclasses; j++) s += probs[(size_t)idx * numclasses + j] * rz[(size_t)idx * numclasses + j];
		for (int i = 0; i < numclasses; i++)
			rError[(size_t)idx * numclasses + i] =
			    probs[(size_t)idx * numclasses + i] * (rz[(size_t)idx * numclasses + i] - s) / (real)rows;
	}
}

static void feature_dims(const CNN_MODEL *model, int *fh, int *fw)
{
	const CONV_LAYER *c = &model->convLayer[model->cLayers - 1];
	const POOL_LAYER *p = &model->poolLayer[model->cLayers - 1];
	*fh = (p->type != NO_POOL) ? p->outHeight : c->outHeight;
	*fw = (p->type != NO_POOL) ? p->outWidth : c->outWidth;
}

/* activation output of conv layer l in the convolution layout (departure D6: the last layer's
 * unpooled output was permuted in place by the forward pass and is rebuilt into tmp) */
static const real *conv_act_out(const CNN_MODEL *model, int l, const real *z, int n, real *tmp)
{
	const CONV_LAYER *c = &model->convLayer[l];
	const real *slab = z + model->zOffsets[l + 1];
	if (l == model->cLayers - 1 && model->poolLayer[l].type == NO_POOL) {
		size_t count = (size_t)n * c->activationVolumn;
		const real *actIn = (c->batchNorm != PERFORM_NO_BATCH_NORM) ? slab + c->batchNormOffset : slab;
		memcpy(tmp, actIn, sizeof(real) * count);
		oracle_activation_forward(model->actFuns[l], tmp, count);
		return tmp;
	}
	return slab + c->activationOffset;
}

/* cnn_hv_forward.cu:53-222.  rz has the layout of z. */
int oracle_cnn_rop_forward(const CNN_MODEL *model, const real *weights, const real *vector, const real *x,
                           const real *z, real *rz, int n)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	int nc = model->cLayers;
	size_t big = max_patch_reals(model, n) + (size_t)model->maxDeltaSize;
	real *scratch = (real *)malloc(sizeof(real) * big), *tmp = (real *)malloc(sizeof(real) * (size_t)model->maxDeltaSize);
	if (!scratch || !tmp) return -1;
	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const POOL_LAYER *p = &model->poolLayer[l];
		const real *slab = z + zOffsets[l + 1];
		real *rslab = rz + zOffsets[l + 1];
		size_t M = (size_t)n * c->outHeight * c->outWidth, count = M * c->outChannels;
		int K = c->kSize * c->kSize * c->inChannels;
		const real *in = (l == 0) ? x : z + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		/* R{conv} = im2col(z_in) * V + im2col(R{z_in}) * W + Vb */
		oracle_im2col(in, n, c->inChannels, c->height, c->width, c->kSize, c->padding, c->stride, scratch);
		oracle_gemm(OP_N, OP_N, (int)M, c->outChannels, K, 1, scratch, (int)M, vector + wOffsets[l], K, 0, rslab, (int)M);
		if (l > 0) {
			const real *rin = rz + zOffsets[l] + model->convLayer[l - 1].outputOffset;
			oracle_im2col(rin, n, c->inChannels, c->height, c->width, c->kSize, c->padding, c->stride, scratch);
			oracle_gemm(OP_N, OP_N, (int)M, c->outChannels, K, 1, scratch, (int)M, weights + wOffsets[l], K, 1, rslab, (int)M);
		}
		if (model->bias != 0)
			for (int o = 0; o < c->outChannels; o++)
				for (size_t i = 0; i < M; i++) rslab[(size_t)o * M + i] += vector[bOffsets[l] + o];
		const real *rpre = rslab, *actIn = slab;
		if (c->batchNorm != PERFORM_NO_BATCH_NORM) {
			/* R{zhat} = (R{x} - <R{x}> - zhat <zhat R{x}>) / s: the backward formula applied to R{x} */
			oracle_batch_norm_backward(rslab, c->outHeight, c->outWidth, c->outChannels, n,
			                           slab + c->batchNormOffset + c->variancesOffset, rslab + c->batchNormOffset,
			                           slab + c->batchNormOffset, BATCH_NORM_EPSILON);
			rpre = rslab + c->batchNormOffset;
			actIn = slab + c->batchNormOffset;
		}
		const real *actOut = conv_act_out(model, l, z, n, tmp);
		real *ract = rslab + c->activationOffset;
		memcpy(ract, rpre, sizeof(real) * count);
		if (oracle_activation_backward(model->actFuns[l], ract, actIn, actOut, count)) return -1;
		if (p->type == MAX_POOL)
			oracle_max_pool_forward_routed(ract, actOut, n, c->outChannels, c->outHeight, c->outWidth, p->pSize, p->stride,
			                               p->padding, p->outHeight, p->outWidth, rslab + c->poolOffset);
		else if (p->type == AVG_POOL)
			oracle_avg_pool_forward(ract, n, c->outChannels, c->outHeight, c->outWidth, p->pSize, p->stride, p->padding,
			                        p->outHeight, p->outWidth, rslab + c->poolOffset);
		else if (p->type != NO_POOL)
			return -1;
	}
	/* feature permute of R{z}, as the forward pass did for z (cnn_hv_forward.cu:178-195) */
	const CONV_LAYER *c = &model->convLayer[nc - 1];
	int fh, fw;
	feature_dims(model, &fh, &fw);
	real *rfeat = rz + zOffsets[nc] + c->outputOffset;
	oracle_reshape(rfeat, c->outChannels, n, fh * fw, scratch);
	oracle_transpose(scratch, c->outChannels * n, fh, fw, rfeat);

	for (int f = 0; f < model->lLayers; f++) {
		const FC_LAYER *fc = &model->fcLayer[f];
		int at = nc + f;
		int off = (f == 0) ? c->outputOffset : 0;
		const real *zin = z + zOffsets[at] + off, *rzin = rz + zOffsets[at] + off;
		const real *zl = z + zOffsets[at + 1];
		real *rzl = rz + zOffsets[at + 1];
		size_t count = (size_t)fc->out * n;
		real *rpre = rzl + fc->offset;
		/* R{W z + b} = V z + W R{z} + Vb (rop_fc_layer.cu:34-133) */
		oracle_gemm(OP_N, OP_N, fc->out, n, fc->in, 1, vector + wOffsets[at], fc->out, zin, fc->in, 0, rpre, fc->out);
		oracle_gemm(OP_N, OP_N, fc->out, n, fc->in, 1, weights + wOffsets[at], fc->out, rzin, fc->in, 1, rpre, fc->out);
		if (model->bias != 0)
			for (int i = 0; i < n; i++)
				for (int r = 0; r < fc->out; r++) rpre[(size_t)i * fc->out + r] += vector[bOffsets[at] + r];
		memcpy(rzl, rpre, sizeof(real) * count);
		if (oracle_activation_backward(fc->actFun, rzl, zl + fc->offset, zl, count)) return -1;
	}
	free(scratch);
	free(tmp);
	return 0;
}

/* cnn_hv_backward.cu:70-912.  rError = R{loss errors}; hv receives R{gradient}. */
int oracle_cnn_rop_backward(const CNN_MODEL *model, const real *weights, const real *vector, const real *x,
                            const real *z, const real *rz, const real *dx, const real *lossFuncErrors,
                            const real *rError, real *hv, int n, int numClasses)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	int nc = model->cLayers;
	size_t dsz = (size_t)model->maxDeltaSize;
	real *scratch = (real *)malloc(sizeof(real) * (max_patch_reals(model, n) + dsz));
	real *rdelta = (real *)calloc(dsz, sizeof(real)), *rnext = (real *)calloc(dsz, sizeof(real));
	real *dout = (real *)calloc(dsz, sizeof(real)), *tmp = (real *)calloc(dsz, sizeof(real));
	real *wtmp = (real *)calloc((size_t)model->pSize, sizeof(real));
	if (!scratch || !rdelta || !rnext || !dout || !tmp || !wtmp) return -1;
	const CONV_LAYER *last = &model->convLayer[nc - 1];
	memcpy(rdelta, rError, sizeof(real) * (size_t)numClasses * n);
	memcpy(dout, lossFuncErrors, sizeof(real) * (size_t)numClasses * n);

	for (int f = model->lLayers - 1; f >= 0; f--) {
		const FC_LAYER *fc = &model->fcLayer[f];
		int at = nc + f;
		int off = (f == 0) ? last->outputOffset : 0;
		const real *zl = z + zOffsets[at + 1], *rzl = rz + zOffsets[at + 1];
		const real *zin = z + zOffsets[at] + off, *rzin = rz + zOffsets[at] + off;
		const real *dpre = dx + zOffsets[at + 1];
		size_t count = (size_t)fc->out * n;
		/* R{delta f'(x)} */
		if (oracle_activation_rop_backward(fc->actFun, rdelta, dout, zl + fc->offset, zl, rzl + fc->offset, tmp, count))
			return -1;
		/* R{dW} = R{d} z' + d R{z}' ; R{db} = R{d} 1 */
		oracle_gemm(OP_N, OP_T, fc->out, fc->in, n, 1, tmp, fc->out, zin, fc->in, 0, hv + wOffsets[at], fc->out);
		oracle_gemm(OP_N, OP_T, fc->out, fc->in, n, 1, dpre, fc->out, rzin, fc->in, 1, hv + wOffsets[at], fc->out);
		if (model->bias != 0)
			for (int r = 0; r < fc->out; r++) {
				real s = 0;
				for (int i = 0; i < n; i++) s += tmp[(size_t)i * fc->out + r];
				hv[bOffsets[at] + r] = s;
			}
		/* R{W' d} = V' d + W' R{d};  and the gradient at the output of the layer below, W' d */
		oracle_gemm(OP_T, OP_N, fc->in, n, fc->out, 1, vector + wOffsets[at], fc->out, dpre, fc->out, 0, rnext, fc->in);
		oracle_gemm(OP_T, OP_N, fc->in, n, fc->out, 1, weights + wOffsets[at], fc->out, tmp, fc->out, 1, rnext, fc->in);
		oracle_gemm(OP_T, OP_N, fc->in, n, fc->out, 1, weights + wOffsets[at], fc->out, dpre, fc->out, 0, dout, fc->in);
		real *t = rdelta;
		rdelta = rnext;
		rnext = t;
	}
	{
		int fh, fw;
		feature_dims(model, &fh, &fw);
		oracle_reshape(rdelta, n, last->outChannels, fh * fw, scratch);
		oracle_transpose_rc(scratch, last->outChannels * n, fh, fw, rdelta);
	}
	for (int c = nc - 1; c >= 0; c--) {
		const CONV_LAYER *l = &model->convLayer[c];
		const POOL_LAYER *p = &model->poolLayer[c];
		const real *slab = z + zOffsets[c + 1], *rslab = rz + zOffsets[c + 1], *dslab = dx + zOffsets[c + 1];
		size_t count = (size_t)n * l->activationVolumn;
		int bn = l->batchNorm != PERFORM_NO_BATCH_NORM;
		const real *actIn = bn ? slab + l->batchNormOffset : slab;
		const real *ractIn = bn ? rslab + l->batchNormOffset : rslab;
		const real *actOut = conv_act_out(model, c, z, n, tmp);
		/* R through the pooling: the same routing as the gradient (dev_pool.cu:346-398) */
		if (p->type == MAX_POOL)
			oracle_max_pool_backward(rdelta, actOut, l->outChannels, p->height, p->width, p->pSize, p->stride, p->padding,
			                         p->outHeight, p->outWidth, n, rnext);
		else if (p->type == AVG_POOL)
			oracle_avg_pool_backward(rdelta, l->outChannels, p->height, p->width, p->pSize, p->stride, p->padding,
			                         p->outHeight, p->outWidth, n, rnext);
		else if (p->type == NO_POOL)
			memcpy(rnext, rdelta, sizeof(real) * count);
		else
			return -1;
		/* R{delta f'(x)}: delta at the activation output is the dx snapshot at +0 */
		if (oracle_activation_rop_backward(model->actFuns[c], rnext, dslab, actIn, actOut, ractIn, rdelta, count)) return -1;
		const real *dc = dslab + l->activationOffset; /* gradient at the convolution output */
		real *rdc = rdelta;
		if (bn) {
			oracle_batch_norm_rop_backward(rdelta, dslab + l->activationOffset, slab + l->batchNormOffset,
			                               rslab + l->batchNormOffset, rslab, dslab + l->batchNormOffset,
			                               slab + l->batchNormOffset + l->variancesOffset, l->outHeight, l->outWidth,
			                               l->outChannels, n, BATCH_NORM_EPSILON, rnext);
			dc = dslab + l->batchNormOffset;
			rdc = rnext;
		}
		size_t M = (size_t)p->height * p->width * n;
		if (model->bias != 0)
			for (int o = 0; o < l->outChannels; o++) {
				real s = 0;
				for (size_t i = 0; i < M; i++) s += rdc[(size_t)o * M + i];
				hv[bOffsets[c] + o] = s;
			}
		const real *in = (c == 0) ? x : z + zOffsets[c] + model->convLayer[c - 1].outputOffset;
		size_t wcount = (size_t)l->outChannels * l->inChannels * l->kSize * l->kSize;
		/* R{dW} = im2col(z_in)' R{dc} + im2col(R{z_in})' dc */
		oracle_conv_weight_gradient(in, rdc, n, l->inChannels, l->height, l->width, l->kSize, l->padding, l->stride,
		                            l->outChannels, hv + wOffsets[c], scratch);
		if (c != 0) {
			const real *rin = rz + zOffsets[c] + model->convLayer[c - 1].outputOffset;
			oracle_conv_weight_gradient(rin, dc, n, l->inChannels, l->height, l->width, l->kSize, l->padding, l->stride,
			                            l->outChannels, wtmp, scratch);
			for (size_t i = 0; i < wcount; i++) hv[wOffsets[c] + i] += wtmp[i];
			/* R{dX} = dX(R{dc}, W) + dX(dc, V) */
			real *other = (rdc == rdelta) ? rnext : rdelta;
			size_t inCount = (size_t)n * l->height * l->width * l->inChannels;
			oracle_conv_input_gradient(rdc, p->height, p->width, l->outChannels, weights + wOffsets[c], l->kSize, l->kSize,
			                           l->height, l->width, l->padding, l->inChannels, n, other, scratch);
			oracle_conv_input_gradient(dc, p->height, p->width, l->outChannels, vector + wOffsets[c], l->kSize, l->kSize,
			                           l->height, l->width, l->padding, l->inChannels, n, tmp, scratch);
			for (size_t i = 0; i < inCount; i++) other[i] += tmp[i];
			if (other != rdelta) {
				real *t = rdelta;
				rdelta = rnext;
				rnext = t;
			}
		}
	}
	free(scratch), free(rdelta), free(rnext), free(dout), free(tmp), free(wtmp);
	return 0;
}

/* cnn_hessian_vec.cu:18-122 (cnnHv): R forward, R of the loss errors, R backward.  z, probs,
 * lossFuncErrors and dx come from oracle_cnn_gradient on the same batch.  No weight-decay term
 * (the reference leaves that to computeQuadraticModel). */
int oracle_cnn_hv(const CNN_MODEL *model, const real *weights, const real *x, const real *z, const real *probs,
                  const real *lossFuncErrors, const real *dx, const real *vector, real *hv, int n, int numClasses)
{
	int nc = model->cLayers;
	real *rz = (real *)calloc((size_t)model->zSize, sizeof(real));
	real *rError = (real *)calloc((size_t)numClasses * n, sizeof(real));
	if (!rz || !rError) return -1;
	int rc = oracle_cnn_rop_forward(model, weights, vector, x, z, rz, n);
	if (rc == 0) {
		const real *rlogits = (model->lLayers == 0)
		                          ? rz + model->zOffsets[nc] + model->convLayer[nc - 1].outputOffset
		                          : rz + model->zOffsets[nc + model->lLayers];
		oracle_cross_entropy_rop_error(rlogits, probs, n, numClasses, rError);
		rc = oracle_cnn_rop_backward(model, weights, vector, x, z, rz, dx, lossFuncErrors, rError, hv, n, numClasses);
	}
	free(rz);
	free(rError);
	return rc;
}

/* ------------------------------------------------------------------ */
/* Input pipeline: batch selection and augmentation                    */
/* ------------------------------------------------------------------ */

/* device/extract_columns.cu:8-20 (kerExtractColumns): column j of tgt is column indices[j] of src,
 * columns of `rows` values. */
void oracle_extract_columns(real *tgt, const real *src, const int *indices, int rows, long numElements)
{
	for (long j = 0; j < numElements; j++) {
		long colId = j / rows, rowId = j % rows;
		tgt[j] = src[(size_t)indices[colId] * rows + rowId];
	}
}

/* augmentation/dev_crop.cu:52-58 (ker_convert): uniform in [0, 1) -> shift in [-padding, padding].
 * The first `samples` values are the row shifts, the next `samples` the column shifts. */
void oracle_crop_shifts(const real *uniforms, int samples, int padding, int *shifts)
{
	for (int i = 0; i < 2 * samples; i++) shifts[i] = (int)((double)uniforms[i] * 100.) % (2 * padding + 1) - padding;
}

/* augmentation/dev_crop.cu:10-50 (ker_random_crop) on [channels][samples][width][height] (height fastest):
 * every image is shifted by (shiftRow, shiftCol); cells that leave the image read defaultVal. */
void oracle_random_crop(const real *input, int samples, int height, int width, int channels, const int *shiftRow,
                        const int *shiftCol, real defaultVal, real *output)
{
	for (int imgIdx = 0; imgIdx < samples; imgIdx++)
		for (int idx = 0; idx < height * width * channels; idx++) {
			int chId = idx / (height * width), chIdx = idx % (height * width);
			int row = chIdx % height, col = chIdx / height;
			int cRow = shiftRow[imgIdx], cCol = shiftCol[imgIdx];
			real val;
			if (cRow + row < 0 || cCol + col < 0 || cRow + row >= height || cCol + col >= width) val = defaultVal;
			else val = input[(size_t)chId * samples * height * width + (size_t)imgIdx * height * width +
				             (size_t)(col + cCol) * height + (row + cRow)];
			output[(size_t)chId * samples * height * width + (size_t)imgIdx * height * width + (size_t)col * height + row] = val;
		}
}

/* augmentation/dev_flip.cu:68-104 (ker_random_flip): images with probs < 0.5 are mirrored along the
 * width (column) axis, the others copied.  (The reference splits the cell index by `width` where the
 * layout needs `height`; the two agree on the square images it is used on, and the layout's own split
 * is restated here.) */
void oracle_random_flip(const real *input, int samples, int channels, int height, int width, const real *probs, real *output)
{
	for (int imgIdx = 0; imgIdx < samples; imgIdx++)
		for (int idx = 0; idx < height * width * channels; idx++) {
			int chId = idx / (height * width), chIdx = idx % (height * width);
			int row = chIdx % height, col = chIdx / height;
			size_t base = (size_t)chId * samples * height * width + (size_t)imgIdx * height * width;
			size_t src = base + (size_t)col * height + row, tgt = src;
			if (probs[imgIdx] < 0.5) tgt = base + (size_t)(width - 1 - col) * height + row;
			output[tgt] = input[src];
		}
}

/* augmentation/dev_normalize.cu:12-36 (ker_normalize): x = (x / nrConstant - mean[c]) / std[c], in place. */
void oracle_normalize(real *input, int samples, int height, int width, int channels, const real *means, const real *std,
                      real nrConstant)
{
	for (int c = 0; c < channels; c++)
		for (size_t i = 0; i < (size_t)samples * height * width; i++) {
			real *x = input + (size_t)c * samples * height * width + i;
			*x /= nrConstant;
			*x = (*x - means[c]) / std[c];
		}
}

/* solvers/kfac_da.cu:22-89 (augmentData) given the uniforms it would draw: [samples][channels][cells] ->
 * [channels][samples][cells] (reshapeMatrix), then with enableDA crop by at most 4 cells (fill 0) and
 * flip, then the data set's normalisation with the pixel scale 255.  cropUniforms: 2*samples values,
 * flipUniforms: samples values.  scratch holds one batch. */
void oracle_augment_data(const real *sampled, int samples, int channels, int height, int width, int enableDA,
                         const real *cropUniforms, const real *flipUniforms, const real *means, const real *std,
                         real *scratch, real *output)
{
	oracle_reshape(sampled, samples, channels, height * width, output);
	if (enableDA >= 1) {
		int *shifts = (int *)malloc(sizeof(int) * 2 * (size_t)samples);
		oracle_crop_shifts(cropUniforms, samples, 4, shifts);
		oracle_random_crop(output, samples, height, width, channels, shifts, shifts + samples, 0, scratch);
		oracle_random_flip(scratch, samples, channels, height, width, flipUniforms, output);
		free(shifts);
	}
	oracle_normalize(output, samples, height, width, channels, means, std, 255.);
}

int oracle_sizeof_real(void) { return (int)sizeof(real); }
