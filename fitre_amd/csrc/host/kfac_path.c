/*
 * Kronecker-factor stage of the KFAC curvature approximation as C host code over the
 * C-ABI device layer: layer walk and data sources of solvers/kfac_inverses.cu:450-630
 * (computeOmegaZ) and :759-857 (computeLambdaDelta), storage offsets of
 * solvers/kfac_utils.cu:6-54.  No scaled copies: each factor is one
 * symmetric product on the device.
 */
#include <stdio.h>
#include <stdlib.h>
#include "fitre_kfac.h"
#include "fitre_hip.h"

#define HIP_CALL(expr)                                                                               \
	do {                                                                                             \
		int rc_ = (expr);                                                                            \
		if (rc_ != FITRE_OK) {                                                                       \
			fprintf(stderr, "%s:%d: %s -> error %d: %s\n", __FILE__, __LINE__, #expr, rc_,           \
			        fitre_hip_last_error());                                                         \
			exit(-1);                                                                                \
		}                                                                                            \
	} while (0)

static fitre_conv_shape conv_shape(const CONV_LAYER *l, int samples)
{
	fitre_conv_shape s;
	s.samples = samples;
	s.inChannels = l->inChannels;
	s.outChannels = l->outChannels;
	s.inA = l->width;
	s.inB = l->height;
	s.outA = l->outWidth;
	s.outB = l->outHeight;
	s.ksize = l->kSize;
	s.stride = l->stride;
	s.padding = l->padding;
	return s;
}

static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }

void computeKFACStorageIndices(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo)
{
	int *omega = kfacInfo->OmegaZOffsets, *lambda = kfacInfo->LambdaGOffsets;
	for (int i = 0; i < MAX_LAYERS; i++) omega[i] = lambda[i] = 0;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		int order = c->inChannels * c->kSize * c->kSize + 1;
		omega[i + 1] = omega[i] + order * order;
		lambda[i + 1] = lambda[i] + c->outChannels * c->outChannels;
	}
	for (int i = 0; i < model->lLayers; i++) {
		const FC_LAYER *f = &model->fcLayer[i];
		int at = model->cLayers + i;
		omega[at + 1] = omega[at] + (f->in + 1) * (f->in + 1);
		lambda[at + 1] = lambda[at] + f->out * f->out;
	}
}

static size_t factor_ws_bytes(const CNN_MODEL *model, int samples)
{
	size_t bytes = 0;
	int withBias = model->bias != 0;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		fitre_conv_shape s = conv_shape(c, samples);
		bytes = max_sz(bytes, fitre_hip_kfac_conv_input_factor_workspace(&s, withBias));
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(c->outChannels, (long)samples * c->outHeight * c->outWidth));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(f->in, samples));
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(f->out, samples));
	}
	return bytes;
}

long kfacFactorsMemRequired(CNN_MODEL *model, int samples)
{
	return (long)((factor_ws_bytes(model, samples) + sizeof(real) - 1) / sizeof(real)) + 64;
}

void computeOmegaZFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                          real *dampedInput, real *dampedZ, real *omegaZZT, int *zOffsets, int *zztOffsets, real *devPtr)
{
	const int *omega = kfac_info->OmegaZOffsets;
	const int withBias = model->bias != 0;
	const size_t wsBytes = factor_ws_bytes(model, samples);
	const int nc = model->cLayers;

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const real *input;
		if (dampedInput != NULL)
			input = (l == 0) ? dampedInput : dampedZ + zztOffsets[l];
		else
			input = (l == 0) ? data->currentBatch : dampedZ + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		fitre_conv_shape s = conv_shape(c, samples);
		HIP_CALL(fitre_hip_kfac_conv_input_factor(&s, input, withBias, omegaZZT + omega[l], devPtr, wsBytes));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		const real *input;
		if (dampedInput != NULL)
			input = dampedZ + zztOffsets[nc + l];
		else if (l == 0)
			input = dampedZ + zOffsets[nc] + model->convLayer[nc - 1].outputOffset;
		else
			input = dampedZ + zOffsets[nc + l];
		HIP_CALL(fitre_hip_kfac_fc_input_factor(input, f->in, samples, withBias, omegaZZT + omega[nc + l], devPtr, wsBytes));
	}
	HIP_CALL(fitre_hip_sync());
}

void computeLambdaDeltaFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx,
                               real *dampedLambda, real *lambdaGGT, int *zOffsets, int *zztOffsets, real *devPtr)
{
	const int *lambda = kfac_info->LambdaGOffsets;
	const size_t wsBytes = factor_ws_bytes(model, samples);
	const int nc = model->cLayers;

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const real *delta;
		if (dampedLambda != NULL)
			delta = dampedLambda + zztOffsets[l + 1];
		else if (c->batchNorm == PERFORM_NO_BATCH_NORM)
			delta = dx + zOffsets[l + 1] + c->activationOffset;
		else
			delta = dx + zOffsets[l + 1] + c->batchNormOffset;
		fitre_conv_shape s = conv_shape(c, samples);
		HIP_CALL(fitre_hip_kfac_conv_output_factor(&s, delta, lambdaGGT + lambda[l], devPtr, wsBytes));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		const real *delta = (dampedLambda != NULL) ? dampedLambda + zztOffsets[nc + l + 1] : dx + zOffsets[nc + l + 1];
		HIP_CALL(fitre_hip_kfac_fc_output_factor(delta, f->out, samples, lambdaGGT + lambda[nc + l], devPtr, wsBytes));
	}
	HIP_CALL(fitre_hip_sync());
}

/* ---- inverses ------------------------------------------------------------------------------ */

static size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static char *aligned_base(real *devPtr) { return (char *)(((size_t)devPtr + 255) & ~(size_t)255); }

/* The reference inverts in double (cusolverDnDpotrf / Dpotrs with real = double, solvers/kfac_inverses.cu:133-186);
 * so does this: the float matrix is widened, inverted in float64 and the inverse rounded to floats. */
void computeMatrixInverse(real *matrix, real *inverse, int n, real *devPtr, real lambda, real dampGamma)
{
	char *base = aligned_base(devPtr);
	const size_t matBytes = round_up((size_t)n * n * sizeof(double), 256);
	int *pivot = (int *)(base + matBytes);
	int host = 0;
	HIP_CALL(fitre_hip_widen_shift(matrix, n, (double)lambda + (double)dampGamma, (double *)base));
	HIP_CALL(fitre_hip_spd_inverse_f64_queued((double *)base, n, inverse, FITRE_MAT_F32, base + matBytes + 256,
	                                          fitre_hip_spd_inverse_f64_workspace(n), pivot));
	HIP_CALL(fitre_hip_sync());
	HIP_CALL(fitre_hip_copy_d2h(&host, pivot, sizeof(int)));
	if (host != 0) {
		fprintf(stderr, "We have a problem with the LU factorization ... %d\n", host);
		exit(-1);
	}
}

long matrixInverseMemRequired(int n)
{
	return (long)((round_up((size_t)n * n * sizeof(double), 256) + 512 + fitre_hip_spd_inverse_f64_workspace(n)) / sizeof(real)) + 64;
}

/* workspace of the float64 factor products of a pass */
static size_t factor64_ws_bytes(const CNN_MODEL *model, int samples)
{
	size_t bytes = 0;
	int withBias = model->bias != 0;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		fitre_conv_shape s = conv_shape(c, samples);
		bytes = max_sz(bytes, fitre_hip_kfac_conv_input_factor_f64_workspace(&s, withBias));
		bytes = max_sz(bytes, fitre_hip_gemm_f64_workspace(c->outChannels, c->outChannels, (long)samples * c->outHeight * c->outWidth,
		                                                   FITRE_GEMM_SYMMETRIC));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		bytes = max_sz(bytes, fitre_hip_gemm_f64_workspace(f->in + 1, f->in + 1, samples, FITRE_GEMM_SYMMETRIC));
		bytes = max_sz(bytes, fitre_hip_gemm_f64_workspace(f->out, f->out, samples, FITRE_GEMM_SYMMETRIC));
	}
	return bytes;
}

/* layout of one slot of the scratch of the two inverse passes: [factor (doubles) | workspace of its product or inverse] */
static size_t inverse_scratch_bytes(const CNN_MODEL *model, int samples, size_t *factorBytes)
{
	size_t order = 1, ws = factor64_ws_bytes(model, samples);
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		size_t k = (size_t)c->inChannels * c->kSize * c->kSize + 1;
		order = max_sz(order, max_sz(k, (size_t)c->outChannels));
	}
	for (int l = 0; l < model->lLayers; l++)
		order = max_sz(order, max_sz((size_t)model->fcLayer[l].in + 1, (size_t)model->fcLayer[l].out));
	ws = max_sz(ws, fitre_hip_spd_inverse_f64_workspace((int)order));
	*factorBytes = round_up(order * order * sizeof(double), 256);
	return *factorBytes + round_up(ws, 256) + 256;
}

/* The inverses of a pass are independent of each other: they are dealt, costliest first, to the four lanes, each
 * of which owns one [factor | workspace] slot; the pivot reports are read once at the end. */
#define KFAC_LANES 4
#define KFAC_INFO_BYTES 1024 /* one int per matrix, 2 * MAX_LAYERS of them */

long kfacInverseMemRequired(CNN_MODEL *model, int samples)
{
	size_t factorBytes;
	return (long)((KFAC_LANES * inverse_scratch_bytes(model, samples, &factorBytes) + KFAC_INFO_BYTES) / sizeof(real)) + 64;
}

/* writes the float64 factor of `layer` (convolution layers, then linear ones), damping included, into `factor` */
typedef void (*FACTOR_FN)(void *ctx, int layer, double shift, double *factor, void *ws, size_t wsBytes);
/* writes the operand R of an input-side factor (factor = alpha R R^T, R order x positions) to `rows` and reports its
 * strides and alpha */
typedef void (*ROWS_FN)(void *ctx, int layer, real *rows, long *rowStride, long *colStride, double *alpha);

/* An input-side factor with fewer positions behind it than half its order (the last layers of a deep network:
 * order 9 Cin + 1 from samples * outH * outW patches) is kept in LOW-RANK FORM instead of as a dense inverse:
 *   (alpha R R^T + s I)^-1 = (I - alpha R S^-1 R^T) / s,   S = s I + alpha R^T R   (positions x positions),
 * i.e. the slot holds R itself and the inverse of the small matrix S -- an inverse of order positions instead of
 * order, and three thin products per application instead of one square one.  The slot then starts with a header
 * whose first word no dense inverse can start with (a negative float on the diagonal of a positive definite
 * matrix), so that computeNaturalGradient can tell the forms apart:
 *   word 0 tag, 1 positions, 2 order, 3 / 4 row and column stride of R, 5-6 alpha, 7-8 s (doubles), 9 the word at which
 *   S^-1 starts;
 *   R at word KFAC_LOWRANK_HEADER, S^-1 behind it as doubles (at the next 8-byte boundary): applying this form subtracts two
 *   nearly equal terms, and the 32 bits a float pair has on its diagonal would cost the result three digits. */
#define KFAC_LOWRANK_TAG 0xF15EED12u
#define KFAC_LOWRANK_HEADER 64
static int lowrank_eligible(int order, long positions)
{
	return positions >= 1 && 2 * positions <= order && order >= 64 &&
	       (size_t)KFAC_LOWRANK_HEADER + (size_t)order * positions + 2 * (size_t)positions * positions + 2 <= (size_t)order * order;
}

/* where S^-1 (doubles) starts in a low-rank slot */
static double *lowrank_sinv(const real *slot, int order, long positions)
{
	return (double *)(((size_t)(slot + KFAC_LOWRANK_HEADER + (size_t)order * positions) + 7) & ~(size_t)7);
}

/* one matrix of a pass: how to make its factor, its order, where its inverse goes */
typedef struct inverse_item {
	FACTOR_FN make;
	ROWS_FN rows; /* non-NULL: the factor may be kept in low-rank form */
	long positions;
	void *ctx;
	int layer;
	int order;
	int group;
	real *inverse;
} INVERSE_ITEM;

typedef struct inverse_job {
	int item;
	double cost;
} INVERSE_JOB;

static int job_by_cost(const void *a, const void *b)
{
	const INVERSE_JOB *x = (const INVERSE_JOB *)a, *y = (const INVERSE_JOB *)b;
	if (x->cost != y->cost) return x->cost < y->cost ? 1 : -1;
	return x->item - y->item;
}

#define KFAC_MAX_ITEMS (2 * MAX_LAYERS)

/* Every item: the factor in float64 with the damping on its diagonal, its float64 inverse, and the inverse stored in
 * the caller's n x n floats as a float pair per element (FITRE_MAT_SYM_PAIR): computeNaturalGradient, the only reader
 * of these arrays (solvers/kfac_natural_gradient.cu:55-56), takes them in that form. */
static void inverse_pass_run(const CNN_MODEL *model, int samples, real *devPtr, const INVERSE_ITEM *items, int count, double shift)
{
	size_t factorBytes;
	const size_t slotBytes = inverse_scratch_bytes(model, samples, &factorBytes);
	const size_t wsBytes = slotBytes - factorBytes - 256;
	char *base = aligned_base(devPtr);
	int *pivots = (int *)base;
	char *slots = base + KFAC_INFO_BYTES;

	INVERSE_JOB jobs[KFAC_MAX_ITEMS];
	for (int i = 0; i < count; i++) {
		jobs[i].item = i;
		/* Milliseconds alone on the chip, fitted to measurements: the inverse is a chain of launches whose length grows
		 * with the order (0.42 / 1.12 / 2.46 / 6.86 ms at order 512 / 1153 / 2305 / 4609) plus the arithmetic; the factor is
		 * a symmetric product over the positions (1.9 ms for order 4609 over 4096 positions).  With the chain's share
		 * underrated (as an earlier form had it) every small matrix of a pass landed on one lane, which then finished last. */
		const int lowrank = items[i].rows != NULL && lowrank_eligible(items[i].order, items[i].positions);
		const double n = lowrank ? (double)items[i].positions : (double)items[i].order;
		const double order = (double)items[i].order, positions = (double)(items[i].positions > 0 ? items[i].positions : 0);
		jobs[i].cost = 0.82e-3 * n + 3.15e-11 * n * n * n +
		               (lowrank ? 1.0e-10 * n * n * order : 2.2e-11 * order * order * positions);
	}
	qsort(jobs, (size_t)count, sizeof(INVERSE_JOB), job_by_cost);
	double load[KFAC_LANES] = { 0, 0, 0, 0 };
	for (int k = 1; k < KFAC_LANES; k++) HIP_CALL(fitre_hip_lane_wait(k, 0)); /* after what lane 0 has queued so far (z, dx) */
	for (int i = 0; i < count; i++) {
		const INVERSE_ITEM *it = &items[jobs[i].item];
		int lane = 0;
		for (int k = 1; k < KFAC_LANES; k++)
			if (load[k] < load[lane]) lane = k;
		load[lane] += jobs[i].cost;
		char *slot = slots + (size_t)lane * slotBytes;
		HIP_CALL(fitre_hip_lane_select(lane));
		if (it->rows != NULL && lowrank_eligible(it->order, it->positions)) {
			const long m = it->positions;
			real *rows = it->inverse + KFAC_LOWRANK_HEADER;
			long rs, cs;
			double alpha;
			it->rows(it->ctx, it->layer, rows, &rs, &cs, &alpha);
			/* S = shift I + alpha R^T R, in the slot's factor area */
			fitre_matrix rt = { rows, cs, rs, FITRE_MAT_F32, -1, -1, 0.0 }, r = { rows, rs, cs, FITRE_MAT_F32, -1, -1, 0.0 };
			fitre_matrix sm = { slot, 1, m, FITRE_MAT_F64, -1, -1, 0.0 };
			HIP_CALL(fitre_hip_gemm_f64(m, m, it->order, alpha, &rt, &r, 0.0, &sm, shift, FITRE_GEMM_SYMMETRIC, slot + factorBytes, wsBytes));
			HIP_CALL(fitre_hip_spd_inverse_f64_queued((double *)slot, (int)m, lowrank_sinv(it->inverse, it->order, m), FITRE_MAT_F64,
			                                          slot + factorBytes, wsBytes, pivots + jobs[i].item));
			union { double d; unsigned int w[2]; } a = { alpha }, sh = { shift };
			unsigned int header[10] = { KFAC_LOWRANK_TAG, (unsigned int)m, (unsigned int)it->order, (unsigned int)rs, (unsigned int)cs,
				                        a.w[0], a.w[1], sh.w[0], sh.w[1],
				                        (unsigned int)((const real *)lowrank_sinv(it->inverse, it->order, m) - it->inverse) };
			HIP_CALL(fitre_hip_write_header(it->inverse, header, 10));
			continue;
		}
		it->make(it->ctx, it->layer, shift, (double *)slot, slot + factorBytes, wsBytes);
		HIP_CALL(fitre_hip_spd_inverse_f64_queued((double *)slot, it->order, it->inverse, FITRE_MAT_SYM_PAIR, slot + factorBytes, wsBytes,
		                                          pivots + jobs[i].item));
	}
	int host[KFAC_MAX_ITEMS];
	HIP_CALL(fitre_hip_lane_select(0));
	HIP_CALL(fitre_hip_sync());
	HIP_CALL(fitre_hip_copy_d2h(host, pivots, sizeof(int) * (size_t)count));
	for (int i = 0; i < count; i++)
		if (host[i] != 0) {
			fprintf(stderr, "We have a problem with the LU factorization ... %d (%s factor of layer %d)\n", host[i],
			        items[i].group < 2 ? "input" : "output", items[i].layer);
			exit(-1);
		}
}

typedef struct omega_ctx {
	const CNN_MODEL *model;
	const DEVICE_DATASET *data;
	int samples, withBias;
	const real *dampedInput, *dampedZ;
	const int *zOffsets, *zztOffsets;
} OMEGA_CTX;

static void omega_factor(void *ctx, int layer, double shift, double *factor, void *ws, size_t wsBytes)
{
	const OMEGA_CTX *o = (const OMEGA_CTX *)ctx;
	const CNN_MODEL *model = o->model;
	const int nc = model->cLayers;
	if (layer < nc) {
		const int l = layer;
		const CONV_LAYER *c = &model->convLayer[l];
		const real *input;
		if (o->dampedInput != NULL)
			input = (l == 0) ? o->dampedInput : o->dampedZ + o->zztOffsets[l];
		else
			input = (l == 0) ? o->data->currentBatch : o->dampedZ + o->zOffsets[l] + model->convLayer[l - 1].outputOffset;
		fitre_conv_shape s = conv_shape(c, o->samples);
		HIP_CALL(fitre_hip_kfac_conv_input_factor_f64(&s, input, o->withBias, shift, factor, ws, wsBytes));
	} else {
		const int l = layer - nc;
		const FC_LAYER *f = &model->fcLayer[l];
		const real *input;
		if (o->dampedInput != NULL)
			input = o->dampedZ + o->zztOffsets[nc + l];
		else if (l == 0)
			input = o->dampedZ + o->zOffsets[nc] + model->convLayer[nc - 1].outputOffset;
		else
			input = o->dampedZ + o->zOffsets[nc + l];
		HIP_CALL(fitre_hip_kfac_fc_input_factor_f64(input, f->in, o->samples, o->withBias, shift, factor, ws, wsBytes));
	}
}

static void omega_rows(void *ctx, int layer, real *rows, long *rowStride, long *colStride, double *alpha)
{
	const OMEGA_CTX *o = (const OMEGA_CTX *)ctx;
	const CNN_MODEL *model = o->model;
	const int nc = model->cLayers;
	if (layer < nc) {
		const int l = layer;
		const CONV_LAYER *c = &model->convLayer[l];
		const real *input;
		if (o->dampedInput != NULL)
			input = (l == 0) ? o->dampedInput : o->dampedZ + o->zztOffsets[l];
		else
			input = (l == 0) ? o->data->currentBatch : o->dampedZ + o->zOffsets[l] + model->convLayer[l - 1].outputOffset;
		fitre_conv_shape s = conv_shape(c, o->samples);
		HIP_CALL(fitre_hip_kfac_conv_input_rows(&s, input, o->withBias, rows));
		const double cells = (double)c->outHeight * c->outWidth;
		*rowStride = (long)o->samples * c->outHeight * c->outWidth, *colStride = 1;
		*alpha = 1.0 / (cells * cells * (double)o->samples);
	} else {
		const int l = layer - nc;
		const FC_LAYER *f = &model->fcLayer[l];
		const real *input;
		if (o->dampedInput != NULL)
			input = o->dampedZ + o->zztOffsets[nc + l];
		else if (l == 0)
			input = o->dampedZ + o->zOffsets[nc] + model->convLayer[nc - 1].outputOffset;
		else
			input = o->dampedZ + o->zOffsets[nc + l];
		HIP_CALL(fitre_hip_kfac_fc_input_rows(input, f->in, o->samples, o->withBias, rows));
		*rowStride = 1, *colStride = f->in + (o->withBias ? 1 : 0);
		*alpha = 1.0 / (double)o->samples;
	}
}

/* items of the input-side factors; returns their number */
static int omega_items(INVERSE_ITEM *items, const KFAC_CURVATURE_INFO *kfac_info, const CNN_MODEL *model, OMEGA_CTX *ctx,
                       real *omegaZInv)
{
	const int nc = model->cLayers, layers = nc + model->lLayers;
	const int *omega = kfac_info->OmegaZOffsets;
	for (int l = 0; l < layers; l++) {
		INVERSE_ITEM *it = &items[l];
		it->make = omega_factor;
		it->rows = omega_rows;
		it->ctx = ctx;
		it->layer = l;
		if (l < nc) {
			const CONV_LAYER *c = &model->convLayer[l];
			it->order = c->inChannels * c->kSize * c->kSize + (ctx->withBias ? 1 : 0);
			it->positions = (long)ctx->samples * c->outHeight * c->outWidth;
			it->group = 0;
		} else {
			it->order = model->fcLayer[l - nc].in + (ctx->withBias ? 1 : 0);
			it->positions = ctx->samples;
			it->group = 1;
		}
		it->inverse = omegaZInv + omega[l];
	}
	return layers;
}

void computeOmegaZ(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                   real *dampedInput, real *dampedZ, real *omegaZInv, int *zOffsets, int *zztOffsets, real *devPtr,
                   real *pageLckPtr, cublasHandle_t blasHandle, cudaStream_t curStream, cusolverDnHandle_t curHandle)
{
	(void)pageLckPtr, (void)blasHandle, (void)curStream, (void)curHandle;
	OMEGA_CTX ctx = { model, data, samples, model->bias != 0, dampedInput, dampedZ, zOffsets, zztOffsets };
	INVERSE_ITEM items[KFAC_MAX_ITEMS];
	const int count = omega_items(items, kfac_info, model, &ctx, omegaZInv);
	inverse_pass_run(model, samples, devPtr, items, count, (double)kfac_info->regLambda + (double)kfac_info->dampGamma);
}

typedef struct lambda_ctx {
	const CNN_MODEL *model;
	int samples;
	const real *dx, *dampedLambda;
	const int *zOffsets, *zztOffsets;
} LAMBDA_CTX;

static void lambda_factor(void *ctx, int layer, double shift, double *factor, void *ws, size_t wsBytes)
{
	const LAMBDA_CTX *o = (const LAMBDA_CTX *)ctx;
	const CNN_MODEL *model = o->model;
	const int nc = model->cLayers;
	if (layer < nc) {
		const int l = layer;
		const CONV_LAYER *c = &model->convLayer[l];
		const real *delta;
		if (o->dampedLambda != NULL)
			delta = o->dampedLambda + o->zztOffsets[l + 1];
		else if (c->batchNorm == PERFORM_NO_BATCH_NORM)
			delta = o->dx + o->zOffsets[l + 1] + c->activationOffset;
		else
			delta = o->dx + o->zOffsets[l + 1] + c->batchNormOffset;
		fitre_conv_shape s = conv_shape(c, o->samples);
		HIP_CALL(fitre_hip_kfac_conv_output_factor_f64(&s, delta, shift, factor, ws, wsBytes));
	} else {
		const int l = layer - nc;
		const FC_LAYER *f = &model->fcLayer[l];
		const real *delta = (o->dampedLambda != NULL) ? o->dampedLambda + o->zztOffsets[nc + l + 1] : o->dx + o->zOffsets[nc + l + 1];
		HIP_CALL(fitre_hip_kfac_fc_output_factor_f64(delta, f->out, o->samples, shift, factor, ws, wsBytes));
	}
}

static int lambda_items(INVERSE_ITEM *items, const KFAC_CURVATURE_INFO *kfac_info, const CNN_MODEL *model, LAMBDA_CTX *ctx,
                        real *lambdaGInv)
{
	const int nc = model->cLayers, layers = nc + model->lLayers;
	const int *lambda = kfac_info->LambdaGOffsets;
	for (int l = 0; l < layers; l++) {
		INVERSE_ITEM *it = &items[l];
		it->make = lambda_factor;
		it->rows = NULL;
		it->positions = 0;
		it->ctx = ctx;
		it->layer = l;
		it->order = l < nc ? model->convLayer[l].outChannels : model->fcLayer[l - nc].out;
		it->group = l < nc ? 2 : 3;
		it->inverse = lambdaGInv + lambda[l];
	}
	return layers;
}

void computeLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx, real *dampedLambda,
                        real *lambdaGInv, int *zOffsets, int *zztOffsets, real *devPtr, real *pageLckPtr,
                        cublasHandle_t blasHandle, cudaStream_t curStream, cusolverDnHandle_t curHandle)
{
	(void)pageLckPtr, (void)blasHandle, (void)curStream, (void)curHandle;
	LAMBDA_CTX ctx = { model, samples, dx, dampedLambda, zOffsets, zztOffsets };
	INVERSE_ITEM items[KFAC_MAX_ITEMS];
	const int count = lambda_items(items, kfac_info, model, &ctx, lambdaGInv);
	inverse_pass_run(model, samples, devPtr, items, count, (double)kfac_info->regLambda + (double)kfac_info->dampGamma);
}

void computeOmegaZAndLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                                 real *dampedInput, real *dampedZ, real *dx, real *dampedLambda, int *zOffsets, int *zztOffsets,
                                 real *devPtr)
{
	OMEGA_CTX octx = { model, data, samples, model->bias != 0, dampedInput, dampedZ, zOffsets, zztOffsets };
	LAMBDA_CTX lctx = { model, samples, dx, dampedLambda, zOffsets, zztOffsets };
	INVERSE_ITEM items[KFAC_MAX_ITEMS];
	int count = omega_items(items, kfac_info, model, &octx, kfac_info->OmegaZInv);
	count += lambda_items(items + count, kfac_info, model, &lctx, kfac_info->LambdaGInv);
	inverse_pass_run(model, samples, devPtr, items, count, (double)kfac_info->regLambda + (double)kfac_info->dampGamma);
}

/* ---- natural gradient ---------------------------------------------------------------------- */

static fitre_matrix mat_of_pair(const real *slot, int order)
{
	fitre_matrix m = { slot, order, order, FITRE_MAT_SYM_PAIR, -1, -1, 0.0 };
	return m;
}

/* A float-pair inverse from this order on is decoded into doubles once per layer and the products read the copy
 * (fitre_hip_pair_to_f64): the pair operand costs two loads per element, one of them across the rows. */
#define NG_DECODE_ORDER 128

/* doubles for the largest decoded inverse of one side */
static size_t decoded_bytes(const CNN_MODEL *model, int inputSide)
{
	const int b = model->bias != 0 ? 1 : 0;
	size_t n = 0;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		n = max_sz(n, inputSide ? (size_t)(c->inChannels * c->kSize * c->kSize + b) : (size_t)c->outChannels);
	}
	for (int l = 0; l < model->lLayers; l++) n = max_sz(n, inputSide ? (size_t)(model->fcLayer[l].in + b) : (size_t)model->fcLayer[l].out);
	return n >= NG_DECODE_ORDER ? round_up(n * n * sizeof(double), 256) : 0;
}

/* the operand a product reads a stored float-pair inverse through: the pairs themselves, or their decoded copy */
static fitre_matrix pair_operand(const real *slot, int order, double *decoded)
{
	if (order < NG_DECODE_ORDER || !decoded) return mat_of_pair(slot, order);
	HIP_CALL(fitre_hip_pair_to_f64(slot, order, order, decoded, order));
	fitre_matrix m = { decoded, 1, order, FITRE_MAT_F64, -1, -1, 0.0 };
	return m;
}

static size_t natural_gradient_bytes(const CNN_MODEL *model, size_t *matBytes)
{
	size_t mat = 256, ws = 256;
	const int b = model->bias != 0 ? 1 : 0;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		int k = c->inChannels * c->kSize * c->kSize + b, o = c->outChannels;
		mat = max_sz(mat, (size_t)k * o * sizeof(double));
		ws = max_sz(ws, max_sz(fitre_hip_gemm_f64_workspace(k, o, o, 0), fitre_hip_gemm_f64_workspace(k, o, k, 0)));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		int k = f->in + b, o = f->out;
		mat = max_sz(mat, (size_t)k * o * sizeof(double));
		ws = max_sz(ws, max_sz(fitre_hip_gemm_f64_workspace(o, k, o, 0), fitre_hip_gemm_f64_workspace(o, k, k, 0)));
	}
	*matBytes = round_up(mat, 256);
	/* [wb | u | zt | t1 | t2 | headers | decoded Omega^-1 | decoded Lambda^-1 | product workspace]; t1, t2 (low-rank form:
	 * positions x Cout, positions <= order / 2) */
	return 5 * *matBytes + KFAC_INFO_BYTES + decoded_bytes(model, 1) + decoded_bytes(model, 0) + round_up(ws, 256) + 256;
}

long kfacNaturalGradientMemRequired(CNN_MODEL *model)
{
	size_t matBytes;
	return (long)(natural_gradient_bytes(model, &matBytes) / sizeof(real)) + 64;
}

static fitre_matrix mat_of(const void *data, long rowStride, long colStride, int kind)
{
	fitre_matrix m = { data, rowStride, colStride, kind, -1, -1, 0.0 };
	return m;
}

/* what the header of an input-side slot says (inverse_pass_run) */
typedef struct omega_form {
	int lowrank;
	long positions, rs, cs;
	double alpha, shift;
} OMEGA_FORM;

/* result (rows x cols, `out`) = Omega^-1 applied to u (doubles) from the left (conv: Omega^-1 * u, u order x cols) or
 * from the right (linear: u * Omega^-1, u rows x order), for either form of the stored inverse */
static void apply_omega(const OMEGA_FORM *form, const real *slot, int order, int other, int fromLeft, const double *u,
                        const fitre_matrix *out, double *t1, double *t2, double *decoded, void *ws, size_t wsBytes)
{
	const long ldu = fromLeft ? order : other;
	const fitre_matrix um = mat_of(u, 1, ldu, FITRE_MAT_F64);
	if (!form->lowrank) {
		const fitre_matrix omega = pair_operand(slot, order, decoded);
		if (fromLeft)
			HIP_CALL(fitre_hip_gemm_f64(order, other, order, 1.0, &omega, &um, 0.0, out, 0.0, 0, ws, wsBytes));
		else
			HIP_CALL(fitre_hip_gemm_f64(other, order, order, 1.0, &um, &omega, 0.0, out, 0.0, 0, ws, wsBytes));
		return;
	}
	/* (I - alpha R S^-1 R^T) u / s, resp. u (I - alpha R S^-1 R^T) / s */
	const long m = form->positions;
	const real *rows = slot + KFAC_LOWRANK_HEADER;
	const fitre_matrix r = mat_of(rows, form->rs, form->cs, FITRE_MAT_F32), rt = mat_of(rows, form->cs, form->rs, FITRE_MAT_F32);
	const fitre_matrix sinv = mat_of(lowrank_sinv(slot, order, m), 1, m, FITRE_MAT_F64);
	if (fromLeft) {
		const fitre_matrix a = mat_of(t1, 1, m, FITRE_MAT_F64), b = mat_of(t2, 1, m, FITRE_MAT_F64); /* positions x other */
		HIP_CALL(fitre_hip_gemm_f64(m, other, order, 1.0, &rt, &um, 0.0, &a, 0.0, 0, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm_f64(m, other, m, 1.0, &sinv, &a, 0.0, &b, 0.0, 0, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm_f64_add(order, other, m, -form->alpha / form->shift, &r, &b, 1.0 / form->shift, &um, out, ws, wsBytes));
	} else {
		const fitre_matrix a = mat_of(t1, 1, other, FITRE_MAT_F64), b = mat_of(t2, 1, other, FITRE_MAT_F64); /* other x positions */
		HIP_CALL(fitre_hip_gemm_f64(other, m, order, 1.0, &um, &r, 0.0, &a, 0.0, 0, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm_f64(other, m, m, 1.0, &a, &sinv, 0.0, &b, 0.0, 0, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm_f64_add(other, order, m, -form->alpha / form->shift, &b, &rt, 1.0 / form->shift, &um, out, ws, wsBytes));
	}
}

void computeNaturalGradient(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo, real *devPtr, real *hostPtr)
{
	(void)hostPtr;
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets;
	const int *omegaOff = kfacInfo->OmegaZOffsets, *lambdaOff = kfacInfo->LambdaGOffsets;
	const real *vec = kfacInfo->gradient;
	real *nGradient = kfacInfo->nGradient;
	const int bias = model->bias != 0, nc = model->cLayers, layers = nc + model->lLayers;
	size_t matBytes;
	const size_t total = natural_gradient_bytes(model, &matBytes);
	char *base = aligned_base(devPtr);
	real *wb = (real *)base, *zt = (real *)(base + 2 * matBytes);
	double *u = (double *)(base + matBytes), *t1 = (double *)(base + 3 * matBytes), *t2 = (double *)(base + 4 * matBytes);
	unsigned int *headers = (unsigned int *)(base + 5 * matBytes);
	const size_t omegaBytes = decoded_bytes(model, 1), lambdaBytes = decoded_bytes(model, 0);
	double *omegaDec = omegaBytes ? (double *)(base + 5 * matBytes + KFAC_INFO_BYTES) : NULL;
	double *lambdaDec = lambdaBytes ? (double *)(base + 5 * matBytes + KFAC_INFO_BYTES + omegaBytes) : NULL;
	void *ws = base + 5 * matBytes + KFAC_INFO_BYTES + omegaBytes + lambdaBytes;
	const size_t wsBytes = total - 5 * matBytes - KFAC_INFO_BYTES - omegaBytes - lambdaBytes - 256;

	/* which form every input-side inverse is stored in: the heads of the slots, with one copy */
	OMEGA_FORM forms[MAX_LAYERS];
	{
		const void *slots[MAX_LAYERS];
		unsigned int host[4 * MAX_LAYERS + 8];
		for (int l = 0; l < layers; l++) slots[l] = kfacInfo->OmegaZInv + omegaOff[l];
		HIP_CALL(fitre_hip_gather_headers(slots, layers, headers));
		HIP_CALL(fitre_hip_sync());
		HIP_CALL(fitre_hip_copy_d2h(host, headers, sizeof(unsigned int) * 4 * (size_t)layers));
		for (int l = 0; l < layers; l++) {
			forms[l].lowrank = host[4 * l] == KFAC_LOWRANK_TAG;
			if (!forms[l].lowrank) continue;
			unsigned int rest[9];
			HIP_CALL(fitre_hip_copy_d2h(rest, (const void *)slots[l], sizeof(rest)));
			union { double d; unsigned int w[2]; } a, sh;
			a.w[0] = rest[5], a.w[1] = rest[6], sh.w[0] = rest[7], sh.w[1] = rest[8];
			forms[l].positions = rest[1], forms[l].rs = rest[3], forms[l].cs = rest[4];
			forms[l].alpha = a.d, forms[l].shift = sh.d;
		}
	}

	/* Both inverses are float pairs, or a low-rank form on the input side (inverse_pass_run); the products of a layer
	 * accumulate in float64, what passes from one to the next stays in doubles, and only the natural gradient itself is
	 * rounded to floats.
	 * Convolution layers.  The reference forms Lambda * wb' * Omega (Cout x (K+1)) and transposes the
	 * weight part back; Lambda and Omega are symmetric, so the transposed product Omega * (wb * Lambda)
	 * is the same matrix already in the parameter layout ((K+1) x Cout, one column per filter). */
	for (int c = 0; c < nc; c++) {
		const CONV_LAYER *l = &model->convLayer[c];
		const int K = l->inChannels * l->kSize * l->kSize, O = l->outChannels, R = K + bias;
		const fitre_matrix lambda = pair_operand(kfacInfo->LambdaGInv + lambdaOff[c], O, lambdaDec);
		const real *v = vec + wOffsets[c];
		real *ng = nGradient + wOffsets[c];
		const real *mat = v;
		if (bias) { /* wb = [filter ; bias] per column, solvers/kfac_natural_gradient.cu:107-119 */
			HIP_CALL(fitre_hip_copy_2d(wb, R, v, K, K, O));
			HIP_CALL(fitre_hip_copy_2d(wb + K, R, vec + bOffsets[c], 1, 1, O));
			mat = wb;
		}
		const fitre_matrix g = mat_of(mat, 1, R, FITRE_MAT_F32), um = mat_of(u, 1, R, FITRE_MAT_F64);
		HIP_CALL(fitre_hip_gemm_f64(R, O, O, 1.0, &g, &lambda, 0.0, &um, 0.0, 0, ws, wsBytes));
		if (bias) {
			const fitre_matrix out = mat_of(zt, 1, R, FITRE_MAT_F32);
			apply_omega(&forms[c], kfacInfo->OmegaZInv + omegaOff[c], R, O, 1, u, &out, t1, t2, omegaDec, ws, wsBytes);
			HIP_CALL(fitre_hip_copy_2d(ng, K, zt, R, K, O));
			HIP_CALL(fitre_hip_copy_2d(nGradient + bOffsets[c], 1, zt + K, R, 1, O));
		} else {
			const fitre_matrix out = mat_of(ng, 1, R, FITRE_MAT_F32);
			apply_omega(&forms[c], kfacInfo->OmegaZInv + omegaOff[c], R, O, 1, u, &out, t1, t2, omegaDec, ws, wsBytes);
		}
	}
	/* Linear layers: the gradient block [W | b] already is the out x (in + 1) matrix
	 * (solvers/kfac_natural_gradient.cu:196-229). */
	for (int f = 0; f < model->lLayers; f++) {
		const FC_LAYER *l = &model->fcLayer[f];
		const int R = l->in + bias, O = l->out;
		const fitre_matrix lambda = pair_operand(kfacInfo->LambdaGInv + lambdaOff[nc + f], O, lambdaDec);
		const fitre_matrix g = mat_of(vec + wOffsets[nc + f], 1, O, FITRE_MAT_F32), um = mat_of(u, 1, O, FITRE_MAT_F64);
		const fitre_matrix out = mat_of(nGradient + wOffsets[nc + f], 1, O, FITRE_MAT_F32);
		HIP_CALL(fitre_hip_gemm_f64(O, R, O, 1.0, &lambda, &g, 0.0, &um, 0.0, 0, ws, wsBytes));
		apply_omega(&forms[nc + f], kfacInfo->OmegaZInv + omegaOff[nc + f], R, O, 0, u, &out, t1, t2, omegaDec, ws, wsBytes);
	}
	HIP_CALL(fitre_hip_sync());
}
