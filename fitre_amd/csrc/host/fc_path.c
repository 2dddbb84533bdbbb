/*
 * The fully connected model family: applyLayerActivation, nnForwardPass, evaluateModel and
 * computeGradient of functions/eval_gradient.cu, as C host code over the C-ABI device layer.
 * Same data flow; the ones-vector products become row sums, the reductions one sum call.
 */
#include <stdio.h>
#include <stdlib.h>
#include "fitre_fc.h"
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

static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }

void fitre_build_nn(NN_MODEL *model, const int *layerSizes, const int *actFuns, int numLayers, int type, int numPoints)
{
	if (numLayers < 1 || numLayers >= MAX_LAYERS) {
		fprintf(stderr, "fitre_build_nn: %d layers (1 .. %d supported)\n", numLayers, MAX_LAYERS - 1);
		exit(-1);
	}
	for (int i = 0; i < MAX_LAYERS; i++) {
		model->layerSizes[i] = model->actFuns[i] = 0;
		model->wOffsets[i] = model->bOffsets[i] = model->zOffsets[i] = 0;
		model->sZOffsets[i] = model->rZOffsets[i] = model->sRZOffsets[i] = 0;
	}
	for (int i = 0; i <= numLayers; i++) model->layerSizes[i] = layerSizes[i];
	for (int i = 0; i < numLayers; i++) model->actFuns[i] = actFuns[i];
	model->actFuns[numLayers] = ACT_NONE;
	model->numLayers = numLayers;
	model->type = type;
	const int l = numLayers;
	int w = 0;
	model->wOffsets[0] = 0;
	model->bOffsets[0] = model->layerSizes[1] * model->layerSizes[0];
	for (int i = 1; i < l; i++) {
		w += model->layerSizes[i] * model->layerSizes[i - 1] + model->layerSizes[i];
		model->wOffsets[i] = w;
		model->bOffsets[i] = w + model->layerSizes[i] * model->layerSizes[i + 1];
	}
	w += model->layerSizes[l] * model->layerSizes[l - 1] + model->layerSizes[l];
	model->pSize = w;
	int zs = 0;
	model->zOffsets[0] = 0;
	for (int i = 1; i <= l; i++) {
		zs += model->layerSizes[i - 1] * numPoints;
		model->zOffsets[i] = zs;
	}
	zs += model->layerSizes[l] * numPoints;
	model->zSize = zs;
	model->sampledZSize = model->sampledRSize = model->rFullSize = 0;
}

void initSampledZOffsets(NN_MODEL *model, int numPoints)
{
	int zSize = 0;
	model->sZOffsets[0] = zSize;
	for (int i = 1; i <= model->numLayers; i++) {
		zSize += model->layerSizes[i - 1] * numPoints;
		model->sZOffsets[i] = zSize;
	}
	zSize += model->layerSizes[model->numLayers] * numPoints;
	model->sampledZSize = zSize;
}

void initRZOffsets(NN_MODEL *model, int datasetSize)
{
	int total = 0;
	model->rZOffsets[0] = total;
	for (int i = 1; i <= model->numLayers; i++) {
		total += model->layerSizes[i] * datasetSize;
		model->rZOffsets[i] = total;
	}
	model->rFullSize = total;
}

void initSampledROffsets(NN_MODEL *model, int sampleSize)
{
	int total = 0;
	model->sRZOffsets[0] = total;
	for (int i = 1; i <= model->numLayers; i++) {
		total += model->layerSizes[i] * sampleSize;
		model->sRZOffsets[i] = total;
	}
	model->sampledRSize = total;
}

static size_t largest_layer(const NN_MODEL *model)
{
	size_t m = 1;
	for (int i = 0; i <= model->numLayers; i++) m = max_sz(m, (size_t)model->layerSizes[i]);
	return m;
}

/* workspace (bytes) of the products of a pass over `points` columns */
static size_t product_ws_bytes(const NN_MODEL *model, int points, int backward)
{
	size_t need = 256;
	for (int i = 0; i < model->numLayers; i++) {
		int in = model->layerSizes[i], out = model->layerSizes[i + 1];
		need = max_sz(need, fitre_hip_gemm_workspace(out, points, in));
		if (backward) {
			need = max_sz(need, fitre_hip_gemm_workspace(out, in, points));
			need = max_sz(need, fitre_hip_gemm_workspace(in, points, out));
		}
	}
	return (need + 255) & ~(size_t)255;
}

long nnForwardMemRequired(NN_MODEL *model, int points)
{
	/* [terms of the output head | product workspace] */
	return (long)model->layerSizes[model->numLayers] * points + (long)(product_ws_bytes(model, points, 0) / sizeof(real)) + 128;
}

long nnGradientMemRequired(NN_MODEL *model, int points)
{
	/* [error term, sized for the widest layer | two spare vectors | forward scratch | product workspace] */
	return (long)largest_layer(model) * points + 2L * points + nnForwardMemRequired(model, points) +
	       (long)(product_ws_bytes(model, points, 1) / sizeof(real)) + 256;
}

static real *align_reals(real *p) { return (real *)(((size_t)p + 255) & ~(size_t)255); }

static void layer_forward(int actFunction, const real *W, int wRows, int wCols, const real *b, const real *z, int zRows,
                          int zCols, real *output, int extendedCopy, void *ws, size_t wsBytes)
{
	const long count = (long)wRows * zCols;
	HIP_CALL(fitre_hip_gemm(0, 0, wRows, zCols, wCols, 1.f, W, wRows, z, zRows, 0.f, output, wRows, b, ws, wsBytes));
	if (extendedCopy) HIP_CALL(fitre_hip_copy_d2d(output + count, output, sizeof(real) * (size_t)count));
	if (actFunction == ACT_SOFTMAX)
		HIP_CALL(fitre_hip_column_softmax(output, wRows, zCols));
	else if (actFunction != ACT_LINEAR && actFunction != ACT_NONE && actFunction != CNN_ACT_NONE) {
		if (fitre_hip_activation_forward(actFunction, output, output, count) != FITRE_OK) {
			fprintf(stderr, "computeGradient: Error Unknown Activation Function \n");
			exit(-1);
		}
	}
}

void applyLayerActivation(int actFunction, real *W, int wRows, int wCols, real *b, int bRows, real *z, int zRows,
                          int zCols, real *output, real *scratch, real *hostPtr)
{
	(void)bRows, (void)scratch, (void)hostPtr;
	layer_forward(actFunction, W, wRows, wCols, b, z, zRows, zCols, output, 1, NULL, 0);
	HIP_CALL(fitre_hip_sync());
}

void nnForwardPass(NN_MODEL *model, DEVICE_DATASET *data, real *weights, real *z, real *errTerm, real *logLikelihood,
                   real *modelError, real *hostPtr, real *devPtr, DATASET_SIZE isGradient, DATA_TYPE dataType)
{
	(void)hostPtr;
	const int numLayers = model->numLayers;
	const int *layerSizes = model->layerSizes;
	const int *zOffsets = (isGradient == FULL_DATASET) ? model->zOffsets : model->sZOffsets;
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets;
	real *dataset, *target;
	int numRows, numCols, numColsTarget;

	if (dataType == TEST_DATA) {
		dataset = data->testSetX, target = data->testSetY;
		numRows = data->features, numCols = data->testSizeX, numColsTarget = data->testSizeY;
	} else if (isGradient == FULL_DATASET) {
		dataset = data->trainSetX, target = data->trainSetY;
		numRows = data->features, numCols = data->trainSizeX, numColsTarget = data->trainSizeY;
	} else {
		dataset = data->sampledTrainX, target = data->sampledTrainX;
		numRows = data->features, numCols = data->sampleSize, numColsTarget = data->sampleSize;
	}
	const int outSize = layerSizes[numLayers];
	const long numElements = (long)outSize * numColsTarget;
	real *terms = devPtr;
	void *ws = align_reals(terms + numElements);
	const size_t wsBytes = product_ws_bytes(model, numCols, 0);

	for (int i = 0; i < numLayers; i++) {
		const real *in = (i == 0) ? dataset : z + zOffsets[i];
		const int inRows = (i == 0) ? numRows : layerSizes[i];
		layer_forward(model->actFuns[i], weights + wOffsets[i], layerSizes[i + 1], layerSizes[i], weights + bOffsets[i], in,
		              inRows, numCols, z + zOffsets[i + 1], 0, ws, wsBytes);
	}

	real *out = z + zOffsets[numLayers];
	real sum = 0;
	const int head = model->actFuns[numLayers - 1];
	if (head == ACT_LINEAR) {
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SQUARED_DIFFERENCE, target, out, numElements, 1.f, terms));
		HIP_CALL(fitre_hip_sum((int)numElements, terms, &sum));
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SCALED_DIFFERENCE, target, out, numElements, 2.f, errTerm));
	} else if (head == ACT_LOGISTIC) {
		/* the logits once more: xi = W z + b of the last layer */
		const real *in = (numLayers == 1) ? dataset : z + zOffsets[numLayers - 1];
		layer_forward(ACT_LINEAR, weights + wOffsets[numLayers - 1], outSize, layerSizes[numLayers - 1],
		              weights + bOffsets[numLayers - 1], in, layerSizes[numLayers - 1], numCols, terms, 0, ws, wsBytes);
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_LOGISTIC_LL, target, terms, numElements, 1.f, terms));
		HIP_CALL(fitre_hip_sum((int)numElements, terms, &sum));
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SCALED_DIFFERENCE, target, out, numElements, 1.f, errTerm));
	} else if (head == ACT_SOFTMAX) {
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SOFTMAX_LL, target, out, numElements, 1.f, terms));
		HIP_CALL(fitre_hip_sum((int)numElements, terms, &sum));
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SCALED_DIFFERENCE, target, out, numElements, 1.f, errTerm));
	}
	*logLikelihood = sum * (real)(-1.0 / (double)numColsTarget);

	*modelError = 0;
	if (model->type == MODEL_TYPE_MSE) {
		real mse = 0;
		HIP_CALL(fitre_hip_output_terms(FITRE_TERM_SQUARED_DIFFERENCE, target, out, numElements, 1.f, terms));
		HIP_CALL(fitre_hip_sum((int)numElements, terms, &mse));
		*modelError = mse / (real)numColsTarget;
	}
	HIP_CALL(fitre_hip_sync());
}

void evaluateModel(NN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *weights, real *logLikelihood,
                   real *modelError, DATASET_SIZE isGradient, DATA_TYPE dataType)
{
	real *z = scratch->nextDevPtr;
	real *errTerm = z + model->zSize;
	const int points = (dataType == TRAIN_DATA) ? data->trainSizeX : data->testSizeX;
	real *nextDevPtr = errTerm + (long)model->layerSizes[model->numLayers] * points;
	*logLikelihood = 0;
	*modelError = 0;
	nnForwardPass(model, data, weights, z, errTerm, logLikelihood, modelError, scratch->nextHostPtr, nextDevPtr, isGradient,
	              dataType);
}

void computeGradient(NN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *weights, real *z, real *dx,
                     real *gradient, real *logLikelihood, real *modelError, DATASET_SIZE isGradient)
{
	const int n = (isGradient == FULL_DATASET) ? data->trainSizeX : data->sampleSize;
	real *dataset = (isGradient == FULL_DATASET) ? data->trainSetX : data->sampledTrainX;
	const int numLayers = model->numLayers;
	const int *layerSizes = model->layerSizes;
	real *dW = gradient;
	real *errorTerm = scratch->nextDevPtr;
	real *oneVector = errorTerm + (long)largest_layer(model) * n; /* kept for the layout; row sums need no ones */
	real *nextDevPtr = oneVector + 2L * n;
	if (z == NULL) {
		z = nextDevPtr;
		dx = z + ((isGradient == SAMPLED_DATASET) ? model->sampledZSize : model->zSize);
		nextDevPtr = dx + ((isGradient == SAMPLED_DATASET) ? model->sampledRSize : model->rFullSize);
	}
	const int *zOffsets = (isGradient == SAMPLED_DATASET) ? model->sZOffsets : model->zOffsets;
	const int *rZOffsets = (isGradient == SAMPLED_DATASET) ? model->sRZOffsets : model->rZOffsets;
	const int *bOffsets = model->bOffsets, *wOffsets = model->wOffsets;

	nnForwardPass(model, data, weights, z, errorTerm, logLikelihood, modelError, scratch->nextHostPtr, nextDevPtr, isGradient,
	              TRAIN_DATA);
	void *ws = align_reals(nextDevPtr + nnForwardMemRequired(model, n));
	const size_t wsBytes = product_ws_bytes(model, n, 1);

	for (int i = numLayers - 1; i >= 0; i--) {
		const int out = layerSizes[i + 1], in = layerSizes[i];
		const long count = (long)out * n;
		if (i < numLayers - 1) { /* the head's derivative is already in the error term */
			const real *xi = z + zOffsets[i + 1];
			const int act = model->actFuns[i];
			if (act == ACT_LOGISTIC || act == ACT_TANH)
				HIP_CALL(fitre_hip_activation_backward(act, errorTerm, NULL, xi, errorTerm, count));
			else if (act != ACT_LINEAR) {
				fprintf(stderr, "computeGradient: Unknown Layer at: %d (%d) \n", i, act);
				exit(-1);
			}
		}
		/* db = sum(err, 2); dW = err * z_i' */
		HIP_CALL(fitre_hip_row_sum(errorTerm, out, n, dW + bOffsets[i]));
		const real *zin = (i == 0) ? dataset : z + zOffsets[i];
		HIP_CALL(fitre_hip_gemm(0, 1, out, in, n, 1.f, errorTerm, out, zin, in, 0.f, dW + wOffsets[i], out, NULL, ws, wsBytes));
		HIP_CALL(fitre_hip_copy_d2d(dx + rZOffsets[i], errorTerm, sizeof(real) * (size_t)count));
		/* err = W_i' * err (not needed below the first layer) */
		if (i > 0)
			HIP_CALL(fitre_hip_gemm(1, 0, in, n, out, 1.f, weights + wOffsets[i], out, dx + rZOffsets[i], out, 0.f, errorTerm, in,
			                        NULL, ws, wsBytes));
	}
	HIP_CALL(fitre_hip_scal(model->pSize, (real)(-1.0 / (double)n), dW));
	HIP_CALL(fitre_hip_sync());
}

/* ---- Hessian-vector products (functions/eval_hessian_vec.cu, eval_gauss_newton_hessian_vec.cu) ---- */

typedef struct hv_layout {
	long n, zReals, rReals;
	size_t wsBytes;
} HV_LAYOUT;

static HV_LAYOUT hv_layout(const NN_MODEL *model, const DEVICE_DATASET *data, DATASET_SIZE allData)
{
	HV_LAYOUT l;
	l.n = (allData == FULL_DATASET) ? data->trainSizeX : data->sampleSize;
	l.zReals = (allData == FULL_DATASET) ? model->zSize : model->sampledZSize;
	l.rReals = (allData == FULL_DATASET) ? model->rFullSize : model->sampledRSize;
	l.wsBytes = product_ws_bytes(model, (int)l.n, 1);
	return l;
}

/* [RdW | Rdz | Rdx | Rz | Rx | 2 x features (the reference's vector of ones) | one layer-sized temporary | products] */
long nnHessianVecMemRequired(NN_MODEL *model, DEVICE_DATASET *data, DATASET_SIZE allData)
{
	const HV_LAYOUT l = hv_layout(model, data, allData);
	return (long)model->pSize + 3 * l.zReals + l.rReals + 2L * data->features + (long)largest_layer(model) * l.n +
	       (long)(l.wsBytes / sizeof(real)) + 256;
}

static void nn_rop(NN_MODEL *model, DEVICE_DATASET *data, real *z, real *dx, real *vec, real *weights, SCRATCH_AREA *scratch,
                   DATASET_SIZE allData, int gaussNewton)
{
	const int *layerSizes = model->layerSizes;
	const int *zOffsets = (allData == FULL_DATASET) ? model->zOffsets : model->sZOffsets;
	const int *rZOffsets = (allData == FULL_DATASET) ? model->rZOffsets : model->sRZOffsets;
	const int *bOffsets = model->bOffsets, *wOffsets = model->wOffsets;
	const int numLayers = model->numLayers;
	const HV_LAYOUT l = hv_layout(model, data, allData);
	const int n = (int)l.n;
	const real *trainX = (allData == FULL_DATASET) ? data->trainSetX : data->sampledTrainX;
	const char *who = gaussNewton ? "gaussNewtonHessianVec" : "hessianVec";

	const int head = model->actFuns[numLayers - 1];
	if (head != ACT_LOGISTIC && head != ACT_SOFTMAX) { /* eval_hessian_vec.cu:300-303: the linear head is not derived */
		fprintf(stderr, "%s: output layer %d is neither logistic nor softmax\n", who, head);
		exit(-1);
	}

	real *RdW = scratch->nextDevPtr;
	real *Rdz = RdW + model->pSize;
	real *Rdx = Rdz + l.zReals;
	real *Rz = Rdx + l.rReals;
	real *Rx = Rz + l.zReals;
	real *oneVector = Rx + l.zReals; /* kept for the layout; row sums need no ones */
	real *tmp = oneVector + 2L * data->features;
	void *ws = align_reals(tmp + (long)largest_layer(model) * n);
	const real *VW = vec;

	HIP_CALL(fitre_hip_memset(RdW, 0, sizeof(real) * (size_t)model->pSize));

	/* forward: Rx_{i+1} = VW_i z_i + Vb_i + W_i Rz_i;  Rz_{i+1} = f'(.) Rx_{i+1} */
	for (int i = 0; i < numLayers; i++) {
		const int out = layerSizes[i + 1], in = layerSizes[i];
		const long count = (long)out * n;
		real *rxi = Rx + zOffsets[i + 1], *rzi = Rz + zOffsets[i + 1];
		const real *zin = (i == 0) ? trainX : z + zOffsets[i];
		const real *zout = z + zOffsets[i + 1];
		HIP_CALL(fitre_hip_gemm(0, 0, out, n, in, 1.f, VW + wOffsets[i], out, zin, in, 0.f, rxi, out, VW + bOffsets[i], ws, l.wsBytes));
		if (i > 0)
			HIP_CALL(fitre_hip_gemm(0, 0, out, n, in, 1.f, weights + wOffsets[i], out, Rz + zOffsets[i], in, 1.f, rxi, out, NULL, ws,
			                        l.wsBytes));
		switch (model->actFuns[i]) {
		case ACT_LOGISTIC:
		case ACT_TANH:
			HIP_CALL(fitre_hip_activation_backward(model->actFuns[i], rxi, NULL, zout, rzi, count));
			break;
		case ACT_LINEAR:
			HIP_CALL(fitre_hip_copy_d2d(rzi, rxi, sizeof(real) * (size_t)count));
			break;
		case ACT_SOFTMAX:
			HIP_CALL(fitre_hip_column_softmax_rop(zout, rxi, out, n, rzi));
			break;
		default:
			fprintf(stderr, "hessianVec: unknown activation function at Layer: %d \n", i);
			exit(-1);
		}
	}

	/* backward, from the head: Rdx_L = -Rz_{L+1} */
	for (int i = numLayers - 1; i >= 0; i--) {
		const int out = layerSizes[i + 1], in = layerSizes[i];
		const long count = (long)out * n;
		real *rdxi = Rdx + rZOffsets[i];
		const real *dxi = dx + rZOffsets[i];
		const real *zin = (i == 0) ? trainX : z + zOffsets[i];
		if (i == numLayers - 1) {
			HIP_CALL(fitre_hip_copy_d2d(rdxi, Rz + zOffsets[numLayers], sizeof(real) * (size_t)count));
			HIP_CALL(fitre_hip_scal((int)count, -1.f, rdxi));
		} else {
			const int act = model->actFuns[i];
			if (act != ACT_LOGISTIC && act != ACT_TANH && act != ACT_LINEAR) {
				fprintf(stderr, "%s: unknown activation function at Layer: %d \n", who, i);
				exit(-1);
			}
			/* the reference's sweep leaves Rdx of a tanh layer unset (eval_hessian_vec.cu:418-420); its derivative is used here */
			HIP_CALL(fitre_hip_fc_rop_backward(act, z + zOffsets[i + 1], Rdz + zOffsets[i + 1], gaussNewton ? NULL : Rx + zOffsets[i + 1],
			                                   gaussNewton ? NULL : dxi, rdxi, count));
		}
		/* RdW_i = Rdx_i z_i' (+ dx_i Rz_i', zero for the first layer);  Rdb_i = sum(Rdx_i, 2) */
		HIP_CALL(fitre_hip_gemm(0, 1, out, in, n, 1.f, rdxi, out, zin, in, 0.f, RdW + wOffsets[i], out, NULL, ws, l.wsBytes));
		if (!gaussNewton && i > 0)
			HIP_CALL(fitre_hip_gemm(0, 1, out, in, n, 1.f, dxi, out, Rz + zOffsets[i], in, 1.f, RdW + wOffsets[i], out, NULL, ws,
			                        l.wsBytes));
		HIP_CALL(fitre_hip_row_sum(rdxi, out, n, RdW + bOffsets[i]));
		/* Rdz_i = W_i' Rdx_i (+ VW_i' dx_i; the Gauss-Newton variant keeps that term for the top layer only,
		 * eval_gauss_newton_hessian_vec.cu:262-275) */
		if (i > 0) {
			real *rdzi = Rdz + zOffsets[i];
			HIP_CALL(fitre_hip_gemm(1, 0, in, n, out, 1.f, weights + wOffsets[i], out, rdxi, out, 0.f, rdzi, in, NULL, ws, l.wsBytes));
			if (!gaussNewton || i == numLayers - 1)
				HIP_CALL(fitre_hip_gemm(1, 0, in, n, out, 1.f, VW + wOffsets[i], out, dxi, out, 1.f, rdzi, in, NULL, ws, l.wsBytes));
		}
	}
	HIP_CALL(fitre_hip_scal(model->pSize, (real)(-1.0 / (double)n), RdW));
	HIP_CALL(fitre_hip_sync());
}

void hessianVec(NN_MODEL *model, DEVICE_DATASET *data, real *z, real *dx, real *vec, real *weights, SCRATCH_AREA *scratch,
                DATASET_SIZE allData)
{
	nn_rop(model, data, z, dx, vec, weights, scratch, allData, 0);
}

void gaussNewtonHessianVec(NN_MODEL *model, DEVICE_DATASET *data, real *z, real *dx, real *vec, real *weights,
                           SCRATCH_AREA *scratch, DATASET_SIZE allData)
{
	nn_rop(model, data, z, dx, vec, weights, scratch, allData, 1);
}
