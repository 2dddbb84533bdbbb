/*
 * The sub-sampled KFAC trust-region solver's loop (solvers/kfac_trust_region.cu:92-660) as C host code
 * over this library's reference-named entry points.  Same order of calls per mini-batch, same
 * acceptance rule, same radius update; every device buffer is carved from the caller's arena at a
 * 256-byte boundary.  One device: the reference's second-device worker for the inverses
 * (solvers/kfac_thread.cu, commented out in the reference's loop as well) has no counterpart.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/time.h>
#include "fitre_solver.h"
#include "fitre_cnn.h"
#include "fitre_hv.h"
#include "fitre_input.h"
#include "fitre_shim.h"
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

#define ARENA_ALIGN 64 /* reals: 256 bytes */
#define MAX_REPORTS 1024

static KFAC_TR_EPOCH_REPORT g_reports[MAX_REPORTS];
static int g_report_count = 0;

static double now_seconds(void)
{
	struct timeval t;
	gettimeofday(&t, NULL);
	return (double)t.tv_sec + (double)t.tv_usec / 1e6;
}

static long round_up(long n) { return (n + ARENA_ALIGN - 1) / ARENA_ALIGN * ARENA_ALIGN; }
static long max_l(long a, long b) { return a > b ? a : b; }

/* bump allocator over the caller's device arena */
typedef struct arena {
	real *next;
} ARENA;

static real *carve(ARENA *a, long reals)
{
	real *p = a->next;
	a->next += round_up(reals);
	return p;
}

void genRandomVector(int *idx, int m, int n)
{
	int im = 0;
	for (int in = 0; in < n && im < m; ++in) {
		int rn = n - in, rm = m - im;
		if (rand() % rn < rm) idx[im++] = in;
	}
	if (im != m) {
		fprintf(stderr, "Failed to generate required number of random numbers ... (%d, %d) ", im, m);
		exit(-1);
	}
	for (int i = m - 1; i >= 0; i--) {
		int j = rand() % (i + 1);
		int t = idx[i];
		idx[i] = idx[j];
		idx[j] = t;
	}
}

void allocSampledDataset(DEVICE_DATASET *data, int sampleSize)
{
	data->sampleSize = sampleSize;
	cuda_malloc((void **)&data->sampledTrainX, (size_t)sampleSize * data->features * sizeof(real), 1, -1);
	/* one label per image (the reference reserves a whole image's worth per label) */
	cuda_malloc((void **)&data->sampledTrainY, (size_t)sampleSize * sizeof(real), 1, -1);
}

void initBatchNormData(CNN_MODEL *model, real *z, int *zOffsets)
{
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		if (c->batchNorm == PERFORM_NO_BATCH_NORM) continue;
		real *bn = z + zOffsets[i + 1] + c->batchNormOffset;
		HIP_CALL(fitre_hip_fill(bn + c->runningMeansOffset, c->outChannels, 0.f));
		HIP_CALL(fitre_hip_fill(bn + c->runningVariancesOffset, c->outChannels, 1.f));
	}
	HIP_CALL(fitre_hip_sync());
}

void updateRunningStats(real *src, real *update, int numElements, real momentum)
{
	if (momentum != 0) {
		HIP_CALL(fitre_hip_scal(numElements, momentum / ((real)1. - momentum), src));
		HIP_CALL(fitre_hip_axpy(numElements, (real)1., update, src));
		HIP_CALL(fitre_hip_scal(numElements, (real)1. - momentum, src));
	} else {
		HIP_CALL(fitre_hip_copy_d2d(src, update, sizeof(real) * (size_t)numElements));
	}
}

static void start_or_update(real *average, real *fresh, long count, int start, real decay)
{
	if (start)
		HIP_CALL(fitre_hip_copy_d2d(average, fresh, sizeof(real) * (size_t)count));
	else
		updateRunningStats(average, fresh, (int)count, decay);
}

void computeSpeedUpOmegaZ(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples, real *z,
                          int *zOffsets, real *dampedInput, real *dampedZ, int *zztOffsets, int iterCount)
{
	const int start = iterCount == 0;
	const real decay = (real)sqrt(kfac_info->stats_decay);
	start_or_update(dampedInput, data->currentBatch, (long)data->features * samples, start, decay);
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		const POOL_LAYER *p = &model->poolLayer[i];
		long cells = (p->type == NO_POOL) ? (long)c->outHeight * c->outWidth : (long)p->outHeight * p->outWidth;
		start_or_update(dampedZ + zztOffsets[i + 1], z + zOffsets[i + 1] + c->outputOffset, cells * c->outChannels * samples, start,
		                decay);
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		int at = l + 1 + model->cLayers;
		start_or_update(dampedZ + zztOffsets[at], z + zOffsets[at], (long)f->out * samples, start, decay);
	}
}

void computeSpeedUpLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx, real *dampedLambda,
                               int *zOffsets, int *zztOffsets, int iterCount)
{
	const int start = iterCount == 0;
	const real decay = (real)sqrt(kfac_info->stats_decay);
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		real *delta = dx + zOffsets[i + 1] + (c->batchNorm == PERFORM_NO_BATCH_NORM ? c->activationOffset : c->batchNormOffset);
		start_or_update(dampedLambda + zztOffsets[i + 1], delta, (long)c->outChannels * c->outHeight * c->outWidth * samples, start,
		                decay);
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		int at = l + 1 + model->cLayers;
		start_or_update(dampedLambda + zztOffsets[at], dx + zOffsets[at], (long)f->out * samples, start, decay);
	}
}

/* the part of the arena that is reused from step to step (everything behind lossFuncErrors) */
static long step_scratch_reals(CNN_MODEL *model, DEVICE_DATASET *data)
{
	const long batch = model->batchSize, classes = data->numClasses;
	const long deltas = 2 * round_up(max_l(model->maxDeltaSize, classes * batch));
	long need = cnnForwardMemRequired(model);
	need = max_l(need, deltas + cnnBackwardMemRequired(model));
	/* second backward and the factor passes keep the sampled-target snapshots alive */
	const long fisher = deltas + round_up(model->zSize) + round_up(batch);
	need = max_l(need, fisher + max_l(cnnBackwardMemRequired(model), 4 * batch));
	need = max_l(need, fisher + kfacInverseMemRequired(model, (int)batch));
	need = max_l(need, kfacNaturalGradientMemRequired(model));
	need = max_l(need, model->pSize + cnnHvMemRequired(model));
	need = max_l(need, 4 * batch);
	return round_up(need) + ARENA_ALIGN;
}

long kfacTrustRegionMemRequired(CNN_MODEL *model, DEVICE_DATASET *data, KFAC_CURVATURE_INFO *kfacInfo)
{
	const int layers = model->cLayers + model->lLayers;
	const long batch = model->batchSize, classes = data->numClasses;
	KFAC_CURVATURE_INFO sizes = *kfacInfo;
	computeKFACStorageIndices(model, &sizes);
	long need = ARENA_ALIGN + round_up(data->trainSizeX);
	if (kfacInfo->inverseFreq != 1) need += round_up((long)data->features * batch) + 2 * round_up(model->zztSize);
	need += round_up(sizes.OmegaZOffsets[layers]) + round_up(sizes.LambdaGOffsets[layers]);
	need += 5 * round_up(model->pSize) + 2 * round_up(model->zSize) + 2 * round_up(classes * batch);
	return need + step_scratch_reals(model, data);
}

long kfacTrustRegionHostMemRequired(DEVICE_DATASET *data) { return round_up(data->trainSizeX) + ARENA_ALIGN; }

int kfacTrustRegionReports(KFAC_TR_EPOCH_REPORT *out, int capacity)
{
	int n = g_report_count < capacity ? g_report_count : capacity;
	if (out != NULL && n > 0) memcpy(out, g_reports, sizeof(KFAC_TR_EPOCH_REPORT) * (size_t)n);
	return g_report_count;
}

static void generateParamReport(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo, TRUST_REGION_PARAMS *trParams)
{
	fprintf(stderr, "********** KFAC_SOLVER_REPORT ***********\n");
	fprintf(stderr, "BatchSize: %d\n", model->batchSize);
	fprintf(stderr, "MaxTRRadius: %f\n", trParams->maxDelta);
	fprintf(stderr, "DampGamma: %f\n", kfacInfo->dampGamma);
	fprintf(stderr, "CheckGrad: %d \n", kfacInfo->checkGrad);
	fprintf(stderr, "BatchNorm: %d \n", model->enableBatchNorm);
	fprintf(stderr, "Bias: %d \n", model->bias);
	fprintf(stderr, "InverseFreq: %d \n", kfacInfo->inverseFreq);
	fprintf(stderr, "Lambda: %f \n", kfacInfo->regLambda);
	fprintf(stderr, "*****************************************\n");
}

void subsampledTrustRegionKFAC(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, KFAC_CURVATURE_INFO *kfacInfo,
                               TRUST_REGION_PARAMS *trParams, SCRATCH_AREA *scratch, int master, int slave)
{
	(void)master;
	(void)slave;
	const DATASET_TYPE datasetType = host != NULL ? host->datasetType : data->datasetType;
	if (host != NULL && host->datasetType != data->datasetType) {
		/* the training loop reads the host set's type, the per-pass sweeps the device set's: they must agree */
		fprintf(stderr, "subsampledTrustRegionKFAC: data set type of the host set (%d) and of the device set (%d) differ\n",
		        (int)host->datasetType, (int)data->datasetType);
		exit(-1);
	}
	/* the third case keeps the training set in host memory and reads mini-batches from there
	 * (selectHostMatrix, solvers/kfac_trust_region.cu:322-337) */
	const int hostResident = datasetType == IMAGENET;
	if (datasetType != CIFAR10 && datasetType != CIFAR100 && datasetType != IMAGENET) {
		fprintf(stderr, "Problem with the dataset initialization.... \n\n");
		exit(-1);
	}
	if (hostResident && (host == NULL || host->trainSetX == NULL || host->trainSetY == NULL)) {
		fprintf(stderr, "subsampledTrustRegionKFAC: a host-resident data set needs the host struct's training arrays\n");
		exit(-1);
	}
	const int layers = model->cLayers + model->lLayers;
	const int components = model->pSize;
	const long batch = model->batchSize, classes = data->numClasses;
	real *pageLckPtr = scratch->nextPageLckPtr;
	/* what the loop carves from the arenas is released when it returns: a second call with the same struct
	 * starts from the same addresses (the reference leaves the pointers advanced) */
	real *const entryDevPtr = scratch->nextDevPtr, *const entryHostPtr = scratch->nextHostPtr;
	real *const entryPageLckPtr = scratch->nextPageLckPtr;
	int *hostIndices = (int *)scratch->nextHostPtr;
	real *nextHostPtr = scratch->nextHostPtr + round_up(data->trainSizeX);

	computeKFACStorageIndices(model, kfacInfo);

	/* device arena, in the reference's order (:112-141) */
	ARENA arena;
	arena.next = (real *)(((size_t)scratch->nextDevPtr + 255) & ~(size_t)255);
	int *shuffleIndices = (int *)carve(&arena, data->trainSizeX);
	real *dampedInput = NULL, *dampedZ = NULL, *dampedLambda = NULL;
	if (kfacInfo->inverseFreq != 1) {
		dampedInput = carve(&arena, (long)data->features * batch);
		dampedZ = carve(&arena, model->zztSize);
		dampedLambda = carve(&arena, model->zztSize);
	}
	real *omegaZInv = carve(&arena, kfacInfo->OmegaZOffsets[layers]);
	real *lambdaGInv = carve(&arena, kfacInfo->LambdaGOffsets[layers]);
	real *gradient = carve(&arena, components);
	real *distGradient = carve(&arena, components);
	real *vector = carve(&arena, components);
	real *prevWeights = carve(&arena, components);
	real *naturalGradient = carve(&arena, components);
	real *z = carve(&arena, model->zSize);
	real *dx = carve(&arena, model->zSize);
	real *probs = carve(&arena, batch * classes);
	real *lossFuncErrors = carve(&arena, batch * classes);
	real *scratchBegin = arena.next;

	/* page-locked scalars (:164-169) */
	real *nextPageLckPtr = pageLckPtr + 4;

	kfacInfo->OmegaZZT = NULL;
	kfacInfo->LambdaGGT = NULL;
	kfacInfo->OmegaZInv = omegaZInv;
	kfacInfo->LambdaGInv = lambdaGInv;
	kfacInfo->vec = vector;
	kfacInfo->nGradient = naturalGradient;
	kfacInfo->gradient = gradient;
	kfacInfo->dampedInput = dampedInput;
	kfacInfo->dampedZ = dampedZ;
	kfacInfo->dampedLambda = dampedLambda;

	generateParamReport(model, kfacInfo, trParams);
	/* As in the reference, every call allocates its sampling buffers and leaves them to the caller, who frees
	 * data->sampledTrainX / sampledTrainY with cuda_free when done with the data set (a caller that runs the solver
	 * again on the same struct frees them in between). */
	fprintf(stderr, "Allocating Sampling Dataset... %d\n", model->batchSize);
	allocSampledDataset(data, 2 * model->batchSize);

	scratch->nextDevPtr = scratchBegin;
	scratch->nextHostPtr = nextHostPtr;
	scratch->nextPageLckPtr = nextPageLckPtr;

	const long deltaReals = round_up(max_l(model->maxDeltaSize, classes * batch));
	unsigned int miniBatchNo = 0;
	g_report_count = 0;
	cuda_memset(prevWeights, 0, sizeof(real) * (size_t)components, -1);
	initBatchNormData(model, z, model->zOffsets);

	for (int iter = 0; iter < trParams->maxIters; iter++) {
		unsigned int offset = 0, curBatchSize = (unsigned int)model->batchSize;
		double sumInverses = 0, sumGrad = 0, sumHessVec = 0, sumAugment = 0, sumNGrad = 0, sumAccuracy = 0, sumRandom = 0;
		double KFACDistTotal = 0, loopTotal = 0, loopSecondTotal = 0;
		int batches = 0, rejected = 0;
		real trainingLikelihood = 0, trainingAccuracy = 0, testLikelihood = 0, testAccuracy = 0, nrmWeights = 0;
		const double start = now_seconds();

		double t0 = now_seconds();
		genRandomVector(hostIndices, data->trainSizeX, data->trainSizeX);
		copy_host_device(hostIndices, shuffleIndices, sizeof(int) * (size_t)data->trainSizeX, cudaMemcpyHostToDevice, -1);
		sumRandom += now_seconds() - t0;

		while (offset < (unsigned int)data->trainSizeX) {
			const double loopSecond = now_seconds();
			/* a last batch that would end exactly at or beyond the end of the set is left out (:310-315) */
			if (offset + model->batchSize < (unsigned int)data->trainSizeX)
				curBatchSize = (unsigned int)model->batchSize;
			else
				break;

			t0 = now_seconds();
			if (hostResident)
				selectHostMatrix(host, data->sampledTrainX, data->sampledTrainY, (int)curBatchSize, hostIndices, (int)offset, NULL);
			else
				selectColumnMatrix(data, (int)curBatchSize, shuffleIndices, (int)offset);
			augmentData(model, data, (int)offset, (int)curBatchSize, scratchBegin, nextHostPtr, 1, datasetType);
			sumAugment += now_seconds() - t0;

			/* loss and gradient (:349-366) */
			t0 = now_seconds();
			scratch->nextDevPtr = scratchBegin;
			trainingLikelihood = cnnForward(model, data, scratch, z, probs, lossFuncErrors, (int)offset, (int)curBatchSize, MODEL_TRAIN);
			real *distErrors_1 = scratchBegin;
			real *distErrors_2 = distErrors_1 + deltaReals;
			real *nextDevPtr = distErrors_2 + deltaReals;
			copy_device(distErrors_1, lossFuncErrors, sizeof(real) * (size_t)(batch * classes), -1);
			cnnBackward(model, data, nextDevPtr, z, gradient, dx, distErrors_1, distErrors_2, (int)offset, (int)curBatchSize, nextHostPtr);
			HIP_CALL(fitre_hip_axpy(components, kfacInfo->regLambda, data->weights, gradient));
			sumGrad += now_seconds() - t0;

			/* backward pass against targets drawn from the prediction: the Fisher statistics (:381-397) */
			t0 = now_seconds();
			real *distributionDX = distErrors_2 + deltaReals;
			real *distTarget = distributionDX + round_up(model->zSize);
			nextDevPtr = distTarget + round_up(batch);
			computeDistributionErrors(probs, distTarget, distErrors_1, (int)curBatchSize, (int)classes, nextDevPtr, nextHostPtr);
			cnnBackward(model, data, nextDevPtr, z, distGradient, distributionDX, distErrors_1, distErrors_2, (int)offset,
			            (int)curBatchSize, nextHostPtr);
			KFACDistTotal += now_seconds() - t0;

			/* factors and their inverses (:401-433) */
			t0 = now_seconds();
			if (dampedInput != NULL && dampedZ != NULL) {
				computeSpeedUpOmegaZ(kfacInfo, model, data, (int)curBatchSize, z, model->zOffsets, dampedInput, dampedZ,
				                     model->zztOffsets, iter + (int)offset);
				computeSpeedUpLambdaDelta(kfacInfo, model, (int)curBatchSize, distributionDX, dampedLambda, model->zOffsets,
				                          model->zztOffsets, iter + (int)offset);
			}
			/* the reference's computeOmegaZ followed by computeLambdaDelta, here as one pass over both sides */
			if (kfacInfo->inverseFreq == 1 || (iter == 0 && miniBatchNo == 0))
				computeOmegaZAndLambdaDelta(kfacInfo, model, data, (int)curBatchSize, NULL, z, distributionDX, NULL, model->zOffsets,
				                            model->zztOffsets, nextDevPtr);
			else if (miniBatchNo % (unsigned int)kfacInfo->inverseFreq == 0)
				computeOmegaZAndLambdaDelta(kfacInfo, model, NULL, (int)curBatchSize, dampedInput, dampedZ, NULL, dampedLambda,
				                            model->zOffsets, model->zztOffsets, nextDevPtr);
			sumInverses += now_seconds() - t0;

			t0 = now_seconds();
			computeNaturalGradient(model, kfacInfo, scratchBegin, nextHostPtr);
			sumNGrad += now_seconds() - t0;

			/* the curvature matrix must be positive semi-definite (:459-465) */
			t0 = now_seconds();
			real assertCondition = 0;
			HIP_CALL(fitre_hip_dot(components, kfacInfo->nGradient, kfacInfo->nGradient, &assertCondition));
			if (assertCondition < 0 || assertCondition != assertCondition) {
				fprintf(stderr, " **** KFAC MATRIX IS NOT PSD.... \n\n\n");
				exit(-1);
			}
			loopTotal += now_seconds() - t0;

			/* model change along the natural gradient, and along the gradient when asked to compare (:481-508) */
			t0 = now_seconds();
			real mErrKfac = computeQuadraticModel(model, data, z, probs, lossFuncErrors, dx, gradient, kfacInfo->nGradient,
			                                      trParams->delta, (int)offset, (int)curBatchSize, kfacInfo->regLambda, scratchBegin,
			                                      nextHostPtr, nextPageLckPtr);
			real mErrGradient = 0;
			if (kfacInfo->checkGrad)
				mErrGradient = computeQuadraticModel(model, data, z, probs, lossFuncErrors, dx, gradient, gradient, trParams->delta,
				                                     (int)offset, (int)curBatchSize, kfacInfo->regLambda, scratchBegin, nextHostPtr,
				                                     nextPageLckPtr);
			sumHessVec += now_seconds() - t0;

			/* step along the better of the two, with momentum (:516-591) */
			real *direction = (!kfacInfo->checkGrad || mErrKfac < mErrGradient) ? kfacInfo->nGradient : gradient;
			real mErr = direction == gradient ? mErrGradient : mErrKfac;
			HIP_CALL(fitre_hip_axpy(components, kfacInfo->momentum, prevWeights, direction));
			HIP_CALL(fitre_hip_axpy(components, (real)-1., direction, data->weights));
			copy_device(prevWeights, direction, sizeof(real) * (size_t)components, -1);

			t0 = now_seconds();
			scratch->nextDevPtr = scratchBegin;
			real newTrainingLikelihood =
			    evaluateCNNModel(model, data, scratch, z, probs, lossFuncErrors, (int)offset, (int)curBatchSize);
			computeAccuracy(probs, data->sampledTrainY, (int)curBatchSize, (int)classes, scratchBegin, nextPageLckPtr);
			sumAccuracy += now_seconds() - t0;
			real rho = (newTrainingLikelihood - trainingLikelihood) / (mErr - (real)1e-16);

			/* radius update and acceptance (:595-611) */
			if (rho > 0.75) trParams->delta = fminf(trParams->maxDelta, (real)2. * trParams->delta);
			if (rho < 0.25) trParams->delta = fmaxf(trParams->minDelta, (real)0.5 * trParams->delta);
			if (rho < 1e-4 || newTrainingLikelihood > (real)10. * trainingLikelihood || rho != rho) {
				HIP_CALL(fitre_hip_axpy(components, (real)1., prevWeights, data->weights));
				rejected++;
			}

			offset += curBatchSize;
			miniBatchNo++;
			batches++;
			loopSecondTotal += now_seconds() - loopSecond;
		}
		const double total = now_seconds() - start;

		/* whole-set statistics (:637-653) */
		scratch->nextDevPtr = scratchBegin;
		computeTestGeneralizationErrors(model, data, scratch, z, probs, lossFuncErrors, &testLikelihood, &testAccuracy);
		computeTrainGeneralizationErrors(model, data, host, scratch, z, probs, lossFuncErrors, &trainingLikelihood, &trainingAccuracy);
		HIP_CALL(fitre_hip_nrm2(components, data->weights, &nrmWeights));

		fprintf(stderr,
		        " Iteration: %d\t, TrainLikelihood: %f\t, TrainAccuracy: %3.2f\t, TestLikelihood: %f\t, TestAccuracy: %3.2f\t, "
		        "Weight: %e\t, IterTime: %6.3f\t, ZZTTime: %6.3f\t, InverseTime: %6.3f\t, GradTime: %6.3f\t, HvTime: %6.3f\t, "
		        "KFACDistPass: %6.3f\t, Augmentation: %6.3f\t, NatGrad: %6.3f\t, AccuracyTime: %6.3f\t, Random: %6.3f\t, "
		        "Loop Variant: %6.3f, second: %6.3f, TR Radius: %f \n\n",
		        iter, trainingLikelihood, trainingAccuracy, testLikelihood, testAccuracy, nrmWeights, total, sumInverses, sumInverses,
		        sumGrad, sumHessVec, KFACDistTotal, sumAugment, sumNGrad, sumAccuracy, sumRandom, loopTotal, loopSecondTotal,
		        trParams->delta);

		if (g_report_count < MAX_REPORTS) {
			KFAC_TR_EPOCH_REPORT *r = &g_reports[g_report_count];
			r->iteration = iter;
			r->miniBatches = batches;
			r->rejectedSteps = rejected;
			r->trainLikelihood = trainingLikelihood;
			r->trainAccuracy = trainingAccuracy;
			r->testLikelihood = testLikelihood;
			r->testAccuracy = testAccuracy;
			r->weightNorm = nrmWeights;
			r->delta = trParams->delta;
			r->seconds = (real)total;
		}
		g_report_count++;
	}
	if (g_report_count > MAX_REPORTS) g_report_count = MAX_REPORTS;
	scratch->nextDevPtr = entryDevPtr;
	scratch->nextHostPtr = entryHostPtr;
	scratch->nextPageLckPtr = entryPageLckPtr;
}
