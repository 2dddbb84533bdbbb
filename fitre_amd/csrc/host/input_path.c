/* Mini-batch selection and augmentation with the reference's names (utilities/sample_matrix.cu,
 * solvers/kfac_da.cu, augmentation/dev_crop.cu, dev_flip.cu, dev_normalize.cu) over the device layer. */
#include <stdio.h>
#include <string.h>
#include <stdlib.h>

#include "fitre_cnn.h"
#include "fitre_hip.h"
#include "fitre_input.h"
#include "fitre_shim.h"

#define HIP_CALL(expr)                                                                       \
	do {                                                                                     \
		int rc_ = (expr);                                                                    \
		if (rc_ != 0) {                                                                      \
			fprintf(stderr, "%s:%d: %s\n  %s\n", __FILE__, __LINE__, #expr, fitre_hip_last_error()); \
			exit(-1);                                                                        \
		}                                                                                    \
	} while (0)

/* augmentation/dev_normalize.cu:55-62 */
static void dataset_statistics(DATASET_TYPE datasetType, const real **mean, const real **std)
{
	static const real mean_cifar10[3] = { 0.4914f, 0.4822f, 0.4465f }, std_cifar10[3] = { 0.2470f, 0.2435f, 0.2616f };
	static const real mean_cifar100[3] = { 0.5071f, 0.4865f, 0.4409f }, std_cifar100[3] = { 0.2673f, 0.2564f, 0.2762f };
	static const real mean_imagenet[3] = { 0.4799f, 0.4478f, 0.3972f }, std_imagenet[3] = { 0.2769f, 0.2690f, 0.2820f };
	switch (datasetType) {
	case CIFAR10: *mean = mean_cifar10, *std = std_cifar10; break;
	case CIFAR100: *mean = mean_cifar100, *std = std_cifar100; break;
	case IMAGENET: *mean = mean_imagenet, *std = std_imagenet; break;
	default: fprintf(stderr, "Unknown DatasetType here... \n\n"); exit(-1);
	}
}

static void need_three_channels(const char *fn, int channels)
{
	if (channels != 3) {
		fprintf(stderr, "%s: the data-set statistics cover 3 channels, the images have %d\n", fn, channels);
		exit(-1);
	}
}

void selectColumnMatrix(DEVICE_DATASET *data, int sampleSize, int *indices, int offset)
{
	HIP_CALL(fitre_hip_extract_columns(data->sampledTrainX, data->trainSetX, indices + offset, data->features, sampleSize));
	HIP_CALL(fitre_hip_extract_columns(data->sampledTrainY, data->trainSetY, indices + offset, 1, sampleSize));
	HIP_CALL(fitre_hip_sync());
}

void randomCrop(real *input, int samples, int height, int width, int channels, int padding, real *output, real *devPtr,
                real *hostPtr, real defaultValue, real *probs)
{
	(void)hostPtr;
	(void)probs;
	getRandomVector(2 * samples, NULL, devPtr, RAND_UNIFORM);
	HIP_CALL(fitre_hip_augment_batch(input, 0, samples, channels, height, width, devPtr, padding, defaultValue, NULL, NULL, NULL,
	                                 1.f, output));
	HIP_CALL(fitre_hip_sync());
}

void flipData(real *input, real *output, int samples, int channels, int height, int width, real *probs, real *devPtr,
              real *hostPtr)
{
	(void)devPtr;
	(void)hostPtr;
	HIP_CALL(fitre_hip_augment_batch(input, 0, samples, channels, height, width, NULL, 0, 0.f, probs, NULL, NULL, 1.f, output));
	HIP_CALL(fitre_hip_sync());
}

void normalizeCIFAR10(real *input, int samples, int channels, int height, int width, real *devPtr, real *hostPtr,
                      DATASET_TYPE datasetType)
{
	(void)devPtr;
	(void)hostPtr;
	const real *mean, *std;
	dataset_statistics(datasetType, &mean, &std);
	need_three_channels("normalizeCIFAR10", channels);
	HIP_CALL(fitre_hip_augment_batch(input, 0, samples, channels, height, width, NULL, 0, 0.f, NULL, mean, std, 255.f, input));
	HIP_CALL(fitre_hip_sync());
}

void augmentData(CNN_MODEL *model, DEVICE_DATASET *data, int offset, int currentBatchSize, real *devPtr, real *hostPtr,
                 int enableDA, DATASET_TYPE datasetType)
{
	(void)offset;
	(void)hostPtr;
	const CONV_LAYER *c = &model->convLayer[0];
	const int channels = c->inChannels, height = c->height, width = c->width, samples = currentBatchSize;
	real *first = data->sampledTrainX;
	real *second = first + (size_t)samples * channels * height * width;
	const real *mean, *std;
	dataset_statistics(datasetType, &mean, &std);
	need_three_channels("augmentData", channels);

	const real *cropUniforms = NULL, *flipUniforms = NULL;
	if (enableDA >= 1) {
		/* the draws of the reference, in its order: one vector it never reads, the crop offsets, the flips */
		getRandomVector(samples, NULL, devPtr, RAND_UNIFORM);
		getRandomVector(2 * samples, NULL, devPtr + samples, RAND_UNIFORM);
		getRandomVector(samples, NULL, devPtr, RAND_UNIFORM);
		cropUniforms = devPtr + samples;
		flipUniforms = devPtr;
	}
	HIP_CALL(fitre_hip_augment_batch(first, 1, samples, channels, height, width, cropUniforms, 4, 0.f, flipUniforms, mean, std,
	                                 255.f, second));
	HIP_CALL(fitre_hip_sync());
	data->currentBatch = second;
}

/* rows indices[offset + i] (indices == NULL: offset + i) of the host set, gathered in a staging buffer and sent
 * as one copy each for images and labels */
static void select_host_rows(HOST_DATASET *host, real *trainX, real *trainY, int numSamples, const int *indices, int offset,
                             real *labelsOut)
{
	const size_t features = (size_t)host->features;
	real *stage = (real *)malloc((size_t)(numSamples > 0 ? numSamples : 1) * (features + 1) * sizeof(real));
	if (stage == NULL) {
		fprintf(stderr, "selectHostMatrix: no host memory for %d images of %zu values\n", numSamples, features);
		exit(-1);
	}
	real *labels = stage + (size_t)numSamples * features;
	for (int i = 0; i < numSamples; i++) {
		const int row = indices != NULL ? indices[offset + i] : offset + i;
		if (row < 0 || row >= host->trainSizeX) {
			fprintf(stderr, "selectHostMatrix: index %d outside the training set of %d images\n", row, host->trainSizeX);
			exit(-1);
		}
		memcpy(stage + (size_t)i * features, host->trainSetX + (size_t)row * features, features * sizeof(real));
		labels[i] = host->trainSetY[row];
		if (labelsOut != NULL) labelsOut[i] = labels[i];
	}
	HIP_CALL(fitre_hip_copy_h2d(trainX, stage, (size_t)numSamples * features * sizeof(real)));
	HIP_CALL(fitre_hip_copy_h2d(trainY, labels, (size_t)numSamples * sizeof(real)));
	free(stage);
}

void selectHostMatrix(HOST_DATASET *host, real *trainX, real *trainY, int numSamples, int *indices, int offset, real *hostPtr)
{
	select_host_rows(host, trainX, trainY, numSamples, indices, offset, hostPtr);
}

/* One evaluation sweep in batches of model->batchSize (the last one shorter): copy the batch's columns
 * and labels, layout change + normalisation (no augmentation), forward pass, accuracy.
 * functions/cnn_accuracy.cu:61-110 (test set) and :112-174 (training set; the reference's sweep stops
 * before a final short batch yet divides by the full size, and so does this one). */
static void generalization_sweep(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs,
                                 real *errors, const real *setX, const real *setY, HOST_DATASET *hostSet, int setSize,
                                 EVAL_TYPE mode, int dropShortTail, real *likelihood, real *accuracy)
{
	real hits = 0;
	int curIdx = 0, curBatchSize = model->batchSize;
	real *nextDevPtr = scratch->nextDevPtr, *nextHostPtr = scratch->nextHostPtr, *nextPageLckPtr = scratch->nextPageLckPtr;
	*likelihood = 0;
	*accuracy = 0;
	if (curBatchSize > setSize) curBatchSize = setSize;
	while (curIdx < setSize && curBatchSize > 0) {
		if (hostSet != NULL) {
			select_host_rows(hostSet, data->sampledTrainX, data->sampledTrainY, curBatchSize, NULL, curIdx, NULL);
		} else {
			HIP_CALL(fitre_hip_copy_d2d(data->sampledTrainX, setX + (size_t)data->features * curIdx,
			                            sizeof(real) * (size_t)data->features * curBatchSize));
			HIP_CALL(fitre_hip_copy_d2d(data->sampledTrainY, setY + curIdx, sizeof(real) * (size_t)curBatchSize));
		}
		augmentData(model, data, curIdx, curBatchSize, nextDevPtr, nextHostPtr, 0, data->datasetType);
		real batchLikelihood = cnnForward(model, data, scratch, z, probs, errors, curIdx, curBatchSize, mode);
		*likelihood += batchLikelihood * curBatchSize;
		computeAccuracy(probs, hostSet != NULL ? data->sampledTrainY : (real *)(setY + curIdx), curBatchSize, data->numClasses,
		                nextDevPtr, nextPageLckPtr);
		hits += *nextPageLckPtr;
		curIdx += curBatchSize;
		if (curIdx + model->batchSize < setSize) {
			curBatchSize = model->batchSize;
		} else {
			curBatchSize = setSize - curIdx;
			if (dropShortTail) break;
		}
	}
	*accuracy = hits * (real)100. / (real)setSize;
	*likelihood /= (real)setSize;
}

void computeTestGeneralizationErrors(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs,
                                     real *errors, real *likelihood, real *accuracy)
{
	generalization_sweep(model, data, scratch, z, probs, errors, data->testSetX, data->testSetY, NULL, data->testSizeX,
	                     MODEL_TEST_ACCURACY, 0, likelihood, accuracy);
}

void computeTrainGeneralizationErrors(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, SCRATCH_AREA *scratch, real *z,
                                      real *probs, real *errors, real *likelihood, real *accuracy)
{
	/* a training set kept in host memory (the reference's IMAGENET case, functions/cnn_accuracy.cu:136-143)
	 * is read through the host struct, batch by batch */
	HOST_DATASET *hostSet = NULL;
	if (data->datasetType == IMAGENET) {
		if (host == NULL || host->trainSetX == NULL || host->trainSetY == NULL) {
			fprintf(stderr, "computeTrainGeneralizationErrors: the training set is neither on the device nor on the host\n");
			exit(-1);
		}
		hostSet = host;
	}
	generalization_sweep(model, data, scratch, z, probs, errors, data->trainSetX, data->trainSetY, hostSet, data->trainSizeX,
	                     MODEL_TRAIN_ACCURACY, 1, likelihood, accuracy);
}
