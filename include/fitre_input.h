/*
 * fitre_input.h -- mini-batch selection and augmentation with the reference's names
 * (utilities/sample_matrix.h, solvers/kfac_da.h, augmentation/dev_crop.h, dev_flip.h, dev_normalize.h).
 *
 * Images are [channels][samples][width][height] with height fastest, pixel values 0..255 before
 * normalisation.  Random numbers come from getRandomVector (the seeded stream of fitre_hip_random_seed),
 * drawn in the reference's order, so a seed fixes the augmented batch.
 */
#ifndef FITRE_INPUT_H
#define FITRE_INPUT_H

#include "fitre_types.h"
#include "fitre_nn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* utilities/sample_matrix.cu:69-92: columns indices[offset .. offset+sampleSize) of trainSetX (features
 * values each) and of trainSetY into sampledTrainX / sampledTrainY.  indices is a DEVICE array. */
void selectColumnMatrix(DEVICE_DATASET *data, int sampleSize, int *indices, int offset);

/* utilities/dataset_utils.c:10-25: the same selection from a training set kept in HOST memory: images
 * indices[offset .. offset+numSamples) of host->trainSetX and their labels into the device buffers trainX,
 * trainY.  indices is a HOST array.  The rows are gathered in a host staging buffer and
 * sent as one copy (the reference sends one copy per image); hostPtr, if not NULL, receives the labels too. */
void selectHostMatrix(HOST_DATASET *host, real *trainX, real *trainY, int numSamples, int *indices, int offset, real *hostPtr);

/* augmentation/dev_crop.cu:60-94: every image shifted by a random (row, column) offset in
 * [-padding, padding], cells from outside read defaultValue.  devPtr: 2*samples reals and as many ints
 * of device scratch; probs and hostPtr are unused, as in the reference. */
void randomCrop(real *input, int samples, int height, int width, int channels, int padding, real *output,
                real *devPtr, real *hostPtr, real defaultValue, real *probs);
/* augmentation/dev_flip.cu:106-117: images with probs[n] < 0.5 mirrored along the width axis */
void flipData(real *input, real *output, int samples, int channels, int height, int width, real *probs,
              real *devPtr, real *hostPtr);
/* augmentation/dev_normalize.cu:51-100: x = (x / 255 - mean[c]) / std[c] in place, with the statistics of
 * the data set (three channels) */
void normalizeCIFAR10(real *input, int samples, int channels, int height, int width, real *devPtr, real *hostPtr,
                      DATASET_TYPE datasetType);

/* solvers/kfac_da.cu:22-89: data->sampledTrainX ([samples][channels][cells]) -> data->currentBatch
 * ([channels][samples][cells], behind the sampled batch in the same buffer, as in the reference); with
 * enableDA >= 1 cropped by up to 4 cells and flipped; normalised.  One pass over the batch.
 * devPtr: 3*currentBatchSize reals of device scratch. */
void augmentData(CNN_MODEL *model, DEVICE_DATASET *data, int offset, int currentBatchSize, real *devPtr, real *hostPtr,
                 int enableDA, DATASET_TYPE datasetType);

/* functions/cnn_accuracy.cu:61-174: mean negative log-likelihood and accuracy (percent) over the whole test
 * resp. training set, in batches of model->batchSize through augmentData (no augmentation) and cnnForward.
 * The sets are device-resident (datasetType IMAGENET: the training set is read from `host`), features x size column-major; pixel values 0..255; data->sampledTrainX must
 * hold two batches (augmentData writes the second), scratch->nextDevPtr cnnForwardMemRequired reals,
 * scratch->nextPageLckPtr one real of host memory.  Batch-norm layers use their running statistics. */
void computeTestGeneralizationErrors(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs,
                                     real *errors, real *likelihood, real *accuracy);
void computeTrainGeneralizationErrors(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, SCRATCH_AREA *scratch,
                                      real *z, real *probs, real *errors, real *likelihood, real *accuracy);

#ifdef __cplusplus
}
#endif
#endif
