/*
 * fitre_dataset.h -- what stands either side of the trust-region solver in the reference's driver:
 * the binary data-set readers (utilities/dataset.h:8-24, utilities/dataset.c:20-42,122-157,373-571,
 * 606-721), their callers (drivers/dataset_driver.c:58-112), and the driver that reads a start point and
 * runs the solver (drivers/kfac_trust_region_driver.cu:59-108,201-498).
 *
 * Host code only.  Record formats (one record per image, bytes):
 *   dataset 1 (CIFAR-10):        label, 3 x 32 x 32 pixels            3073 per record
 *   dataset 2 (CIFAR-100):       coarse label, fine label, pixels      3074 per record (the fine label is kept)
 *   dataset 3 (Tiny ImageNet):   label, 3 x 64 x 64 pixels            12289 per record
 * Pixels are channel-major, each channel row-major.  In memory every image keeps its channel order and
 * each channel is stored column-major (element (row, col) at col * height + row), pixel values 0..255 as
 * reals, labels 1-based as reals -- the layout selectColumnMatrix and augmentData read.
 */
#ifndef FITRE_DATASET_H
#define FITRE_DATASET_H

#include "fitre_types.h"
#include "fitre_nn.h"
#include "fitre_kfac.h"
#include "fitre_solver.h"

#ifdef __cplusplus
extern "C" {
#endif

/* utilities/dataset.c:20-24: rows x cols row-major -> column-major */
void convertToColumnMajor(real *src, int rows, int cols, real *tgt);

/* utilities/dataset.c:27-42: every channel of every image from row-major to column-major.  The reference
 * derives the column as v % height, which is the transposition only for square images (all it is used on);
 * here the column is v % width, so that non-square images are transposed too. */
void convertCIFARToColumnMajor(real *src, real *tgt, int datasetSize, int channels, int height, int width);

/* utilities/dataset.c:122-157: src = (src / constant - mean[c]) / std[c] over a [channel][image][cell] tensor;
 * datasetType 1, 2, 3 selects the CIFAR-10, CIFAR-100 or ImageNet statistics; anything else exits(-1). */
void imageNormalization(real *src, int numImages, int channels, int height, int width, real constant, int datasetType);

/* utilities/dataset.c:198-240: a text matrix, one row per line, values separated by commas or blanks, into a
 * malloc'ed row-major array; the last line's token count is the column count (as there), an empty line ends the
 * matrix, short rows are padded with zeros.  Lines of any length (the reference stops at 4 MiB). */
void readDelimitedMatrix(char *fileName, real **data, int *rows, int *cols);

/* utilities/dataset.c:373-571.  Reads dir + train + "1.bin" .. dir + train + "<numFiles>.bin" and the test file
 * dir + test (dataset 3: dir + test + "1.bin" and "2.bin") into malloc'ed host arrays of `data`, sets
 * trainSizeX/Y, testSizeX/Y, features and numClasses (10, 100, 200).  A trailing partial record counts as a
 * record padded with zeros, as in the reference.  scratch, raw and batchSize are unused (the reference
 * transposes through the host arena; here each record is transposed as it is read).  A missing file: message
 * on stderr, exit(-1). */
void readCIFARDataset(char *dir, char *train, int numFiles, char *test, HOST_DATASET *data, SCRATCH_AREA *s, int raw,
                      int batchSize, int datasetType, int height, int width);

/* utilities/dataset.c:606-654: sizes into the device struct, the four arrays allocated on the device and
 * copied.  initialize_device_image (:656-706): the same for the test set only; the training set stays on the
 * host (trainSetX / trainSetY = NULL). */
void initialize_device_data(HOST_DATASET *s, DEVICE_DATASET *t);
void initialize_device_image(HOST_DATASET *s, DEVICE_DATASET *t);
/* utilities/dataset.c:709-721 */
void cleanup_dataset(HOST_DATASET *s, DEVICE_DATASET *t);

/* The folders the reference hard-codes (drivers/dataset_driver.c:66,85,104 and
 * drivers/kfac_trust_region_driver.cu:205) stay the defaults; a NULL argument restores the default.  The strings
 * are copied.  datasetType 1, 2, 3.  No counterpart in the reference. */
void fitreSetDatasetFolder(int datasetType, const char *dir);
void fitreSetWeightsFolder(const char *dir);

/* drivers/dataset_driver.c:58-112: 32 x 32 (64 x 64) images, datasetType CIFAR10 / CIFAR100 / IMAGENET on both
 * structs, the reference's file names (data_batch_1..5 + test_batch.bin; train_1 + test.bin; train_1..19 +
 * test_1..2), then the device copy.  Return 0. */
int getCIFAR10(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch);
int getCIFAR100(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch);
int getTinyImageNet(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch);

/* nn/read_nn.c:867-880: the device parameter vector (pSize reals) */
void cnnInitializations(CNN_MODEL *model, DEVICE_DATASET *data);

/* drivers/kfac_trust_region_driver.cu:59-83 and :85-108: the driver's defaults */
void initKFACTrustRegionParams(TRUST_REGION_PARAMS *params, int n);
void initKFACInfo(KFAC_CURVATURE_INFO *kfacInfo);

/* drivers/kfac_trust_region_driver.cu:225-488: <weights folder><cifar10|cifar100|imagenet>/<net>_<init>[_bias].params
 * with net of lenet, alexnet, vgg11, vgg13, vgg16, vgg19 (model->name) and init of default, kaiming, xavier
 * (initialization 0, 1, 2).  Returns 0, or -1 (nothing written) for an unknown dataset, network or initialization or
 * a buffer that is too small; the reference exits there, and so does testKFACTrustRegion. */
int kfacParamsFileName(CNN_MODEL *model, int dataset, int initialization, char *out, int outBytes);

/* drivers/kfac_trust_region_driver.cu:201-498: defaults, the arguments over them, the start point read from the
 * parameter file into data->weights, then subsampledTrustRegionKFAC. */
void testKFACTrustRegion(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, SCRATCH_AREA *scratch, real dampGamma,
                         real trMaxRadius, int checkGrad, int master, int slave, int inverseFreq, int epochs, int dataset,
                         real regLambda, int initialization);

#ifdef __cplusplus
}
#endif
#endif
