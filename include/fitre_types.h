/*
 * fitre_types.h -- scalar type, status codes and the workspace / dataset
 * records that cross the C boundary of the MI355X CNN gradient path.
 *
 * The records keep the field names and field order of the reference trainer
 * so that its solver sources compile against this header unchanged:
 *   real                      core/datadefs.h:5   (reference: double; this build: float)
 *   status codes              core/errors.h:4-20
 *   SCRATCH_AREA              core/structdefs.h:25-33
 *   HOST_DATASET              core/structdefs.h:35-53
 *   DEVICE_DATASET            core/structdefs.h:55-83
 *   SparseDataset             core/sparsedefs.h:18-29 (the vendor sparse-matrix
 *                             descriptor becomes an opaque pointer)
 */
#ifndef FITRE_TYPES_H
#define FITRE_TYPES_H

#include <stddef.h>

/* All tensors on the gradient path are IEEE binary32.  The oracle alone is
 * built a second time with -DFITRE_REAL_DOUBLE. */
#ifdef FITRE_REAL_DOUBLE
#define real double
#else
#define real float
#endif

/* Exit codes used when a device-shim call fails (process exits with the code,
 * as the reference's device/cuda_utils.c:8-12 does). */
#define ERROR_MEM_ALLOC             0x01
#define ERROR_MEM_CLEANUP           0x02
#define ERROR_MEMCPY_DEVICE_HOST    0x03
#define ERR_MEM_ALLOC               0x04
#define ERR_MEM_FREE                0x05
#define ERROR_MEMCPY_TRAINSETX      0x06
#define ERROR_MEMCPY_TESTSETX       0x07
#define ERROR_MEMCPY_TRAINSETY      0x08
#define ERROR_MEMCPY_TESTSETY       0x09
#define ERROR_DEBUG                 0x10
#define ERROR_MEMSET                0x11
#define ERROR_MEMCPY_DEVICE_DEVICE  0x13
#define ERROR_MEMCPY_HOST_DEVICE    0x14

/* Arena sizes.  The reference grabs 12 GiB of host memory at start-up
 * (core/memsizes.h:6); here the host arena size is a run-time argument of
 * fitre_env_init and these are only the defaults. */
#define FITRE_DEFAULT_HOST_WORKSPACE   ((size_t)1 << 28)
#define PAGE_LOCKED_WORKSPACE_SIZE     ((size_t)1 << 20)

typedef enum data_type { TEST_DATA = 0, TRAIN_DATA = 1 } DATA_TYPE;

typedef enum DATASET_SIZE { FULL_DATASET = 0, SAMPLED_DATASET = 1 } DATASET_SIZE;

typedef enum dataset_type { CIFAR10 = 10, CIFAR100 = 20, IMAGENET = 30 } DATASET_TYPE;

/* Bump-allocated arenas.  A callee may carve buffers from next*Ptr but must
 * put the three cursors back before it returns. */
typedef struct scratch_space {
	real *hostWorkspace;
	real *devWorkspace;
	real *pageLckWorkspace;

	real *nextDevPtr;
	real *nextHostPtr;
	real *nextPageLckPtr;
} SCRATCH_AREA;

typedef struct host_dataset {
	real *trainSetX;
	real *trainSetY;
	real *testSetX;
	real *testSetY;

	int trainSizeX;
	int trainSizeY;
	int testSizeX;
	int testSizeY;

	int features;
	int height;
	int width;
	int numClasses;
	DATASET_TYPE datasetType;
} HOST_DATASET;

/* CSR sampling matrix of the data pipeline; not touched by the gradient path
 * but part of DEVICE_DATASET, so its size must match. */
typedef struct spData {
	int *rowPtr, *colPtr, *rowCsrPtr;
	real *valPtr;
	int nnz;
	real *sortedVals;
	int *P;
	void *descr;
} SparseDataset;

/* Device-resident data.  The gradient path reads: weights (flat parameter
 * vector), currentBatch (layer-0 input, [C][N][W][H]), sampledTrainY (labels,
 * 1-based class ids stored as real), numClasses, features. */
typedef struct dev_dataset {
	real *trainSetX;
	real *trainSetY;
	real *testSetX;
	real *testSetY;

	real *weights;

	int numClasses;
	DATASET_TYPE datasetType;

	int features;
	int height;
	int width;
	int testSizeX;
	int testSizeY;
	int trainSizeX;
	int trainSizeY;

	int sampleSize;
	real *sampledTrainX;
	real *sampledTrainY;
	real *currentBatch;

	SparseDataset spSamplingMatrix;
} DEVICE_DATASET;

#endif
