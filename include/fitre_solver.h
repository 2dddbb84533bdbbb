/*
 * fitre_solver.h -- the sub-sampled KFAC trust-region solver's host loop with the reference's
 * names (solvers/kfac_trust_region.h:11-13, solvers/params.h:12-35, solvers/kfac_inverses.h,
 * utilities/alloc_sampled_dataset.h, device/gen_random.h:15).
 *
 * The loop is host code over the entry points of fitre_input.h, fitre_cnn.h, fitre_kfac.h and
 * fitre_hv.h: per mini-batch it selects and augments the batch, runs forward and backward, a second
 * backward against targets sampled from the model's own prediction (the Fisher statistics), both
 * factor/inverse passes, the natural gradient, the quadratic model along it, the step, and the
 * trust-region update.  One device; the reference's second-device inverse worker (master / slave)
 * is not part of it and both arguments are ignored.
 */
#ifndef FITRE_SOLVER_H
#define FITRE_SOLVER_H

#include "fitre_types.h"
#include "fitre_nn.h"
#include "fitre_kfac.h"

#ifdef __cplusplus
extern "C" {
#endif

/* solvers/params.h:7-10 */
typedef enum hessian_type { TRUE_HESSIAN = 0, GAUSS_NEWTON } HESSIAN_TYPE;

/* solvers/params.h:12-35 (field order and types as there) */
typedef struct trust_region_params {
	real delta;
	real minDelta;
	real maxDelta;
	real eta1;
	real eta2;
	real gamma1;
	real gamma2;
	unsigned long int maxProps;
	int maxMatVecs;
	int maxEpochs;
	int maxIters;
	int hessianType;
	real alpha;
	int curIteration;
	real hs;
	real lambda;
} TRUST_REGION_PARAMS;

/* device/gen_random.cu:76-98: m distinct indices out of 0..n-1 in random order (selection sampling,
 * then a Fisher-Yates shuffle), drawn with the C library's rand(): srand() fixes the sequence. */
void genRandomVector(int *idx, int m, int n);

/* utilities/alloc_sampled_dataset.cu:9-19: device buffers for sampleSize images and labels */
void allocSampledDataset(DEVICE_DATASET *data, int sampleSize);

/* solvers/kfac_trust_region.cu:64-75: running mean 0, running variance 1 in every batch-norm layer */
void initBatchNormData(CNN_MODEL *model, real *z, int *zOffsets);

/* solvers/kfac_inverses.cu:106-124: src = momentum*src + (1-momentum)*update, in the reference's three
 * steps (scale, add, scale); momentum == 0 copies */
void updateRunningStats(real *src, real *update, int numElements, real momentum);

/* solvers/kfac_inverses.cu:386-446 and :699-755: running averages (decay sqrt(stats_decay)) of the layer
 * inputs resp. of the sampled-target deltas, packed at zztOffsets; iterCount == 0 starts them with a copy */
void computeSpeedUpOmegaZ(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples, real *z,
                          int *zOffsets, real *dampedInput, real *dampedZ, int *zztOffsets, int iterCount);
void computeSpeedUpLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx, real *dampedLambda,
                               int *zOffsets, int *zztOffsets, int iterCount);

/* Reals of device arena (scratch->nextDevPtr), host arena (scratch->nextHostPtr) and page-locked arena
 * (scratch->nextPageLckPtr) the solver carves; kfacInfo->inverseFreq must be set.  No counterpart in the
 * reference, which takes all free device memory. */
long kfacTrustRegionMemRequired(CNN_MODEL *model, DEVICE_DATASET *data, KFAC_CURVATURE_INFO *kfacInfo);
long kfacTrustRegionHostMemRequired(DEVICE_DATASET *data);
#define KFAC_TR_PAGE_LOCKED_REALS 8

/* What one pass over the training set left behind (the reference prints these to stderr and keeps
 * nothing; the line is printed here too). */
typedef struct kfac_tr_epoch_report {
	int iteration;
	int miniBatches;
	int rejectedSteps;
	real trainLikelihood;
	real trainAccuracy;
	real testLikelihood;
	real testAccuracy;
	real weightNorm;
	real delta;
	real seconds;
} KFAC_TR_EPOCH_REPORT;
/* Copies up to `capacity` reports of the last subsampledTrustRegionKFAC call; returns how many epochs it ran
 * (no counterpart in the reference). */
int kfacTrustRegionReports(KFAC_TR_EPOCH_REPORT *out, int capacity);

/* solvers/kfac_trust_region.cu:92-660.  data: trainSetX/Y and testSetX/Y device-resident
 * (features x size, pixel values 0..255, labels 1-based reals), weights the start point (updated in
 * place), datasetType CIFAR10 or CIFAR100.  kfacInfo: regLambda, dampGamma, momentum, stats_decay,
 * checkGrad, inverseFreq (1: factors and inverses from every mini-batch; k > 1: from running averages,
 * every k-th mini-batch).  trParams: delta (updated), minDelta, maxDelta, maxIters = passes over the
 * training set.  The sampled-batch buffers are allocated here (allocSampledDataset) and stay with data.
 * scratch->nextDevPtr / nextHostPtr / nextPageLckPtr move while the loop runs and are back at their entry values on
 * return. */
void subsampledTrustRegionKFAC(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, KFAC_CURVATURE_INFO *kfacInfo,
                               TRUST_REGION_PARAMS *trParams, SCRATCH_AREA *scratch, int master, int slave);

#ifdef __cplusplus
}
#endif
#endif
