/*
 * KFAC curvature bookkeeping and the Kronecker-factor stage of the reference's
 * computeOmegaZ / computeLambdaDelta (solvers/kfac_inverses.cu:450-630, 759-857).
 *
 * The reference computes each factor and hands it straight to
 * computeMatrixInverseCusolver; here the factor stage stands alone and writes the
 * factors into caller-owned storage at the offsets of computeKFACStorageIndices, so
 * that an inverse routine can be applied to them afterwards.  Argument meaning
 * follows the reference functions; the cuBLAS / cuSOLVER / stream handles are gone.
 */
#ifndef FITRE_KFAC_H
#define FITRE_KFAC_H

#include "fitre_nn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* solvers/kfac_structs.h:13-52, same fields in the same order */
typedef struct kfac_curvature {
	real *OmegaZZT;
	real *LambdaGGT;
	real *OmegaZInv;
	real *LambdaGInv;
	real *vec;
	real *nGradient;
	real *gradient;
	int OmegaZOffsets[MAX_LAYERS];
	int LambdaGOffsets[MAX_LAYERS];
	real stats_decay;
	real momentum;
	real regLambda;
	real dampGamma;
	int checkGrad;
	int dampedInputSize;
	real *dampedInput;
	real *dampedZ;
	real *dampedLambda;
	int inverseFreq;
} KFAC_CURVATURE_INFO;

/* solvers/kfac_utils.cu:6-54: offsets of the per-layer factors, convolution layers first.
 * Input-side slots always have room for the bias column: (Cin*k*k + 1)^2 resp. (in + 1)^2;
 * output-side slots Cout^2 resp. out^2.  Entry [cLayers + lLayers] is the total. */
void computeKFACStorageIndices(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo);

/* Scratch (in reals) the two factor passes may carve from devPtr. */
long kfacFactorsMemRequired(CNN_MODEL *model, int samples);

/* Input-side factors of every layer (solvers/kfac_inverses.cu:450-630 without the inverses):
 * convolution layer l: P^T P / samples with P = [im2col(input_l)/(outH*outW), 1] (the ones column
 * only when model->bias != 0), order Cin*k*k (+1), stored densely at omegaZZT + OmegaZOffsets[l];
 * linear layer l: [z;1][z;1]^T / samples, order in (+1), at omegaZZT + OmegaZOffsets[cLayers+l].
 * dampedInput == NULL: layer inputs are read from data->currentBatch and from dampedZ (= z of
 * cnnForward) at zOffsets; otherwise from dampedInput / dampedZ at zztOffsets, as in the reference. */
void computeOmegaZFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                          real *dampedInput, real *dampedZ, real *omegaZZT, int *zOffsets, int *zztOffsets,
                          real *devPtr);

/* Output-side factors (solvers/kfac_inverses.cu:759-857 without the inverses): convolution layer l:
 * delta^T delta * (samples*outH*outW) with delta = dx + zOffsets[l+1] + (batchNormOffset if the layer
 * is batch-normalised, else activationOffset), order Cout, at lambdaGGT + LambdaGOffsets[l];
 * linear layer l: delta delta^T * samples with delta = dx + zOffsets[cLayers+l+1], order out.
 * dampedLambda != NULL: deltas are read from dampedLambda + zztOffsets[...] instead. */
void computeLambdaDeltaFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx,
                               real *dampedLambda, real *lambdaGGT, int *zOffsets, int *zztOffsets, real *devPtr);

#ifdef __cplusplus
}
#endif
#endif
