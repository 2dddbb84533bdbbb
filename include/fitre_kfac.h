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

/* inverse = (matrix + (lambda + dampGamma) I)^-1, order n, both dense n x n
 * (solvers/kfac_inverses.cu:133-186, computeMatrixInverseCusolver without the cuSOLVER handles).  As in the
 * reference the arithmetic is double: the matrix is widened, factored and inverted in float64, and the inverse
 * rounded to reals.  devPtr: matrixInverseMemRequired(n) reals of scratch.  Exits with the reference's message
 * when the matrix is not positive definite. */
void computeMatrixInverse(real *matrix, real *inverse, int n, real *devPtr, real lambda, real dampGamma);
long matrixInverseMemRequired(int n);

/* Scratch (in reals) computeOmegaZ / computeLambdaDelta may carve from devPtr: four lanes, each with the largest
 * factor in doubles plus the workspaces of its product and of its inverse. */
long kfacInverseMemRequired(CNN_MODEL *model, int samples);

/* solvers/kfac_inverses.cu:450-630 and :759-857 in full: every layer's factor (built in scratch, as in
 * the reference) and its damped inverse, stored at omegaZInv + OmegaZOffsets[l] resp.
 * lambdaGInv + LambdaGOffsets[l].  Damping: kfac_info->regLambda + kfac_info->dampGamma on the diagonal.
 * pageLckPtr is unused (the reference reads cuSOLVER's devInfo through it).
 * Precision: the reference does this leg in double.  Here reals are floats, and the factors of a network with a small
 * damping are too ill-conditioned for float arithmetic (condition 1e4 .. 1e6 at lambda = 1e-3), so every factor is
 * accumulated, factored and inverted in float64 on the device and the inverse is stored in the caller's n x n reals
 * as a PAIR of floats per element: the inverse rounded to float on and above the diagonal, the rounding remainder
 * below it (FITRE_MAT_SYM_PAIR, fitre_hip.h).  The upper triangle alone is the float inverse; computeNaturalGradient,
 * the only reader of these arrays in the reference (solvers/kfac_natural_gradient.cu:55-56), takes the pairs.
 * An input-side factor with few positions behind it (2 * positions <= order, positions = samples * outH * outW of a
 * convolution layer resp. samples of a linear layer: VGG-11's layers on 2x2 maps at batch 256, its linear layer) is
 * not inverted at its own order: with A = alpha R R' (R: order x positions),
 *     (A + s I)^-1 = (I - alpha R S^-1 R') / s,   S = s I + alpha R' R   (order = positions),
 * and the slot holds, in its n x n words: word 0 = 0xF15EED12 (as a float a negative number, which no diagonal entry
 * of a positive definite inverse is), word 1 = positions, word 2 = order, words 3, 4 = row / column stride of R in
 * words, words 5-6 = alpha and 7-8 = s as doubles, word 9 = the word offset of S^-1; R as floats from word 64 on;
 * S^-1 (positions x positions doubles) at that offset.  computeNaturalGradient reads either form. */
/* The three trailing arguments are the reference's vendor handles (cublasHandle_t, cudaStream_t,
 * cusolverDnHandle_t, solvers/kfac_inverses.h:28-34), kept so that its solver source compiles against this
 * header unchanged; they are opaque pointers and are ignored (the device layer owns its streams). */
#ifndef FITRE_VENDOR_HANDLES_DEFINED /* define it before this header where another header already declares the three names */
#define FITRE_VENDOR_HANDLES_DEFINED
typedef void *cublasHandle_t;
typedef void *cudaStream_t;
typedef void *cusolverDnHandle_t;
#endif
void computeOmegaZ(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                   real *dampedInput, real *dampedZ, real *omegaZInv, int *zOffsets, int *zztOffsets, real *devPtr,
                   real *pageLckPtr, cublasHandle_t blasHandle, cudaStream_t curStream, cusolverDnHandle_t curHandle);
void computeLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx, real *dampedLambda,
                        real *lambdaGInv, int *zOffsets, int *zztOffsets, real *devPtr, real *pageLckPtr,
                        cublasHandle_t blasHandle, cudaStream_t curStream, cusolverDnHandle_t curHandle);

/* Both passes as one (no counterpart in the reference, whose solver calls them one after the other): the small
 * output-side inverses run on the lanes that the large input-side ones leave idle.  Same results, written to
 * kfac_info->OmegaZInv and kfac_info->LambdaGInv; devPtr as for the single passes. */
void computeOmegaZAndLambdaDelta(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                                 real *dampedInput, real *dampedZ, real *dx, real *dampedLambda, int *zOffsets,
                                 int *zztOffsets, real *devPtr);

/* Scratch (in reals) of computeNaturalGradient. */
long kfacNaturalGradientMemRequired(CNN_MODEL *model);
/* solvers/kfac_natural_gradient.cu:36-241: per layer nGradient = Lambda^-1 * gradient * Omega^-1 with the
 * layer's gradient seen as a Cout x (K + bias) matrix (convolution) resp. out x (in + bias) (linear);
 * reads kfacInfo->gradient, OmegaZInv, LambdaGInv, writes kfacInfo->nGradient in the flat parameter
 * layout.  hostPtr is unused. */
void computeNaturalGradient(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo, real *devPtr, real *hostPtr);

#ifdef __cplusplus
}
#endif
#endif
