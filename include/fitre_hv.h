/*
 * Hessian-vector product of the CNN loss by R-operator passes, and the quadratic-model step the
 * trust-region solver takes from it: functions/cnn_hessian_vec.h:9-13 and
 * functions/model_reduction.h:9-12 of the reference, same names, argument order and meaning.
 */
#ifndef FITRE_HV_H
#define FITRE_HV_H

#include "fitre_cnn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Reals of device scratch cnnHv carves from devPtr (R{z}, R{errors}, the delta buffers and the
 * workspaces of both R passes; the reference sizes this with zSize + maxDeltaSize +
 * cnnROpForwardMemRequired + cnnROpBackwardMemRequired). */
long cnnHvMemRequired(CNN_MODEL *model);

/* hv = H * vector, H the Hessian of the mean loss of the current batch at data->weights.
 * z, probs, lossFuncErrors and dx must come from computeCNNGradient on the same batch (z: activations,
 * dx: the gradient snapshots).  No weight-decay term is added (weightDecay is unused here, as in the
 * reference, whose computeQuadraticModel adds it).  s and hostPtr are unused.
 * functions/cnn_hessian_vec.cu:18-122 with cnn_hv_forward.cu:53-222 and cnn_hv_backward.cu:70-912. */
void cnnHv(CNN_MODEL *model, DEVICE_DATASET *data, real *z, real *probs, real *lossFuncErrors, real *dx, real *vector,
           real *hv, int s, int curBatchSize, real *devPtr, real *hostPtr, real weightDecay);

/* functions/model_reduction.cu:20-93: hv = H*vector + weightDecay*weights (in devPtr), vHv, and the step
 * along `vector` inside the trust region of radius delta: negative curvature -> to the boundary,
 * else min(g'v / (vHv + 1e-6), delta / |v|).  Scales `vector` by the step and returns the model
 * change 0.5 vHv step^2 - g'v step.  devPtr: pSize + cnnHvMemRequired(model) reals; pageLckPtr: three
 * host reals (g'v, vHv, |v|). */
real computeQuadraticModel(CNN_MODEL *model, DEVICE_DATASET *data, real *z, real *probs, real *lossFuncErrors, real *dx,
                           real *gradient, real *vector, real delta, int offset, int curBatchSize, real weightDecay,
                           real *devPtr, real *hostPtr, real *pageLckPtr);

#ifdef __cplusplus
}
#endif
#endif
