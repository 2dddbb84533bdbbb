/*
 * Fully connected model family of the reference (the auto-encoder / classifier networks of its
 * first-order and trust-region solvers): functions/eval_gradient.h:9-25 with the same names,
 * argument order and meaning.  All data pointers are device pointers; results returned through
 * logLikelihood / modelError are host scalars, complete on return.
 *
 * Layout (nn/read_nn.c:779-805): layer i maps layerSizes[i] -> layerSizes[i+1] with weights
 * column-major layerSizes[i+1] x layerSizes[i] at weights + wOffsets[i] and bias at
 * weights + bOffsets[i]; activations z_i (layerSizes[i] x points, column-major, one column per
 * point) at z + zOffsets[i] for i >= 1; back-propagated errors of layer i at dx + rZOffsets[i].
 * The output head is chosen by actFuns[numLayers-1]: ACT_LINEAR (squared error), ACT_LOGISTIC
 * (Bernoulli likelihood of the logits), ACT_SOFTMAX (cross entropy).
 *
 * Where this differs from the reference, on purpose:
 *  - nnForwardPass does not write the copy of W z + b behind each layer's output (the reference's
 *    applyLayerActivation does, eval_gradient.cu:137-138, and for the last layer that copy lies past
 *    zSize); the exported applyLayerActivation still writes it, as the CNN path relies on it;
 *  - a one-layer model takes the data set, not the never-written z slot 0, as input of its weight
 *    gradient (eval_gradient.cu:704);
 *  - the number of output elements is layerSizes[numLayers] x points (the reference multiplies
 *    data->features, the same number for its auto-encoders).
 */
#ifndef FITRE_FC_H
#define FITRE_FC_H

#include "fitre_nn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Fills numLayers, layerSizes, actFuns, type and the weight / z offsets for numPoints columns
 * (the arithmetic of readNeuralNet, nn/read_nn.c:776-805, for any layer list).
 * layerSizes has numLayers + 1 entries, actFuns numLayers. */
void fitre_build_nn(NN_MODEL *model, const int *layerSizes, const int *actFuns, int numLayers, int type, int numPoints);
void initSampledZOffsets(NN_MODEL *model, int numPoints); /* nn/read_nn.c:808-820 */
void initRZOffsets(NN_MODEL *model, int datasetSize);     /* nn/read_nn.c:822-834 */
void initSampledROffsets(NN_MODEL *model, int sampleSize); /* nn/read_nn.c:838-850 */

/* Reals of device scratch nnForwardPass (devPtr) resp. computeGradient / evaluateModel
 * (scratch->nextDevPtr, z and dx not included) may use for `points` columns. */
long nnForwardMemRequired(NN_MODEL *model, int points);
long nnGradientMemRequired(NN_MODEL *model, int points);

/* output = f(W z + b), W wRows x wCols, z zRows x zCols, all column-major; also leaves W z + b at
 * output + wRows*zCols.  scratch and hostPtr are unused.  eval_gradient.cu:29-229. */
void applyLayerActivation(int actFunction, real *W, int wRows, int wCols, real *b, int bRows, real *z, int zRows,
                          int zCols, real *output, real *scratch, real *hostPtr);

/* eval_gradient.cu:275-555: forward pass over the chosen data (TEST_DATA: testSet; TRAIN_DATA with
 * FULL_DATASET: trainSet; with SAMPLED_DATASET: sampledTrainX, which is also the target), fills z and
 * errTerm = scale * (target - output), *logLikelihood = -(1/points) * sum of the head's terms,
 * *modelError = mean squared error per point for MODEL_TYPE_MSE, else 0. */
void nnForwardPass(NN_MODEL *model, DEVICE_DATASET *data, real *weights, real *z, real *errTerm, real *logLikelihood,
                   real *modelError, real *hostPtr, real *devPtr, DATASET_SIZE dSize, DATA_TYPE d);

/* eval_gradient.cu:231-268: forward pass with z and the error term carved from scratch->nextDevPtr. */
void evaluateModel(NN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *w, real *logLikelihood,
                   real *modelError, DATASET_SIZE dSize, DATA_TYPE s);

/* eval_gradient.cu:561-914: forward + backward; gradient[pSize] = d(loss)/d(weights) with the loss
 * averaged over the points, dx = the back-propagated errors per layer.  z == NULL: z and dx are
 * carved from scratch->nextDevPtr as the reference does. */
void computeGradient(NN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *weights, real *z, real *dx,
                     real *gradient, real *ll, real *err, DATASET_SIZE dSize);

/* functions/eval_hessian_vec.h:9-11 and functions/eval_gauss_newton_hessian_vec.h:9-11: the Hessian resp. the
 * Gauss-Newton matrix of the loss computeGradient differentiates, times vec, by the R-operator; z and dx are the
 * ones computeGradient left at the same weights and data (allData selects the full or the sampled set and its
 * offsets).  The product, scaled by -1/n like the gradient, is left in the first pSize reals behind
 * scratch->nextDevPtr, as in the reference; nnHessianVecMemRequired (no counterpart there) is how many reals it
 * uses from that pointer.  Heads: logistic and softmax (the linear head exits, eval_hessian_vec.cu:300-303).
 * Hidden layers: logistic, linear, and tanh -- for tanh the reference's backward sweep leaves the layer's term unset
 * (:418-420) and the derivative is used here.  The Gauss-Newton variant keeps the reference's VW' dx term of the top
 * layer (eval_gauss_newton_hessian_vec.cu:262-275). */
long nnHessianVecMemRequired(NN_MODEL *model, DEVICE_DATASET *data, DATASET_SIZE allData);
void hessianVec(NN_MODEL *model, DEVICE_DATASET *data, real *z, real *dx, real *vec, real *weights, SCRATCH_AREA *scratch,
                DATASET_SIZE allData);
void gaussNewtonHessianVec(NN_MODEL *model, DEVICE_DATASET *data, real *z, real *dx, real *vec, real *weights,
                           SCRATCH_AREA *scratch, DATASET_SIZE allData);

#ifdef __cplusplus
}
#endif
#endif
