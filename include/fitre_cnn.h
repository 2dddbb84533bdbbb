/*
 * fitre_cnn.h -- host-side C interface of the CNN gradient path.
 *
 * These are the free functions the reference's solvers and drivers call
 * (solvers/kfac_trust_region.cu:352,361,395; utilities/cnn_derivative_test.cu:158-168).
 * Names, argument order and argument meaning are the reference's; every
 * function is device-complete when it returns.  On an unrecoverable error a
 * message goes to stderr and the process exits, as in the reference
 * (functions/cnn_backward.cu:171-174).
 *
 * All pointers named z, dx, probs, errors, gradient, delta, devPtr and the
 * DEVICE_DATASET members are DEVICE pointers owned by the caller.
 */
#ifndef FITRE_CNN_H
#define FITRE_CNN_H

#include "fitre_nn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- shape and flat-layout arithmetic (reference: nn/utils.c:12-172) ---- */

/* (height + 2*padding - kernel)/stride + 1, integer division. nn/utils.c:12-17 */
void getDimensions(int height, int width, int padding, int stride, int kernel, int *h, int *w);
/* pSize = number of reals in the flat parameter vector. nn/utils.c:19-42 */
void computeParamSize(CNN_MODEL *model);
/* wOffsets for a model without biases; bOffsets := INT_MAX. nn/utils.c:44-71 */
void computeWeightOffsets(CNN_MODEL *model);
/* interleaved [W_l | b_l] offsets for a model with biases. nn/utils.c:74-105 */
void computeWeightBiasOffsets(CNN_MODEL *model);
/* zOffsets, zztOffsets, zSize, zztSize, maxDeltaSize. nn/utils.c:108-172 */
void computeZOffsets(CNN_MODEL *model, int height, int width, int batchSize);
/* 3x3 / stride 1 / pad 1 convolution + optional 2x2 pool, with the slab
 * offsets of nn/read_vgg.c:25-120. */
void makeLayer(CONV_LAYER *conv, POOL_LAYER *pool, POOL_TYPE poolFun, int inChannels, int outChannels,
               int height, int width, int *outHeight, int *outWidth, int batchSize,
               BATCH_NORM_TYPES batchnorm);
/* VGG-11 as the reference builds it (swish; nn/read_vgg.c:216-300). */
void readVGG11(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels,
               int bias, int enableBatchNorm, DATASET_TYPE datasetType);
/* nn/read_nn.h:18-19 and nn/read_alexnet.h:7-8: the reference's two small networks as it builds them -- LeNet with
 * swish and 2 / 2 average pools (6 and 16 channels; linear 120, 84, 10), and its CIFAR-sized "AlexNet" (two 5x5 / pad 2
 * convolutions of 64 channels with 3 / 2 / 1 max pools; linear 384, 192, numClasses).  fitre_build_lenet /
 * fitre_build_alexnet below take activations and pooling as arguments (the latter is the five-convolution network). */
void readLenetCNN(CNN_MODEL *model, int channels, int width, int height, int batchSize, int enableBias, int enableBatchNorm);
void readAlexNetCNN(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int enableBias, int enableBatchNorm);
/* nn/read_vgg.h:10-12: 10, 13 and 16 convolutions (64,64,M,128,128,M,256,256[,256[,256]],M,512,...), same arguments */
void readVGG13(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType);
void readVGG16(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType);
void readVGG19(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType);

/* ---- builders that have no counterpart in the reference: the same slab
 * scheme as makeLayer for arbitrary kernel / stride / padding / pooling ---- */
void fitre_make_conv_layer(CONV_LAYER *conv, POOL_LAYER *pool, int inChannels, int outChannels,
                           int height, int width, int kSize, int stride, int padding,
                           POOL_TYPE poolFun, int poolSize, int poolStride, int poolPadding,
                           int batchSize, BATCH_NORM_TYPES batchnorm, int *outHeight, int *outWidth);
/* Fills pSize, w/b/z offsets and sizes once cLayers/lLayers/layers/bias are set. */
void fitre_finalize_model(CNN_MODEL *model, int height, int width, int batchSize);
/* LeNet-style: conv5x5 C->6, pool2, conv5x5 6->16, pool2, FC 400-120-84-classes (32x32 input). */
void fitre_build_lenet(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                       int numClasses, int bias, int enableBatchNorm, int convAct, int fcAct);
/* VGG-11-style with a chosen activation. */
void fitre_build_vgg11(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                       int numClasses, int bias, int enableBatchNorm, int convAct);
/* ImageNet AlexNet-style: 11x11/s4/p2, 5x5/p2, 3x3 x3, maxpool 3/2 after 1,2,5; FC 9216-4096-4096-classes. */
void fitre_build_alexnet(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                         int numClasses, int bias, int convAct, int fcAct);

/* ---- the gradient path (reference: functions/cnn_forward.h:9-13,
 * functions/cnn_backward.h:11-16, functions/cnn_gradient.h:9-12,
 * functions/cnn_eval_model.cu:7-13) ---- */

/* Scratch (in reals) the forward pass may carve from scratch->nextDevPtr. */
long cnnForwardMemRequired(CNN_MODEL *model);
/* Fills z, probs (classes x batch, class fastest) and errors = (p - onehot)/batch;
 * returns the mean negative log-likelihood. */
real cnnForward(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs,
                real *errors, int s, int curBatchSize, EVAL_TYPE forTesting);
/* Scratch (in reals) cnnBackward may carve from devPtr. */
long cnnBackwardMemRequired(CNN_MODEL *model);
/* gradient[pSize] and the dx snapshots from z and delta (= errors of cnnForward).
 * delta and delta_new (each >= maxDeltaSize reals) are clobbered. */
void cnnBackward(CNN_MODEL *model, DEVICE_DATASET *data, real *devPtr, real *z, real *gradient, real *dx,
                 real *delta, real *delta_new, int offset, int batchSize, real *hostPtr);
/* Back-propagation goes through stride-1 convolutions only: every convolution layer above the first must have
 * stride 1 (the first layer's input gradient is never taken, so its stride is free -- AlexNet's 11x11 / 4).  The
 * reference's backpropConvolution (functions/dev_backprop_convolution.cu:173-247) has the same limit (its patch
 * gather is written for stride 1).  Returns 0 when `model` can be back-propagated through, else the 1-based index of
 * the first offending layer; cnnBackward and cnnHv call it before their first launch and exit(-1) with a message. */
int fitreBackwardUnsupportedLayer(const CNN_MODEL *model);
/* cnnBackward queues a pass on one stream or spreads it over the device layer's lanes (weight gradients beside the
 * chain of input gradients); by default it decides from the network's convolution work (one lane below 1e9
 * multiply-adds per pass, a limit fitted on LeNet, VGG-11 and AlexNet).  mode 0: always one
 * lane, 1: always the lanes, -1: the default rule.  The results do not depend on it, bit for bit.  No counterpart in
 * the reference (one stream).  fitreBackwardUsesLanes: what a pass of this model and batch would do now.
 * Weights, z and delta must be complete on lane 0 when cnnBackward is called; the other lanes order themselves behind it. */
void fitreSetBackwardLanes(int mode);
int fitreBackwardUsesLanes(CNN_MODEL *model, int batchSize);

real evaluateCNNModel(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z,
                      real *probs, real *lossFuncErrors, int offset, int curBatchSize);
/* forward + backward + gradient += weightDecay * weights; returns the loss. */
real computeCNNGradient(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *dx,
                        real *probs, real *lossFuncErrors, real *gradient, int offset, int curBatchSize,
                        real weightDecay);

/* errors = (probs - onehot(target)) / rows (functions/softmax_loss.cu:141-175 as called from :131). */
void computeCrossEntropyError(real *probs, int rows, int num_classes, real *target, real *errors);
/* One class per sample drawn from the model's own predictive distribution
 * (functions/dev_dist_errors.cu:39-53); devPtr: samples (+1) reals of scratch for the uniform draws. */
void getMultinomialDistSample(real *probs, int samples, int numClasses, real *distClasses, real *devPtr);
/* Sampled targets and the loss errors against them -- the input of the backward pass that builds the
 * Fisher (KFAC) statistics (functions/softmax_loss.cu:104-136).  hostPtr is unused. */
void computeDistributionErrors(real *probs, real *distTarget, real *distError, int rows, int num_classes,
                               real *devPtr, real *hostPtr);

/* Percentage of rows whose most probable class (first maximum) is the label; *pageLckPtr receives the
 * number of hits, as callers read it (functions/cnn_accuracy.cu:39-59, :89-91).  devPtr: rows reals
 * of device scratch; pageLckPtr: a host pointer. */
real computeAccuracy(real *probs, real *target, int rows, int numClasses, real *devPtr, real *pageLckPtr);

#ifdef __cplusplus
}
#endif
#endif
