/*
 * fitre_nn.h -- network description records of the CNN gradient path.
 *
 * Field names, field order and enumerator values follow the reference's
 * nn/nn_decl.h:4-215 exactly: CNN_MODEL is filled by the caller (or by the
 * builders in fitre_cnn.h) and read by cnnForward / cnnBackward, and the
 * reference's solvers index into it directly.
 *
 * Offsets are counted in reals.  "Volumn" is the reference's spelling and is
 * part of the field names.
 */
#ifndef FITRE_NN_H
#define FITRE_NN_H

#include <stdio.h>
#include <stdlib.h>
#include "fitre_types.h"

#define MAX_LAYERS 20

typedef enum network_name {
	CNN_LENET = 0,
	CNN_ALEXNET = 1,
	CNN_VGG11NET = 2,
	CNN_VGG13NET = 3,
	CNN_VGG16NET = 4,
	CNN_VGG19NET = 5
} NETWORK_NAME;

typedef enum batch_norm_types {
	PERFORM_NO_BATCH_NORM = 0,
	PERFORM_BATCH_NORM = 10,
	PERFORM_BATCH_NORM_TRAINABLE = 20
} BATCH_NORM_TYPES;

typedef enum eval_type {
	MODEL_TRAIN = 10,
	MODEL_TRAIN_ACCURACY = 20,
	MODEL_TEST_ACCURACY = 30
} EVAL_TYPE;

/* activations of fully connected layers */
typedef enum act_funs {
	ACT_NONE = 0,
	ACT_LOGISTIC = 1,
	ACT_TANH = 2,
	ACT_LINEAR = 3,
	ACT_SOFTMAX = 4
} ACTIVATION_FUNCTIONS;

/* activations of convolution layers (also accepted on FC layers) */
typedef enum cnn_act_funs {
	CNN_ACT_NONE = 10,
	CNN_ACT_SOFTPLUS = 11,
	CNN_ACT_ELU = 12,
	CNN_ACT_RELU = 13,
	CNN_ACT_SWISH = 14
} CNN_ACTIVATION_FUNCTIONS;

typedef enum model_type {
	MODEL_TYPE_MSE = 0,
	MODEL_TYPE_CLASSIFICATION = 1
} MODEL_TYPES;

/* One convolution layer.  The *Offset fields locate the stages of the layer
 * inside its slab of the activation store z (and of dx): the convolution
 * output sits at 0, then -- with batch norm -- the normalised output at
 * batchNormOffset followed by four per-channel vectors (batch mean, batch
 * variance, running mean, running variance; their offsets are relative to
 * the normalised output), then the activation output at activationOffset
 * and the pooled output at poolOffset.  outputOffset is whichever of the
 * last two feeds the next layer.  Unused offsets hold INT_MAX. */
typedef struct conv {
	int inChannels;
	int outChannels;

	int width;
	int height;
	int outWidth;
	int outHeight;

	int kSize;

	int stride;
	int padding;

	int activationOffset;
	int poolOffset;
	int batchNormOffset;
	int outputOffset;

	BATCH_NORM_TYPES batchNorm;
	int meansOffset;
	int variancesOffset;

	int runningMeansOffset;
	int runningVariancesOffset;

	int convVolumn;
	int activationVolumn;
	int poolVolumn;
	int batchNormVolumn;
} CONV_LAYER;

typedef enum pool_type { MAX_POOL = 0, AVG_POOL = 1, NO_POOL = 2 } POOL_TYPE;

/* Pooling stage attached to a convolution layer; height/width are the
 * convolution's output extent, also when type is NO_POOL. */
typedef struct pool {
	int height;
	int width;
	int outHeight;
	int outWidth;
	int type;
	int pSize;
	int padding;
	int stride;
} POOL_LAYER;

/* Fully connected layer; offset = out * batch locates the saved
 * pre-activation copy inside the layer's 2*out*batch slab of z. */
typedef struct full_connect {
	int in;
	int out;
	int actFun;
	int batchNorm;
	int offset;
} FC_LAYER;

typedef struct cnn {
	CONV_LAYER convLayer[MAX_LAYERS];
	int actFuns[MAX_LAYERS];
	POOL_LAYER poolLayer[MAX_LAYERS];
	int cLayers;

	int lLayers;
	FC_LAYER fcLayer[MAX_LAYERS];

	int bias;
	int pSize;
	int zSize;
	int batchSize;
	int maxDeltaSize;
	int name;
	int enableBatchNorm;

	int wOffsets[MAX_LAYERS];
	int bOffsets[MAX_LAYERS];
	int zOffsets[MAX_LAYERS];

	int zztSize;
	int zztOffsets[MAX_LAYERS];

	int rZOffsets[MAX_LAYERS];
} CNN_MODEL;

/* Fully connected auto-encoder model of the first-order solvers. */
typedef struct nn {
	int layerSizes[MAX_LAYERS];
	int actFuns[MAX_LAYERS];

	int numLayers;
	int type;

	int pSize;
	int zSize;
	int sampledZSize;
	int sampledRSize;
	int rFullSize;

	int wOffsets[MAX_LAYERS];
	int bOffsets[MAX_LAYERS];

	int zOffsets[MAX_LAYERS];
	int sZOffsets[MAX_LAYERS];

	int rZOffsets[MAX_LAYERS];
	int sRZOffsets[MAX_LAYERS];
} NN_MODEL;

#define BATCH_NORM_EPSILON  1e-5
#define BATCH_NORM_MOMENTUM 0.9

#endif
