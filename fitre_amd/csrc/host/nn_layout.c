/*
 * Shape arithmetic and the flat parameter / activation-store layouts.
 *
 * Restates nn/utils.c:12-172 and the slab scheme of nn/read_vgg.c:25-120 of
 * the reference; the generalised layer builder keeps that scheme for any
 * kernel size, stride, padding and pooling window.
 */
#include <limits.h>
#include <string.h>
#include "fitre_cnn.h"

static int conv_weight_count(const CONV_LAYER *c)
{
	return c->outChannels * c->kSize * c->kSize * c->inChannels;
}

static int has_bn(const CONV_LAYER *c)
{
	return c->batchNorm == PERFORM_BATCH_NORM || c->batchNorm == PERFORM_BATCH_NORM_TRAINABLE;
}

void getDimensions(int height, int width, int padding, int stride, int kernel, int *h, int *w)
{
	*h = (height + 2 * padding - kernel) / stride + 1;
	*w = (width + 2 * padding - kernel) / stride + 1;
}

void computeParamSize(CNN_MODEL *model)
{
	int total = 0;
	for (int i = 0; i < model->cLayers; i++) {
		total += conv_weight_count(&model->convLayer[i]);
		if (model->bias >= 1) total += model->convLayer[i].outChannels;
	}
	for (int i = 0; i < model->lLayers; i++) {
		total += model->fcLayer[i].out * model->fcLayer[i].in;
		if (model->bias >= 1) total += model->fcLayer[i].out;
	}
	model->pSize = total;
}

static void clear_offsets(CNN_MODEL *model)
{
	for (int i = 0; i < MAX_LAYERS; i++)
		model->wOffsets[i] = model->bOffsets[i] = model->zOffsets[i] = 0;
}

void computeWeightOffsets(CNN_MODEL *model)
{
	clear_offsets(model);
	for (int i = 0; i < MAX_LAYERS; i++) model->bOffsets[i] = INT_MAX;

	int nc = model->cLayers, nl = model->lLayers;
	int cursor = 0;
	for (int i = 0; i < nc; i++) {
		model->wOffsets[i] = cursor;
		cursor += conv_weight_count(&model->convLayer[i]);
	}
	for (int i = 0; i < nl; i++) {
		model->wOffsets[nc + i] = cursor;
		cursor += model->fcLayer[i].out * model->fcLayer[i].in;
	}
	model->wOffsets[nc + nl] = cursor;
}

void computeWeightBiasOffsets(CNN_MODEL *model)
{
	clear_offsets(model);

	int nc = model->cLayers, nl = model->lLayers;
	int cursor = 0;
	for (int i = 0; i < nc; i++) {
		model->wOffsets[i] = cursor;
		cursor += conv_weight_count(&model->convLayer[i]);
		model->bOffsets[i] = cursor;
		cursor += model->convLayer[i].outChannels;
	}
	for (int i = 0; i < nl; i++) {
		model->wOffsets[nc + i] = cursor;
		cursor += model->fcLayer[i].out * model->fcLayer[i].in;
		model->bOffsets[nc + i] = cursor;
		cursor += model->fcLayer[i].out;
	}
}

void computeZOffsets(CNN_MODEL *model, int height, int width, int batchSize)
{
	(void)height;
	(void)width;
	for (int i = 0; i < MAX_LAYERS; i++) {
		model->zOffsets[i] = 0;
		model->zztOffsets[i] = 0;
	}
	model->maxDeltaSize = 0;
	model->zztSize = 0;

	int nc = model->cLayers;
	for (int i = 1; i <= nc; i++) {
		const CONV_LAYER *t = &model->convLayer[i - 1];
		const POOL_LAYER *p = &model->poolLayer[i - 1];
		int vol = t->outHeight * t->outWidth * t->outChannels;

		/* convolution output + activation output */
		int slab = batchSize * vol * 2;
		/* normalised output + (mean, variance, running mean, running variance) */
		if (has_bn(t)) slab += batchSize * vol + 4 * t->outChannels;
		if (p->type != NO_POOL) slab += batchSize * (p->outHeight * p->outWidth * t->outChannels);

		model->zOffsets[i + 1] = model->zOffsets[i] + slab;
		model->zztOffsets[i + 1] = model->zztOffsets[i] + batchSize * vol;
		model->zztSize += batchSize * vol;
		if (slab > model->maxDeltaSize) model->maxDeltaSize = slab;
	}

	for (int i = 1; i <= model->lLayers; i++) {
		const FC_LAYER *t = &model->fcLayer[i - 1];
		/* activation output + saved pre-activation */
		int slab = t->out * batchSize * 2;
		model->zOffsets[i + nc + 1] = model->zOffsets[i + nc] + slab;
		model->zztOffsets[i + 1 + nc] = model->zztOffsets[i + nc] + t->out * batchSize;
		model->zztSize += t->out * batchSize;
		if (slab > model->maxDeltaSize) model->maxDeltaSize = slab;
	}
	model->zSize = model->zOffsets[nc + model->lLayers + 1];
}

void fitre_make_conv_layer(CONV_LAYER *conv, POOL_LAYER *pool, int inChannels, int outChannels,
                           int height, int width, int kSize, int stride, int padding,
                           POOL_TYPE poolFun, int poolSize, int poolStride, int poolPadding,
                           int batchSize, BATCH_NORM_TYPES batchnorm, int *outHeight, int *outWidth)
{
	conv->height = height;
	conv->width = width;
	conv->stride = stride;
	conv->padding = padding;
	conv->kSize = kSize;
	conv->inChannels = inChannels;
	conv->outChannels = outChannels;
	conv->batchNorm = batchnorm;
	getDimensions(height, width, padding, stride, kSize, &conv->outHeight, &conv->outWidth);

	pool->type = poolFun;
	pool->pSize = poolSize;
	pool->stride = poolStride;
	pool->padding = poolPadding;
	pool->height = conv->outHeight;
	pool->width = conv->outWidth;
	if (poolFun == NO_POOL) {
		pool->outHeight = pool->height;
		pool->outWidth = pool->width;
	} else {
		getDimensions(pool->height, pool->width, poolPadding, poolStride, poolSize,
		              &pool->outHeight, &pool->outWidth);
	}
	*outHeight = pool->outHeight;
	*outWidth = pool->outWidth;

	int stage = conv->outHeight * conv->outWidth * conv->outChannels * batchSize;
	if (batchnorm == PERFORM_NO_BATCH_NORM) {
		conv->activationOffset = stage;
		conv->batchNormOffset = INT_MAX;
		conv->meansOffset = conv->variancesOffset = INT_MAX;
		conv->runningMeansOffset = conv->runningVariancesOffset = INT_MAX;
	} else {
		conv->batchNormOffset = stage;
		conv->meansOffset = stage;
		conv->variancesOffset = conv->meansOffset + conv->outChannels;
		conv->runningMeansOffset = conv->variancesOffset + conv->outChannels;
		conv->runningVariancesOffset = conv->runningMeansOffset + conv->outChannels;
		conv->activationOffset = 2 * stage + 4 * conv->outChannels;
	}
	if (poolFun == NO_POOL) {
		conv->poolOffset = INT_MAX;
		conv->outputOffset = conv->activationOffset;
	} else {
		conv->poolOffset = conv->activationOffset + stage;
		conv->outputOffset = conv->poolOffset;
	}

	conv->convVolumn = conv->outHeight * conv->outWidth * conv->outChannels;
	conv->batchNormVolumn = (batchnorm != PERFORM_NO_BATCH_NORM) ? INT_MAX : conv->convVolumn;
	conv->activationVolumn = conv->convVolumn;
	conv->poolVolumn = (poolFun == NO_POOL) ? INT_MAX
	                                        : pool->outHeight * pool->outWidth * conv->outChannels;
}

void makeLayer(CONV_LAYER *conv, POOL_LAYER *pool, POOL_TYPE poolFun, int inChannels, int outChannels,
               int height, int width, int *outHeight, int *outWidth, int batchSize,
               BATCH_NORM_TYPES batchnorm)
{
	fitre_make_conv_layer(conv, pool, inChannels, outChannels, height, width, 3, 1, 1, poolFun, 2, 2, 0,
	                      batchSize, batchnorm, outHeight, outWidth);
}

void fitre_finalize_model(CNN_MODEL *model, int height, int width, int batchSize)
{
	model->batchSize = batchSize;
	computeParamSize(model);
	if (model->bias != 0)
		computeWeightBiasOffsets(model);
	else
		computeWeightOffsets(model);
	computeZOffsets(model, height, width, batchSize);
}

static void set_fc(CNN_MODEL *model, int l, int in, int out, int act, int batchSize)
{
	model->fcLayer[l].in = in;
	model->fcLayer[l].out = out;
	model->fcLayer[l].actFun = act;
	model->fcLayer[l].batchNorm = 0;
	model->fcLayer[l].offset = batchSize * out;
}

/* The VGG family of nn/read_vgg.c: 3x3 / pad 1 convolutions of the given widths, max pool 2 after the marked
 * ones, one linear layer on the flattened features. */
static void build_vgg(CNN_MODEL *model, int name, const int *channels, const int *pooled, int count, int batchSize,
                      int height, int width, int inChannels, int numClasses, int bias, int enableBatchNorm, int convAct)
{
	BATCH_NORM_TYPES bn = enableBatchNorm ? PERFORM_BATCH_NORM : PERFORM_NO_BATCH_NORM;

	memset(model, 0, sizeof(*model));
	model->enableBatchNorm = enableBatchNorm;
	int h = height, w = width, cin = inChannels;
	for (int l = 0; l < count; l++) {
		model->actFuns[l] = convAct;
		makeLayer(&model->convLayer[l], &model->poolLayer[l], pooled[l] ? MAX_POOL : NO_POOL, cin, channels[l], h, w, &h, &w,
		          batchSize, bn);
		cin = channels[l];
	}
	model->cLayers = count;
	set_fc(model, 0, cin * h * w, numClasses, CNN_ACT_NONE, batchSize);
	model->lLayers = 1;
	model->bias = bias;
	model->name = name;
	fitre_finalize_model(model, height, width, batchSize);
}

void fitre_build_vgg11(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                       int numClasses, int bias, int enableBatchNorm, int convAct)
{
	static const int channels[8] = { 64, 128, 256, 256, 512, 512, 512, 512 };
	static const int pooled[8] = { 1, 1, 0, 1, 0, 1, 0, 1 };
	build_vgg(model, CNN_VGG11NET, channels, pooled, 8, batchSize, height, width, inChannels, numClasses, bias, enableBatchNorm,
	          convAct);
}

void readVGG11(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels,
               int bias, int enableBatchNorm, DATASET_TYPE datasetType)
{
	(void)datasetType; /* FC fan-in follows from the image size: 512 at 32x32, 2048 at 64x64 */
	fitre_build_vgg11(model, batchSize, height, width, inChannels, numClasses, bias, enableBatchNorm,
	                  CNN_ACT_SWISH);
}

/* nn/read_vgg.c:345-424, :486-579, :642-750: the deeper members, swish after every convolution as there */
void readVGG13(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType)
{
	static const int channels[10] = { 64, 64, 128, 128, 256, 256, 512, 512, 512, 512 };
	static const int pooled[10] = { 0, 1, 0, 1, 0, 1, 0, 1, 0, 1 };
	(void)datasetType;
	build_vgg(model, CNN_VGG13NET, channels, pooled, 10, batchSize, height, width, inChannels, numClasses, bias, enableBatchNorm,
	          CNN_ACT_SWISH);
}

void readVGG16(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType)
{
	static const int channels[13] = { 64, 64, 128, 128, 256, 256, 256, 512, 512, 512, 512, 512, 512 };
	static const int pooled[13] = { 0, 1, 0, 1, 0, 0, 1, 0, 0, 1, 0, 0, 1 };
	(void)datasetType;
	build_vgg(model, CNN_VGG16NET, channels, pooled, 13, batchSize, height, width, inChannels, numClasses, bias, enableBatchNorm,
	          CNN_ACT_SWISH);
}

void readVGG19(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int inChannels, int bias,
               int enableBatchNorm, DATASET_TYPE datasetType)
{
	static const int channels[16] = { 64, 64, 128, 128, 256, 256, 256, 256, 512, 512, 512, 512, 512, 512, 512, 512 };
	static const int pooled[16] = { 0, 1, 0, 1, 0, 0, 0, 1, 0, 0, 0, 1, 0, 0, 0, 1 };
	(void)datasetType;
	build_vgg(model, CNN_VGG19NET, channels, pooled, 16, batchSize, height, width, inChannels, numClasses, bias, enableBatchNorm,
	          CNN_ACT_SWISH);
}

void fitre_build_lenet(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                       int numClasses, int bias, int enableBatchNorm, int convAct, int fcAct)
{
	BATCH_NORM_TYPES bn = enableBatchNorm ? PERFORM_BATCH_NORM : PERFORM_NO_BATCH_NORM;
	memset(model, 0, sizeof(*model));
	model->enableBatchNorm = enableBatchNorm;
	int h = height, w = width;
	model->actFuns[0] = convAct;
	fitre_make_conv_layer(&model->convLayer[0], &model->poolLayer[0], inChannels, 6, h, w, 5, 1, 0,
	                      MAX_POOL, 2, 2, 0, batchSize, bn, &h, &w);
	model->actFuns[1] = convAct;
	fitre_make_conv_layer(&model->convLayer[1], &model->poolLayer[1], 6, 16, h, w, 5, 1, 0, MAX_POOL, 2,
	                      2, 0, batchSize, bn, &h, &w);
	model->cLayers = 2;
	set_fc(model, 0, 16 * h * w, 120, fcAct, batchSize);
	set_fc(model, 1, 120, 84, fcAct, batchSize);
	set_fc(model, 2, 84, numClasses, CNN_ACT_NONE, batchSize);
	model->lLayers = 3;
	model->bias = bias;
	model->name = CNN_LENET;
	fitre_finalize_model(model, height, width, batchSize);
}

void fitre_build_alexnet(CNN_MODEL *model, int batchSize, int height, int width, int inChannels,
                         int numClasses, int bias, int convAct, int fcAct)
{
	static const int cout[5] = { 96, 256, 384, 384, 256 };
	static const int ksz[5] = { 11, 5, 3, 3, 3 };
	static const int strd[5] = { 4, 1, 1, 1, 1 };
	static const int padd[5] = { 2, 2, 1, 1, 1 };
	static const int pooled[5] = { 1, 1, 0, 0, 1 };

	memset(model, 0, sizeof(*model));
	int h = height, w = width, cin = inChannels;
	for (int l = 0; l < 5; l++) {
		model->actFuns[l] = convAct;
		fitre_make_conv_layer(&model->convLayer[l], &model->poolLayer[l], cin, cout[l], h, w, ksz[l],
		                      strd[l], padd[l], pooled[l] ? MAX_POOL : NO_POOL, 3, 2, 0, batchSize,
		                      PERFORM_NO_BATCH_NORM, &h, &w);
		cin = cout[l];
	}
	model->cLayers = 5;
	set_fc(model, 0, cin * h * w, 4096, fcAct, batchSize);
	set_fc(model, 1, 4096, 4096, fcAct, batchSize);
	set_fc(model, 2, 4096, numClasses, CNN_ACT_NONE, batchSize);
	model->lLayers = 3;
	model->bias = bias;
	model->name = CNN_ALEXNET;
	fitre_finalize_model(model, height, width, batchSize);
}

/* nn/read_nn.c:500-700: the reference's LeNet -- 5x5 convolutions of 6 and 16 channels, each with swish and a
 * 2 / 2 AVERAGE pool, linear layers 120, 84 (swish) and 10.  (width before height, as there.)  With batch norm on,
 * the slab of a layer is laid out as makeLayer does for the VGG family; the reference's own offsets for this
 * network place the normalisation behind the pool, which its forward pass does not follow. */
void readLenetCNN(CNN_MODEL *model, int channels, int width, int height, int batchSize, int enableBias, int enableBatchNorm)
{
	BATCH_NORM_TYPES bn = enableBatchNorm ? PERFORM_BATCH_NORM : PERFORM_NO_BATCH_NORM;
	memset(model, 0, sizeof(*model));
	model->enableBatchNorm = enableBatchNorm;
	int h = height, w = width;
	model->actFuns[0] = CNN_ACT_SWISH;
	fitre_make_conv_layer(&model->convLayer[0], &model->poolLayer[0], channels, 6, h, w, 5, 1, 0, AVG_POOL, 2, 2, 0, batchSize, bn,
	                      &h, &w);
	model->actFuns[1] = CNN_ACT_SWISH;
	fitre_make_conv_layer(&model->convLayer[1], &model->poolLayer[1], 6, 16, h, w, 5, 1, 0, AVG_POOL, 2, 2, 0, batchSize, bn, &h, &w);
	model->cLayers = 2;
	set_fc(model, 0, 16 * h * w, 120, CNN_ACT_SWISH, batchSize);
	set_fc(model, 1, 120, 84, CNN_ACT_SWISH, batchSize);
	set_fc(model, 2, 84, 10, CNN_ACT_NONE, batchSize);
	model->lLayers = 3;
	model->bias = enableBias;
	model->name = CNN_LENET;
	fitre_finalize_model(model, height, width, batchSize);
}

/* nn/read_alexnet.c:14-215: the reference's CIFAR-sized "AlexNet" -- two 5x5 / pad 2 convolutions of 64 channels,
 * each with swish and a 3 / 2 / 1 max pool, linear layers 384, 192 (swish) and numClasses. */
void readAlexNetCNN(CNN_MODEL *model, int batchSize, int height, int width, int numClasses, int enableBias, int enableBatchNorm)
{
	BATCH_NORM_TYPES bn = enableBatchNorm ? PERFORM_BATCH_NORM : PERFORM_NO_BATCH_NORM;
	memset(model, 0, sizeof(*model));
	model->enableBatchNorm = enableBatchNorm;
	int h = height, w = width, cin = 3;
	for (int l = 0; l < 2; l++) {
		model->actFuns[l] = CNN_ACT_SWISH;
		fitre_make_conv_layer(&model->convLayer[l], &model->poolLayer[l], cin, 64, h, w, 5, 1, 2, MAX_POOL, 3, 2, 1, batchSize, bn,
		                      &h, &w);
		cin = 64;
	}
	model->cLayers = 2;
	set_fc(model, 0, 64 * h * w, 384, CNN_ACT_SWISH, batchSize);
	set_fc(model, 1, 384, 192, CNN_ACT_SWISH, batchSize);
	set_fc(model, 2, 192, numClasses, CNN_ACT_NONE, batchSize);
	model->lLayers = 3;
	model->bias = enableBias;
	model->name = CNN_ALEXNET;
	fitre_finalize_model(model, height, width, batchSize);
}
