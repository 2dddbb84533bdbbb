/*
 * Kronecker-factor stage of the KFAC curvature approximation as C host code over the
 * C-ABI device layer: layer walk and data sources of solvers/kfac_inverses.cu:450-630
 * (computeOmegaZ) and :759-857 (computeLambdaDelta), storage offsets of
 * solvers/kfac_utils.cu:6-54.  No patch matrix, no scaled copies: each factor is one
 * symmetric product on the device.
 */
#include <stdio.h>
#include <stdlib.h>
#include "fitre_kfac.h"
#include "fitre_hip.h"

#define HIP_CALL(expr)                                                                               \
	do {                                                                                             \
		int rc_ = (expr);                                                                            \
		if (rc_ != FITRE_OK) {                                                                       \
			fprintf(stderr, "%s:%d: %s -> error %d: %s\n", __FILE__, __LINE__, #expr, rc_,           \
			        fitre_hip_last_error());                                                         \
			exit(-1);                                                                                \
		}                                                                                            \
	} while (0)

static fitre_conv_shape conv_shape(const CONV_LAYER *l, int samples)
{
	fitre_conv_shape s;
	s.samples = samples;
	s.inChannels = l->inChannels;
	s.outChannels = l->outChannels;
	s.inA = l->width;
	s.inB = l->height;
	s.outA = l->outWidth;
	s.outB = l->outHeight;
	s.ksize = l->kSize;
	s.stride = l->stride;
	s.padding = l->padding;
	return s;
}

static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }

void computeKFACStorageIndices(CNN_MODEL *model, KFAC_CURVATURE_INFO *kfacInfo)
{
	int *omega = kfacInfo->OmegaZOffsets, *lambda = kfacInfo->LambdaGOffsets;
	for (int i = 0; i < MAX_LAYERS; i++) omega[i] = lambda[i] = 0;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		int order = c->inChannels * c->kSize * c->kSize + 1;
		omega[i + 1] = omega[i] + order * order;
		lambda[i + 1] = lambda[i] + c->outChannels * c->outChannels;
	}
	for (int i = 0; i < model->lLayers; i++) {
		const FC_LAYER *f = &model->fcLayer[i];
		int at = model->cLayers + i;
		omega[at + 1] = omega[at] + (f->in + 1) * (f->in + 1);
		lambda[at + 1] = lambda[at] + f->out * f->out;
	}
}

static size_t factor_ws_bytes(const CNN_MODEL *model, int samples)
{
	size_t bytes = 0;
	int withBias = model->bias != 0;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		fitre_conv_shape s = conv_shape(c, samples);
		bytes = max_sz(bytes, fitre_hip_kfac_conv_input_factor_workspace(&s, withBias));
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(c->outChannels, (long)samples * c->outHeight * c->outWidth));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(f->in, samples));
		bytes = max_sz(bytes, fitre_hip_kfac_gram_workspace(f->out, samples));
	}
	return bytes;
}

long kfacFactorsMemRequired(CNN_MODEL *model, int samples)
{
	return (long)((factor_ws_bytes(model, samples) + sizeof(real) - 1) / sizeof(real)) + 64;
}

void computeOmegaZFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, DEVICE_DATASET *data, int samples,
                          real *dampedInput, real *dampedZ, real *omegaZZT, int *zOffsets, int *zztOffsets, real *devPtr)
{
	const int *omega = kfac_info->OmegaZOffsets;
	const int withBias = model->bias != 0;
	const size_t wsBytes = factor_ws_bytes(model, samples);
	const int nc = model->cLayers;

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const real *input;
		if (dampedInput != NULL)
			input = (l == 0) ? dampedInput : dampedZ + zztOffsets[l];
		else
			input = (l == 0) ? data->currentBatch : dampedZ + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		fitre_conv_shape s = conv_shape(c, samples);
		HIP_CALL(fitre_hip_kfac_conv_input_factor(&s, input, withBias, omegaZZT + omega[l], devPtr, wsBytes));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		const real *input;
		if (dampedInput != NULL)
			input = dampedZ + zztOffsets[nc + l];
		else if (l == 0)
			input = dampedZ + zOffsets[nc] + model->convLayer[nc - 1].outputOffset;
		else
			input = dampedZ + zOffsets[nc + l];
		HIP_CALL(fitre_hip_kfac_fc_input_factor(input, f->in, samples, withBias, omegaZZT + omega[nc + l], devPtr, wsBytes));
	}
	HIP_CALL(fitre_hip_sync());
}

void computeLambdaDeltaFactors(KFAC_CURVATURE_INFO *kfac_info, CNN_MODEL *model, int samples, real *dx,
                               real *dampedLambda, real *lambdaGGT, int *zOffsets, int *zztOffsets, real *devPtr)
{
	const int *lambda = kfac_info->LambdaGOffsets;
	const size_t wsBytes = factor_ws_bytes(model, samples);
	const int nc = model->cLayers;

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const real *delta;
		if (dampedLambda != NULL)
			delta = dampedLambda + zztOffsets[l + 1];
		else if (c->batchNorm == PERFORM_NO_BATCH_NORM)
			delta = dx + zOffsets[l + 1] + c->activationOffset;
		else
			delta = dx + zOffsets[l + 1] + c->batchNormOffset;
		fitre_conv_shape s = conv_shape(c, samples);
		HIP_CALL(fitre_hip_kfac_conv_output_factor(&s, delta, lambdaGGT + lambda[l], devPtr, wsBytes));
	}
	for (int l = 0; l < model->lLayers; l++) {
		const FC_LAYER *f = &model->fcLayer[l];
		const real *delta = (dampedLambda != NULL) ? dampedLambda + zztOffsets[nc + l + 1] : dx + zOffsets[nc + l + 1];
		HIP_CALL(fitre_hip_kfac_fc_output_factor(delta, f->out, samples, lambdaGGT + lambda[nc + l], devPtr, wsBytes));
	}
	HIP_CALL(fitre_hip_sync());
}
