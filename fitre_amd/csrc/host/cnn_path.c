/*
 * cnnForward / cnnBackward / computeCNNGradient: the model-level passes of the
 * gradient path, as C host code over the C-ABI device layer.
 *
 * Data flow and z / dx contents follow functions/cnn_forward.cu:49-383,
 * functions/cnn_backward.cu:76-857 and functions/cnn_gradient.cu:13-64 of the
 * reference; what differs is below the layer calls: no patch matrices, no
 * ones-vector products, no staging copies -- the dx slots themselves are the
 * working buffers of the backward pass.
 */
#include <stdio.h>
#include <stdlib.h>
#include "fitre_cnn.h"
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

static int has_bn(const CONV_LAYER *c) { return c->batchNorm != PERFORM_NO_BATCH_NORM; }

static fitre_conv_shape conv_shape(const CONV_LAYER *l, int samples)
{
	fitre_conv_shape s;
	s.samples = samples;
	s.inChannels = l->inChannels;
	s.outChannels = l->outChannels;
	s.inA = l->width; /* A = image column index, B = image row index (fastest) */
	s.inB = l->height;
	s.outA = l->outWidth;
	s.outB = l->outHeight;
	s.ksize = l->kSize;
	s.stride = l->stride;
	s.padding = l->padding;
	return s;
}

static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }

/* extent of the feature map handed to the first FC layer */
static void feature_extent(const CNN_MODEL *model, int *extA, int *extB)
{
	const CONV_LAYER *c = &model->convLayer[model->cLayers - 1];
	const POOL_LAYER *p = &model->poolLayer[model->cLayers - 1];
	if (p->type != NO_POOL) {
		*extA = p->outWidth;
		*extB = p->outHeight;
	} else {
		*extA = c->outWidth;
		*extB = c->outHeight;
	}
}

static size_t forward_ws_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 256;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		fitre_conv_shape s = conv_shape(c, batch);
		need = max_sz(need, fitre_hip_conv_forward_workspace(&s));
		if (has_bn(c)) need = max_sz(need, fitre_hip_batch_norm_workspace(c->outChannels, (long)batch * c->outWidth * c->outHeight));
	}
	if (model->cLayers > 0) {
		int extA, extB;
		feature_extent(model, &extA, &extB);
		need = max_sz(need, sizeof(real) * (size_t)extA * extB * batch * model->convLayer[model->cLayers - 1].outChannels);
	}
	for (int i = 0; i < model->lLayers; i++)
		need = max_sz(need, fitre_hip_gemm_workspace(model->fcLayer[i].out, batch, model->fcLayer[i].in));
	return need;
}

/* cnnBackward carves two workspaces from devPtr: one for the chain that produces each layer's
 * delta (pool / activation / batch norm / input gradient, lane 0) and one for the weight gradients,
 * which run beside that chain on lane 1. */
/* The chain workspace has two parts that are live at the same time: the input gradient's split partials,
 * which the pool / activation pass of the layer below sums while it reads them, and that pass's
 * batch-norm sums. */
static size_t backward_dx_ws_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 256;
	for (int i = 1; i < model->cLayers; i++) {
		fitre_conv_shape s = conv_shape(&model->convLayer[i], batch);
		need = max_sz(need, fitre_hip_conv_input_grad_workspace(&s));
	}
	for (int i = 0; i < model->lLayers; i++) {
		const FC_LAYER *f = &model->fcLayer[i];
		need = max_sz(need, fitre_hip_gemm_workspace(f->in, batch, f->out));
	}
	if (model->cLayers > 0) {
		/* the first linear layer's delta in the convolution layout, until the last convolution layer has read it */
		int extA, extB;
		feature_extent(model, &extA, &extB);
		need = max_sz(need, sizeof(real) * (size_t)extA * extB * batch * model->convLayer[model->cLayers - 1].outChannels);
	}
	return (need + 255) & ~(size_t)255;
}

static size_t backward_bn_ws_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 256;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		need = max_sz(need, fitre_hip_batch_norm_workspace(c->outChannels, (long)batch * c->outWidth * c->outHeight));
	}
	return (need + 255) & ~(size_t)255;
}

static size_t backward_chain_ws_bytes(const CNN_MODEL *model, int batch)
{
	return backward_dx_ws_bytes(model, batch) + backward_bn_ws_bytes(model, batch);
}

/* the linear layers as the fused tail sees them (shapes only; tail_layers fills in the pointers); 0 when they do not fit it */
static int tail_shapes(const CNN_MODEL *model, int n, fitre_fc_tail_layer *tail)
{
	if (model->lLayers < 2 || model->lLayers > 4) return 0; /* one layer alone: the two per-layer launches are the shorter way */
	for (int f = 0; f < model->lLayers; f++) {
		fitre_fc_tail_layer t = { model->fcLayer[f].in, model->fcLayer[f].out, model->fcLayer[f].actFun, NULL, NULL, NULL, NULL, NULL, NULL, NULL };
		tail[f] = t;
	}
	return fitre_hip_fc_tail_fits(model->lLayers, tail, n);
}

static size_t backward_side_ws_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 256;
	fitre_fc_tail_layer tail[4];
	if (tail_shapes(model, batch, tail)) need = max_sz(need, fitre_hip_fc_tail_workspace(model->lLayers, tail, batch));
	size_t held = 0; /* layers whose reduction is held back until the end of the pass keep their blocks: a slice each */
	for (int i = 0; i < model->cLayers; i++) {
		fitre_conv_shape s = conv_shape(&model->convLayer[i], batch);
		need = max_sz(need, fitre_hip_conv_weight_grad_workspace(&s));
		held += fitre_hip_thin_reduce_bytes(&s);
		if (!has_bn(&model->convLayer[i]))
			need = max_sz(need, fitre_hip_channel_sum_workspace(model->convLayer[i].outChannels,
			                                                    (long)batch * model->convLayer[i].outWidth * model->convLayer[i].outHeight));
	}
	for (int i = 0; i < model->lLayers; i++) {
		const FC_LAYER *f = &model->fcLayer[i];
		need = max_sz(need, fitre_hip_linear_weight_grad_workspace(f->in, f->out, batch));
	}
	return ((need + 255) & ~(size_t)255) + held;
}

/* Rearranged weight copies that some input gradients multiply by (fitre_hip_conv_input_grad_prepare): made at the
 * start of the pass on a lane of their own, one buffer per layer that has one. */
static size_t backward_prepared_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 0;
	for (int i = 1; i < model->cLayers; i++) {
		fitre_conv_shape s = conv_shape(&model->convLayer[i], batch);
		need += (fitre_hip_conv_input_grad_prepared_bytes(&s) + 255) & ~(size_t)255;
	}
	return need;
}

static size_t backward_ws_bytes(const CNN_MODEL *model, int batch)
{
	return backward_chain_ws_bytes(model, batch) + backward_side_ws_bytes(model, batch) + backward_prepared_bytes(model, batch);
}

int fitreBackwardUnsupportedLayer(const CNN_MODEL *model)
{
	for (int c = 1; c < model->cLayers; c++)
		if (model->convLayer[c].stride != 1) return c + 1;
	return 0;
}

long cnnForwardMemRequired(CNN_MODEL *model)
{
	return (long)((forward_ws_bytes(model, model->batchSize) + sizeof(real) - 1) / sizeof(real));
}

long cnnBackwardMemRequired(CNN_MODEL *model)
{
	return (long)((backward_ws_bytes(model, model->batchSize) + sizeof(real) - 1) / sizeof(real));
}

real cnnForward(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs, real *errors,
                int s, int curBatchSize, EVAL_TYPE forTesting)
{
	(void)s;
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	const real *weights = data->weights;
	const int nc = model->cLayers, n = curBatchSize;
	void *ws = (void *)scratch->nextDevPtr;
	const size_t wsBytes = sizeof(real) * (size_t)cnnForwardMemRequired(model);

	if (forTesting != MODEL_TRAIN && forTesting != MODEL_TRAIN_ACCURACY && forTesting != MODEL_TEST_ACCURACY) {
		fprintf(stderr, "Unknown EVAL_TYPE... \n\n");
		exit(-1);
	}
	if (nc < 1 || n < 1 || n > model->batchSize) {
		fprintf(stderr, "cnnForward: needs at least one convolution layer and 1 <= batch (%d) <= model batch (%d)\n", n,
		        model->batchSize);
		exit(-1);
	}

	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *cv = &model->convLayer[l];
		const POOL_LAYER *pl = &model->poolLayer[l];
		const real *in = (l == 0) ? data->currentBatch : z + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		real *slab = z + zOffsets[l + 1];
		real *actOut = slab + cv->activationOffset;
		fitre_conv_shape shape = conv_shape(cv, n);

		HIP_CALL(fitre_hip_conv_forward(&shape, in, weights + wOffsets[l],
		                                (model->bias == 0) ? NULL : weights + bOffsets[l], slab, ws, wsBytes));
		/* batch norm (where the layer has it), activation and pooling: one pass over the convolution output where the
		 * shapes allow, the separate passes otherwise */
		{
			real *bnOut = has_bn(cv) ? slab + cv->batchNormOffset : NULL;
			const int pooled = pl->type != NO_POOL;
			HIP_CALL(fitre_hip_bn_act_pool_forward(
			    slab, cv->outChannels, n, pooled ? pl->width : cv->outWidth, pooled ? pl->height : cv->outHeight, bnOut,
			    bnOut ? bnOut + cv->meansOffset : NULL, bnOut ? bnOut + cv->variancesOffset : NULL,
			    bnOut ? bnOut + cv->runningMeansOffset : NULL, bnOut ? bnOut + cv->runningVariancesOffset : NULL,
			    (real)BATCH_NORM_EPSILON, (real)BATCH_NORM_MOMENTUM, forTesting == MODEL_TRAIN, model->actFuns[l], actOut, pl->type,
			    pl->pSize, pl->stride, pl->padding, pl->outWidth, pl->outHeight, pooled ? slab + cv->poolOffset : NULL, ws, wsBytes));
		}
	}

	/* [C][N][a*B+b] -> [N][C][b*A+a], in place through the workspace */
	const CONV_LAYER *last = &model->convLayer[nc - 1];
	int extA, extB;
	feature_extent(model, &extA, &extB);
	real *feat = z + zOffsets[nc] + last->outputOffset;
	const size_t featCount = (size_t)extA * extB * n * last->outChannels;
	HIP_CALL(fitre_hip_conv_to_fc(feat, last->outChannels, n, extA, extB, (real *)ws));
	HIP_CALL(fitre_hip_copy_d2d(feat, ws, sizeof(real) * featCount));

	int outputOffset = last->outputOffset;
	for (int l = 0; l < model->lLayers; l++) {
		if (l != 0) outputOffset = 0;
		const FC_LAYER *f = &model->fcLayer[l];
		real *out = z + zOffsets[l + 1 + nc];
		const long count = (long)f->out * n;
		/* W z + b, then the saved copy behind it, then the activation in place */
		HIP_CALL(fitre_hip_gemm(0, 0, f->out, n, f->in, 1.f, weights + wOffsets[l + nc], f->out,
		                        z + zOffsets[l + nc] + outputOffset, f->in, 0.f, out, f->out,
		                        (model->bias == 0) ? NULL : weights + bOffsets[l + nc], ws, wsBytes));
		HIP_CALL(fitre_hip_copy_d2d(out + count, out, sizeof(real) * (size_t)count));
		HIP_CALL(fitre_hip_activation_forward(f->actFun, out, out, count));
	}

	const real *logits = (model->lLayers == 0) ? feat : z + zOffsets[model->lLayers + nc];
	real loss = 0;
	HIP_CALL(fitre_hip_softmax_cross_entropy(logits, data->sampledTrainY, n, data->numClasses, probs, errors, &loss));
	HIP_CALL(fitre_hip_sync());
	return loss;
}

/* Multiply-adds of the convolution layers' two gradient products: what decides whether a pass is long enough for
 * the lanes to pay.  Ordering two lanes costs the host two runtime calls per dependency, a few microseconds each:
 * a pass of LeNet at batch 128 (1.5e8, kernels of 5 to 17 us) takes the same time either way (0.092 ms) and stays on
 * one lane; LeNet with batch norm at batch 1024 (1.2e9) takes 0.217 ms on two lanes against 0.227 on one, AlexNet
 * at batch 64 2.82 against 2.90 ms, VGG-11 with batch norm at batch 256 1.37 against 1.52 ms.  (While the largest
 * weight-gradient kernels filled the register file, two lanes lost on networks with little pooling / batch-norm
 * traffic per multiply-add, such as AlexNet, and a second limit kept those on one lane; the kernels of the delta
 * chain now find room beside every weight gradient and the limit is gone.) */
static double backward_conv_work(const CNN_MODEL *model, int n)
{
	double macs = 0;
	for (int c = 0; c < model->cLayers; c++) {
		const CONV_LAYER *l = &model->convLayer[c];
		macs += 2.0 * n * l->outHeight * l->outWidth * (double)l->outChannels * l->inChannels * l->kSize * l->kSize;
	}
	return macs;
}
#define LANE_WORK_THRESHOLD 1.0e9
/* The chain's bandwidth-bound steps (pooling, activation, batch norm: about 28 bytes per activation with batch norm, 16
 * without) of layer c - 1 run beside the weight gradient of layer c on lane 1, and the next input gradient waits for
 * them.  Where they are many per multiply-add of that weight gradient, it is planned for fewer compute units and the
 * chain has the rest of the chip to itself (fitre_hip_weight_grad_share).  Measured on VGG-11 with batch norm at batch
 * 256, bytes per thousand FLOP / best share: layer 1 49 / six eighths, layer 2 24 and layer 4 12 / seven or six
 * eighths (equal within the noise), layers 3 and 5 6 and 3 / the whole chip; the pass 1.32 against 1.37 ms.  A pass with
 * few such bytes overall (AlexNet at batch 64: about 400 FLOP per byte against 140) keeps the whole chip for every weight
 * gradient: 2.82 against 3.00 ms with the shares.  The share depends on the network alone, not on whether the lanes are
 * in use, so that one lane and two give the same bits. */
static double elementwise_bytes(const CONV_LAYER *l, int n)
{
	return (double)n * l->outHeight * l->outWidth * l->outChannels * (has_bn(l) ? 28.0 : 16.0);
}
static double backward_flop_per_elementwise_byte(const CNN_MODEL *model, int n)
{
	double bytes = 0;
	for (int c = 0; c < model->cLayers; c++) bytes += elementwise_bytes(&model->convLayer[c], n);
	return bytes > 0 ? 2.0 * backward_conv_work(model, n) / bytes : 0.0;
}
#define SHARE_INTENSITY_LIMIT 250.0
static int backward_shares_chip(const CNN_MODEL *model, int n)
{
	return backward_conv_work(model, n) >= LANE_WORK_THRESHOLD && backward_flop_per_elementwise_byte(model, n) < SHARE_INTENSITY_LIMIT;
}
/* eighths of the compute units the weight gradient of layer c is planned for */
static int weight_grad_eighths(const CNN_MODEL *model, int n, int c)
{
	if (c < 1) return 8;
	const CONV_LAYER *l = &model->convLayer[c];
	const double flops = 2.0 * n * l->outHeight * l->outWidth * (double)l->outChannels * l->inChannels * l->kSize * l->kSize;
	const double perKiloFlop = 1000.0 * elementwise_bytes(&model->convLayer[c - 1], n) / flops;
	return perKiloFlop >= 40.0 ? 6 : (perKiloFlop >= 10.0 ? 7 : 8);
}
/* -1: by the limit above (fitted on LeNet, VGG-11 and AlexNet); 0: one lane; 1: lanes, whatever the network */
static int g_backward_lanes = -1;
void fitreSetBackwardLanes(int mode) { g_backward_lanes = mode < 0 ? -1 : (mode ? 1 : 0); }
int fitreBackwardUsesLanes(CNN_MODEL *model, int batchSize)
{
	if (g_backward_lanes >= 0) return g_backward_lanes;
	return backward_conv_work(model, batchSize) >= LANE_WORK_THRESHOLD;
}
#define LANE_SELECT(lane_) do { if (lanes) HIP_CALL(fitre_hip_lane_select(lane_)); } while (0)
#define LANE_WAIT(waiter_, signaller_) do { if (lanes) HIP_CALL(fitre_hip_lane_wait(waiter_, signaller_)); } while (0)

void cnnBackward(CNN_MODEL *model, DEVICE_DATASET *data, real *devPtr, real *z, real *gradient, real *dx, real *delta,
                 real *delta_new, int offset, int batchSize, real *hostPtr)
{
	(void)offset;
	(void)hostPtr;
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	const real *weights = data->weights;
	const int n = batchSize, nc = model->cLayers;
	const int lanes = fitreBackwardUsesLanes(model, n);
	void *ws = (void *)devPtr; /* input-gradient partials (and the FC products' splits) */
	const size_t wsBytes = backward_dx_ws_bytes(model, model->batchSize);
	void *bnWs = (void *)((char *)devPtr + wsBytes);
	const size_t bnBytes = backward_bn_ws_bytes(model, model->batchSize);
	void *sideWs = (void *)((char *)bnWs + bnBytes);
	const size_t sideBytes = backward_side_ws_bytes(model, model->batchSize);
	char *preparedWs = (char *)sideWs + sideBytes;
	const void *prepared[MAX_LAYERS] = { NULL };
	int preparedPending = 0;

	if (nc < 1 || n < 1 || n > model->batchSize) {
		fprintf(stderr, "cnnBackward: needs at least one convolution layer and 1 <= batch (%d) <= model batch (%d)\n", n,
		        model->batchSize);
		exit(-1);
	}
	if (fitreBackwardUnsupportedLayer(model)) {
		fprintf(stderr, "cnnBackward: convolution layer %d has stride %d; only the first layer may be strided (the input "
		                "gradient is implemented for stride 1)\n",
		        fitreBackwardUnsupportedLayer(model), model->convLayer[fitreBackwardUnsupportedLayer(model) - 1].stride);
		exit(-1);
	}
	const CONV_LAYER *last = &model->convLayer[nc - 1];
	const int sharesChip = backward_shares_chip(model, n);

	/* Weight copies of the layers whose input gradient reads one: they depend on the weights only, so lane 2 makes
	 * them while the chain works through the linear layers. */
	{
		int any = 0;
		for (int c = 1; c < nc; c++) {
			fitre_conv_shape shape = conv_shape(&model->convLayer[c], n);
			/* the buffers are laid out for the model's batch size; a shape's need does not depend on the batch */
			const size_t bytes = fitre_hip_conv_input_grad_prepared_bytes(&shape);
			prepared[c] = NULL;
			if (bytes == 0 || !has_bn(&model->convLayer[c - 1])) continue;
			if (!any) {
				/* behind whatever the caller has queued on lane 0 (a weight update, say): the copies read the weights */
				LANE_WAIT(2, 0);
				LANE_SELECT(2);
			}
			any = 1;
			HIP_CALL(fitre_hip_conv_input_grad_prepare(&shape, weights + wOffsets[c], preparedWs, bytes));
			prepared[c] = preparedWs;
			preparedWs += (bytes + 255) & ~(size_t)255;
		}
		if (any) LANE_SELECT(0);
		preparedPending = any;
	}

	/* Linear layers, top down.  The delta of a layer (after its activation derivative) is written once, into the
	 * layer's dx slot -- the snapshot the Hessian-vector product and the KFAC factors read -- and everything that
	 * follows reads it there: the chain (lane 0) never writes a buffer that lane 1 still reads, so it never waits
	 * for lane 1.  The last product leaves the first convolution-side delta in the chain workspace, already in
	 * the convolution layout [C][N][a*B+b] (the reference permutes it separately, functions/cnn_backward.cu:330-348);
	 * the workspace is free until the last convolution layer's input gradient, which is queued behind the pass
	 * that reads this tensor. */
	real *features = (real *)ws;
	int extA, extB;
	feature_extent(model, &extA, &extB);
	fitre_fc_tail_layer tail[4];
	const int fusedTail = tail_shapes(model, n, tail);
	int tailFoldedPool = 0;
	if (fusedTail) {
		/* small layers (LeNet's 400-120-84-10): the whole tail in two launches on the chain's lane -- every delta into its
		 * slot, every weight and bias gradient, and the first convolution-side delta */
		for (int f = 0; f < model->lLayers; f++) {
			const FC_LAYER *l = &model->fcLayer[f];
			real *zl = z + zOffsets[f + nc + 1];
			tail[f].W = weights + wOffsets[f + nc];
			tail[f].zPre = zl + l->offset, tail[f].zPost = zl;
			tail[f].zin = z + zOffsets[f + nc] + ((f == 0) ? last->outputOffset : 0);
			tail[f].slot = dx + zOffsets[f + nc + 1];
			tail[f].dW = gradient + wOffsets[f + nc];
			tail[f].db = (model->bias != 0) ? gradient + bOffsets[f + nc] : NULL;
		}
		const POOL_LAYER *pl = &model->poolLayer[nc - 1];
		if (!has_bn(last) && pl->type == MAX_POOL && pl->pSize == 2 && pl->stride == 2 && pl->padding == 0 && pl->width == 2 * extA &&
		    pl->height == 2 * extB && pl->outWidth == extA && pl->outHeight == extB) {
			/* the top convolution layer's pool and activation steps ride on the launch that produces their delta */
			const real *slabT = z + zOffsets[nc];
			real *dslabT = dx + zOffsets[nc];
			HIP_CALL(fitre_hip_fc_tail_backward_pool_act(model->lLayers, tail, n, delta, extA, extB, features, model->actFuns[nc - 1], slabT,
			                                             slabT + last->activationOffset, dslabT, dslabT + last->activationOffset, sideWs,
			                                             sideBytes));
			tailFoldedPool = 1;
		} else {
			HIP_CALL(fitre_hip_fc_tail_backward(model->lLayers, tail, n, delta, extA, extB, features, sideWs, sideBytes));
		}
	}
	for (int f = fusedTail ? -1 : model->lLayers - 1; f >= 0; f--) {
		const FC_LAYER *l = &model->fcLayer[f];
		real *zl = z + zOffsets[f + nc + 1];
		real *slot = dx + zOffsets[f + nc + 1];
		const real *zin = z + zOffsets[f + nc] + ((f == 0) ? last->outputOffset : 0);

		/* delta .* f'(.) of the output layer; the layers below get theirs from the epilogue of the product above them.
		 * Without an activation it is the caller's delta as it stands: the product reads it there and leaves the copy in
		 * the slot on its way. */
		const real *cur_delta = slot;
		real *snapshot = NULL;
		if (f == model->lLayers - 1) {
			if (l->actFun == CNN_ACT_NONE || l->actFun == ACT_LINEAR) {
				cur_delta = delta;
				snapshot = slot;
			} else {
				HIP_CALL(fitre_hip_activation_backward(l->actFun, delta, zl + l->offset, zl, slot, (long)l->out * n));
			}
		}
		if (!snapshot) LANE_WAIT(1, 0);
		/* the chain goes straight on: delta of the layer below = f'(.) .* (W' * delta) */
		if (f > 0) {
			const FC_LAYER *below = &model->fcLayer[f - 1];
			real *zb = z + zOffsets[f + nc];
			HIP_CALL(fitre_hip_linear_input_grad(l->in, l->out, n, weights + wOffsets[f + nc], cur_delta, below->actFun,
			                                     zb + below->offset, zb, 0, 0, dx + zOffsets[f + nc], NULL, ws, wsBytes, snapshot));
		} else {
			HIP_CALL(fitre_hip_linear_input_grad(l->in, l->out, n, weights + wOffsets[f + nc], cur_delta, -1, NULL, NULL, extA, extB,
			                                     features, delta_new, ws, wsBytes, snapshot));
		}
		if (snapshot) LANE_WAIT(1, 0); /* lane 1 reads the slot the product has just filled */
		/* beside it, on lane 1, what nothing later in this pass reads: dW = delta * z', db = delta * 1 */
		LANE_SELECT(1);
		HIP_CALL(fitre_hip_linear_weight_grad(l->in, l->out, n, slot, zin, gradient + wOffsets[f + nc],
		                                      (model->bias != 0) ? gradient + bOffsets[f + nc] : NULL, sideWs, sideBytes));
		LANE_SELECT(0);
	}
	if (model->lLayers == 0) HIP_CALL(fitre_hip_fc_to_conv(delta, last->outChannels, n, extA, extB, features));

	/* delta as the layer above left it: a plain tensor, or the unsummed split partials of its input
	 * gradient (summed by the pool / activation pass below while it reads them) */
	fitre_split_view dview = { features, 1, 0 };
	/* The weight gradients of layers with very few channels end in a short reduction launch each: they are held back and
	 * made as one launch at the end of the pass.  Until then such a layer's blocks stay in a slice of lane 1's workspace of
	 * their own, and the layers after it work in what follows the slices. */
	size_t sideHeld = 0;
	HIP_CALL(fitre_hip_thin_reduce_defer(1));
	int poolFolded = tailFoldedPool;
	for (int c = nc - 1; c >= 0; c--) {
		const CONV_LAYER *l = &model->convLayer[c];
		const POOL_LAYER *p = &model->poolLayer[c];
		const real *slab = z + zOffsets[c + 1];
		real *dslab = dx + zOffsets[c + 1];
		const long perChannel = (long)n * l->outWidth * l->outHeight;
		const int act = model->actFuns[c];

		if (p->type != MAX_POOL && p->type != AVG_POOL && p->type != NO_POOL) {
			fprintf(stderr, "Unknown Pool Function... \n");
			exit(-1);
		}
		const real *actIn = has_bn(l) ? slab + l->batchNormOffset : slab;
		const real *actOut = slab + l->activationOffset;
		/* With batch norm and ReLU the fused pass derives the activation output from its input. */
		const int fusedRelu = has_bn(l) && act == CNN_ACT_RELU;
		if (c == nc - 1 && p->type == NO_POOL) {
			/* The forward pass rewrote this layer's activation output into the FC layout in place;
			 * rebuild it from the activation input (the reference reads the permuted buffer,
			 * functions/cnn_backward.cu:574-580). */
			if (!fusedRelu) HIP_CALL(fitre_hip_activation_forward(act, actIn, delta_new, perChannel * l->outChannels));
			actOut = delta_new;
		}
		const real *cur;
		if (poolFolded) {
			/* the layer above's input gradient went on through this layer's pool and activation in its own launch */
			poolFolded = 0;
			cur = dslab + l->activationOffset;
		} else if (has_bn(l)) {
			/* pool backward -> dx slab + 0; times f'(.) -> dx slab + activationOffset; batch-norm backward ->
			 * dx slab + batchNormOffset, its column sums being the bias gradient */
			HIP_CALL(fitre_hip_pool_act_bn_backward(p->type, act, dview.base, dview.splits, dview.stride, actIn,
			                                        fusedRelu ? NULL : actOut,
			                                        slab + l->batchNormOffset + l->variancesOffset, l->outChannels, n, p->width,
			                                        p->height, p->pSize, p->stride, p->padding, p->outWidth, p->outHeight,
			                                        (real)BATCH_NORM_EPSILON, dslab, dslab + l->activationOffset,
			                                        dslab + l->batchNormOffset,
			                                        (model->bias != 0) ? gradient + bOffsets[c] : NULL, bnWs, bnBytes));
			cur = dslab + l->batchNormOffset;
		} else {
			/* pool backward -> dx slab + 0; times f'(.) -> dx slab + activationOffset */
			HIP_CALL(fitre_hip_pool_act_backward(p->type, act, dview.base, actIn, actOut, l->outChannels, n, p->width, p->height,
			                                     p->pSize, p->stride, p->padding, p->outWidth, p->outHeight, dslab,
			                                     dslab + l->activationOffset));
			cur = dslab + l->activationOffset; /* its channel sums (the bias gradient) are taken on lane 1, below */
		}

		const real *input = (c == 0) ? data->currentBatch : z + zOffsets[c] + model->convLayer[c - 1].outputOffset;
		fitre_conv_shape shape = conv_shape(l, n);
		/* The weight gradient, whose result nothing later reads, goes to lane 1 as soon as this layer's delta is
		 * complete: it shares the matrix pipes with the input gradient below, and its kernels leave registers
		 * free on every SIMD, on which the bandwidth-bound kernels of the layer below (split reduction, pooling,
		 * batch norm) run while it keeps the pipes busy.  Queued only behind the input gradient it started 10 us
		 * after that had ended, with no matrix kernel running in between (measured: the pass 0.8 % longer). */
		const int beside = fitre_hip_conv_weight_grad_runs_beside(&shape);
		if (beside) LANE_WAIT(1, 0);
		if (c != 0) {
			if (has_bn(&model->convLayer[c - 1])) {
				if (prepared[c] && preparedPending) { /* the chain's first use of a copy lane 2 made */
					LANE_WAIT(0, 2);
					preparedPending = 0;
				}
				HIP_CALL(fitre_hip_conv_input_grad_split_prepared(&shape, cur, weights + wOffsets[c], prepared[c], delta, ws, wsBytes,
				                                                  &dview));
			} else {
				const CONV_LAYER *lb = &model->convLayer[c - 1];
				const POOL_LAYER *pb = &model->poolLayer[c - 1];
				if (pb->type == MAX_POOL && pb->pSize == 2 && pb->stride == 2 && pb->padding == 0 && pb->width == 2 * shape.inA &&
				    pb->height == 2 * shape.inB && pb->outWidth == shape.inA && pb->outHeight == shape.inB &&
				    fitre_hip_conv_input_grad_folds_pool(&shape)) {
					const real *slabB = z + zOffsets[c];
					real *dslabB = dx + zOffsets[c];
					HIP_CALL(fitre_hip_conv_input_grad_pool_act(&shape, cur, weights + wOffsets[c], delta, model->actFuns[c - 1], slabB,
					                                            slabB + lb->activationOffset, dslabB, dslabB + lb->activationOffset, ws,
					                                            wsBytes));
					poolFolded = 1;
				} else {
					HIP_CALL(fitre_hip_conv_input_grad(&shape, cur, weights + wOffsets[c], delta, ws, wsBytes));
				}
				dview.base = delta, dview.splits = 1, dview.stride = 0;
			}
		}
		/* A weight gradient the device layer does not want beside other matrix kernels (none by now) stays in line; its
		 * workspace is lane 1's, so the lanes are ordered around it. */
		if (!beside) LANE_WAIT(1, 0);
		if (beside) {
			LANE_SELECT(1);
		} else {
			LANE_WAIT(0, 1);
		}
		/* without batch norm the bias gradient is taken here as well (with batch norm it is a by-product of its
		 * backward pass above); nothing in the chain reads either */
		HIP_CALL(fitre_hip_weight_grad_share(sharesChip ? weight_grad_eighths(model, n, c) : 8));
		HIP_CALL(fitre_hip_conv_weight_bias_grad(&shape, input, cur, gradient + wOffsets[c],
		                                         (!has_bn(l) && model->bias != 0) ? gradient + bOffsets[c] : NULL,
		                                         (char *)sideWs + sideHeld, sideBytes - sideHeld));
		sideHeld += fitre_hip_thin_reduce_bytes(&shape);
		if (c == 0) HIP_CALL(fitre_hip_thin_reduce_defer(0)); /* every held reduction, on the lane their blocks were made on */
		if (beside) LANE_SELECT(0);
	}
	HIP_CALL(fitre_hip_weight_grad_share(8));
	HIP_CALL(fitre_hip_sync());
}

real evaluateCNNModel(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *probs,
                      real *lossFuncErrors, int offset, int curBatchSize)
{
	return cnnForward(model, data, scratch, z, probs, lossFuncErrors, offset, curBatchSize, MODEL_TRAIN);
}

real computeCNNGradient(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *dx, real *probs,
                        real *lossFuncErrors, real *gradient, int offset, int curBatchSize, real weightDecay)
{
	real *oldDevPtr = scratch->nextDevPtr;
	real *oldHostPtr = scratch->nextHostPtr;
	real *oldPagePtr = scratch->nextPageLckPtr;

	real *errors = scratch->nextDevPtr;
	real *errors_1 = errors + model->maxDeltaSize;
	real *nextDevPtr = errors_1 + model->maxDeltaSize;
	scratch->nextDevPtr = nextDevPtr;

	real lossVal = evaluateCNNModel(model, data, scratch, z, probs, lossFuncErrors, offset, curBatchSize);

	HIP_CALL(fitre_hip_copy_d2d(errors, lossFuncErrors, sizeof(real) * (size_t)data->numClasses * curBatchSize));
	cnnBackward(model, data, nextDevPtr, z, gradient, dx, errors, errors_1, offset, curBatchSize, scratch->nextHostPtr);

	if (weightDecay != 0) HIP_CALL(fitre_hip_axpy(model->pSize, weightDecay, data->weights, gradient));
	HIP_CALL(fitre_hip_sync());

	scratch->nextDevPtr = oldDevPtr;
	scratch->nextHostPtr = oldHostPtr;
	scratch->nextPageLckPtr = oldPagePtr;
	return lossVal;
}

real computeAccuracy(real *probs, real *target, int rows, int numClasses, real *devPtr, real *pageLckPtr)
{
	HIP_CALL(fitre_hip_accuracy_hits(probs, target, rows, numClasses, devPtr));
	HIP_CALL(fitre_hip_dot(rows, devPtr, devPtr, pageLckPtr)); /* complete on return */
	return (real)((*pageLckPtr * 100.) / (real)rows);
}

void computeCrossEntropyError(real *probs, int rows, int num_classes, real *target, real *errors)
{
	HIP_CALL(fitre_hip_cross_entropy_error(probs, target, rows, num_classes, errors));
	HIP_CALL(fitre_hip_sync());
}

void getMultinomialDistSample(real *probs, int samples, int numClasses, real *distClasses, real *devPtr)
{
	HIP_CALL(fitre_hip_random_uniform(devPtr, samples));
	HIP_CALL(fitre_hip_multinomial_classes(probs, devPtr, samples, numClasses, distClasses));
	HIP_CALL(fitre_hip_sync());
}

void computeDistributionErrors(real *probs, real *distTarget, real *distError, int rows, int num_classes, real *devPtr,
                               real *hostPtr)
{
	(void)hostPtr;
	getMultinomialDistSample(probs, rows, num_classes, distTarget, devPtr);
	computeCrossEntropyError(probs, rows, num_classes, distTarget, distError);
}
