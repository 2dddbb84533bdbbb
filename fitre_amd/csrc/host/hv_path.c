/*
 * Hessian-vector product by R-operator passes (functions/cnn_hessian_vec.cu:18-122,
 * cnn_hv_forward.cu:53-222, cnn_hv_backward.cu:70-912, rop_fc_layer.cu:34-133) and the
 * quadratic-model step (functions/model_reduction.cu:20-93), as C host code over the C-ABI
 * device layer.  R{.} is the directional derivative along `vector` in weight space.  Every
 * product is one of the convolution / GEMM entry points of the gradient path applied to a
 * different pair of operands: R{conv(z, W)} = conv(z, V) + conv(R{z}, W), and likewise for the
 * weight and input gradients; batch-norm forward's R-operator is its backward formula.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include "fitre_hv.h"
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
static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }
static size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

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

static size_t largest_weight_block(const CNN_MODEL *model)
{
	size_t m = 1;
	for (int l = 0; l < model->cLayers; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		m = max_sz(m, (size_t)c->outChannels * c->inChannels * c->kSize * c->kSize);
	}
	return m;
}

static size_t hv_ws_bytes(const CNN_MODEL *model, int batch)
{
	size_t need = 256;
	for (int i = 0; i < model->cLayers; i++) {
		const CONV_LAYER *c = &model->convLayer[i];
		fitre_conv_shape s = conv_shape(c, batch);
		need = max_sz(need, fitre_hip_conv_forward_workspace(&s));
		need = max_sz(need, fitre_hip_conv_weight_grad_workspace(&s));
		if (i != 0) need = max_sz(need, fitre_hip_conv_input_grad_workspace(&s));
		for (int kind = 0; kind < 3; kind++) need = max_sz(need, fitre_hip_conv_pair_workspace(&s, kind));
		need = max_sz(need, fitre_hip_batch_norm_workspace(c->outChannels, (long)batch * c->outWidth * c->outHeight));
	}
	if (model->cLayers > 0) {
		int extA, extB;
		feature_extent(model, &extA, &extB);
		need = max_sz(need, sizeof(real) * (size_t)extA * extB * batch * model->convLayer[model->cLayers - 1].outChannels);
	}
	for (int i = 0; i < model->lLayers; i++) {
		const FC_LAYER *f = &model->fcLayer[i];
		need = max_sz(need, fitre_hip_gemm_workspace(f->out, batch, f->in));
		need = max_sz(need, fitre_hip_gemm_workspace(f->out, f->in, batch));
		need = max_sz(need, fitre_hip_gemm_workspace(f->in, batch, f->out));
	}
	return up256(need);
}

/* [rz | rError | four delta-sized buffers | one weight block | workspace], each 256-byte aligned */
long cnnHvMemRequired(CNN_MODEL *model)
{
	size_t bytes = up256(sizeof(real) * (size_t)model->zSize) + 5 * up256(sizeof(real) * (size_t)model->maxDeltaSize) +
	               up256(sizeof(real) * largest_weight_block(model)) + hv_ws_bytes(model, model->batchSize) + 512;
	return (long)(bytes / sizeof(real));
}

/* activation output of conv layer l in the convolution layout: the forward pass permuted the last
 * layer's unpooled output in place, so it is rebuilt from the activation input into tmp */
static const real *conv_act_out(const CNN_MODEL *model, int l, const real *z, int n, real *tmp)
{
	const CONV_LAYER *c = &model->convLayer[l];
	const real *slab = z + model->zOffsets[l + 1];
	if (l == model->cLayers - 1 && model->poolLayer[l].type == NO_POOL) {
		const real *actIn = has_bn(c) ? slab + c->batchNormOffset : slab;
		HIP_CALL(fitre_hip_activation_forward(model->actFuns[l], actIn, tmp, (long)n * c->activationVolumn));
		return tmp;
	}
	return slab + c->activationOffset;
}

static void rop_forward(CNN_MODEL *model, const real *weights, const real *vector, const real *x, const real *z, real *rz,
                        int n, real *tmp, real *actbuf, void *ws, size_t wsBytes)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	const int nc = model->cLayers, bias = model->bias != 0;
	for (int l = 0; l < nc; l++) {
		const CONV_LAYER *c = &model->convLayer[l];
		const POOL_LAYER *p = &model->poolLayer[l];
		const real *slab = z + zOffsets[l + 1];
		real *rslab = rz + zOffsets[l + 1];
		const long perChannel = (long)n * c->outWidth * c->outHeight, count = perChannel * c->outChannels;
		const real *in = (l == 0) ? x : z + zOffsets[l] + model->convLayer[l - 1].outputOffset;
		fitre_conv_shape shape = conv_shape(c, n);
		/* R{conv} = conv(z_in, V) + Vb + conv(R{z_in}, W): one launch whose reduction runs over both products where the
		 * shape allows, else two products and an addition */
		const real *vb = bias ? vector + bOffsets[l] : NULL;
		if (l > 0 && fitre_hip_conv_pair_supported(&shape, 0)) {
			const real *rin = rz + zOffsets[l] + model->convLayer[l - 1].outputOffset;
			HIP_CALL(fitre_hip_conv_forward_pair(&shape, in, vector + wOffsets[l], rin, weights + wOffsets[l], vb, rslab, ws, wsBytes));
		} else {
			HIP_CALL(fitre_hip_conv_forward(&shape, in, vector + wOffsets[l], vb, rslab, ws, wsBytes));
			if (l > 0) {
				const real *rin = rz + zOffsets[l] + model->convLayer[l - 1].outputOffset;
				HIP_CALL(fitre_hip_conv_forward(&shape, rin, weights + wOffsets[l], NULL, tmp, ws, wsBytes));
				HIP_CALL(fitre_hip_axpy((int)count, 1.f, tmp, rslab));
			}
		}
		const real *actOut = conv_act_out(model, l, z, n, actbuf);
		real *ract = rslab + c->activationOffset;
		if (has_bn(c)) {
			/* batch norm forward's R-operator is its backward formula on R{x}; with the activation's and the pooling's in one
			 * pass over R{x} and zhat where the shapes allow */
			const int pooled = p->type == MAX_POOL || p->type == AVG_POOL;
			if (p->type != NO_POOL && !pooled) {
				fprintf(stderr, "Unknown Pool Function... \n");
				exit(-1);
			}
			HIP_CALL(fitre_hip_bn_act_pool_rop_forward(rslab, slab + c->batchNormOffset, actOut,
			                                           slab + c->batchNormOffset + c->variancesOffset, c->outChannels, n,
			                                           pooled ? p->width : c->outWidth, pooled ? p->height : c->outHeight,
			                                           (real)BATCH_NORM_EPSILON, model->actFuns[l], rslab + c->batchNormOffset, ract, p->type,
			                                           p->pSize, p->stride, p->padding, p->outWidth, p->outHeight,
			                                           pooled ? rslab + c->poolOffset : NULL, ws, wsBytes));
		} else {
			HIP_CALL(fitre_hip_activation_backward(model->actFuns[l], rslab, slab, actOut, ract, count));
			if (p->type == MAX_POOL || p->type == AVG_POOL)
				HIP_CALL(fitre_hip_pool_forward_routed(p->type, ract, actOut, c->outChannels, n, p->width, p->height, p->pSize,
				                                       p->stride, p->padding, p->outWidth, p->outHeight, rslab + c->poolOffset));
			else if (p->type != NO_POOL) {
				fprintf(stderr, "Unknown Pool Function... \n");
				exit(-1);
			}
		}
	}
	/* the feature permute of the forward pass, on R{z} */
	const CONV_LAYER *last = &model->convLayer[nc - 1];
	int extA, extB;
	feature_extent(model, &extA, &extB);
	real *rfeat = rz + zOffsets[nc] + last->outputOffset;
	const size_t featCount = (size_t)extA * extB * n * last->outChannels;
	HIP_CALL(fitre_hip_conv_to_fc(rfeat, last->outChannels, n, extA, extB, (real *)ws));
	HIP_CALL(fitre_hip_copy_d2d(rfeat, ws, sizeof(real) * featCount));

	for (int f = 0; f < model->lLayers; f++) {
		const FC_LAYER *fc = &model->fcLayer[f];
		const int at = nc + f, off = (f == 0) ? last->outputOffset : 0;
		const real *zin = z + zOffsets[at] + off, *rzin = rz + zOffsets[at] + off;
		const real *zl = z + zOffsets[at + 1];
		real *rzl = rz + zOffsets[at + 1];
		real *rpre = rzl + fc->offset;
		/* R{W z + b} = V z + Vb + W R{z} */
		HIP_CALL(fitre_hip_gemm(0, 0, fc->out, n, fc->in, 1.f, vector + wOffsets[at], fc->out, zin, fc->in, 0.f, rpre, fc->out,
		                        bias ? vector + bOffsets[at] : NULL, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm(0, 0, fc->out, n, fc->in, 1.f, weights + wOffsets[at], fc->out, rzin, fc->in, 1.f, rpre, fc->out,
		                        NULL, ws, wsBytes));
		HIP_CALL(fitre_hip_activation_backward(fc->actFun, rpre, zl + fc->offset, zl, rzl, (long)fc->out * n));
	}
}

static void rop_backward(CNN_MODEL *model, const real *weights, const real *vector, const real *x, const real *z,
                         const real *rz, const real *dx, const real *lossFuncErrors, const real *rError, real *hv, int n,
                         int numClasses, real *rdelta, real *rnext, real *dout, real *tmp, real *wtmp, void *ws, size_t wsBytes)
{
	const int *wOffsets = model->wOffsets, *bOffsets = model->bOffsets, *zOffsets = model->zOffsets;
	const int nc = model->cLayers, bias = model->bias != 0;
	const CONV_LAYER *last = &model->convLayer[nc - 1];
	real *t;
	HIP_CALL(fitre_hip_copy_d2d(rdelta, rError, sizeof(real) * (size_t)numClasses * n));
	HIP_CALL(fitre_hip_copy_d2d(dout, lossFuncErrors, sizeof(real) * (size_t)numClasses * n));

	for (int f = model->lLayers - 1; f >= 0; f--) {
		const FC_LAYER *fc = &model->fcLayer[f];
		const int at = nc + f, off = (f == 0) ? last->outputOffset : 0;
		const real *zl = z + zOffsets[at + 1], *rzl = rz + zOffsets[at + 1];
		const real *zin = z + zOffsets[at] + off, *rzin = rz + zOffsets[at] + off;
		const real *dpre = dx + zOffsets[at + 1];
		/* R{delta f'(x)} -> tmp */
		HIP_CALL(fitre_hip_activation_rop_backward(fc->actFun, rdelta, dout, zl + fc->offset, zl, rzl + fc->offset, tmp,
		                                           (long)fc->out * n));
		/* R{dW} = R{d} z' + d R{z}',  R{db} = R{d} 1 */
		HIP_CALL(fitre_hip_gemm(0, 1, fc->out, fc->in, n, 1.f, tmp, fc->out, zin, fc->in, 0.f, hv + wOffsets[at], fc->out, NULL, ws,
		                        wsBytes));
		HIP_CALL(fitre_hip_gemm(0, 1, fc->out, fc->in, n, 1.f, dpre, fc->out, rzin, fc->in, 1.f, hv + wOffsets[at], fc->out, NULL,
		                        ws, wsBytes));
		if (bias) HIP_CALL(fitre_hip_row_sum(tmp, fc->out, n, hv + bOffsets[at]));
		/* R{W' d} = V' d + W' R{d}; the gradient at the output of the layer below is W' d */
		HIP_CALL(fitre_hip_gemm(1, 0, fc->in, n, fc->out, 1.f, vector + wOffsets[at], fc->out, dpre, fc->out, 0.f, rnext, fc->in,
		                        NULL, ws, wsBytes));
		HIP_CALL(fitre_hip_gemm(1, 0, fc->in, n, fc->out, 1.f, weights + wOffsets[at], fc->out, tmp, fc->out, 1.f, rnext, fc->in,
		                        NULL, ws, wsBytes));
		if (f > 0)
			HIP_CALL(fitre_hip_gemm(1, 0, fc->in, n, fc->out, 1.f, weights + wOffsets[at], fc->out, dpre, fc->out, 0.f, dout, fc->in,
			                        NULL, ws, wsBytes));
		t = rdelta, rdelta = rnext, rnext = t;
	}
	{
		int extA, extB;
		feature_extent(model, &extA, &extB);
		HIP_CALL(fitre_hip_fc_to_conv(rdelta, last->outChannels, n, extA, extB, rnext));
		t = rdelta, rdelta = rnext, rnext = t;
	}
	for (int c = nc - 1; c >= 0; c--) {
		const CONV_LAYER *l = &model->convLayer[c];
		const POOL_LAYER *p = &model->poolLayer[c];
		const real *slab = z + zOffsets[c + 1], *rslab = rz + zOffsets[c + 1], *dslab = dx + zOffsets[c + 1];
		const long perChannel = (long)n * l->outWidth * l->outHeight, count = perChannel * l->outChannels;
		const int bn = has_bn(l);
		const real *actIn = bn ? slab + l->batchNormOffset : slab;
		const real *ractIn = bn ? rslab + l->batchNormOffset : rslab;
		const real *actOut = conv_act_out(model, c, z, n, dout); /* dout is free once the FC layers are done */
		const real *dc = dslab + l->activationOffset; /* gradient at the convolution output */
		real *rdc;
		if (bn) {
			/* routing through the pooling, R{delta f'(x)} and the batch-norm R-step: one pass that leaves the sums, one that
			 * applies the formula (the separate passes where the shape does not allow it).  delta at the activation output is
			 * the dx snapshot at +0; tmp takes the routed R{delta} when the passes run separately. */
			const int pooled = p->type != NO_POOL;
			HIP_CALL(fitre_hip_pool_act_bn_rop_backward(
			    p->type, model->actFuns[c], rdelta, dslab, slab + l->batchNormOffset, actOut, rslab + l->batchNormOffset,
			    dslab + l->activationOffset, rslab, dslab + l->batchNormOffset, slab + l->batchNormOffset + l->variancesOffset,
			    l->outChannels, n, pooled ? p->width : l->outWidth, pooled ? p->height : l->outHeight, p->pSize, p->stride, p->padding,
			    p->outWidth, p->outHeight, (real)BATCH_NORM_EPSILON, tmp, rnext, rdelta, ws, wsBytes));
			dc = dslab + l->batchNormOffset;
			rdc = rdelta;
		} else {
			/* R through the pooling: the routing of the gradient itself */
			if (p->type == NO_POOL) {
				t = rdelta, rdelta = rnext, rnext = t; /* rnext now holds R{delta at the activation output} */
			} else {
				HIP_CALL(fitre_hip_pool_backward(p->type, rdelta, actOut, l->outChannels, n, p->width, p->height, p->pSize, p->stride,
				                                 p->padding, p->outWidth, p->outHeight, rnext));
			}
			/* R{delta f'(x)}; delta at the activation output is the dx snapshot at +0 */
			HIP_CALL(fitre_hip_activation_rop_backward(model->actFuns[c], rnext, dslab, actIn, actOut, ractIn, rdelta, count));
			rdc = rdelta;
		}
		if (bias) HIP_CALL(fitre_hip_channel_sum(rdc, l->outChannels, perChannel, hv + bOffsets[c], ws, wsBytes));
		const real *in = (c == 0) ? x : z + zOffsets[c] + model->convLayer[c - 1].outputOffset;
		const long wcount = (long)l->outChannels * l->inChannels * l->kSize * l->kSize;
		fitre_conv_shape shape = conv_shape(l, n);
		/* R{dW} = dW(z_in, R{dc}) + dW(R{z_in}, dc); the input of the first layer carries no R term */
		if (c == 0) {
			HIP_CALL(fitre_hip_conv_weight_grad(&shape, in, rdc, hv + wOffsets[c], ws, wsBytes));
		} else {
			const real *rin = rz + zOffsets[c] + model->convLayer[c - 1].outputOffset;
			if (fitre_hip_conv_pair_supported(&shape, 2)) {
				HIP_CALL(fitre_hip_conv_weight_grad_pair(&shape, in, rdc, rin, dc, hv + wOffsets[c], ws, wsBytes));
			} else {
				HIP_CALL(fitre_hip_conv_weight_grad(&shape, in, rdc, hv + wOffsets[c], ws, wsBytes));
				HIP_CALL(fitre_hip_conv_weight_grad(&shape, rin, dc, wtmp, ws, wsBytes));
				HIP_CALL(fitre_hip_axpy((int)wcount, 1.f, wtmp, hv + wOffsets[c]));
			}
			/* R{dX} = dX(R{dc}, W) + dX(dc, V) */
			real *other = (rdc == rdelta) ? rnext : rdelta;
			const long inCount = (long)n * l->height * l->width * l->inChannels;
			if (fitre_hip_conv_pair_supported(&shape, 1)) {
				HIP_CALL(fitre_hip_conv_input_grad_pair(&shape, rdc, weights + wOffsets[c], dc, vector + wOffsets[c], other, ws, wsBytes));
			} else {
				HIP_CALL(fitre_hip_conv_input_grad(&shape, rdc, weights + wOffsets[c], other, ws, wsBytes));
				HIP_CALL(fitre_hip_conv_input_grad(&shape, dc, vector + wOffsets[c], tmp, ws, wsBytes));
				HIP_CALL(fitre_hip_axpy((int)inCount, 1.f, tmp, other));
			}
			if (other != rdelta) t = rdelta, rdelta = rnext, rnext = t;
		}
	}
}

void cnnHv(CNN_MODEL *model, DEVICE_DATASET *data, real *z, real *probs, real *lossFuncErrors, real *dx, real *vector,
           real *hv, int s, int curBatchSize, real *devPtr, real *hostPtr, real weightDecay)
{
	(void)s, (void)hostPtr, (void)weightDecay;
	const int n = curBatchSize, nc = model->cLayers;
	if (nc < 1 || model->lLayers < 1 || n < 1 || n > model->batchSize) {
		fprintf(stderr, "cnnHv: needs convolution and linear layers and 1 <= batch (%d) <= model batch (%d)\n", n, model->batchSize);
		exit(-1);
	}
	if (fitreBackwardUnsupportedLayer(model)) {
		fprintf(stderr, "cnnHv: convolution layer %d has stride %d; only the first layer may be strided\n",
		        fitreBackwardUnsupportedLayer(model), model->convLayer[fitreBackwardUnsupportedLayer(model) - 1].stride);
		exit(-1);
	}
	const size_t dBytes = up256(sizeof(real) * (size_t)model->maxDeltaSize);
	char *base = (char *)(((size_t)devPtr + 255) & ~(size_t)255);
	real *rz = (real *)base;
	base += up256(sizeof(real) * (size_t)model->zSize);
	real *rError = (real *)base, *rdelta = (real *)(base + dBytes), *rnext = (real *)(base + 2 * dBytes);
	real *dout = (real *)(base + 3 * dBytes), *tmp = (real *)(base + 4 * dBytes);
	base += 5 * dBytes;
	real *wtmp = (real *)base;
	base += up256(sizeof(real) * largest_weight_block(model));
	void *ws = base;
	const size_t wsBytes = hv_ws_bytes(model, model->batchSize);

	rop_forward(model, data->weights, vector, data->currentBatch, z, rz, n, tmp, dout, ws, wsBytes);
	const real *rlogits = rz + model->zOffsets[nc + model->lLayers];
	HIP_CALL(fitre_hip_cross_entropy_rop_error(rlogits, probs, n, data->numClasses, rError));
	rop_backward(model, data->weights, vector, data->currentBatch, z, rz, dx, lossFuncErrors, rError, hv, n, data->numClasses,
	             rdelta, rnext, dout, tmp, wtmp, ws, wsBytes);
	HIP_CALL(fitre_hip_sync());
}

real computeQuadraticModel(CNN_MODEL *model, DEVICE_DATASET *data, real *z, real *probs, real *lossFuncErrors, real *dx,
                           real *gradient, real *vector, real delta, int offset, int curBatchSize, real weightDecay,
                           real *devPtr, real *hostPtr, real *pageLckPtr)
{
	real *gradVecDot = pageLckPtr, *vHv = pageLckPtr + 1, *nrmVec = pageLckPtr + 2;
	real *hv = devPtr;
	real *nextDevPtr = hv + model->pSize;
	const int components = model->pSize;
	real alpha, step;

	cnnHv(model, data, z, probs, lossFuncErrors, dx, vector, hv, offset, curBatchSize, nextDevPtr, hostPtr, weightDecay);
	/* the reference adds weightDecay * weights (not * vector) here, functions/model_reduction.cu:50-52 */
	HIP_CALL(fitre_hip_axpy(components, weightDecay, data->weights, hv));
	HIP_CALL(fitre_hip_dot(components, hv, vector, vHv));
	HIP_CALL(fitre_hip_nrm2(components, vector, nrmVec));
	HIP_CALL(fitre_hip_dot(components, gradient, vector, gradVecDot));
	if (*vHv < 0) { /* negative curvature: go to the boundary */
		alpha = delta / (*nrmVec);
		HIP_CALL(fitre_hip_scal(components, alpha, vector));
		HIP_CALL(fitre_hip_sync());
		return (real)(0.5 * (*vHv) * alpha * alpha - (*gradVecDot) * alpha);
	}
	step = (*gradVecDot) / (*vHv + (real)1e-6);
	step = fminf(step, delta / (*nrmVec + (real)1e-16));
	HIP_CALL(fitre_hip_scal(components, step, vector));
	HIP_CALL(fitre_hip_sync());
	return (real)((*vHv) * 0.5 * step * step - (*gradVecDot) * step);
}
