// Convolution gradients of layers with very few channels (LeNet: 3 -> 6 and 6 -> 16 with 5 x 5 windows).
//
// With six or sixteen output channels a 32 x 32 MFMA block is a tenth to a half full and the tile engine's
// 64-row tiles a tenth: such layers are bound by launch and load latency there, not by arithmetic (two
// GFLOP per pass at batch 1024).  Here both gradients are computed with ordinary vector multiply-adds by
// workgroups that keep one image at a time in LDS:
//
//   input gradient   one thread per input cell (n, a, b), Cin accumulators in registers; the image's delta
//                    (all output channels) and the weights ([co][tap][ci]: the channels of a tap are one or two
//                    broadcast 16-byte reads) in LDS;
//   weight gradient  one thread per (patch index k = (ci, ta, tb), position slice), Cout accumulators in
//                    registers; per position one LDS read of the input cell and Cout / 4 broadcast 16-byte
//                    reads of delta (stored [position][channel]); slices are added in a fixed order, every
//                    workgroup leaves one partial Cout x K block and splitk_reduce sums the blocks in
//                    workgroup order -- the result does not depend on scheduling.
#pragma once
#include "conv_common.h"

namespace fitre {

constexpr int kThinMaxChannels = 16; // accumulators a thread holds
constexpr int kThinLdsFloats = 12288; // 48 KB of staging per workgroup

struct ThinConvParams {
	const float *x;     // [Cin][N][inA][inB]   (weight gradient)
	const float *delta; // [Cout][N][outA][outB]
	const float *w;     // [Cout][Cin][k][k]     (input gradient)
	int cin, cout, samples, inA, inB, outA, outB, ksize, stride, pad;
	int imagesPerGroup;
	FastDiv divInB, divOutB, divK, divKK, divCells, divOcells;
};

// ---- input gradient (stride 1): dx[ci][n][a][b] = sum_co sum_taps W[co][ci][ta][tb] * delta[co][n][a - ta + p][b - tb + p]
// LDS: [weights as [co][tap][CIN] | delta of the group's images as [image][co][outA * outB]]
// KS: window extent known at compile time (the tap loops are unrolled: all of a channel's delta reads in flight), 0: any
template <int CIN, int KS>
__global__ void __launch_bounds__(256) thin_input_grad_kernel(const ThinConvParams p, float *dx)
{
	extern __shared__ __align__(16) float thin_lds[];
	const int tid = threadIdx.x;
	const int cells = p.inA * p.inB, ocells = p.outA * p.outB, taps = p.ksize * p.ksize;
	const int n0 = blockIdx.x * p.imagesPerGroup;
	const int imgs = (p.samples - n0 < p.imagesPerGroup) ? p.samples - n0 : p.imagesPerGroup;
	const size_t oplane = (size_t)p.samples * ocells, iplane = (size_t)p.samples * cells;
	float *wl = thin_lds;
	float *dl = thin_lds + p.cout * taps * CIN;
	// weights: W[co][ci][tap] -> wl[(co * taps + tap) * CIN + ci], zero for ci >= cin
	for (int i = tid; i < p.cout * taps * CIN; i += 256) {
		const int ci = i % CIN, r = i / CIN;
		uint32_t co, tap;
		p.divKK.divmod((uint32_t)r, co, tap);
		wl[i] = (ci < p.cin) ? p.w[((size_t)co * p.cin + ci) * taps + tap] : 0.f;
	}
	// delta, eight loads of a thread in flight at a time
	const int total = imgs * p.cout * ocells;
	for (int base = tid; base < total; base += 256 * 8) {
		float v[8];
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int i = base + 256 * u;
			uint32_t t, q, img, co;
			p.divOcells.divmod((uint32_t)(i < total ? i : 0), t, q);
			img = t / (uint32_t)p.cout, co = t - img * (uint32_t)p.cout;
			v[u] = (i < total) ? p.delta[(size_t)co * oplane + (size_t)(n0 + (int)img) * ocells + q] : 0.f;
		}
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int i = base + 256 * u;
			if (i < total) dl[i] = v[u];
		}
	}
	__syncthreads();
	for (int pos = tid; pos < imgs * cells; pos += 256) {
		uint32_t img, cell, a, b;
		p.divCells.divmod((uint32_t)pos, img, cell);
		p.divInB.divmod(cell, a, b);
		float acc[CIN];
#pragma unroll
		for (int ci = 0; ci < CIN; ci++) acc[ci] = 0.f;
		const float *dimg = dl + (int)img * p.cout * ocells;
		for (int co = 0; co < p.cout; co++) {
			const float *wco = wl + co * taps * CIN;
			const float *dco = dimg + co * ocells;
			auto tap = [&](int ta, int tb, int ks) {
				const int oa = (int)a - ta + p.pad, ob = (int)b - tb + p.pad;
				const bool ok = ((unsigned)oa < (unsigned)p.outA) & ((unsigned)ob < (unsigned)p.outB);
				const float d = dco[ok ? oa * p.outB + ob : 0] * (ok ? 1.f : 0.f);
				const float4 *wq = reinterpret_cast<const float4 *>(wco + (ta * ks + tb) * CIN); // the same for every lane
#pragma unroll
				for (int g = 0; g < CIN / 4; g++) {
					const float4 wv = wq[g];
					acc[4 * g] = fmaf(wv.x, d, acc[4 * g]);
					acc[4 * g + 1] = fmaf(wv.y, d, acc[4 * g + 1]);
					acc[4 * g + 2] = fmaf(wv.z, d, acc[4 * g + 2]);
					acc[4 * g + 3] = fmaf(wv.w, d, acc[4 * g + 3]);
				}
			};
			if constexpr (KS > 0) {
#pragma unroll
				for (int ta = 0; ta < KS; ta++)
#pragma unroll
					for (int tb = 0; tb < KS; tb++) tap(ta, tb, KS);
			} else {
				for (int ta = 0; ta < p.ksize; ta++)
					for (int tb = 0; tb < p.ksize; tb++) tap(ta, tb, p.ksize);
			}
		}
#pragma unroll
		for (int ci = 0; ci < CIN; ci++)
			if (ci < p.cin) dx[(size_t)ci * iplane + (size_t)n0 * cells + pos] = acc[ci];
	}
}

// ---- weight gradient: dW[co][k] = sum over positions of delta[co][position] * patch[position][k]
// blockDim = 512.  LDS: [x of one image | delta of one image as [position][COUT] | slice sums]
template <int COUT>
__global__ void __launch_bounds__(512) thin_weight_grad_kernel(const ThinConvParams p, float *partial)
{
	extern __shared__ __align__(16) float thin_lds[];
	const int tid = threadIdx.x;
	const int K = p.cin * p.ksize * p.ksize;
	const int cells = p.inA * p.inB, ocells = p.outA * p.outB;
	const int slices = 512 / K; // >= 1 (host checks K <= 512)
	float *xs = thin_lds;
	float *ds = thin_lds + ((cells * p.cin + 3) & ~3);
	const int k = tid % K, slice = tid / K;
	const bool live = slice < slices;
	uint32_t ci, tap, ta, tb;
	p.divKK.divmod((uint32_t)k, ci, tap);
	p.divK.divmod(tap, ta, tb);
	float acc[COUT];
#pragma unroll
	for (int c = 0; c < COUT; c++) acc[c] = 0.f;
	const size_t oplane = (size_t)p.samples * ocells, iplane = (size_t)p.samples * cells;
	const int n0 = blockIdx.x * p.imagesPerGroup;
	const int imgs = (p.samples - n0 < p.imagesPerGroup) ? p.samples - n0 : p.imagesPerGroup;
	for (int img = 0; img < imgs; img++) {
		const int n = n0 + img;
		__syncthreads(); // the previous image's readers are done
		// eight loads of a thread in flight at a time
		const int xTotal = p.cin * cells, dTotal = COUT * ocells;
		for (int base = tid; base < xTotal; base += 512 * 8) {
			float v[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int i = base + 512 * u;
				uint32_t c, q;
				p.divCells.divmod((uint32_t)(i < xTotal ? i : 0), c, q);
				v[u] = (i < xTotal) ? p.x[(size_t)c * iplane + (size_t)n * cells + q] : 0.f;
			}
#pragma unroll
			for (int u = 0; u < 8; u++)
				if (base + 512 * u < xTotal) xs[base + 512 * u] = v[u];
		}
		for (int base = tid; base < dTotal; base += 512 * 8) {
			float v[8];
			uint32_t c[8], q[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int i = base + 512 * u; // reads contiguous along the positions of a channel
				p.divOcells.divmod((uint32_t)(i < dTotal ? i : 0), c[u], q[u]);
				v[u] = (i < dTotal && (int)c[u] < p.cout) ? p.delta[(size_t)c[u] * oplane + (size_t)n * ocells + q[u]] : 0.f;
			}
#pragma unroll
			for (int u = 0; u < 8; u++)
				if (base + 512 * u < dTotal) ds[q[u] * COUT + c[u]] = v[u];
		}
		__syncthreads();
		if (live) {
			const float *xc = xs + ci * cells;
			for (int q = slice; q < ocells; q += slices) {
				uint32_t oa, ob;
				p.divOutB.divmod((uint32_t)q, oa, ob);
				const int a = (int)oa * p.stride + (int)ta - p.pad, b = (int)ob * p.stride + (int)tb - p.pad;
				const bool ok = ((unsigned)a < (unsigned)p.inA) & ((unsigned)b < (unsigned)p.inB);
				const float xv = ok ? xc[a * p.inB + b] : 0.f;
				const float4 *dq = reinterpret_cast<const float4 *>(ds + q * COUT);
#pragma unroll
				for (int g = 0; g < COUT / 4; g++) {
					const float4 d = dq[g];
					acc[4 * g] = fmaf(d.x, xv, acc[4 * g]);
					acc[4 * g + 1] = fmaf(d.y, xv, acc[4 * g + 1]);
					acc[4 * g + 2] = fmaf(d.z, xv, acc[4 * g + 2]);
					acc[4 * g + 3] = fmaf(d.w, xv, acc[4 * g + 3]);
				}
			}
		}
	}
	// slices of one k are added in slice order; the sums go out as one Cout x K block per workgroup
	__syncthreads();
	float *red = thin_lds; // [slice][k][COUT]
	if (live) {
#pragma unroll
		for (int c = 0; c < COUT; c++) red[(slice * K + k) * COUT + c] = acc[c];
	}
	__syncthreads();
	float *out = partial + (size_t)blockIdx.x * p.cout * K;
	for (int i = tid; i < p.cout * K; i += 512) {
		const int c = i / K, kk = i - c * K;
		float s = 0.f;
		for (int sl = 0; sl < slices; sl++) s += red[(sl * K + kk) * COUT + c];
		out[i] = s;
	}
}

static inline ThinConvParams thin_params(const fitre_conv_shape *s)
{
	ThinConvParams p;
	p.x = p.delta = p.w = nullptr;
	p.cin = s->inChannels, p.cout = s->outChannels, p.samples = s->samples;
	p.inA = s->inA, p.inB = s->inB, p.outA = s->outA, p.outB = s->outB;
	p.ksize = s->ksize, p.stride = s->stride, p.pad = s->padding;
	p.imagesPerGroup = 1;
	p.divInB = FastDiv((uint32_t)s->inB);
	p.divOutB = FastDiv((uint32_t)s->outB);
	p.divK = FastDiv((uint32_t)s->ksize);
	p.divKK = FastDiv((uint32_t)(s->ksize * s->ksize));
	p.divCells = FastDiv((uint32_t)(s->inA * s->inB));
	p.divOcells = FastDiv((uint32_t)(s->outA * s->outB));
	return p;
}

// ---- input gradient --------------------------------------------------------------------------------------------
constexpr int kThinDxLdsFloats = 15360; // 60 KB: weights + delta of the group's images
static inline int thin_dx_cin_pad(const fitre_conv_shape *s) { return s->inChannels <= 4 ? 4 : (s->inChannels <= 8 ? 8 : 16); }
static inline int thin_dx_weight_floats(const fitre_conv_shape *s) { return s->outChannels * s->ksize * s->ksize * thin_dx_cin_pad(s); }
static inline int thin_dx_images(const fitre_conv_shape *s)
{
	const int perImage = s->outChannels * s->outA * s->outB, cells = s->inA * s->inB;
	const int room = kThinDxLdsFloats - thin_dx_weight_floats(s);
	int imgs = (256 + cells - 1) / cells;
	if (imgs * perImage > room) imgs = room / perImage;
	if (s->samples / (imgs > 0 ? imgs : 1) < 2 * device_compute_units()) imgs = 1; // few images: spread them over the chip
	return imgs < 1 ? 1 : imgs;
}
static inline bool thin_dx_eligible(const fitre_conv_shape *s)
{
	return s->stride == 1 && s->inChannels <= kThinMaxChannels && s->outChannels <= 32 && s->ksize <= 7 &&
	       s->inChannels * s->outChannels <= 256 &&
	       thin_dx_weight_floats(s) + s->outChannels * s->outA * s->outB <= kThinDxLdsFloats;
}
static int launch_thin_dx(const fitre_conv_shape *s, const float *delta, const float *w, float *dx)
{
	ThinConvParams p = thin_params(s);
	p.delta = delta, p.w = w;
	p.imagesPerGroup = thin_dx_images(s);
	const int groups = (s->samples + p.imagesPerGroup - 1) / p.imagesPerGroup;
	const size_t lds = sizeof(float) * ((size_t)p.imagesPerGroup * s->outChannels * s->outA * s->outB + (size_t)thin_dx_weight_floats(s));
	LaunchScope scope(FITRE_KC_CONV_DX, conv_flops(s), 0);
#define THIN_DX(CIN_, KS_) thin_input_grad_kernel<CIN_, KS_><<<groups, 256, lds, stream()>>>(p, dx)
	if (s->inChannels <= 4) {
		if (s->ksize == 5) THIN_DX(4, 5);
		else if (s->ksize == 3) THIN_DX(4, 3);
		else THIN_DX(4, 0);
	} else if (s->inChannels <= 8) {
		if (s->ksize == 5) THIN_DX(8, 5);
		else if (s->ksize == 3) THIN_DX(8, 3);
		else THIN_DX(8, 0);
	} else {
		THIN_DX(16, 0);
	}
#undef THIN_DX
	return check_launch("thin_input_grad_kernel");
}

// ---- weight gradient -------------------------------------------------------------------------------------------
static inline int thin_dw_pad(int cout) { return cout <= 8 ? 8 : 16; }
static inline size_t thin_dw_lds_floats(const fitre_conv_shape *s)
{
	const int K = s->inChannels * s->ksize * s->ksize, cp = thin_dw_pad(s->outChannels);
	const size_t stage = (size_t)((s->inA * s->inB * s->inChannels + 3) & ~3) + (size_t)s->outA * s->outB * cp;
	const size_t red = (size_t)(512 / K) * K * cp;
	return stage > red ? stage : red;
}
static inline bool thin_dw_general_eligible(const fitre_conv_shape *s)
{
	const int K = s->inChannels * s->ksize * s->ksize;
	return s->outChannels <= kThinMaxChannels && K <= 512 && K >= 16 && thin_dw_lds_floats(s) <= (size_t)kThinLdsFloats;
}
static inline int thin_dw_general_groups(const fitre_conv_shape *s, int *imagesPerGroup)
{
	int groups = 2 * device_compute_units();
	if (groups > s->samples) groups = s->samples;
	const int per = (s->samples + groups - 1) / groups;
	*imagesPerGroup = per;
	return (s->samples + per - 1) / per;
}
static inline size_t thin_dw_general_workspace(const fitre_conv_shape *s)
{
	int per;
	return sizeof(float) * (size_t)thin_dw_general_groups(s, &per) * s->outChannels * s->inChannels * s->ksize * s->ksize;
}
static int launch_thin_dw_general(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws)
{
	ThinConvParams p = thin_params(s);
	p.x = x, p.delta = delta;
	const int groups = thin_dw_general_groups(s, &p.imagesPerGroup);
	const int K = s->inChannels * s->ksize * s->ksize;
	const size_t lds = sizeof(float) * thin_dw_lds_floats(s);
	{
		LaunchScope scope(FITRE_KC_CONV_DW, conv_flops(s), 0);
		if (thin_dw_pad(s->outChannels) == 8) thin_weight_grad_kernel<8><<<groups, 512, lds, stream()>>>(p, (float *)ws);
		else thin_weight_grad_kernel<16><<<groups, 512, lds, stream()>>>(p, (float *)ws);
	}
	OutParams out{ dW, (long)K, 0, nullptr, nullptr, 1.f, 0.f };
	launch_splitk_reduce((const float *)ws, groups, s->outChannels, K, out);
	return check_launch("thin_weight_grad_kernel");
}

} // namespace fitre
