// Shape checks and patch geometry shared by the convolution products and the Kronecker factors.
#pragma once
#include "gemm_engine.h"

namespace fitre {

static inline int check_conv(const char *fn, const fitre_conv_shape *s)
{
	FITRE_REQUIRE(s != nullptr, "%s: null shape", fn);
	FITRE_REQUIRE(s->samples > 0 && s->inChannels > 0 && s->outChannels > 0 && s->inA > 0 && s->inB > 0 && s->ksize > 0 &&
	                  s->stride > 0 && s->padding >= 0,
	              "%s: non-positive shape (N=%d Cin=%d Cout=%d A=%d B=%d k=%d s=%d p=%d)", fn, s->samples, s->inChannels,
	              s->outChannels, s->inA, s->inB, s->ksize, s->stride, s->padding);
	FITRE_REQUIRE(s->outA == (s->inA + 2 * s->padding - s->ksize) / s->stride + 1 &&
	                  s->outB == (s->inB + 2 * s->padding - s->ksize) / s->stride + 1 && s->outA > 0 && s->outB > 0,
	              "%s: output extent %dx%d does not follow from input %dx%d, k=%d s=%d p=%d", fn, s->outA, s->outB, s->inA,
	              s->inB, s->ksize, s->stride, s->padding);
	FITRE_REQUIRE(s->ksize < 256, "%s: window %d too large", fn, s->ksize);
	double lim = 1073741800.0; /* operands are read through 32-bit byte offsets, the last 16 bytes of the range mark invalid groups */
	FITRE_REQUIRE((double)s->samples * s->inA * s->inB * s->inChannels < lim &&
	                  (double)s->samples * s->outA * s->outB * s->outChannels < lim &&
	                  (double)s->inChannels * s->ksize * s->ksize * s->outChannels < lim,
	              "%s: a tensor exceeds 2^30 elements", fn);
	return FITRE_OK;
}

// patches of `src` (srcA x srcB per map) taken on an outA x outB grid
static inline PatchGeom make_patch_geom(const float *src, int channels, int samples, int srcA, int srcB, int outA, int outB, int ksize,
                                 int stride, int pad)
{
	PatchGeom g;
	g.src = src;
	g.bytes = (uint32_t)((size_t)channels * samples * srcA * srcB * sizeof(float));
	g.samples = samples;
	g.srcA = srcA;
	g.srcB = srcB;
	g.outA = outA;
	g.outB = outB;
	g.ksize = ksize;
	g.stride = stride;
	g.pad = pad;
	g.positions = samples * outA * outB;
	g.taps = ksize * ksize;
	g.patchLen = channels * g.taps;
	g.chanStride = samples * srcA * srcB;
	g.divOutB = FastDiv((uint32_t)outB);
	g.divOutA = FastDiv((uint32_t)outA);
	g.divTaps = FastDiv((uint32_t)g.taps);
	g.divK = FastDiv((uint32_t)ksize);
	g.onesValue = 0.f;
	g.ktable = nullptr;
	return g;
}

static inline double conv_flops(const fitre_conv_shape *s)
{
	return 2.0 * (double)s->samples * s->outA * s->outB * (double)s->inChannels * s->ksize * s->ksize * (double)s->outChannels;
}

} // namespace fitre
