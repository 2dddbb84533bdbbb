// Convolution forward / weight gradient / input gradient and the general
// column-major GEMM, all on the fp32-MFMA tile engine.
#include "gemm_engine.h"

namespace fitre {

static int check_conv(const char *fn, const fitre_conv_shape *s)
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
	double lim = 1073741823.0; /* operands are read through 32-bit byte offsets */
	FITRE_REQUIRE((double)s->samples * s->inA * s->inB * s->inChannels < lim &&
	                  (double)s->samples * s->outA * s->outB * s->outChannels < lim &&
	                  (double)s->inChannels * s->ksize * s->ksize * s->outChannels < lim,
	              "%s: a tensor exceeds 2^30 elements", fn);
	return FITRE_OK;
}

// patches of `src` (srcA x srcB per map) taken on an outA x outB grid
static PatchGeom make_patch_geom(const float *src, int channels, int samples, int srcA, int srcB, int outA, int outB, int ksize,
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
	g.ktable = nullptr;
	return g;
}

// Device table of the patch decode, owned by the layer and grown on demand; every use is
// ordered on the layer's stream.
static unsigned long long *g_ktable = nullptr;
static int g_ktable_cap = 0;

// bn = tile extent along the positions, which fixes how the waves stride through a slice
static int attach_patch_table(PatchGeom &g, int bn)
{
	const int kstep = kGemmThreads / bn;
	const int padded = ((g.patchLen + kGemmBK - 1) / kGemmBK) * kGemmBK;
	if (padded > g_ktable_cap) {
		FITRE_HIP_TRY(hipStreamSynchronize(stream()));
		if (g_ktable) FITRE_HIP_TRY(hipFree(g_ktable));
		g_ktable = nullptr;
		g_ktable_cap = 0;
		int cap = padded < 16384 ? 16384 : padded;
		FITRE_HIP_TRY(hipMalloc((void **)&g_ktable, sizeof(unsigned long long) * (size_t)cap));
		g_ktable_cap = cap;
	}
	patch_table_kernel<<<(padded + 255) / 256, 256, 0, stream()>>>(g_ktable, padded, g.patchLen, g.chanStride, g.srcB,
	                                                             g.divTaps, g.divK, kGemmBK, kstep);
	g.ktable = g_ktable;
	return check_launch("patch_table_kernel");
}

static double conv_flops(const fitre_conv_shape *s)
{
	return 2.0 * (double)s->samples * s->outA * s->outB * (double)s->inChannels * s->ksize * s->ksize * (double)s->outChannels;
}

} // namespace fitre

using namespace fitre;

extern "C" {

// ---- forward: I = Cout, J = positions, R = Cin*k*k ---------------------------
size_t fitre_hip_conv_forward_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	return plan_gemm(s->outChannels, (long)s->samples * s->outA * s->outB, (long)s->inChannels * s->ksize * s->ksize).wsBytes;
}

int fitre_hip_conv_forward(const fitre_conv_shape *s, const float *x, const float *w, const float *bias, float *y, void *ws,
                           size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_forward", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && w && y, "fitre_hip_conv_forward: null pointer");
	const int I = s->outChannels, J = s->samples * s->outA * s->outB, R = s->inChannels * s->ksize * s->ksize;
	GemmPlan plan = plan_gemm(I, J, R);
	PlainParams pa{ w, (uint32_t)((size_t)I * R * sizeof(float)), R, I };
	PatchGeom pb = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	OutParams out{ y, (long)J, 0, bias, nullptr, 1.f, 0.f };
	rc = attach_patch_table(pb, plan.bn);
	if (rc) return rc;
	return launch_gemm<PlainKContig, PatchRowContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_FWD, conv_flops(s));
}

// ---- weight gradient: I = Cout, J = Cin*k*k, R = positions -------------------
size_t fitre_hip_conv_weight_grad_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	return plan_gemm(s->outChannels, (long)s->inChannels * s->ksize * s->ksize, (long)s->samples * s->outA * s->outB).wsBytes;
}

int fitre_hip_conv_weight_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_weight_grad", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && delta && dW, "fitre_hip_conv_weight_grad: null pointer");
	const int I = s->outChannels, J = s->inChannels * s->ksize * s->ksize, R = s->samples * s->outA * s->outB;
	GemmPlan plan = plan_gemm(I, J, R);
	PlainParams pa{ delta, (uint32_t)((size_t)I * R * sizeof(float)), R, I };
	PatchGeom pb = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	OutParams out{ dW, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	return launch_gemm<PlainKContig, PatchKContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_DW, conv_flops(s));
}

// ---- input gradient: I = Cin, J = input positions, R = Cout*k*k ----------------
size_t fitre_hip_conv_input_grad_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	return plan_gemm(s->inChannels, (long)s->samples * s->inA * s->inB, (long)s->outChannels * s->ksize * s->ksize).wsBytes;
}

int fitre_hip_conv_input_grad(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_input_grad", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && w && dx, "fitre_hip_conv_input_grad: null pointer");
	if (s->stride != 1)
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_input_grad: stride %d (only stride 1 is back-propagated through)", s->stride);
	FITRE_REQUIRE(s->padding < s->ksize, "fitre_hip_conv_input_grad: padding %d >= window %d", s->padding, s->ksize);
	const int I = s->inChannels, J = s->samples * s->inA * s->inB, R = s->outChannels * s->ksize * s->ksize;
	GemmPlan plan = plan_gemm(I, J, R);
	FlipWeightParams pa;
	pa.w = w;
	pa.bytes = (uint32_t)((size_t)s->outChannels * s->inChannels * s->ksize * s->ksize * sizeof(float));
	pa.cin = s->inChannels;
	pa.taps = s->ksize * s->ksize;
	pa.outStride = s->inChannels * pa.taps;
	pa.divTaps = FastDiv((uint32_t)pa.taps);
	// a full correlation of delta with the flipped window: pad' = k - 1 - p
	PatchGeom pb = make_patch_geom(delta, s->outChannels, s->samples, s->outA, s->outB, s->inA, s->inB, s->ksize, 1,
	                               s->ksize - 1 - s->padding);
	OutParams out{ dx, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	rc = attach_patch_table(pb, plan.bn);
	if (rc) return rc;
	return launch_gemm<FlipWeightKContig, PatchRowContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_DX, conv_flops(s));
}

// ---- general column-major GEMM ---------------------------------------------------
// C(MxN) column-major is C[n*ldc + m]: engine i = n (column), j = m (row, contiguous).
// A operand of the engine (rows i = n) is op(B)^T, B operand (rows j = m) is op(A).
size_t fitre_hip_gemm_workspace(int M, int N, int K)
{
	if (M <= 0 || N <= 0 || K <= 0) return 0;
	return plan_gemm(N, M, K).wsBytes;
}

int fitre_hip_gemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb,
                   float beta, float *C, int ldc, const float *bias, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(A && B && C, "fitre_hip_gemm: null pointer");
	FITRE_REQUIRE(M > 0 && N > 0 && K > 0, "fitre_hip_gemm: non-positive shape %d x %d x %d", M, N, K);
	FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "fitre_hip_gemm: bad transpose flags");
	FITRE_REQUIRE(lda >= (transA ? K : M) && ldb >= (transB ? N : K) && ldc >= M, "fitre_hip_gemm: leading dimension too small");
	const size_t aElems = (size_t)lda * (transA ? M : K), bElems = (size_t)ldb * (transB ? K : N);
	FITRE_REQUIRE(aElems < ((size_t)1 << 30) && bElems < ((size_t)1 << 30), "fitre_hip_gemm: an operand exceeds 2^30 elements");
	const int I = N, J = M, R = K;
	GemmPlan plan = plan_gemm(I, J, R);
	OutParams out{ C, (long)ldc, 0, nullptr, bias, alpha, beta };
	const double flops = 2.0 * (double)M * N * K;
	// engine A(i = n, k): op(B)(k, n).  transB == 0: B[n*ldb + k] (contiguous along k); else B[k*ldb + n]
	// engine B(j = m, k): op(A)(m, k).  transA == 0: A[k*lda + m] (contiguous along m); else A[m*lda + k]
	PlainParams bk{ B, (uint32_t)(bElems * sizeof(float)), ldb, I };
	PlainParams br = bk;
	PlainParams ar{ A, (uint32_t)(aElems * sizeof(float)), lda, J };
	PlainParams ak = ar;
	if (!transB && !transA) return launch_gemm<PlainKContig, PlainRowContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, FITRE_KC_FC_GEMM, flops);
	if (!transB && transA) return launch_gemm<PlainKContig, PlainKContig>(bk, ak, out, I, J, R, plan, ws, wsBytes, FITRE_KC_FC_GEMM, flops);
	if (transB && !transA) return launch_gemm<PlainRowContig, PlainRowContig>(br, ar, out, I, J, R, plan, ws, wsBytes, FITRE_KC_FC_GEMM, flops);
	return launch_gemm<PlainRowContig, PlainKContig>(br, ak, out, I, J, R, plan, ws, wsBytes, FITRE_KC_FC_GEMM, flops);
}

} // extern "C"
