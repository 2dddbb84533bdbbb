// Kronecker factors of the KFAC curvature approximation, as symmetric products on the fp32-MFMA
// tile engine.  Only the tiles on and above the diagonal are computed; the rest is mirrored.
//
//   convolution, input side   A = P^T P / samples,  P = [ im2col(x) / (outA*outB) , 1 ]
//   convolution, output side  G = D^T D * (samples*outA*outB),  D = delta as (positions x Cout)
//   fully connected, input    A = Z Z^T / samples,  Z = [ z ; 1 ]   (z is in x samples)
//   fully connected, output   G = D D^T * samples,  D = delta (out x samples)
//
// The patch matrix P is never materialised: both operands of P^T P gather their elements
// from the image, and the column of ones is a constant row of the operand.
#include "conv_common.h"

namespace fitre {

// last row and column of the fully connected input factor: A[n][j] = A[j][n] = mean_s z[j][s], A[n][n] = 1.
// `sums` holds the row sums of z and may alias the factor's last row.
__global__ void __launch_bounds__(256) fc_factor_border_kernel(float *factor, const float *sums, int in, float invSamples)
{
	const int n = in + 1;
	const int j = blockIdx.x * blockDim.x + threadIdx.x;
	if (j < in) {
		float v = sums[j] * invSamples;
		factor[(size_t)in * n + j] = v;
		factor[(size_t)j * n + in] = v;
	} else if (j == in) {
		factor[(size_t)in * n + in] = 1.f;
	}
}

} // namespace fitre

using namespace fitre;

extern "C" {

size_t fitre_hip_kfac_conv_input_factor_workspace(const fitre_conv_shape *s, int withBias)
{
	if (!s) return 0;
	const long n = (long)s->inChannels * s->ksize * s->ksize + (withBias ? 1 : 0);
	return plan_gemm_workspace(n, n, (long)s->samples * s->outA * s->outB, true);
}

int fitre_hip_kfac_conv_input_factor(const fitre_conv_shape *s, const float *x, int withBias, float *factor, void *ws,
                                     size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_kfac_conv_input_factor", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && factor, "fitre_hip_kfac_conv_input_factor: null pointer");
	const int K = s->inChannels * s->ksize * s->ksize, n = K + (withBias ? 1 : 0);
	const int R = s->samples * s->outA * s->outB;
	FITRE_REQUIRE((double)n * n < 2147483647.0, "fitre_hip_kfac_conv_input_factor: factor of order %d too large", n);
	const float cells = (float)(s->outA * s->outB);
	PatchGeom g = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	// patches are used unscaled and the ones column carries outA*outB, so that one factor
	// 1 / (cells^2 * samples) on the product gives P^T P / samples
	g.onesValue = cells;
	GemmPlan plan = plan_gemm(n, n, R, true);
	OutParams out{ factor, (long)n, 0, nullptr, nullptr, 1.f / (cells * cells * (float)s->samples), 0.f, 1 };
	const double flops = (double)n * (n + 1) * (double)R; // 2 flops per element of the upper triangle and position
	if (withBias)
		return launch_gemm<PatchKContigOnes, PatchKContigOnes>(g, g, out, n, n, R, plan, ws, wsBytes, FITRE_KC_KFAC_FACTOR, flops);
	return launch_gemm<PatchKContig, PatchKContig>(g, g, out, n, n, R, plan, ws, wsBytes, FITRE_KC_KFAC_FACTOR, flops);
}

size_t fitre_hip_kfac_gram_workspace(int order, long reduce)
{
	if (order <= 0 || reduce <= 0) return 0;
	return plan_gemm_workspace(order, order, reduce, true);
}

int fitre_hip_kfac_conv_output_factor(const fitre_conv_shape *s, const float *delta, float *factor, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_kfac_conv_output_factor", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && factor, "fitre_hip_kfac_conv_output_factor: null pointer");
	const int n = s->outChannels, R = s->samples * s->outA * s->outB;
	GemmPlan plan = plan_gemm(n, n, R, true);
	PlainParams d{ delta, (uint32_t)((size_t)n * R * sizeof(float)), R, n };
	OutParams out{ factor, (long)n, 0, nullptr, nullptr, (float)R, 0.f, 1 };
	return launch_gemm<PlainKContig, PlainKContig>(d, d, out, n, n, R, plan, ws, wsBytes, FITRE_KC_KFAC_FACTOR,
	                                               (double)n * (n + 1) * (double)R);
}

int fitre_hip_kfac_fc_input_factor(const float *z, int in, int samples, int withBias, float *factor, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(z && factor, "fitre_hip_kfac_fc_input_factor: null pointer");
	FITRE_REQUIRE(in > 0 && samples > 0, "fitre_hip_kfac_fc_input_factor: non-positive shape %d x %d", in, samples);
	FITRE_REQUIRE((double)in * samples < 1073741823.0 && in < 46000, "fitre_hip_kfac_fc_input_factor: operand too large");
	const int n = in + (withBias ? 1 : 0);
	GemmPlan plan = plan_gemm(in, in, samples, true);
	PlainParams zp{ z, (uint32_t)((size_t)in * samples * sizeof(float)), in, in };
	OutParams out{ factor, (long)n, 0, nullptr, nullptr, 1.f / (float)samples, 0.f, 1 };
	int rc = launch_gemm<PlainRowContig, PlainRowContig>(zp, zp, out, in, in, samples, plan, ws, wsBytes, FITRE_KC_KFAC_FACTOR,
	                                                     (double)in * (in + 1) * (double)samples);
	if (rc || !withBias) return rc;
	// border: row sums of z land in the factor's last row, then are scaled and mirrored
	float *last = factor + (size_t)in * n;
	rc = fitre_hip_row_sum(z, in, samples, last);
	if (rc) return rc;
	fc_factor_border_kernel<<<blocks_for(n, 256), 256, 0, stream()>>>(factor, last, in, 1.f / (float)samples);
	return check_launch("fc_factor_border_kernel");
}

int fitre_hip_kfac_fc_output_factor(const float *delta, int outDim, int samples, float *factor, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && factor, "fitre_hip_kfac_fc_output_factor: null pointer");
	FITRE_REQUIRE(outDim > 0 && samples > 0, "fitre_hip_kfac_fc_output_factor: non-positive shape %d x %d", outDim, samples);
	FITRE_REQUIRE((double)outDim * samples < 1073741823.0 && outDim < 46000, "fitre_hip_kfac_fc_output_factor: operand too large");
	GemmPlan plan = plan_gemm(outDim, outDim, samples, true);
	PlainParams d{ delta, (uint32_t)((size_t)outDim * samples * sizeof(float)), outDim, outDim };
	OutParams out{ factor, (long)outDim, 0, nullptr, nullptr, (float)samples, 0.f, 1 };
	return launch_gemm<PlainRowContig, PlainRowContig>(d, d, out, outDim, outDim, samples, plan, ws, wsBytes, FITRE_KC_KFAC_FACTOR,
	                                                   (double)outDim * (outDim + 1) * (double)samples);
}

} // extern "C"
