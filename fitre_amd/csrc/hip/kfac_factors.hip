// Kronecker factors of the KFAC curvature approximation, as symmetric products on the fp32-MFMA
// tile engine.  Only the tiles on and above the diagonal are computed; the rest is mirrored.
//
//   convolution, input side   A = P^T P / samples,  P = [ im2col(x) / (outA*outB) , 1 ]
//   convolution, output side  G = D^T D * (samples*outA*outB),  D = delta as (positions x Cout)
//   fully connected, input    A = Z Z^T / samples,  Z = [ z ; 1 ]   (z is in x samples)
//   fully connected, output   G = D D^T * samples,  D = delta (out x samples)
//
// The input-side factor of a convolution first writes P^T (one row per patch index, positions
// contiguous, the row of ones last) into its workspace and then runs the plain symmetric product
// on it: 150 MB at most for VGG-11 at batch 256, written and read at HBM speed, against operand
// fetches that decode every element's patch coordinates (measured: 100-124 TFLOP/s on the rows
// against 63 with the gather).  With a workspace too small for the rows both operands gather their
// elements from the image and the column of ones is a constant row of the operand.
#include "conv_common.h"

namespace fitre {

// last row and column of an input factor of order in + 1 (the bias): A[n][j] = A[j][n] = sums[j] * scale, A[n][n] = corner.
// `sums` holds the row sums of the operand and may alias the factor's last row.
__global__ void __launch_bounds__(256) fc_factor_border_kernel(float *factor, const float *sums, int in, float scale, float corner)
{
	const int n = in + 1;
	const int j = blockIdx.x * blockDim.x + threadIdx.x;
	if (j < in) {
		float v = sums[j] * scale;
		factor[(size_t)in * n + j] = v;
		factor[(size_t)j * n + in] = v;
	} else if (j == in) {
		factor[(size_t)in * n + in] = corner;
	}
}

// rows[row][m] = src[c][n][oa*stride - pad + ta][ob*stride - pad + tb] for row = (c, ta, tb) and position m = (n, oa, ob),
// zero outside the image.  blockIdx.y: row.
__global__ void __launch_bounds__(256) patch_rows_kernel(PatchGeom g, float *rows)
{
	const uint32_t row = blockIdx.y;
	float *dst = rows + (size_t)row * g.positions;
	const long stride = (long)gridDim.x * blockDim.x;
	uint32_t c, tap, ta, tb;
	g.divTaps.divmod(row, c, tap);
	g.divK.divmod(tap, ta, tb);
	const float *src = g.src + (size_t)c * g.chanStride;
	for (long m = (long)blockIdx.x * blockDim.x + threadIdx.x; m < g.positions; m += stride) {
		uint32_t q, ob, n, oa;
		g.divOutB.divmod((uint32_t)m, q, ob);
		g.divOutA.divmod(q, n, oa);
		const int a = (int)oa * g.stride - g.pad + (int)ta, b = (int)ob * g.stride - g.pad + (int)tb;
		const bool ok = ((unsigned)a < (unsigned)g.srcA) & ((unsigned)b < (unsigned)g.srcB);
		dst[m] = ok ? src[(size_t)n * g.srcA * g.srcB + (size_t)a * g.srcB + b] : 0.f;
	}
}

static size_t patch_rows_bytes(const fitre_conv_shape *s)
{
	const size_t bytes = (size_t)s->inChannels * s->ksize * s->ksize * (size_t)s->samples * s->outA * s->outB * sizeof(float);
	return (bytes + 255) & ~(size_t)255;
}

// workspace behind the rows: the product's split partials, then (the product queued) the partial sums of the rows
static size_t patch_rows_tail_bytes(const fitre_conv_shape *s, int withBias)
{
	const long K = (long)s->inChannels * s->ksize * s->ksize, R = (long)s->samples * s->outA * s->outB;
	size_t tail = plan_gemm_workspace(K, K, R, true);
	if (withBias) {
		const size_t sums = fitre_hip_channel_sum_workspace((int)K, R);
		tail = sums > tail ? sums : tail;
	}
	return (tail + 255) & ~(size_t)255;
}

} // namespace fitre

using namespace fitre;

extern "C" {

size_t fitre_hip_kfac_conv_input_factor_workspace(const fitre_conv_shape *s, int withBias)
{
	if (!s) return 0;
	const long n = (long)s->inChannels * s->ksize * s->ksize + (withBias ? 1 : 0);
	const size_t product = plan_gemm_workspace(n, n, (long)s->samples * s->outA * s->outB, true);
	const size_t rows = patch_rows_bytes(s);
	// the rows of P^T in front of the product's own workspace, when an operand of that size can be addressed
	if (rows / sizeof(float) >= ((size_t)1 << 30)) return product;
	const size_t withRows = rows + patch_rows_tail_bytes(s, withBias);
	return withRows > product ? withRows : product;
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
	// Rows of P^T in the workspace, the plain symmetric product on them (order K: whole tiles for the usual channel
	// counts), and the bias row and column from the row sums: A[n][j] = sum_m P[m][j] / samples.
	const size_t rowBytes = patch_rows_bytes(s);
	if (ws && (((uintptr_t)ws) & 255) == 0 && rowBytes / sizeof(float) < ((size_t)1 << 30) &&
	    wsBytes >= rowBytes + patch_rows_tail_bytes(s, withBias)) {
		float *rows = (float *)ws;
		void *tail = (char *)ws + rowBytes;
		const size_t tailBytes = wsBytes - rowBytes;
		{
			LaunchScope scope(FITRE_KC_BLAS1, 2.0 * (double)rowBytes);
			const dim3 grid(blocks_for(R, 256, 64), (unsigned)K);
			patch_rows_kernel<<<grid, 256, 0, stream()>>>(g, rows);
		}
		PlainParams pr{ rows, (uint32_t)rowBytes, R, K };
		rc = launch_gemm<PlainKContig, PlainKContig>(pr, pr, out, K, K, R, plan_gemm(K, K, R, true), tail, tailBytes,
		                                             FITRE_KC_KFAC_FACTOR, flops);
		if (rc || !withBias) return rc;
		float *last = factor + (size_t)K * n;
		rc = fitre_hip_channel_sum(rows, K, R, last, tail, tailBytes);
		if (rc) return rc;
		fc_factor_border_kernel<<<blocks_for(n, 256), 256, 0, stream()>>>(factor, last, K, 1.f / (cells * (float)s->samples), cells);
		return check_launch("fc_factor_border_kernel");
	}
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
	fc_factor_border_kernel<<<blocks_for(n, 256), 256, 0, stream()>>>(factor, last, in, 1.f / (float)samples, 1.f);
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
