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

// The same rows in tap-major order over cell-major positions: row t * channels + c for tap t = (ta, tb), position
// (oa * outB + ob) * samples + n.  A row is then zero on whole runs of `samples` positions (the cells at which its tap
// leaves the image) and the product of two rows only needs the cells at which both taps are inside.
// Workgroup (image chunk, channel, tap row ta): the chunk's images of the channel go into LDS as they lie in memory (one
// word of padding per image: lanes that hold consecutive images then read different banks) and leave as the ksize rows of
// the taps (ta, .), in runs of consecutive images.  chunk * (srcA * srcB + 1) floats of dynamic LDS.
__global__ void __launch_bounds__(256) patch_rows_by_tap_kernel(PatchGeom g, int channels, int chunk, float *rows)
{
	extern __shared__ float img[];
	const int c = blockIdx.y, ta = blockIdx.z, img0 = blockIdx.x * chunk;
	const int count = (g.samples - img0 < chunk) ? g.samples - img0 : chunk;
	const int srcCells = g.srcA * g.srcB, ld = srcCells + 1;
	const float *src = g.src + (size_t)c * g.chanStride + (size_t)img0 * srcCells;
	for (int e = threadIdx.x; e < count * srcCells; e += blockDim.x) {
		const int n = e / srcCells, cell = e - n * srcCells;
		img[n * ld + cell] = src[e];
	}
	__syncthreads();
	const int outCells = g.outA * g.outB;
	for (int tb = 0; tb < g.ksize; tb++) {
		float *dst = rows + (size_t)((ta * g.ksize + tb) * channels + c) * g.positions + img0;
		for (int e = threadIdx.x; e < outCells * count; e += blockDim.x) {
			const int cell = e / count, n = e - cell * count;
			const int oa = cell / g.outB, ob = cell - oa * g.outB;
			const int a = oa * g.stride - g.pad + ta, b = ob * g.stride - g.pad + tb;
			const bool ok = ((unsigned)a < (unsigned)g.srcA) & ((unsigned)b < (unsigned)g.srcB);
			const float v = img[ok ? n * ld + a * g.srcB + b : 0];
			dst[(size_t)cell * g.samples + n] = ok ? v : 0.f;
		}
	}
}

// factor[(c1 * taps + t1) * ld + c2 * taps + t2] = byTap[(t1 * channels + c1) * K + t2 * channels + c2], K = taps * channels:
// the product of tap-major rows back in the order of the patch index.  One workgroup per row: the source row is read as it
// lies in memory, goes through LDS (each tap's segment 8 words behind a multiple of 32: a wave's reads of one destination
// run then spread over the banks) and leaves as one contiguous row.  Dynamic LDS: taps * (channels + 8) floats.
__global__ void __launch_bounds__(256) tap_order_to_patch_order_kernel(const float *byTap, int channels, int taps, float *factor, long ld)
{
	extern __shared__ float seg[];
	const int K = channels * taps, segLd = channels + 8;
	const int r = blockIdx.x; // destination row
	const int c1 = r / taps, t1 = r - c1 * taps;
	const float *srcRow = byTap + (size_t)(t1 * channels + c1) * K;
	for (int q = threadIdx.x; q < K; q += blockDim.x) {
		const int t2 = q / channels, c2 = q - t2 * channels;
		seg[t2 * segLd + c2] = srcRow[q];
	}
	__syncthreads();
	float *dstRow = factor + (size_t)r * ld;
	for (int j = threadIdx.x; j < K; j += blockDim.x) {
		const int c2 = j / taps, t2 = j - c2 * taps;
		dstRow[j] = seg[t2 * segLd + c2];
	}
}

// Products of tap-major rows pay where a good part of every row is zero: small maps (on an 8 x 8 map a sixth of the
// reduction is skipped, on 4 x 4 a third, on 2 x 2 four fifths; on 16 x 16 one fourteenth, less than the reordering costs).
static bool tap_major_eligible(const fitre_conv_shape *s)
{
	return s->stride == 1 && s->ksize >= 2 && s->ksize <= 7 && s->inChannels % 128 == 0 && s->outA * s->outB <= 64 && s->inA * s->inB <= 1024 && s->samples % 16 == 0 &&
	       (size_t)(s->inChannels + 8) * s->ksize * s->ksize * sizeof(float) <= 64 * 1024;
}

static size_t tap_major_bytes(const fitre_conv_shape *s)
{
	if (!tap_major_eligible(s)) return 0;
	const size_t K = (size_t)s->inChannels * s->ksize * s->ksize;
	return (K * K * sizeof(float) + 255) & ~(size_t)255;
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


// ---- the operand of an input-side factor itself, for factors kept in low-rank form -----------------------------
// rows[r][m] (row r contiguous): the patch rows of patch_rows_kernel, and under them (withBias) one row that is outA * outB
// everywhere: R with P^T P / samples = R R^T / (cells^2 samples).
__global__ void __launch_bounds__(256) fill_row_kernel(float *row, long n, float v)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) row[idx] = v;
}

// out (n x samples, column-major) = [ z ; 1 ] for z (in x samples, column-major)
__global__ void __launch_bounds__(256) rows_with_ones_kernel(const float *z, int in, int samples, int withBias, float *out)
{
	const int n = in + (withBias ? 1 : 0);
	const long total = (long)n * samples;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const int s = (int)(idx / n), r = (int)(idx - (long)s * n);
		out[idx] = r < in ? z[(size_t)s * in + r] : 1.f;
	}
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
	const size_t withRows = rows + patch_rows_tail_bytes(s, withBias) + tap_major_bytes(s);
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
		// on small maps: rows by tap, the product into a buffer behind the tail, and from there into the factor
		const size_t byTapBytes = tap_major_bytes(s);
		const bool byTap = byTapBytes != 0 && wsBytes >= rowBytes + patch_rows_tail_bytes(s, withBias) + byTapBytes;
		const size_t tailBytes = byTap ? patch_rows_tail_bytes(s, withBias) : wsBytes - rowBytes;
		{
			LaunchScope scope(FITRE_KC_BLAS1, 2.0 * (double)rowBytes);
			const dim3 grid(blocks_for(R, 256, 64), (unsigned)K);
			if (byTap) {
				const int perImage = s->inA * s->inB + 1;
				int chunk = (int)(48 * 1024 / sizeof(float)) / perImage;
				chunk = chunk >= 64 ? chunk / 64 * 64 : chunk; // whole waves of images per cell
				if (chunk > s->samples) chunk = s->samples;
				const dim3 byTapGrid((unsigned)((s->samples + chunk - 1) / chunk), (unsigned)s->inChannels, (unsigned)s->ksize);
				patch_rows_by_tap_kernel<<<byTapGrid, 256, (size_t)chunk * perImage * sizeof(float), stream()>>>(g, s->inChannels, chunk, rows);
			} else {
				patch_rows_kernel<<<grid, 256, 0, stream()>>>(g, rows);
			}
		}
		PlainParams pr{ rows, (uint32_t)rowBytes, R, K };
		if (byTap) {
			float *product = (float *)((char *)tail + tailBytes);
			OutParams tapOut{ product, (long)K, 0, nullptr, nullptr, out.alpha, 0.f, 1 };
			tapOut.tapRows = s->inChannels, tapOut.tapImages = s->samples, tapOut.tapKs = s->ksize, tapOut.tapPad = s->padding;
			tapOut.tapOutA = s->outA, tapOut.tapOutB = s->outB, tapOut.tapSrcA = s->inA, tapOut.tapSrcB = s->inB;
			rc = launch_gemm<PlainKContig, PlainKContig>(pr, pr, tapOut, K, K, R, plan_gemm(K, K, R, true), tail, tailBytes,
			                                             FITRE_KC_KFAC_FACTOR, flops);
			if (rc) return rc;
			const int taps = s->ksize * s->ksize;
			LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)K * K);
			tap_order_to_patch_order_kernel<<<K, 256, (size_t)taps * (s->inChannels + 8) * sizeof(float), stream()>>>(product, s->inChannels,
			                                                                                                      taps, factor, n);
			rc = check_launch("tap_order_to_patch_order_kernel");
		} else {
			rc = launch_gemm<PlainKContig, PlainKContig>(pr, pr, out, K, K, R, plan_gemm(K, K, R, true), tail, tailBytes,
			                                             FITRE_KC_KFAC_FACTOR, flops);
		}
		if (rc || !withBias) return rc;
		// the row sums do not depend on the order of the positions, but they come in the order of the rows
		float *last = factor + (size_t)K * n;
		if (byTap) {
			float *sums = (float *)((char *)tail + tailBytes); // the product buffer is free again
			rc = fitre_hip_channel_sum(rows, K, R, sums, tail, tailBytes);
			if (rc) return rc;
			tap_order_to_patch_order_kernel<<<1, 256, (size_t)s->ksize * s->ksize * (s->inChannels + 8) * sizeof(float), stream()>>>(
			    sums, s->inChannels, s->ksize * s->ksize, last, n);
			rc = check_launch("tap_order_to_patch_order_kernel");
			if (rc) return rc;
			fc_factor_border_kernel<<<blocks_for(n, 256), 256, 0, stream()>>>(factor, last, K, 1.f / (cells * (float)s->samples), cells);
			return check_launch("fc_factor_border_kernel");
		}
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

// ---- the same factors accumulated in float64 -----------------------------------------------------------------
size_t fitre_hip_kfac_conv_input_factor_f64_workspace(const fitre_conv_shape *s, int withBias)
{
	if (!s) return 0;
	const long n = (long)s->inChannels * s->ksize * s->ksize + (withBias ? 1 : 0);
	return patch_rows_bytes(s) + dgemm_workspace(n, n, (long)s->samples * s->outA * s->outB, kDgMirror);
}

int fitre_hip_kfac_conv_input_factor_f64(const fitre_conv_shape *s, const float *x, int withBias, double shift, double *factor,
                                         void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_kfac_conv_input_factor_f64", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && factor && ws, "fitre_hip_kfac_conv_input_factor_f64: null pointer");
	FITRE_REQUIRE((((uintptr_t)ws) & 255) == 0, "fitre_hip_kfac_conv_input_factor_f64: workspace must be 256-byte aligned");
	const int K = s->inChannels * s->ksize * s->ksize, n = K + (withBias ? 1 : 0);
	const long R = (long)s->samples * s->outA * s->outB;
	const size_t rowBytes = patch_rows_bytes(s);
	if (wsBytes < rowBytes)
		return fail(FITRE_E_WORKSPACE, "fitre_hip_kfac_conv_input_factor_f64: workspace of %zu bytes is smaller than the %zu of the patch rows",
		            wsBytes, rowBytes);
	const double cells = (double)(s->outA * s->outB);
	PatchGeom g = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	float *rows = (float *)ws;
	{
		LaunchScope scope(FITRE_KC_BLAS1, 2.0 * (double)rowBytes);
		const dim3 grid(blocks_for(R, 256, 64), (unsigned)K);
		patch_rows_kernel<<<grid, 256, 0, stream()>>>(g, rows);
	}
	// rows of P^T unscaled, the row of ones as outA * outB: one factor 1 / (cells^2 * samples) on the product gives P^T P / samples
	DMat a = dmat32(rows, R, 1);
	if (withBias) a.onesRow = K, a.onesValue = cells;
	DMat b = a;
	b.rs = a.cs, b.cs = a.rs, b.onesRow = -1, b.onesCol = a.onesRow;
	return dgemm(n, n, R, 1.0 / (cells * cells * (double)s->samples), a, b, 0.0, DOut{ factor, 1, n, FITRE_MAT_F64 }, shift, kDgMirror,
	             FITRE_KC_KFAC_FACTOR, (char *)ws + rowBytes, wsBytes - rowBytes);
}

int fitre_hip_kfac_conv_output_factor_f64(const fitre_conv_shape *s, const float *delta, double shift, double *factor, void *ws,
                                          size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_kfac_conv_output_factor_f64", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && factor, "fitre_hip_kfac_conv_output_factor_f64: null pointer");
	const int n = s->outChannels;
	const long R = (long)s->samples * s->outA * s->outB;
	return dgemm(n, n, R, (double)R, dmat32(delta, R, 1), dmat32(delta, 1, R), 0.0, DOut{ factor, 1, n, FITRE_MAT_F64 }, shift, kDgMirror,
	             FITRE_KC_KFAC_FACTOR, ws, wsBytes);
}

int fitre_hip_kfac_fc_input_factor_f64(const float *z, int in, int samples, int withBias, double shift, double *factor, void *ws,
                                       size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(z && factor, "fitre_hip_kfac_fc_input_factor_f64: null pointer");
	FITRE_REQUIRE(in > 0 && samples > 0, "fitre_hip_kfac_fc_input_factor_f64: non-positive shape %d x %d", in, samples);
	const int n = in + (withBias ? 1 : 0);
	DMat a = dmat32(z, 1, in);
	if (withBias) a.onesRow = in, a.onesValue = 1.0;
	DMat b = a;
	b.rs = a.cs, b.cs = a.rs, b.onesRow = -1, b.onesCol = a.onesRow;
	return dgemm(n, n, samples, 1.0 / (double)samples, a, b, 0.0, DOut{ factor, 1, n, FITRE_MAT_F64 }, shift, kDgMirror, FITRE_KC_KFAC_FACTOR, ws,
	             wsBytes);
}

int fitre_hip_kfac_fc_output_factor_f64(const float *delta, int outDim, int samples, double shift, double *factor, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && factor, "fitre_hip_kfac_fc_output_factor_f64: null pointer");
	FITRE_REQUIRE(outDim > 0 && samples > 0, "fitre_hip_kfac_fc_output_factor_f64: non-positive shape %d x %d", outDim, samples);
	return dgemm(outDim, outDim, samples, (double)samples, dmat32(delta, 1, outDim), dmat32(delta, outDim, 1), 0.0,
	             DOut{ factor, 1, outDim, FITRE_MAT_F64 }, shift, kDgMirror, FITRE_KC_KFAC_FACTOR, ws, wsBytes);
}

int fitre_hip_kfac_conv_input_rows(const fitre_conv_shape *s, const float *x, int withBias, float *rows)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_kfac_conv_input_rows", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && rows, "fitre_hip_kfac_conv_input_rows: null pointer");
	const int K = s->inChannels * s->ksize * s->ksize;
	const long R = (long)s->samples * s->outA * s->outB;
	PatchGeom g = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	LaunchScope scope(FITRE_KC_BLAS1, 4.0 * (double)(K + 1) * (double)R);
	const dim3 grid(blocks_for(R, 256, 64), (unsigned)K);
	patch_rows_kernel<<<grid, 256, 0, stream()>>>(g, rows);
	if (withBias) fill_row_kernel<<<blocks_for(R, 256, 256), 256, 0, stream()>>>(rows + (size_t)K * R, R, (float)(s->outA * s->outB));
	return check_launch("fitre_hip_kfac_conv_input_rows");
}

int fitre_hip_kfac_fc_input_rows(const float *z, int in, int samples, int withBias, float *rows)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(z && rows && in > 0 && samples > 0, "fitre_hip_kfac_fc_input_rows: bad argument");
	rows_with_ones_kernel<<<blocks_for((long)(in + 1) * samples, 256, 4096), 256, 0, stream()>>>(z, in, samples, withBias, rows);
	return check_launch("rows_with_ones_kernel");
}

} // extern "C"
