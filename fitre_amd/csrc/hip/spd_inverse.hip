// Inverse of a symmetric positive definite matrix (plus a multiple of the identity): what the
// reference obtains from cusolverDnDpotrf + cusolverDnDpotrs with an identity right-hand side
// (solvers/kfac_inverses.cu:133-186), for the KFAC factors (order up to Cin*k*k + 1 = 4609).
//
//   1. W = A + shift*I = L L^T      blocked right-looking Cholesky, 64-wide block columns:
//                                   a one-wave kernel factors the diagonal block and inverts its
//                                   factor, the panel and the symmetric trailing update are
//                                   products on the MFMA tile engine;
//   2. X = L^-1                     pairwise block recursion  [X11 0; -X22 L21 X11, X22]  bottom-up,
//                                   two engine products per pair;
//   3. A^-1 = X^T X                 one symmetric engine product whose reduction skips the zero
//                                   part of the triangular operand.
// All matrices are column-major with leading dimension n; only lower triangles are meaningful
// in W and X (X's upper triangle is kept at zero).
#include "common.h"

namespace fitre {

constexpr int kNb = 64; // block order of the factorization

// value of v in lane `lane` (a compile-time lane index), as a wave-uniform scalar
__device__ __forceinline__ float lane_value(float v, int lane)
{
	return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// One wave factors the nb x nb (nb <= 64) diagonal block in place (lower triangle) and writes the
// inverse of the factor, 64 x 64 column-major, padded with the identity.  Lane i holds row i in
// registers; what a step needs from another lane's row comes through v_readlane as a scalar, so
// there is no LDS traffic and no barrier in the 2 x 2016 multiply-adds.
// info: set to the 1-based global index of the first non-positive pivot.
__global__ void __launch_bounds__(64) chol_diag_kernel(float *W, int ld, int k0, int nb, float *Linv, int *info)
{
	const int i = threadIdx.x;
	float a[kNb];
	float *blk = W + (size_t)k0 * ld + k0;
#pragma unroll
	for (int j = 0; j < kNb; j++) {
		const bool inside = (i < nb) & (j < nb);
		a[j] = inside ? blk[(size_t)j * ld + i] : ((i == j) ? 1.f : 0.f);
	}
	float rdiag[kNb]; // 1 / L[j][j], wave-uniform
	int bad = 0;
#pragma unroll
	for (int j = 0; j < kNb; j++) {
		const float ajj = lane_value(a[j], j);
		if (!(ajj > 0.f) && bad == 0) bad = k0 + j + 1;
		const float d = rsqrtf(ajj);
		rdiag[j] = d;
		a[j] = (i == j) ? ajj * d : a[j] * d; // column j of L; sqrt(ajj) on the diagonal
#pragma unroll
		for (int k = j + 1; k < kNb; k++) a[k] -= a[j] * lane_value(a[j], k); // entries above the diagonal are never used
	}
	if (bad != 0 && i == 0) atomicCAS(info, 0, bad);
#pragma unroll
	for (int j = 0; j < kNb; j++)
		if ((i < nb) & (j < nb) & (j <= i)) blk[(size_t)j * ld + i] = a[j];
	// lane c solves L x = e_c by forward substitution; L[r][k] is lane r's a[k]
	float x[kNb];
#pragma unroll
	for (int r = 0; r < kNb; r++) {
		float acc0 = (r == i) ? 1.f : 0.f, acc1 = 0.f;
#pragma unroll
		for (int k = 0; k < r; k++) {
			const float l = lane_value(a[k], r);
			if (k & 1) acc1 -= l * x[k];
			else acc0 -= l * x[k];
		}
		x[r] = (acc0 + acc1) * rdiag[r];
	}
#pragma unroll
	for (int r = 0; r < kNb; r++) Linv[(size_t)i * kNb + r] = x[r];
}

__global__ void __launch_bounds__(256) shifted_copy_kernel(const float *A, float *W, int n, float shift)
{
	const long total = (long)n * n;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const int c = (int)(idx / n), r = (int)(idx - (long)c * n);
		W[idx] = A[idx] + ((r == c) ? shift : 0.f);
	}
}

// dst (rows x cols, ld ldd) = src (ld lds)
__global__ void __launch_bounds__(256) block_copy_kernel(const float *src, int lds_, float *dst, int ldd, int rows, int cols)
{
	const long total = (long)rows * cols;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const int c = (int)(idx / rows), r = (int)(idx - (long)c * rows);
		dst[(size_t)c * ldd + r] = src[(size_t)c * lds_ + r];
	}
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float *p, long n)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) p[idx] = 0.f;
}

struct InverseLayout {
	size_t w, x, linv, panel, info, gemm, total; // byte offsets / sizes
	size_t gemmBytes;
};

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static InverseLayout inverse_layout(int n)
{
	InverseLayout l;
	const size_t nn = (size_t)n * n * sizeof(float);
	const int blocks = (n + kNb - 1) / kNb;
	size_t g = 0;
	// the largest split workspaces the products below can ask for
	g = gemm_ex_workspace(n, n, kNb, kGemmMirror) > g ? gemm_ex_workspace(n, n, kNb, kGemmMirror) : g;
	g = gemm_ex_workspace(n, kNb, kNb, 0) > g ? gemm_ex_workspace(n, kNb, kNb, 0) : g;
	for (int s = kNb; s < n; s *= 2) {
		int m = (s < n - s) ? s : n - s; // rows of the lower block can be up to s
		size_t a = gemm_ex_workspace(s, s, s, 0);
		g = a > g ? a : g;
		(void)m;
	}
	size_t c = gemm_ex_workspace(n, n, n, kGemmMirror);
	g = c > g ? c : g;
	l.w = 0;
	l.x = align256(l.w + nn);
	l.linv = align256(l.x + nn);
	l.panel = align256(l.linv + (size_t)blocks * kNb * kNb * sizeof(float));
	l.info = align256(l.panel + (size_t)n * kNb * sizeof(float));
	l.gemm = align256(l.info + 256);
	l.gemmBytes = align256(g + 256);
	l.total = l.gemm + l.gemmBytes;
	return l;
}

} // namespace fitre

using namespace fitre;

extern "C" {

size_t fitre_hip_spd_inverse_workspace(int n)
{
	if (n <= 0) return 0;
	return inverse_layout(n).total;
}

// queues the whole inverse on the selected lane; pivotInfo: device int that receives the 1-based index of the
// first non-positive pivot, or stays zero (null: a slot of the workspace)
static int spd_inverse_run(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes, int *pivotInfo,
                           int **infoSlot)
{
	FITRE_REQUIRE(matrix && inverse && ws, "fitre_hip_spd_inverse: null pointer");
	FITRE_REQUIRE(n > 0 && n <= 23000, "fitre_hip_spd_inverse: order %d out of range", n);
	FITRE_REQUIRE((((uintptr_t)ws) & 255) == 0, "fitre_hip_spd_inverse: workspace must be 256-byte aligned");
	const InverseLayout lay = inverse_layout(n);
	if (wsBytes < lay.total)
		return fail(FITRE_E_WORKSPACE, "fitre_hip_spd_inverse: workspace of %zu bytes is smaller than the %zu required", wsBytes,
		            lay.total);
	char *base = (char *)ws;
	float *W = (float *)(base + lay.w), *X = (float *)(base + lay.x), *Linv = (float *)(base + lay.linv);
	float *P = (float *)(base + lay.panel);
	int *dInfo = pivotInfo ? pivotInfo : (int *)(base + lay.info);
	if (infoSlot) *infoSlot = dInfo;
	void *gws = base + lay.gemm;
	const size_t gBytes = lay.gemmBytes;
	float *T = inverse; // free until the last product
	const int blocks = (n + kNb - 1) / kNb;
	const int KC = FITRE_KC_SPD_INVERSE;
	int rc;

	{
		LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)n * n);
		shifted_copy_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(matrix, W, n, shift);
		fill_zero_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(X, (long)n * n);
		fill_zero_kernel<<<1, 64, 0, stream()>>>((float *)dInfo, 1);
	}
	// ---- 1. Cholesky ----------------------------------------------------------------------------
	for (int b = 0; b < blocks; b++) {
		const int k0 = b * kNb, nb = (n - k0 < kNb) ? n - k0 : kNb, m = n - k0 - nb;
		{
			LaunchScope scope(KC, 2.0 * kNb * kNb * kNb / 3.0);
			chol_diag_kernel<<<1, 64, 0, stream()>>>(W, n, k0, nb, Linv + (size_t)b * kNb * kNb, dInfo);
		}
		if (m <= 0) break;
		float *A21 = W + (size_t)k0 * n + k0 + nb;
		// L21 = A21 * L11^-T  (m x nb) through the panel buffer, then back into W
		rc = gemm_ex(0, 1, m, nb, nb, 1.f, A21, n, Linv + (size_t)b * kNb * kNb, kNb, 0.f, P, m, nullptr, 0, KC, gws, gBytes);
		if (rc) return rc;
		block_copy_kernel<<<blocks_for((long)m * nb, 256, 4096), 256, 0, stream()>>>(P, m, A21, n, m, nb);
		// A22 -= L21 L21^T
		float *A22 = W + (size_t)(k0 + nb) * n + k0 + nb;
		rc = gemm_ex(0, 1, m, m, nb, -1.f, P, m, P, m, 1.f, A22, n, nullptr, kGemmMirror, KC, gws, gBytes);
		if (rc) return rc;
	}
	// ---- 2. X = L^-1 ----------------------------------------------------------------------------
	for (int b = 0; b < blocks; b++) {
		const int k0 = b * kNb, nb = (n - k0 < kNb) ? n - k0 : kNb;
		block_copy_kernel<<<blocks_for((long)nb * nb, 256, 64), 256, 0, stream()>>>(Linv + (size_t)b * kNb * kNb, kNb,
		                                                                           X + (size_t)k0 * n + k0, n, nb, nb);
	}
	for (int s = 1; s < blocks; s *= 2) {
		for (int lo = 0; lo + s < blocks; lo += 2 * s) {
			const int mid = lo + s, hi = (lo + 2 * s < blocks) ? lo + 2 * s : blocks;
			const int r1 = lo * kNb, m1 = s * kNb;
			const int r2 = mid * kNb, m2 = ((hi * kNb < n) ? hi * kNb : n) - r2;
			const float *L21 = W + (size_t)r1 * n + r2;
			const float *X11 = X + (size_t)r1 * n + r1;
			const float *X22 = X + (size_t)r2 * n + r2;
			float *X21 = X + (size_t)r1 * n + r2;
			// T = L21 * X11 (m2 x m1), X21 = -X22 * T
			rc = gemm_ex(0, 0, m2, m1, m1, 1.f, L21, n, X11, n, 0.f, T, m2, nullptr, 0, KC, gws, gBytes);
			if (rc) return rc;
			rc = gemm_ex(0, 0, m2, m1, m2, -1.f, X22, n, T, m2, 0.f, X21, n, nullptr, 0, KC, gws, gBytes);
			if (rc) return rc;
		}
	}
	// ---- 3. A^-1 = X^T X ------------------------------------------------------------------------
	rc = gemm_ex(1, 0, n, n, n, 1.f, X, n, X, n, 0.f, inverse, n, nullptr, kGemmMirror | kGemmTriK, KC, gws, gBytes);
	if (rc) return rc;
	return check_launch("fitre_hip_spd_inverse");
}

int fitre_hip_spd_inverse(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes, int *info)
{
	FITRE_NEED_INIT();
	int *dInfo = nullptr;
	int rc = spd_inverse_run(matrix, n, shift, inverse, ws, wsBytes, nullptr, &dInfo);
	if (rc) return rc;
	if (info) {
		int h = 0;
		FITRE_HIP_TRY(hipMemcpyAsync(&h, dInfo, sizeof(int), hipMemcpyDeviceToHost, stream()));
		FITRE_HIP_TRY(hipStreamSynchronize(stream()));
		*info = h;
		if (h != 0) return fail(FITRE_E_ARGUMENT, "fitre_hip_spd_inverse: the matrix is not positive definite (pivot %d)", h);
	}
	return FITRE_OK;
}

int fitre_hip_spd_inverse_queued(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes, int *pivotInfo)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(pivotInfo != nullptr, "fitre_hip_spd_inverse_queued: null pivot slot");
	return spd_inverse_run(matrix, n, shift, inverse, ws, wsBytes, pivotInfo, nullptr);
}

} // extern "C"
