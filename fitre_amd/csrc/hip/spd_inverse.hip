// Inverse of a symmetric positive definite matrix (plus a multiple of the identity): what the
// reference obtains from cusolverDnDpotrf + cusolverDnDpotrs with an identity right-hand side
// (solvers/kfac_inverses.cu:133-186), for the KFAC factors (order up to Cin*k*k + 1 = 4609).
//
//   1. W = A + shift*I = L L^T and X = L^-1 together, by halving: for W = [A11 .; A21 A22]
//        (L11, X11) of A11;  L21 = A21 X11^T;  A22 -= L21 L21^T;  (L22, X22) of that;
//        X21 = -X22 (L21 X11).
//      Every product is as large as the halves it joins (rank n/2, n/4, ... updates on the MFMA
//      tile engine instead of n/64 rank-64 ones), and a 64 x 64 leaf is one one-wave kernel that
//      factors the block and inverts its factor;
//   2. A^-1 = X^T X                 one symmetric engine product whose reduction skips the zero
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
// inverse of the factor into the same block of Xout (lower triangle, leading dimension ld).  Lane i holds row i in
// registers; what a step needs from another lane's row comes through v_readlane as a scalar, so
// there is no LDS traffic and no barrier in the 2 x 2016 multiply-adds.
// info: set to the 1-based global index of the first non-positive pivot.
__global__ void __launch_bounds__(64) chol_diag_kernel(float *W, int ld, int k0, int nb, float *Xout, int *info)
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
	// x[r] is element (r, i) of the inverse, i.e. this lane holds column i.  Columns are contiguous in
	// memory: turn the block through LDS so that a store instruction writes 64 consecutive rows of one column.
	__shared__ float turn[kNb][kNb + 1];
#pragma unroll
	for (int r = 0; r < kNb; r++) turn[i][r] = x[r];
	__syncthreads();
	float *xblk = Xout + (size_t)k0 * ld + k0;
	for (int c = 0; c < nb; c++)
		if ((i < nb) & (i >= c)) xblk[(size_t)c * ld + i] = turn[c][i];
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

// largest split-K workspace the products of a node of `blocks` 64-wide block columns (order nn) ask for
static size_t node_gemm_workspace(int blocks, int nn)
{
	if (blocks <= 1) return 0;
	const int b1 = blocks / 2, n1 = b1 * kNb, m = nn - n1;
	size_t g = gemm_ex_workspace(m, n1, n1, 0);
	size_t a = gemm_ex_workspace(m, m, n1, kGemmMirror);
	g = a > g ? a : g;
	a = gemm_ex_workspace(m, n1, m, 0);
	g = a > g ? a : g;
	a = node_gemm_workspace(b1, n1);
	g = a > g ? a : g;
	a = node_gemm_workspace(blocks - b1, m);
	return a > g ? a : g;
}

static InverseLayout inverse_layout(int n)
{
	InverseLayout l;
	const size_t nn = (size_t)n * n * sizeof(float);
	const int blocks = (n + kNb - 1) / kNb;
	size_t g = node_gemm_workspace(blocks, n);
	size_t c = gemm_ex_workspace(n, n, n, kGemmMirror);
	g = c > g ? c : g;
	l.w = 0;
	l.x = align256(l.w + nn);
	l.linv = align256(l.x + nn);
	l.panel = align256(l.linv + (size_t)kNb * kNb * sizeof(float));
	l.info = l.panel; // no panel buffer: the products' temporaries live in the result matrix
	l.gemm = align256(l.info + 256);
	l.gemmBytes = align256(g + 256);
	l.total = l.gemm + l.gemmBytes;
	return l;
}

// state of one inverse while its launches are queued
constexpr int kMaxDepth = 16;
struct InverseRun {
	float *W, *X;
	float *L21[kMaxDepth]; // per recursion depth: the off-diagonal block of the factor (a node's children work one level down)
	float *T2;             // temporary of the last product of a node
	int n;
	int *dInfo;
	void *gws;
	size_t gBytes;
};

// floats of the largest L21 block at every recursion depth
static void l21_sizes(int blocks, int nn, int depth, size_t *need)
{
	if (blocks <= 1 || depth >= kMaxDepth) return;
	const int b1 = blocks / 2, n1 = b1 * kNb, m = nn - n1;
	const size_t sz = (size_t)m * n1;
	if (sz > need[depth]) need[depth] = sz;
	l21_sizes(b1, n1, depth + 1, need);
	l21_sizes(blocks - b1, m, depth + 1, need);
}

// L and X = L^-1 of the diagonal block of `blocks` block columns that starts at row/column r0 (order nn)
static int chol_and_inverse(const InverseRun &r, int r0, int blocks, int nn, int depth = 0)
{
	const int KC = FITRE_KC_SPD_INVERSE;
	const int n = r.n;
	if (blocks == 1) {
		LaunchScope scope(KC, 2.0 * kNb * kNb * kNb / 3.0);
		chol_diag_kernel<<<1, 64, 0, stream()>>>(r.W, n, r0, nn, r.X, r.dInfo);
		return check_launch("chol_diag_kernel");
	}
	const int b1 = blocks / 2, n1 = b1 * kNb, m = nn - n1, r1 = r0 + n1;
	FITRE_REQUIRE(depth < kMaxDepth, "fitre_hip_spd_inverse: recursion deeper than %d", kMaxDepth);
	int rc = chol_and_inverse(r, r0, b1, n1, depth + 1);
	if (rc) return rc;
	const float *A21 = r.W + (size_t)r0 * n + r1;
	float *A22 = r.W + (size_t)r1 * n + r1;
	const float *X11 = r.X + (size_t)r0 * n + r0;
	float *L21 = r.L21[depth];
	// L21 = A21 * X11^T (m x n1); W keeps A21: only X is needed in the end
	rc = gemm_ex(0, 1, m, n1, n1, 1.f, A21, n, X11, n, 0.f, L21, m, nullptr, 0, KC, r.gws, r.gBytes);
	if (rc) return rc;
	// A22 -= L21 L21^T
	rc = gemm_ex(0, 1, m, m, n1, -1.f, L21, m, L21, m, 1.f, A22, n, nullptr, kGemmMirror, KC, r.gws, r.gBytes);
	if (rc) return rc;
	rc = chol_and_inverse(r, r1, blocks - b1, m, depth + 1);
	if (rc) return rc;
	// X21 = -X22 * (L21 * X11)
	const float *X22 = r.X + (size_t)r1 * n + r1;
	float *X21 = r.X + (size_t)r0 * n + r1;
	rc = gemm_ex(0, 0, m, n1, n1, 1.f, L21, m, X11, n, 0.f, r.T2, m, nullptr, 0, KC, r.gws, r.gBytes);
	if (rc) return rc;
	return gemm_ex(0, 0, m, n1, m, -1.f, X22, n, r.T2, m, 0.f, X21, n, nullptr, 0, KC, r.gws, r.gBytes);
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
	float *W = (float *)(base + lay.w), *X = (float *)(base + lay.x);
	int *dInfo = pivotInfo ? pivotInfo : (int *)(base + lay.info);
	if (infoSlot) *infoSlot = dInfo;
	void *gws = base + lay.gemm;
	const size_t gBytes = lay.gemmBytes;
	const int blocks = (n + kNb - 1) / kNb;
	const int KC = FITRE_KC_SPD_INVERSE;
	int rc;

	{
		LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)n * n);
		shifted_copy_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(matrix, W, n, shift);
		fill_zero_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(X, (long)n * n);
		fill_zero_kernel<<<1, 64, 0, stream()>>>((float *)dInfo, 1);
	}
	// ---- 1. Cholesky factor and its inverse ---------------------------------------------------
	// The result matrix is free until the last product and holds the temporaries: T2 (at most a
	// quarter of the matrix) in its second half, the per-depth L21 blocks (a quarter, a sixteenth,
	// ... of it) in the first.
	InverseRun run;
	run.W = W, run.X = X, run.n = n, run.dInfo = dInfo, run.gws = gws, run.gBytes = gBytes;
	run.T2 = inverse + ((size_t)n * n + 1) / 2;
	{
		size_t need[kMaxDepth] = {};
		l21_sizes(blocks, n, 0, need);
		size_t off = 0;
		for (int d = 0; d < kMaxDepth; d++) {
			run.L21[d] = inverse + off;
			off += (need[d] + 63) & ~(size_t)63;
		}
		FITRE_REQUIRE(off <= ((size_t)n * n + 1) / 2, "fitre_hip_spd_inverse: temporaries do not fit (order %d)", n);
	}
	rc = chol_and_inverse(run, 0, blocks, n);
	if (rc) return rc;
	// ---- 2. A^-1 = X^T X ------------------------------------------------------------------------
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
