// Inverse of a symmetric positive definite matrix (plus a multiple of the identity): what the
// reference obtains from cusolverDnDpotrf + cusolverDnDpotrs with an identity right-hand side
// (solvers/kfac_inverses.cu:133-186), for the KFAC factors (order up to Cin*k*k + 1 = 4609).
//
//   1. W = A + shift*I = L L^T and X = L^-1 together, by halving: for W = [A11 .; A21 A22]
//        (L11, X11) of A11;  L21 = A21 X11^T;  A22 -= L21 L21^T;  (L22, X22) of that;
//        X21 = -X22 (L21 X11).
//      Every product is as large as the halves it joins (rank n/2, n/4, ... updates on the MFMA
//      tile engine instead of n/64 rank-64 ones), and a leaf of order <= 128 is one workgroup that
//      factors the block and inverts its factor without leaving LDS;
//   2. A^-1 = X^T X                 one symmetric engine product whose reduction skips the zero
//                                   part of the triangular operand.
// All matrices are column-major with leading dimension n; only lower triangles are meaningful
// in W and X (X's upper triangle is kept at zero).
#include "common.h"

namespace fitre {

constexpr int kNb = 64; // block order of the factorization
typedef float v16f __attribute__((ext_vector_type(16)));

// value of v in lane `lane` (a compile-time lane index), as a wave-uniform scalar
__device__ __forceinline__ float lane_value(float v, int lane)
{
	return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// ---- leaf of the recursion: a diagonal block of order <= 128, one workgroup, everything in LDS --------
//
// The block is cut into 32 x 32 sub-blocks.  A sub-block on the diagonal is factored, and its factor
// inverted, by one wave with a row per lane (what a step needs from another lane's row comes through
// v_readlane as a scalar: no LDS traffic, no barrier inside the 2 x 496 multiply-adds); everything off
// the diagonal is 32 x 32 x 32 products on the matrix pipes, one tile per wave, operands read from LDS:
//     for kb:  (L[kb][kb], X[kb][kb]) of W[kb][kb];   L[ib][kb] = W[ib][kb] X[kb][kb]^T  (ib > kb);
//              W[ib][jb] -= L[ib][kb] L[jb][kb]^T  (ib >= jb > kb)
//     for ib:  X[ib][jb] = -X[ib][ib] * sum_{jb <= k < ib} L[ib][k] X[k][jb]  (jb < ib)
// The matrix is column-major in LDS with a leading dimension of 129 words, which makes the
// stride-129 accesses of the transposed operands and of the accumulator layout conflict-free.
constexpr int kSub = 32;                 // order of a sub-block
constexpr int kLeafBlocks = 2;           // 64-wide block columns a leaf covers
constexpr int kLeaf = kLeafBlocks * kNb; // largest leaf order
constexpr int kLeafLd = kLeaf + 1;

// One wave: factor diagonal sub-block kb of Ms in registers and put the inverse of its factor in its place (zeros
// above the diagonal).  Returns the 1-based index inside the leaf of the first non-positive pivot of this sub-block,
// or 0.
//
// The lower half of the wave holds the block, lane i its row i; the upper half holds the inverse in the making, lane
// 32 + i its column i, which starts as the unit vector e_i and is forward-substituted column by column.  Both live in the
// SAME registers v[0..31] (one column each), because both take the same steps: step j scales column j, and then every
// later column k takes v[k] -= v[j] * L[k][j] -- the factorization in the lower half, the substitution in the upper,
// one multiply-add for the two -- with the scalar L[k][j] = lane k's v[j] fetched through v_readlane.  The scalars are
// fetched eight at a time ahead of their eight multiply-adds: with one wave on the SIMD a multiply-add right behind its
// own v_readlane waits for it.
// columns K0 .. K0+7 (those below kSub) of step J
template <int J, int K0>
__device__ __forceinline__ void factor_update_group(float (&v)[kSub])
{
	constexpr int N = (kSub - K0 < 8) ? (kSub - K0) : 8;
	int s[N];
#pragma unroll
	for (int q = 0; q < N; q++) s[q] = __builtin_amdgcn_readlane(__float_as_int(v[J]), K0 + q);
	// all lane reads of the group before its first multiply-add
	if constexpr (N == 8)
		asm volatile("" : "+s"(s[0]), "+s"(s[1]), "+s"(s[2]), "+s"(s[3]), "+s"(s[4]), "+s"(s[5]), "+s"(s[6]), "+s"(s[7]));
#pragma unroll
	for (int q = 0; q < N; q++) v[K0 + q] -= v[J] * __int_as_float(s[q]); // entries above the diagonal are never used
	// the updates stay in this step: left to itself the compiler postpones each until column k is needed and keeps
	// the 496 scalars alive (spilled) until then
	if constexpr (N == 8) {
		asm volatile("" : "+v"(v[K0]), "+v"(v[K0 + 1]), "+v"(v[K0 + 2]), "+v"(v[K0 + 3]), "+v"(v[K0 + 4]), "+v"(v[K0 + 5]),
		             "+v"(v[K0 + 6]), "+v"(v[K0 + 7]));
	} else {
#pragma unroll
		for (int q = 0; q < N; q++) asm volatile("" : "+v"(v[K0 + q]));
	}
	if constexpr (K0 + 8 < kSub) factor_update_group<J, K0 + 8>(v);
}

// steps J .. kSub-1; first: base of the 1-based pivot numbering
template <int J>
__device__ __forceinline__ void factor_steps(float (&v)[kSub], int first, int &bad)
{
	const float ajj = lane_value(v[J], J);
	if (!(ajj > 0.f) && bad == 0) bad = first + J + 1;
	const float d = rsqrtf(ajj);
	v[J] *= d; // column J of L (lane J's own entry becomes ajj / sqrt(ajj), the diagonal); row J of the inverse is complete
	if constexpr (J + 1 < kSub) {
		factor_update_group<J, J + 1>(v);
		factor_steps<J + 1>(v, first, bad);
	}
}

__device__ __forceinline__ int factor_sub_block(float *Ms, int kb, int lane)
{
	const int i = lane & (kSub - 1);
	const bool inverseHalf = lane >= kSub;
	float *wb = Ms + (kb * kSub) * kLeafLd + kb * kSub;
	float v[kSub];
#pragma unroll
	for (int j = 0; j < kSub; j++) {
		const float a = wb[j * kLeafLd + i];
		v[j] = inverseHalf ? ((i == j) ? 1.f : 0.f) : a;
	}
	int bad = 0;
	factor_steps<0>(v, kb * kSub, bad);
	// in the upper half v[r] is element (r, i) of the inverse: the lane holds column i.  The inverse replaces the block:
	// nothing reads a diagonal sub-block of the factor itself again.
	if (inverseHalf) {
#pragma unroll
		for (int j = 0; j < kSub; j++) wb[i * kLeafLd + j] = v[j];
	}
	return bad;
}

// acc += A * B for 32 x 32 operands in LDS.  element (r, k) of A is at A[k * aK + r * aR], element
// (k, c) of B at B[k * bK + c * bC].
__device__ __forceinline__ void sub_block_product(const float *A, int aR, int aK, const float *B, int bK, int bC, int lane,
                                                  v16f &acc)
{
	const int l32 = lane & 31, khalf = lane >> 5;
	const float *ap = A + l32 * aR + khalf * aK;
	const float *bp = B + l32 * bC + khalf * bK;
#pragma unroll
	for (int s = 0; s < kSub / 2; s++)
		acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ap[2 * s * aK], bp[2 * s * bK], acc, 0, 0, 0);
}

// register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32 of a 32 x 32 accumulator
__device__ __forceinline__ void store_sub_block(float *M, int lane, const v16f &acc, float scale)
{
	float *col = M + (lane & 31) * kLeafLd + 4 * (lane >> 5);
#pragma unroll
	for (int v = 0; v < 16; v++) col[8 * (v / 4) + (v % 4)] = acc[v] * scale;
}

__device__ __forceinline__ void load_sub_block(const float *M, int lane, v16f &acc)
{
	const float *col = M + (lane & 31) * kLeafLd + 4 * (lane >> 5);
#pragma unroll
	for (int v = 0; v < 16; v++) acc[v] = col[8 * (v / 4) + (v % 4)];
}

// sub-block (rb, cb) of a matrix held column-major in LDS
__device__ __forceinline__ float *sub_block(float *M, int rb, int cb) { return M + (cb * kSub) * kLeafLd + rb * kSub; }

// The diagonal block of order nn (1..128) that starts at row/column k0 of W (column-major, leading dimension
// ld, lower triangle read): X = L^-1 of its Cholesky factor into the same block of Xout (lower triangle written).
// info: set to the 1-based global index of the first non-positive pivot.
// Workgroup b of the launch works on the b-th matrix of a batch (wStride / xStride floats behind the one before).
__global__ void __launch_bounds__(256) chol_leaf_kernel(const float *W, int ld, int k0, int nn, float *Xout, int *info, long wStride,
                                                        long xStride)
{
	W += (size_t)blockIdx.x * wStride;
	Xout += (size_t)blockIdx.x * xStride;
	info += blockIdx.x;
	// ONE matrix in LDS (66 KB), turned from W into L and then into X in place: with both kept side by side (132 KB) the
	// workgroup only fits on a compute unit that runs next to nothing else, and beside another lane's chip-filling
	// product every leaf of the chain waited for that product's tail.
	__shared__ float Ws[kLeaf * kLeafLd];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int nb = (nn + kSub - 1) / kSub, order = nb * kSub;
	const float *blk = W + (size_t)k0 * ld + k0;
	// Thread (r, h) moves row r, columns of parity h: the sub-blocks on and below the diagonal only (the rest of Ws is
	// scratch), a sub-block column of sixteen loads in flight at a time.
	const int row = tid & (kLeaf - 1), half = tid >> 7, rowBlock = row >> 5;
	if (row < order) {
#pragma unroll
		for (int b = 0; b < kLeaf / kSub; b++) {
			if (b > rowBlock) break;
			float v[kSub / 2];
#pragma unroll
			for (int q = 0; q < kSub / 2; q++) {
				const int c = b * kSub + half + 2 * q;
				// rows and columns beyond the block: identity, which factors to itself
				v[q] = ((row < nn) & (c < nn)) ? blk[(size_t)c * ld + row] : ((row == c) ? 1.f : 0.f);
			}
#pragma unroll
			for (int q = 0; q < kSub / 2; q++) Ws[(b * kSub + half + 2 * q) * kLeafLd + row] = v[q];
		}
	}
	__syncthreads();

	for (int kb = 0; kb < nb; kb++) {
		if (wave == 0) {
			const int bad = factor_sub_block(Ws, kb, lane);
			if (bad != 0 && lane == 0) atomicCAS(info, 0, k0 + bad);
		}
		__syncthreads();
		// column kb of the factor below the diagonal: one sub-block per wave
		{
			const int ib = kb + 1 + wave;
			v16f acc = {};
			if (ib < nb) {
				// A = W[ib][kb]; B[k][c] = X[kb][kb][c][k]
				sub_block_product(sub_block(Ws, ib, kb), 1, kLeafLd, sub_block(Ws, kb, kb), kLeafLd, 1, lane, acc);
				store_sub_block(sub_block(Ws, ib, kb), lane, acc, 1.f);
			}
		}
		__syncthreads();
		// what is left of the lower triangle: W[ib][jb] -= L[ib][kb] L[jb][kb]^T
		{
			const int left = nb - kb - 1, tiles = left * (left + 1) / 2;
			for (int t = wave; t < tiles; t += 4) {
				int ib = 0, first = 0; // tile t of the triangle, row by row
				while (first + ib + 1 <= t) first += ++ib;
				const int jb = t - first;
				float *C = sub_block(Ws, kb + 1 + ib, kb + 1 + jb);
				v16f acc = {};
				// A = L[ib][kb]; B[k][c] = L[jb][kb][c][k]
				sub_block_product(sub_block(Ws, kb + 1 + ib, kb), 1, kLeafLd, sub_block(Ws, kb + 1 + jb, kb), kLeafLd, 1, lane, acc);
				v16f old;
				load_sub_block(C, lane, old);
#pragma unroll
				for (int v = 0; v < 16; v++) acc[v] = old[v] - acc[v];
				store_sub_block(C, lane, acc, 1.f);
			}
		}
		__syncthreads();
	}

	// The inverse of the factor below its diagonal sub-blocks, one row of sub-blocks after the other, each row of X
	// taking the place of that row of L once every wave has read it; the sums go through the unused upper triangle of
	// Ws on their way from accumulator to operand layout.
	for (int ib = 1; ib < nb; ib++) {
		const int jb = wave;
		if (jb < ib) {
			v16f acc = {};
			for (int k = jb; k < ib; k++) // A = L[ib][k]; B = X[k][jb]
				sub_block_product(sub_block(Ws, ib, k), 1, kLeafLd, sub_block(Ws, k, jb), 1, kLeafLd, lane, acc);
			store_sub_block(sub_block(Ws, jb, ib), lane, acc, 1.f);
		}
		__syncthreads();
		if (jb < ib) {
			v16f acc = {};
			// A = X[ib][ib]; B = the sum above
			sub_block_product(sub_block(Ws, ib, ib), 1, kLeafLd, sub_block(Ws, jb, ib), 1, kLeafLd, lane, acc);
			store_sub_block(sub_block(Ws, ib, jb), lane, acc, -1.f);
		}
		__syncthreads();
	}

	float *xblk = Xout + (size_t)k0 * ld + k0;
	if (row < nn) {
#pragma unroll
		for (int b = 0; b < kLeaf / kSub; b++) {
			if (b > rowBlock) break;
#pragma unroll
			for (int q = 0; q < kSub / 2; q++) {
				const int c = b * kSub + half + 2 * q;
				if (c <= row) xblk[(size_t)c * ld + row] = Ws[c * kLeafLd + row];
			}
		}
	}
}

// blockIdx.y: matrix of a batch
__global__ void __launch_bounds__(256) shifted_copy_kernel(const float *A, float *W, int n, float shift, long aStride, long wStride)
{
	A += (size_t)blockIdx.y * aStride;
	W += (size_t)blockIdx.y * wStride;
	const long total = (long)n * n;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const int c = (int)(idx / n), r = (int)(idx - (long)c * n);
		W[idx] = A[idx] + ((r == c) ? shift : 0.f);
	}
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float *p, long n, long batchStride)
{
	p += (size_t)blockIdx.y * batchStride;
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
	if (blocks <= kLeafBlocks) return 0;
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
	int batch;       // matrices worked on side by side, every launch covers all of them
	long sWs, sInv;  // floats between the workspaces (W, X, product workspace) resp. the result matrices of two of them
	long wsStrideBytes;
	float *W, *X;
	float *L21[kMaxDepth]; // per recursion depth: the off-diagonal block of the factor (a node's children work one level down)
	float *T2[kMaxDepth];  // per recursion depth: L21 * X11, the inner product of X21 (same sizes as L21)
	int n;
	int *dInfo;
	void *gws;
	size_t gBytes;
};

// floats of the largest L21 block at every recursion depth
static void l21_sizes(int blocks, int nn, int depth, size_t *need)
{
	if (blocks <= kLeafBlocks || depth >= kMaxDepth) return;
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
	if (blocks <= kLeafBlocks) {
		LaunchScope scope(KC, 2.0 * nn * (double)nn * nn / 3.0 * r.batch);
		chol_leaf_kernel<<<r.batch, 256, 0, stream()>>>(r.W, n, r0, nn, r.X, r.dInfo, r.sWs, r.sWs);
		return check_launch("chol_leaf_kernel");
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
	rc = gemm_ex_batched(r.batch, 0, 1, m, n1, n1, 1.f, A21, n, r.sWs, X11, n, r.sWs, 0.f, L21, m, r.sInv, kGemmBUpperTri, KC, r.gws, r.gBytes,
	                     r.wsStrideBytes);
	if (rc) return rc;
	// A22 -= L21 L21^T and, side by side with it, T2 = L21 * X11, the inner product of X21 = -X22 * (L21 * X11): nothing
	// needs it before the right half is done, and nothing it reads changes until then.
	float *T2 = r.T2[depth];
	const BatchedProduct update{ 0, 1, m, m, n1, -1.f, L21, m, r.sInv, L21, m, r.sInv, 1.f, A22, n, r.sWs, kGemmMirror };
	const BatchedProduct inner{ 0, 0, m, n1, n1, 1.f, L21, m, r.sInv, X11, n, r.sWs, 0.f, T2, m, r.sInv, kGemmBLowerTri };
	rc = gemm_pair_batched(r.batch, update, inner, KC, r.gws, r.gBytes, r.wsStrideBytes);
	if (rc) return rc;
	rc = chol_and_inverse(r, r1, blocks - b1, m, depth + 1);
	if (rc) return rc;
	// X21 = -X22 * (L21 * X11)
	const float *X22 = r.X + (size_t)r1 * n + r1;
	float *X21 = r.X + (size_t)r0 * n + r1;
	return gemm_ex_batched(r.batch, 0, 0, m, n1, m, -1.f, X22, n, r.sWs, T2, m, r.sInv, 0.f, X21, n, r.sWs, kGemmALowerTri, KC, r.gws, r.gBytes,
	                       r.wsStrideBytes);
}

} // namespace fitre

using namespace fitre;

extern "C" {

size_t fitre_hip_spd_inverse_workspace(int n)
{
	if (n <= 0) return 0;
	return inverse_layout(n).total;
}

// Everything one call needs to know about the matrices it inverts side by side: problem b reads
// matrix + b*matrixStride, writes inverse + b*inverseStride (floats), works in (char *)ws + b*wsStrideBytes and
// reports its pivot in pivotInfo[b].
struct InverseBatch {
	int batch;
	long matrixStride, inverseStride, wsStrideBytes;
};

// queues the whole inverse on the selected lane; pivotInfo: device ints (one per matrix) that receive the 1-based
// index of the first non-positive pivot, or stay zero (null: a slot of the workspace, single matrices only)
static int spd_inverse_run(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes, int *pivotInfo,
                           int **infoSlot, const InverseBatch &ib)
{
	FITRE_REQUIRE(matrix && inverse && ws, "fitre_hip_spd_inverse: null pointer");
	FITRE_REQUIRE(n > 0 && n <= 23000, "fitre_hip_spd_inverse: order %d out of range", n);
	FITRE_REQUIRE((((uintptr_t)ws) & 255) == 0, "fitre_hip_spd_inverse: workspace must be 256-byte aligned");
	FITRE_REQUIRE(ib.batch >= 1 && ib.batch <= 16, "fitre_hip_spd_inverse: batch of %d", ib.batch);
	const InverseLayout lay = inverse_layout(n);
	if (wsBytes < lay.total)
		return fail(FITRE_E_WORKSPACE, "fitre_hip_spd_inverse: workspace of %zu bytes is smaller than the %zu required", wsBytes,
		            lay.total);
	if (ib.batch > 1) {
		FITRE_REQUIRE(pivotInfo != nullptr, "fitre_hip_spd_inverse: a batch needs pivot slots");
		FITRE_REQUIRE(ib.wsStrideBytes % 256 == 0 && (size_t)ib.wsStrideBytes >= lay.total,
		              "fitre_hip_spd_inverse: workspaces of a batch overlap or are misaligned");
		FITRE_REQUIRE(ib.inverseStride >= (long)n * n && ib.matrixStride >= (long)n * n, "fitre_hip_spd_inverse: matrices of a batch overlap");
	}
	char *base = (char *)ws;
	float *W = (float *)(base + lay.w), *X = (float *)(base + lay.x);
	int *dInfo = pivotInfo ? pivotInfo : (int *)(base + lay.info);
	if (infoSlot) *infoSlot = dInfo;
	void *gws = base + lay.gemm;
	const size_t gBytes = lay.gemmBytes;
	const int blocks = (n + kNb - 1) / kNb;
	const int KC = FITRE_KC_SPD_INVERSE;
	const long sWs = ib.wsStrideBytes / 4;
	int rc;

	{
		LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)n * n * ib.batch);
		const dim3 grid(blocks_for((long)n * n, 256, 8192), (unsigned)ib.batch);
		shifted_copy_kernel<<<grid, 256, 0, stream()>>>(matrix, W, n, shift, ib.matrixStride, sWs);
		fill_zero_kernel<<<grid, 256, 0, stream()>>>(X, (long)n * n, sWs);
		fill_zero_kernel<<<1, 64, 0, stream()>>>((float *)dInfo, ib.batch, 0);
	}
	// ---- 1. Cholesky factor and its inverse ---------------------------------------------------
	// The result matrix is free until the last product and holds the temporaries: the per-depth L21 blocks (a quarter, a
	// sixteenth, ... of it) in its first half, the per-depth T2 blocks, of the same sizes, in the second.
	InverseRun run;
	run.batch = ib.batch, run.sWs = sWs, run.sInv = ib.inverseStride, run.wsStrideBytes = ib.wsStrideBytes;
	run.W = W, run.X = X, run.n = n, run.dInfo = dInfo, run.gws = gws, run.gBytes = gBytes;
	{
		size_t need[kMaxDepth] = {};
		l21_sizes(blocks, n, 0, need);
		size_t off = 0;
		for (int d = 0; d < kMaxDepth; d++) {
			run.L21[d] = inverse + off;
			run.T2[d] = inverse + ((size_t)n * n + 1) / 2 + off;
			off += (need[d] + 63) & ~(size_t)63;
		}
		FITRE_REQUIRE(off <= (size_t)n * n / 2, "fitre_hip_spd_inverse: temporaries do not fit (order %d)", n);
	}
	rc = chol_and_inverse(run, 0, blocks, n);
	if (rc) return rc;
	// ---- 2. A^-1 = X^T X ------------------------------------------------------------------------
	rc = gemm_ex_batched(ib.batch, 1, 0, n, n, n, 1.f, X, n, sWs, X, n, sWs, 0.f, inverse, n, ib.inverseStride, kGemmMirror | kGemmTriK,
	                     KC, gws, gBytes, ib.wsStrideBytes);
	if (rc) return rc;
	return check_launch("fitre_hip_spd_inverse");
}

int fitre_hip_spd_inverse(const float *matrix, int n, float shift, float *inverse, void *ws, size_t wsBytes, int *info)
{
	FITRE_NEED_INIT();
	int *dInfo = nullptr;
	int rc = spd_inverse_run(matrix, n, shift, inverse, ws, wsBytes, nullptr, &dInfo, InverseBatch{ 1, 0, 0, 0 });
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
	return spd_inverse_run(matrix, n, shift, inverse, ws, wsBytes, pivotInfo, nullptr, InverseBatch{ 1, 0, 0, 0 });
}

int fitre_hip_spd_inverse_batched_queued(int batch, const float *matrix, long matrixStride, int n, float shift, float *inverse,
                                         long inverseStride, void *ws, size_t wsBytes, long wsStrideBytes, int *pivotInfo)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(pivotInfo != nullptr, "fitre_hip_spd_inverse_batched_queued: null pivot slots");
	return spd_inverse_run(matrix, n, shift, inverse, ws, wsBytes, pivotInfo, nullptr,
	                       InverseBatch{ batch, matrixStride, inverseStride, wsStrideBytes });
}

} // extern "C"
