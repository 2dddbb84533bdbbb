// Float64 matrix products on v_mfma_f64_16x16x4_f64 and, built from them, the float64 inverse of a symmetric positive
// definite matrix.  The KFAC leg of the reference is double throughout (core/datadefs.h:5; cusolverDnDpotrf / Dpotrs,
// solvers/kfac_inverses.cu:133-186; cublasDgemm in solvers/kfac_natural_gradient.cu:36-241), and with the benchmark's
// damping of 1e-3 its factors have condition numbers of 1e4 .. 1e6: a float32 factor, a float32 Cholesky or a float32
// inverse each cost the natural gradient several digits.  So the factors are accumulated, factored, inverted and applied
// in float64 here; only what has to cross the caller's float arrays is stored as floats (a symmetric inverse as a pair
// of floats per element: the rounded value in the upper triangle, the remainder in the lower one).
//
// One kernel serves every product: operands are read through a small descriptor (float, double or such a float pair;
// any strides; an optional constant row or column, the bias row of a KFAC input factor), converted to double on their
// way into LDS, and multiplied on the float64 matrix instruction, which is slow enough (a 16 x 16 x 4 block per 64
// cycles) that neither the conversion nor element-wise loads show.
#include "common.h"

namespace fitre {

typedef double v4d __attribute__((ext_vector_type(4)));

struct DgemmArgs {
	int M, N, K;
	DMat A, B; // A(i, k), B(k, j)
	DOut C;
	double alpha, beta, diagAdd;
	int flags, splits, tilesM, tilesN;
	double *partials;
	float *diagRemainder; // float-pair results: the remainders of the diagonal, folded into the matrix by a pass of its own
	int aKContig, bKContig;
};

constexpr int kDgBK = 16;
static size_t dalign(size_t v) { return (v + 255) & ~(size_t)255; }

__device__ __forceinline__ double dmat_load(const DMat &m, long r, long c)
{
	if (m.kind == FITRE_MAT_F64) return ((const double *)m.p)[r * m.rs + c * m.cs];
	const float *f = (const float *)m.p;
	if (m.kind == FITRE_MAT_F32) {
		const bool ones = (r == m.onesRow) | (c == m.onesCol);
		const float v = f[ones ? 0 : r * m.rs + c * m.cs];
		return ones ? m.onesValue : (double)v;
	}
	// symmetric float pair of order rs: rounded value on and above the diagonal, remainder below; the remainder of diagonal
	// element k shares a word with that of element (k, k + 1) (16 bits each, see pair_fold_diagonal_kernel)
	const long a = r < c ? r : c, b = r < c ? c : r, n = m.rs;
	const double hi = (double)f[b * m.cs + a];
	if (a == b) {
		if (n < 3) return hi;
		const uint32_t w = __float_as_uint(f[(a + 1 < n) ? a * m.cs + a + 1 : n - 1]);
		return hi + (double)__uint_as_float(w << 16);
	}
	uint32_t w = __float_as_uint(f[a * m.cs + b]);
	if (n >= 3 && (b == a + 1 || (a == 0 && b == n - 1))) w &= 0xFFFF0000u;
	return hi + (double)__uint_as_float(w);
}

// C(i, j) = alpha * v + beta * C(i, j) (+ diagAdd on the diagonal); offDiagonalTile: also store the mirrored element
__device__ __forceinline__ void dgemm_store(const DgemmArgs &g, long i, long j, double v, bool mirrorToo, bool diagonalTile)
{
	if (i >= g.M || j >= g.N) return;
	double r = g.alpha * v;
	if (g.C.kind == FITRE_MAT_SYM_PAIR) {
		if (i > j) return; // diagonal tiles hold both halves
		float *f = (float *)g.C.p;
		if (i == j) r += g.diagAdd;
		const float hi = (float)r;
		f[j * g.C.cs + i] = hi;
		if (i < j) f[i * g.C.cs + j] = (float)(r - (double)hi);
		else g.diagRemainder[i] = (float)(r - (double)hi);
		return;
	}
	(void)diagonalTile;
	const long idx = i * g.C.rs + j * g.C.cs;
	if (g.C.kind == FITRE_MAT_F64) {
		double *c = (double *)g.C.p;
		if (g.beta != 0.0) r += g.beta * c[idx];
		if (i == j) r += g.diagAdd;
		c[idx] = r;
		if (mirrorToo) c[j * g.C.rs + i * g.C.cs] = r;
	} else {
		float *c = (float *)g.C.p;
		if (g.beta != 0.0) r += g.beta * (double)c[idx];
		if (i == j) r += g.diagAdd;
		c[idx] = (float)r;
		if (mirrorToo) c[j * g.C.rs + i * g.C.cs] = (float)r;
	}
}

// Tile TM x TN, 256 threads = 2 x 2 waves, a wave (TM/2) x (TN/2) = MI x NI blocks of 16 x 16.
// Lane l of a block holds A(i = l % 16, k = l / 16), B(k = l / 16, j = l % 16) and, in register r of the accumulator,
// C(i = 4 r + l / 16, j = l % 16).
// blockIdx.x: tile (row-major over tilesM x tilesN), blockIdx.y: split of the reduction.
template <int TM, int TN>
__global__ void __launch_bounds__(256) dgemm_kernel(const DgemmArgs g)
{
	constexpr int BK = kDgBK;
	constexpr int LDA = TM + 16, LDB = TN + 16; // row offsets of 16 doubles mod 32: the four k rows of a fragment read hit different banks
	constexpr int WTM = TM / 2, WTN = TN / 2, MI = WTM / 16, NI = WTN / 16;
	constexpr int EA = TM * BK / 256, EB = TN * BK / 256;
	__shared__ double As[BK * LDA];
	__shared__ double Bs[BK * LDB];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int tile = blockIdx.x, ti = tile / g.tilesN, tj = tile - ti * g.tilesN;
	if ((g.flags & kDgMirror) && tj < ti) return;
	const int i0 = ti * TM, j0 = tj * TN;
	int kb = 0, ke = g.K;
	if (g.flags & kDgAUpper) kb = max(kb, i0);
	if (g.flags & kDgBLower) kb = max(kb, j0);
	if (g.flags & kDgALower) ke = min(ke, i0 + TM);
	if (g.flags & kDgBUpper) ke = min(ke, j0 + TN);
	kb &= ~(BK - 1);
	int k0 = kb, k1 = ke;
	if (g.splits > 1) {
		int chunk = (ke - kb + g.splits - 1) / g.splits;
		chunk = (chunk + BK - 1) / BK * BK;
		k0 = kb + (int)blockIdx.y * chunk;
		k1 = min(ke, k0 + chunk);
	}

	v4d acc[MI][NI];
#pragma unroll
	for (int mi = 0; mi < MI; mi++)
#pragma unroll
		for (int ni = 0; ni < NI; ni++) acc[mi][ni] = v4d{ 0.0, 0.0, 0.0, 0.0 };

	double ra[EA], rb[EB];
	auto fetch = [&](int kk) {
#pragma unroll
		for (int q = 0; q < EA; q++) {
			int row, k;
			if (g.aKContig) k = tid & 15, row = (tid >> 4) + 16 * q;
			else row = tid % TM, k = tid / TM + (256 / TM) * q;
			const long gi = i0 + row, gk = kk + k;
			ra[q] = (gi < g.M && gk < k1) ? dmat_load(g.A, gi, gk) : 0.0;
		}
#pragma unroll
		for (int q = 0; q < EB; q++) {
			int col, k;
			if (g.bKContig) k = tid & 15, col = (tid >> 4) + 16 * q;
			else col = tid % TN, k = tid / TN + (256 / TN) * q;
			const long gj = j0 + col, gk = kk + k;
			rb[q] = (gj < g.N && gk < k1) ? dmat_load(g.B, gk, gj) : 0.0;
		}
	};
	auto stage = [&]() {
#pragma unroll
		for (int q = 0; q < EA; q++) {
			int row, k;
			if (g.aKContig) k = tid & 15, row = (tid >> 4) + 16 * q;
			else row = tid % TM, k = tid / TM + (256 / TM) * q;
			As[k * LDA + row] = ra[q];
		}
#pragma unroll
		for (int q = 0; q < EB; q++) {
			int col, k;
			if (g.bKContig) k = tid & 15, col = (tid >> 4) + 16 * q;
			else col = tid % TN, k = tid / TN + (256 / TN) * q;
			Bs[k * LDB + col] = rb[q];
		}
	};

	if (k0 < k1) fetch(k0);
	for (int kk = k0; kk < k1; kk += BK) {
		__syncthreads(); // the previous slice has been read
		stage();
		__syncthreads();
		if (kk + BK < k1) fetch(kk + BK); // in flight while this slice is multiplied
		const double *ap = As + (lane >> 4) * LDA + wm * WTM + (lane & 15);
		const double *bp = Bs + (lane >> 4) * LDB + wn * WTN + (lane & 15);
#pragma unroll
		for (int k4 = 0; k4 < BK / 4; k4++) {
			double a[MI], b[NI];
#pragma unroll
			for (int mi = 0; mi < MI; mi++) a[mi] = ap[k4 * 4 * LDA + mi * 16];
#pragma unroll
			for (int ni = 0; ni < NI; ni++) b[ni] = bp[k4 * 4 * LDB + ni * 16];
#pragma unroll
			for (int mi = 0; mi < MI; mi++)
#pragma unroll
				for (int ni = 0; ni < NI; ni++) acc[mi][ni] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
		}
	}

	if (g.splits > 1) {
		// partial tile, element e of thread tid at [e][tid]: coalesced for the reduction kernel, which has the same mapping
		constexpr int ACC = MI * NI * 4;
		double *dst = g.partials + ((size_t)blockIdx.y * gridDim.x + tile) * (size_t)(ACC * 256) + tid;
#pragma unroll
		for (int mi = 0; mi < MI; mi++)
#pragma unroll
			for (int ni = 0; ni < NI; ni++)
#pragma unroll
				for (int r = 0; r < 4; r++) dst[(size_t)((mi * NI + ni) * 4 + r) * 256] = acc[mi][ni][r];
		return;
	}
	const bool mirrorToo = (g.flags & kDgMirror) && tj > ti && g.C.kind != FITRE_MAT_SYM_PAIR;
#pragma unroll
	for (int mi = 0; mi < MI; mi++)
#pragma unroll
		for (int ni = 0; ni < NI; ni++)
#pragma unroll
			for (int r = 0; r < 4; r++)
				dgemm_store(g, i0 + wm * WTM + mi * 16 + 4 * r + (lane >> 4), j0 + wn * WTN + ni * 16 + (lane & 15), acc[mi][ni][r], mirrorToo,
				            ti == tj);
}

// adds the partial tiles of the splits in split order and stores the result (one workgroup per tile)
template <int TM, int TN>
__global__ void __launch_bounds__(256) dgemm_reduce_kernel(const DgemmArgs g)
{
	constexpr int WTM = TM / 2, WTN = TN / 2, MI = WTM / 16, NI = WTN / 16, ACC = MI * NI * 4;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int tile = blockIdx.x, ti = tile / g.tilesN, tj = tile - ti * g.tilesN;
	if ((g.flags & kDgMirror) && tj < ti) return;
	const int i0 = ti * TM, j0 = tj * TN;
	const bool mirrorToo = (g.flags & kDgMirror) && tj > ti && g.C.kind != FITRE_MAT_SYM_PAIR;
	const size_t tiles = gridDim.x;
	for (int e = 0; e < ACC; e++) {
		double sum = 0.0;
		for (int s = 0; s < g.splits; s++) sum += g.partials[((size_t)s * tiles + tile) * (size_t)(ACC * 256) + (size_t)e * 256 + tid];
		const int mi = e / (NI * 4), ni = (e / 4) % NI, r = e & 3;
		dgemm_store(g, i0 + wm * WTM + mi * 16 + 4 * r + (lane >> 4), j0 + wn * WTN + ni * 16 + (lane & 15), sum, mirrorToo, ti == tj);
	}
}

// A float-pair matrix of order n has n (n + 1) / 2 values and n (n - 1) / 2 words below the diagonal for their
// remainders: none for the diagonal's.  The word of element (k + 1, k) -- (n - 1, 0) for the last diagonal element --
// is therefore shared: its upper 16 bits keep the remainder of its own element, truncated, its lower 16 bits take the
// upper 16 bits of the diagonal element's remainder.  Both values then have 32 significant bits instead of 48 resp. 24.
// Orders below 3 keep the diagonal at float precision.
__global__ void __launch_bounds__(256) pair_fold_diagonal_kernel(float *pairs, long ld, int n, const float *diagRemainder)
{
	const int k = blockIdx.x * blockDim.x + threadIdx.x;
	if (k >= n || n < 3) return;
	float *word = pairs + ((k + 1 < n) ? (long)k * ld + k + 1 : (long)(n - 1));
	*word = __uint_as_float((__float_as_uint(*word) & 0xFFFF0000u) | (__float_as_uint(diagRemainder[k]) >> 16));
}

struct DgemmPlan {
	int tile;   // 128 or 64
	int splits;
	int tilesM, tilesN;
};

static DgemmPlan plan_dgemm(long M, long N, long K, int flags)
{
	DgemmPlan p;
	const int cus = device_compute_units() > 0 ? device_compute_units() : 256;
	auto count = [&](int t) {
		const long tm = (M + t - 1) / t, tn = (N + t - 1) / t;
		return (flags & kDgMirror) ? tm * (tm + 1) / 2 : tm * tn;
	};
	p.tile = count(128) >= cus ? 128 : 64;
	p.tilesM = (int)((M + p.tile - 1) / p.tile);
	p.tilesN = (int)((N + p.tile - 1) / p.tile);
	const long live = count(p.tile);
	long splits = 1;
	if (live < cus) {
		splits = (2 * cus + live - 1) / live;
		const long deepest = K / 256 > 0 ? K / 256 : 1; // at least 256 reduction steps per split
		if (splits > deepest) splits = deepest;
		if (splits > 64) splits = 64;
	}
	p.splits = (int)splits;
	return p;
}

static size_t dgemm_partial_bytes(const DgemmPlan &p)
{
	if (p.splits <= 1) return 0;
	return (size_t)p.splits * p.tilesM * p.tilesN * (size_t)p.tile * p.tile * sizeof(double);
}

static DMat transposed(const DMat &m)
{
	DMat t = m;
	if (m.kind != FITRE_MAT_SYM_PAIR) t.rs = m.cs, t.cs = m.rs;
	t.onesRow = m.onesCol, t.onesCol = m.onesRow;
	return t;
}

size_t dgemm_workspace(long M, long N, long K, int flags)
{
	// the kernel may work on the transposed problem; the plan is symmetric in M and N
	return dalign(dgemm_partial_bytes(plan_dgemm(M, N, K, flags))) + dalign((size_t)(M > N ? M : N) * sizeof(float)) + 256;
}

// C(M x N) = alpha * A(M x K) * B(K x N) + beta * C (+ diagAdd on the diagonal), on the selected lane
int dgemm(long M, long N, long K, double alpha, DMat A, DMat B, double beta, DOut C, double diagAdd, int flags, int kernelClass,
          void *ws, size_t wsBytes)
{
	FITRE_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1l << 30) && N < (1l << 30) && K < (1l << 30), "float64 product: shape %ld x %ld x %ld", M, N, K);
	FITRE_REQUIRE(A.p && B.p && C.p, "float64 product: null pointer");
	FITRE_REQUIRE(!(flags & kDgMirror) || M == N, "float64 product: a mirrored product must be square");
	FITRE_REQUIRE(C.kind != FITRE_MAT_SYM_PAIR || ((flags & kDgMirror) && beta == 0.0), "float64 product: a float-pair result needs a symmetric product and beta = 0");
	// the lanes of an accumulator block run along j: make that the direction in which the result is contiguous
	if (C.kind != FITRE_MAT_SYM_PAIR && C.rs < C.cs) {
		const DMat a = transposed(B), b = transposed(A);
		A = a, B = b;
		const long t = M;
		M = N, N = t;
		const long s = C.rs;
		C.rs = C.cs, C.cs = s;
		int f = flags & kDgMirror;
		if (flags & kDgALower) f |= kDgBUpper;
		if (flags & kDgAUpper) f |= kDgBLower;
		if (flags & kDgBLower) f |= kDgAUpper;
		if (flags & kDgBUpper) f |= kDgALower;
		flags = f;
	}
	float *diagRemainder = nullptr;
	if (C.kind == FITRE_MAT_SYM_PAIR) {
		const size_t tail = dalign((size_t)M * sizeof(float));
		FITRE_REQUIRE(ws && (((uintptr_t)ws) & 255) == 0 && wsBytes >= tail + 256, "float64 product: a float-pair result needs %zu bytes of workspace", tail + 256);
		wsBytes = (wsBytes - tail) & ~(size_t)255;
		diagRemainder = (float *)((char *)ws + wsBytes);
	}
	DgemmPlan p = plan_dgemm(M, N, K, flags);
	while (p.splits > 1 && (((uintptr_t)ws & 255) != 0 || dgemm_partial_bytes(p) > wsBytes)) p.splits--;
	DgemmArgs g;
	g.M = (int)M, g.N = (int)N, g.K = (int)K;
	g.A = A, g.B = B, g.C = C;
	g.alpha = alpha, g.beta = beta, g.diagAdd = diagAdd;
	g.flags = flags, g.splits = p.splits, g.tilesM = p.tilesM, g.tilesN = p.tilesN;
	g.partials = (double *)ws;
	g.diagRemainder = diagRemainder;
	g.aKContig = (A.kind != FITRE_MAT_SYM_PAIR && A.cs == 1 && A.rs != 1);
	g.bKContig = (B.kind != FITRE_MAT_SYM_PAIR && B.rs == 1 && B.cs != 1);
	const dim3 grid((unsigned)(p.tilesM * p.tilesN), (unsigned)p.splits);
	const double flops = ((flags & kDgMirror) ? 1.0 : 2.0) * (double)M * (double)N * (double)K;
	LaunchScope scope(kernelClass, flops);
	if (p.tile == 128) {
		dgemm_kernel<128, 128><<<grid, 256, 0, stream()>>>(g);
		if (p.splits > 1) dgemm_reduce_kernel<128, 128><<<grid.x, 256, 0, stream()>>>(g);
	} else {
		dgemm_kernel<64, 64><<<grid, 256, 0, stream()>>>(g);
		if (p.splits > 1) dgemm_reduce_kernel<64, 64><<<grid.x, 256, 0, stream()>>>(g);
	}
	if (diagRemainder) pair_fold_diagonal_kernel<<<blocks_for(M, 256), 256, 0, stream()>>>((float *)C.p, C.cs, (int)M, diagRemainder);
	return check_launch("float64 product");
}

// ---- leaf of the inverse: a diagonal block of order <= 64, one workgroup, float64 in LDS ----------------------------
//
// One sweep of 64 steps, one barrier each, does the Cholesky factorisation W = L L^T (right-looking) and the inverse of
// the factor together: the column operations that turn L^T into the identity (scale column j by 1 / l_jj, then column
// k -= column j * l_kj for k > j) turn the identity into L^-T, and step j of them needs exactly column j of L, which
// step j of the factorisation has just produced.  Thread (i, q) = (tid % 64, tid / 64) owns row i of the trailing
// update (columns k = j+1+q, j+5+q, ...) and column i of the inverse in the making (rows q, q+4, ...).  A finished
// row of X = L^-1 goes to the unused upper triangle of W's copy.
constexpr int kDLeaf = 64, kDLd = kDLeaf + 1;

__global__ void __launch_bounds__(256) dchol_leaf_kernel(const double *W, long ld, int k0, int nn, double *X, int *info)
{
	__shared__ double Ws[kDLeaf * kDLd]; // column-major: (i, k) at k * kDLd + i
	__shared__ double Ys[kDLeaf * kDLd]; // L^-T in the making, column-major
	__shared__ double diagX[kDLeaf];
	const int tid = threadIdx.x, i = tid & 63, q = tid >> 6;
	const double *blk = W + (size_t)k0 * ld + k0;
	for (int c = q; c < kDLeaf; c += 4) {
		double v = (i == c) ? 1.0 : 0.0; // beyond the block: identity, which factors to itself
		if (i < nn && c < nn && i >= c) v = blk[(size_t)c * ld + i];
		Ws[c * kDLd + i] = v;
		Ys[c * kDLd + i] = (i == c) ? 1.0 : 0.0;
	}
	for (int j = 0; j < kDLeaf; j++) {
		__syncthreads();
		const double ajj = Ws[j * kDLd + j];
		if (!(ajj > 0.0) && tid == 0) atomicCAS(info, 0, k0 + j + 1);
		const double d = 1.0 / sqrt(ajj);
		if (i > j) {
			const double lij = Ws[j * kDLd + i] * d;
			for (int k = j + 1 + q; k <= i; k += 4) Ws[k * kDLd + i] -= lij * (Ws[j * kDLd + k] * d);
			for (int r = q; r <= j; r += 4) Ys[i * kDLd + r] -= (Ys[j * kDLd + r] * d) * lij;
		} else if (q == 0) {
			// row j of X = column j of L^-T, scaled: final
			if (i == j) diagX[j] = d;
			else Ws[j * kDLd + i] = Ys[j * kDLd + i] * d; // (i, j) with i < j: above the diagonal, read by nobody
		}
	}
	__syncthreads();
	double *xblk = X + (size_t)k0 * ld + k0;
	// X(j, r), r <= j, from Ws(r, j); thread: row j = i, columns r = q, q + 4, ...
	if (i < nn)
		for (int r = q; r <= i; r += 4) xblk[(size_t)r * ld + i] = (r == i) ? diagX[i] : Ws[i * kDLd + r];
}

__global__ void __launch_bounds__(256) dfill_zero_kernel(double *p, long n)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) p[idx] = 0.0;
}

// float matrix (+ shift on the diagonal) -> double matrix, both n x n dense
__global__ void __launch_bounds__(256) widen_shift_kernel(const float *A, double *W, int n, double shift)
{
	const long total = (long)n * n;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const int c = (int)(idx / n), r = (int)(idx - (long)c * n);
		W[idx] = (double)A[idx] + ((r == c) ? shift : 0.0);
	}
}

__global__ void fill_int_kernel(int *p, int n, int v)
{
	const int i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) p[i] = v;
}

constexpr int kDMaxDepth = 16;
struct DInverseLayout {
	size_t x, l21[kDMaxDepth], t2[kDMaxDepth], info, gemm, gemmBytes, total;
};

static void dnode_sizes(int blocks, int nn, int depth, size_t *need, size_t *gemm)
{
	if (blocks <= 1 || depth >= kDMaxDepth) return;
	const int b1 = blocks / 2, n1 = b1 * kDLeaf, m = nn - n1;
	const size_t sz = (size_t)m * n1;
	if (sz > need[depth]) need[depth] = sz;
	size_t g = dgemm_workspace(m, n1, n1, 0);
	size_t a = dgemm_workspace(m, m, n1, kDgMirror);
	g = a > g ? a : g;
	a = dgemm_workspace(m, n1, m, 0);
	g = a > g ? a : g;
	if (g > *gemm) *gemm = g;
	dnode_sizes(b1, n1, depth + 1, need, gemm);
	dnode_sizes(blocks - b1, m, depth + 1, need, gemm);
}

static DInverseLayout dinverse_layout(int n)
{
	DInverseLayout l;
	const int blocks = (n + kDLeaf - 1) / kDLeaf;
	size_t need[kDMaxDepth] = {};
	size_t g = dgemm_workspace(n, n, n, kDgMirror);
	dnode_sizes(blocks, n, 0, need, &g);
	size_t off = 0;
	l.x = off, off = dalign(off + (size_t)n * n * sizeof(double));
	for (int d = 0; d < kDMaxDepth; d++) l.l21[d] = off, off = dalign(off + need[d] * sizeof(double));
	for (int d = 0; d < kDMaxDepth; d++) l.t2[d] = off, off = dalign(off + need[d] * sizeof(double));
	l.info = off, off += 256;
	l.gemm = off, l.gemmBytes = dalign(g);
	l.total = off + l.gemmBytes;
	return l;
}

struct DInverseRun {
	double *W, *X;
	double *L21[kDMaxDepth], *T2[kDMaxDepth];
	int n;
	int *dInfo;
	void *gws;
	size_t gBytes;
};

// L and X = L^-1 of the diagonal block of `blocks` 64-wide block columns that starts at row / column r0 (order nn), by
// halving (the scheme of the float32 inverse): (L11, X11) of A11; L21 = A21 X11^T; A22 -= L21 L21^T; (L22, X22) of
// that; X21 = -X22 (L21 X11).  Column-major, leading dimension n; X's upper triangle stays zero.
static int dchol_and_inverse(const DInverseRun &r, int r0, int blocks, int nn, int depth)
{
	const int KC = FITRE_KC_SPD_INVERSE;
	const long n = r.n;
	if (blocks <= 1) {
		LaunchScope scope(KC, 2.0 * nn * (double)nn * nn / 3.0);
		dchol_leaf_kernel<<<1, 256, 0, stream()>>>(r.W, n, r0, nn, r.X, r.dInfo);
		return check_launch("dchol_leaf_kernel");
	}
	FITRE_REQUIRE(depth < kDMaxDepth, "float64 inverse: recursion deeper than %d", kDMaxDepth);
	const int b1 = blocks / 2, n1 = b1 * kDLeaf, m = nn - n1, r1 = r0 + n1;
	int rc = dchol_and_inverse(r, r0, b1, n1, depth + 1);
	if (rc) return rc;
	const double *A21 = r.W + (size_t)r0 * n + r1;
	double *A22 = r.W + (size_t)r1 * n + r1;
	const double *X11 = r.X + (size_t)r0 * n + r0;
	double *L21 = r.L21[depth], *T2 = r.T2[depth];
	// L21(m x n1) = A21 * X11^T: B(k, j) = X11(j, k), zero for k > j
	rc = dgemm(m, n1, n1, 1.0, dmat64(A21, 1, n), dmat64(X11, n, 1), 0.0, DOut{ L21, 1, m, FITRE_MAT_F64 }, 0.0, kDgBUpper, KC, r.gws, r.gBytes);
	if (rc) return rc;
	// A22 -= L21 L21^T
	rc = dgemm(m, m, n1, -1.0, dmat64(L21, 1, m), dmat64(L21, m, 1), 1.0, DOut{ A22, 1, n, FITRE_MAT_F64 }, 0.0, kDgMirror, KC, r.gws, r.gBytes);
	if (rc) return rc;
	// T2(m x n1) = L21 * X11: B(k, j) = X11(k, j), zero for k < j
	rc = dgemm(m, n1, n1, 1.0, dmat64(L21, 1, m), dmat64(X11, 1, n), 0.0, DOut{ T2, 1, m, FITRE_MAT_F64 }, 0.0, kDgBLower, KC, r.gws, r.gBytes);
	if (rc) return rc;
	rc = dchol_and_inverse(r, r1, blocks - b1, m, depth + 1);
	if (rc) return rc;
	// X21 = -X22 * T2: A(i, k) = X22(i, k), zero for k > i
	const double *X22 = r.X + (size_t)r1 * n + r1;
	double *X21 = r.X + (size_t)r0 * n + r1;
	return dgemm(m, n1, m, -1.0, dmat64(X22, 1, n), dmat64(T2, 1, m), 0.0, DOut{ X21, 1, n, FITRE_MAT_F64 }, 0.0, kDgALower, KC, r.gws, r.gBytes);
}

size_t dspd_inverse_workspace(int n) { return n > 0 ? dinverse_layout(n).total : 0; }

// W: n x n doubles, symmetric positive definite (destroyed).  result = W^-1 as `kind` (double, float, or float pair),
// dense with leading dimension n.  Queued on the selected lane.
int dspd_inverse_run(double *W, int n, void *result, int kind, void *ws, size_t wsBytes, int *pivotInfo)
{
	FITRE_REQUIRE(W && result && ws && pivotInfo, "float64 inverse: null pointer");
	FITRE_REQUIRE(n > 0 && n <= 23000, "float64 inverse: order %d out of range", n);
	FITRE_REQUIRE((((uintptr_t)ws) & 255) == 0, "float64 inverse: workspace must be 256-byte aligned");
	const DInverseLayout lay = dinverse_layout(n);
	if (wsBytes < lay.total) return fail(FITRE_E_WORKSPACE, "float64 inverse: workspace of %zu bytes is smaller than the %zu required", wsBytes, lay.total);
	char *base = (char *)ws;
	DInverseRun run;
	run.W = W, run.X = (double *)(base + lay.x), run.n = n, run.dInfo = pivotInfo;
	for (int d = 0; d < kDMaxDepth; d++) run.L21[d] = (double *)(base + lay.l21[d]), run.T2[d] = (double *)(base + lay.t2[d]);
	run.gws = base + lay.gemm, run.gBytes = lay.gemmBytes;
	{
		LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)n * n);
		dfill_zero_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(run.X, (long)n * n);
		fill_int_kernel<<<1, 64, 0, stream()>>>(pivotInfo, 1, 0);
	}
	const int blocks = (n + kDLeaf - 1) / kDLeaf;
	int rc = dchol_and_inverse(run, 0, blocks, n, 0);
	if (rc) return rc;
	// W^-1 = X^T X: A(i, k) = X(k, i), zero for k < i; B(k, j) = X(k, j), zero for k < j
	return dgemm(n, n, n, 1.0, dmat64(run.X, n, 1), dmat64(run.X, 1, n), 0.0, DOut{ result, 1, n, kind }, 0.0, kDgMirror | kDgAUpper | kDgBLower,
	             FITRE_KC_SPD_INVERSE, run.gws, run.gBytes);
}

} // namespace fitre

using namespace fitre;

extern "C" {

static int to_dmat(const fitre_matrix *m, DMat *out, const char *what)
{
	FITRE_REQUIRE(m && m->data, "%s: null operand", what);
	FITRE_REQUIRE(m->kind == FITRE_MAT_F32 || m->kind == FITRE_MAT_F64 || m->kind == FITRE_MAT_SYM_PAIR, "%s: unknown operand kind %d", what, m->kind);
	out->p = m->data, out->rs = m->rowStride, out->cs = m->colStride, out->kind = m->kind;
	out->onesRow = m->kind == FITRE_MAT_F32 ? m->onesRow : -1;
	out->onesCol = m->kind == FITRE_MAT_F32 ? m->onesCol : -1;
	out->onesValue = m->onesValue;
	return FITRE_OK;
}

size_t fitre_hip_gemm_f64_workspace(long M, long N, long K, int flags) { return dgemm_workspace(M, N, K, flags); }

int fitre_hip_gemm_f64(long M, long N, long K, double alpha, const fitre_matrix *A, const fitre_matrix *B, double beta,
                       const fitre_matrix *C, double diagAdd, int flags, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	DMat a, b;
	int rc = to_dmat(A, &a, "fitre_hip_gemm_f64");
	if (rc) return rc;
	rc = to_dmat(B, &b, "fitre_hip_gemm_f64");
	if (rc) return rc;
	FITRE_REQUIRE(C && C->data, "fitre_hip_gemm_f64: null result");
	FITRE_REQUIRE((flags & ~(FITRE_GEMM_SYMMETRIC | FITRE_GEMM_A_LOWER | FITRE_GEMM_A_UPPER | FITRE_GEMM_B_LOWER | FITRE_GEMM_B_UPPER)) == 0,
	              "fitre_hip_gemm_f64: unknown flags %d", flags);
	DOut c{ (void *)C->data, C->rowStride, C->colStride, C->kind };
	return dgemm(M, N, K, alpha, a, b, beta, c, diagAdd, flags, FITRE_KC_FC_GEMM, ws, wsBytes);
}

size_t fitre_hip_spd_inverse_f64_workspace(int n) { return dspd_inverse_workspace(n); }

int fitre_hip_spd_inverse_f64_queued(double *matrix, int n, void *inverse, int inverseKind, void *ws, size_t wsBytes, int *pivotInfo)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(inverseKind == FITRE_MAT_F32 || inverseKind == FITRE_MAT_F64 || inverseKind == FITRE_MAT_SYM_PAIR,
	              "fitre_hip_spd_inverse_f64_queued: unknown result kind %d", inverseKind);
	FITRE_REQUIRE(pivotInfo != nullptr, "fitre_hip_spd_inverse_f64_queued: null pivot slot");
	return dspd_inverse_run(matrix, n, inverse, inverseKind, ws, wsBytes, pivotInfo);
}

int fitre_hip_widen_shift(const float *matrix, int n, double shift, double *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(matrix && out && n > 0, "fitre_hip_widen_shift: bad argument");
	widen_shift_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(matrix, out, n, shift);
	return check_launch("widen_shift_kernel");
}

} // extern "C"
