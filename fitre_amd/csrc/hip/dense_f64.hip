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
	uint32_t bytesA, bytesB; // extent of the operands in memory
	float *diagRemainder; // float-pair results: the remainders of the diagonal, folded into the matrix by a pass of its own
	int aKContig, bKContig;
};

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
	if (g.C.add) r += g.C.addScale * g.C.add[i * g.C.addRs + j * g.C.addCs];
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

// Global reads go through raw buffer resources: 32-bit byte offsets, no address arithmetic per slice (the slice moves the
// resource's base, scalar work), and an element outside the matrix gets the offset 0xFFFFFFFF, which the hardware's range
// check answers with zero.  Every operand must therefore be smaller than 4 GiB.
constexpr uint32_t kDgOutOfRange = 0xFFFFFFFFu;
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dg_rsrc(const void *p, uint32_t bytes)
{
	return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, bytes, 0x00020000);
}

// What a load leaves in registers until its slice goes to LDS: the bits as they came (a float, a double, or the two
// words of a float pair).  Converting at once would be a use of the value, and the wave would wait for every load
// right behind it instead of a slice later.
template <int KIND>
struct DgRaw {
	uint32_t w[KIND == FITRE_MAT_F32 ? 1 : 2];
};

template <int KIND>
__device__ __forceinline__ DgRaw<KIND> dg_load(__amdgpu_buffer_rsrc_t r, uint32_t byteOffset)
{
	DgRaw<KIND> v;
	if constexpr (KIND == FITRE_MAT_F64) {
		const v2u t = __builtin_amdgcn_raw_buffer_load_b64(r, (int)byteOffset, 0, 0);
		v.w[0] = t.x, v.w[1] = t.y;
	} else {
		v.w[0] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)byteOffset, 0, 0);
	}
	return v;
}

// the two words of element (r, c) of a symmetric float pair of order n (see dmat_load); rs covers the whole array
__device__ __forceinline__ DgRaw<FITRE_MAT_SYM_PAIR> dg_load_pair(__amdgpu_buffer_rsrc_t rs, int n, int ld, int r, int c, bool ok)
{
	const int a = r < c ? r : c, b = r < c ? c : r;
	const int below = (a == b) ? ((a + 1 < n) ? a * ld + a + 1 : n - 1) : a * ld + b;
	DgRaw<FITRE_MAT_SYM_PAIR> v;
	v.w[0] = __builtin_amdgcn_raw_buffer_load_b32(rs, ok ? 4 * (b * ld + a) : (int)kDgOutOfRange, 0, 0);
	v.w[1] = __builtin_amdgcn_raw_buffer_load_b32(rs, ok ? 4 * below : (int)kDgOutOfRange, 0, 0);
	return v;
}

template <int KIND>
__device__ __forceinline__ double dg_value(const DgRaw<KIND> &v, int n, int r, int c)
{
	if constexpr (KIND == FITRE_MAT_F64) {
		return __hiloint2double((int)v.w[1], (int)v.w[0]);
	} else if constexpr (KIND == FITRE_MAT_F32) {
		return (double)__uint_as_float(v.w[0]);
	} else {
		const int a = r < c ? r : c, b = r < c ? c : r;
		uint32_t w = v.w[1];
		if (a == b) w = (n < 3) ? 0u : w << 16;
		else if (n >= 3 && (b == a + 1 || (a == 0 && b == n - 1))) w &= 0xFFFF0000u;
		return (double)__uint_as_float(v.w[0]) + (double)__uint_as_float(w);
	}
}

// Tile TM x TN, 256 threads = 2 x 2 waves, a wave (TM/2) x (TN/2) = MI x NI blocks of 16 x 16; slices of BK reduction
// indices, double-buffered in LDS (one barrier per slice; the next slice's global loads are in flight while this one is
// multiplied).  Lane l of a block holds A(i = l % 16, k = l / 16), B(k = l / 16, j = l % 16) and, in register r of the
// accumulator, C(i = 4 r + l / 16, j = l % 16).
// KA / KB: operand kinds (compile-time: the loads of the float and double kinds are one add and one load per element,
// their offsets computed once per thread).  blockIdx.x: tile (row-major over tilesM x tilesN), blockIdx.y: split.
// AKC / BKC: whether the operand is contiguous along the reduction (1), along its rows (0), or decided at run time (-1):
// with the layout known at compile time every LDS offset of the loop is an immediate.
template <int TM, int TN, int BK, int KA, int KB, int AKC, int BKC>
__device__ __forceinline__ void dgemm_tile(const DgemmArgs &g, const int tile, const int split, const int tiles)
{
	const bool aKC = AKC < 0 ? (g.aKContig != 0) : (AKC != 0), bKC = BKC < 0 ? (g.bKContig != 0) : (BKC != 0);
	// An operand's slice sits in LDS as [k][row], rows TM + 16 doubles apart (a row offset of 16 mod 32: the four k rows of a
	// fragment read hit different banks), when its lanes run along the rows; as [row][k], rows BK + 1 doubles apart, when
	// they run along k (a k-contiguous operand): the stores of a wave are then contiguous runs of BK doubles, and the
	// sixteen rows of a fragment read, 2 (BK + 1) words apart, spread over the banks.
	constexpr int LDA = TM + 16, LDB = TN + 16, LDK = BK + 1;
	constexpr int BUFA = (BK * LDA > TM * LDK) ? BK * LDA : TM * LDK, BUFB = (BK * LDB > TN * LDK) ? BK * LDB : TN * LDK;
	constexpr int WTM = TM / 2, WTN = TN / 2, MI = WTM / 16, NI = WTN / 16;
	constexpr int EA = TM * BK / 256, EB = TN * BK / 256;
	extern __shared__ double lds[];
	double *As = lds, *Bs = lds + 2 * BUFA; // two buffers each
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int ti = tile / g.tilesN, tj = tile - ti * g.tilesN;
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
		k0 = kb + split * chunk;
		k1 = min(ke, k0 + chunk);
	}

	v4d acc[MI][NI];
#pragma unroll
	for (int mi = 0; mi < MI; mi++)
#pragma unroll
		for (int ni = 0; ni < NI; ni++) acc[mi][ni] = v4d{ 0.0, 0.0, 0.0, 0.0 };

	// Which elements of a slice a thread moves: element q is (row0 + q * rowStep, kq0 + q * kStep) of the tile's slice,
	// with the lanes along the direction in which the operand is contiguous; its place in LDS and (float / double
	// operands) its byte offset in memory at reduction index 0 are affine in q as well.
	constexpr int SA = KA == FITRE_MAT_F64 ? 8 : 4, SB = KB == FITRE_MAT_F64 ? 8 : 4;
	const int kq0A = aKC ? tid % BK : tid / TM, kStepA = aKC ? 0 : 256 / TM;
	const int row0A = aKC ? tid / BK : tid % TM, rowStepA = aKC ? 256 / BK : 0;
	const int kq0B = bKC ? tid % BK : tid / TN, kStepB = bKC ? 0 : 256 / TN;
	const int row0B = bKC ? tid / BK : tid % TN, rowStepB = bKC ? 256 / BK : 0;
	const int ldsRowA = aKC ? LDK : 1, ldsKA = aKC ? 1 : LDA; // LDS strides along the rows / along k
	const int ldsRowB = bKC ? LDK : 1, ldsKB = bKC ? 1 : LDB;
	const int lds0A = kq0A * ldsKA + row0A * ldsRowA, ldsStepA = kStepA * ldsKA + rowStepA * ldsRowA;
	const int lds0B = kq0B * ldsKB + row0B * ldsRowB, ldsStepB = kStepB * ldsKB + rowStepB * ldsRowB;
	const int stepA = (int)g.A.cs, stepB = (int)g.B.rs; // elements per reduction index
	uint32_t voffA[EA], voffB[EB];
	uint32_t onesA = 0, onesB = 0; // elements of the constant row / column
#pragma unroll
	for (int q = 0; q < EA; q++) {
		const int gi = i0 + row0A + q * rowStepA;
		const bool ones = gi == g.A.onesRow;
		if (ones) onesA |= 1u << q;
		voffA[q] = (gi < g.M && !ones) ? (uint32_t)SA * (uint32_t)(gi * (int)g.A.rs + (kq0A + q * kStepA) * stepA) : kDgOutOfRange;
	}
#pragma unroll
	for (int q = 0; q < EB; q++) {
		const int gj = j0 + row0B + q * rowStepB;
		const bool ones = gj == g.B.onesCol;
		if (ones) onesB |= 1u << q;
		voffB[q] = (gj < g.N && !ones) ? (uint32_t)SB * (uint32_t)(gj * (int)g.B.cs + (kq0B + q * kStepB) * stepB) : kDgOutOfRange;
	}

	// two slices of loads in flight: slice s + 2 is requested while slice s is multiplied and reaches LDS a slice later
	DgRaw<KA> ra[2][EA];
	DgRaw<KB> rb[2][EB];
	auto fetch = [&](int kk, DgRaw<KA> (&va)[EA], DgRaw<KB> (&vb)[EB]) {
		const bool whole = kk + BK <= k1;
		if constexpr (KA == FITRE_MAT_SYM_PAIR) {
			const __amdgpu_buffer_rsrc_t rs = dg_rsrc(g.A.p, g.bytesA);
#pragma unroll
			for (int q = 0; q < EA; q++) {
				const int gi = i0 + row0A + q * rowStepA, gk = kk + kq0A + q * kStepA;
				va[q] = dg_load_pair(rs, (int)g.A.rs, (int)g.A.cs, gi, gk, gi < g.M && gk < k1);
			}
		} else {
			const uint32_t adv = (uint32_t)__builtin_amdgcn_readfirstlane(SA * kk * stepA); // wave-uniform: the resource stays in scalar registers
			const __amdgpu_buffer_rsrc_t rs = dg_rsrc((const char *)g.A.p + adv, g.bytesA - adv);
#pragma unroll
			for (int q = 0; q < EA; q++) va[q] = dg_load<KA>(rs, voffA[q] | ((whole | (kk + kq0A + q * kStepA < k1)) ? 0u : kDgOutOfRange));
		}
		if constexpr (KB == FITRE_MAT_SYM_PAIR) {
			const __amdgpu_buffer_rsrc_t rs = dg_rsrc(g.B.p, g.bytesB);
#pragma unroll
			for (int q = 0; q < EB; q++) {
				const int gj = j0 + row0B + q * rowStepB, gk = kk + kq0B + q * kStepB;
				vb[q] = dg_load_pair(rs, (int)g.B.rs, (int)g.B.cs, gk, gj, gj < g.N && gk < k1);
			}
		} else {
			const uint32_t adv = (uint32_t)__builtin_amdgcn_readfirstlane(SB * kk * stepB);
			const __amdgpu_buffer_rsrc_t rs = dg_rsrc((const char *)g.B.p + adv, g.bytesB - adv);
#pragma unroll
			for (int q = 0; q < EB; q++) vb[q] = dg_load<KB>(rs, voffB[q] | ((whole | (kk + kq0B + q * kStepB < k1)) ? 0u : kDgOutOfRange));
		}
	};
	// slice kk from registers to LDS buffer buf, as doubles, the constant row / column put in
	auto stage = [&](int buf, int kk, const DgRaw<KA> (&va)[EA], const DgRaw<KB> (&vb)[EB]) {
#pragma unroll
		for (int q = 0; q < EA; q++) {
			const int gk = kk + kq0A + q * kStepA;
			const double v = dg_value<KA>(va[q], (int)g.A.rs, i0 + row0A + q * rowStepA, gk);
			As[buf * BUFA + lds0A + q * ldsStepA] = (((onesA >> q) & 1) && gk < k1) ? g.A.onesValue : v;
		}
#pragma unroll
		for (int q = 0; q < EB; q++) {
			const int gk = kk + kq0B + q * kStepB;
			const double v = dg_value<KB>(vb[q], (int)g.B.rs, gk, j0 + row0B + q * rowStepB);
			Bs[buf * BUFB + lds0B + q * ldsStepB] = (((onesB >> q) & 1) && gk < k1) ? g.B.onesValue : v;
		}
	};
	auto multiply = [&](int buf) {
		const double *ap = As + buf * BUFA + (lane >> 4) * ldsKA + (wm * WTM + (lane & 15)) * ldsRowA;
		const double *bp = Bs + buf * BUFB + (lane >> 4) * ldsKB + (wn * WTN + (lane & 15)) * ldsRowB;
#pragma unroll
		for (int k4 = 0; k4 < BK / 4; k4++) {
			double a[MI], b[NI];
#pragma unroll
			for (int mi = 0; mi < MI; mi++) a[mi] = ap[k4 * 4 * ldsKA + mi * 16 * ldsRowA];
#pragma unroll
			for (int ni = 0; ni < NI; ni++) b[ni] = bp[k4 * 4 * ldsKB + ni * 16 * ldsRowB];
#pragma unroll
			for (int mi = 0; mi < MI; mi++)
#pragma unroll
				for (int ni = 0; ni < NI; ni++) acc[mi][ni] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
		}
		// the accumulators stay in the accumulation registers from slice to slice (left alone, the compiler carries them
		// through the loop in vector registers and copies all of them in and out around every slice)
		if constexpr (TM == 128) {
#pragma unroll
			for (int mi = 0; mi < MI; mi++)
#pragma unroll
				for (int ni = 0; ni < NI; ni++) asm volatile("" : "+a"(acc[mi][ni]));
		}
	};

	if (k0 < k1) {
		fetch(k0, ra[0], rb[0]);
		stage(0, k0, ra[0], rb[0]);
		if (k0 + BK < k1) fetch(k0 + BK, ra[1], rb[1]);
	}
	__syncthreads();
	// two slices per round, so that the register sets and LDS buffers have constant indices
	for (int kk = k0; kk < k1; kk += 2 * BK) {
		if (kk + 2 * BK < k1) fetch(kk + 2 * BK, ra[0], rb[0]);
		multiply(0);
		if (kk + BK < k1) stage(1, kk + BK, ra[1], rb[1]);
		__syncthreads();
		if (kk + BK >= k1) break;
		if (kk + 3 * BK < k1) fetch(kk + 3 * BK, ra[1], rb[1]);
		multiply(1);
		if (kk + 2 * BK < k1) stage(0, kk + 2 * BK, ra[0], rb[0]);
		__syncthreads();
	}

	if (g.splits > 1) {
		// partial tile, element e of thread tid at [e][tid]: coalesced for the reduction kernel, which has the same mapping
		constexpr int ACC = MI * NI * 4;
		double *dst = g.partials + ((size_t)split * tiles + tile) * (size_t)(ACC * 256) + tid;
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

template <int TM, int TN, int BK, int KA, int KB, int AKC, int BKC>
__global__ void __launch_bounds__(256, (TM == 64 ? 2 : 1)) dgemm_kernel(const DgemmArgs g)
{
	dgemm_tile<TM, TN, BK, KA, KB, AKC, BKC>(g, (int)blockIdx.x, (int)blockIdx.y, (int)gridDim.x);
}

// two unsplit products that do not depend on each other as one launch: the first `tiles1` workgroups take the first
template <int TM, int TN, int BK, int KA, int KB>
__global__ void __launch_bounds__(256, 2) dgemm_pair_kernel(const DgemmArgs g1, const DgemmArgs g2, int tiles1)
{
	if ((int)blockIdx.x < tiles1) dgemm_tile<TM, TN, BK, KA, KB, -1, -1>(g1, (int)blockIdx.x, 0, tiles1);
	else dgemm_tile<TM, TN, BK, KA, KB, -1, -1>(g2, (int)blockIdx.x - tiles1, 0, (int)gridDim.x - tiles1);
}

// adds the partial tiles of the splits in split order and stores the result: blockIdx.x = tile, blockIdx.y = which
// kDgReduceElements of a thread's elements (a tile with hundreds of splits behind it is shared by several workgroups)
constexpr int kDgReduceElements = 4;
template <int TM, int TN>
__global__ void __launch_bounds__(256) dgemm_reduce_kernel(const DgemmArgs g)
{
	constexpr int WTM = TM / 2, WTN = TN / 2, MI = WTM / 16, NI = WTN / 16, ACC = MI * NI * 4;
	static_assert(ACC % kDgReduceElements == 0, "elements per thread");
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int tile = blockIdx.x, ti = tile / g.tilesN, tj = tile - ti * g.tilesN;
	if ((g.flags & kDgMirror) && tj < ti) return;
	const int i0 = ti * TM, j0 = tj * TN;
	const bool mirrorToo = (g.flags & kDgMirror) && tj > ti && g.C.kind != FITRE_MAT_SYM_PAIR;
	const size_t tiles = gridDim.x, perSplit = tiles * (size_t)(ACC * 256);
	const int e0 = (int)blockIdx.y * kDgReduceElements;
	const double *base = g.partials + (size_t)tile * (size_t)(ACC * 256) + (size_t)e0 * 256 + tid;
	double sum[kDgReduceElements];
#pragma unroll
	for (int e = 0; e < kDgReduceElements; e++) sum[e] = 0.0;
	int s = 0;
	for (; s + 4 <= g.splits; s += 4) { // sixteen loads in flight; every sum in split order
		double v[4][kDgReduceElements];
#pragma unroll
		for (int u = 0; u < 4; u++)
#pragma unroll
			for (int e = 0; e < kDgReduceElements; e++) v[u][e] = base[(size_t)(s + u) * perSplit + (size_t)e * 256];
#pragma unroll
		for (int u = 0; u < 4; u++)
#pragma unroll
			for (int e = 0; e < kDgReduceElements; e++) sum[e] += v[u][e];
	}
	for (; s < g.splits; s++)
#pragma unroll
		for (int e = 0; e < kDgReduceElements; e++) sum[e] += base[(size_t)s * perSplit + (size_t)e * 256];
#pragma unroll
	for (int k = 0; k < kDgReduceElements; k++) {
		const int e = e0 + k;
		const int mi = e / (NI * 4), ni = (e / 4) % NI, r = e & 3;
		dgemm_store(g, i0 + wm * WTM + mi * 16 + 4 * r + (lane >> 4), j0 + wn * WTN + ni * 16 + (lane & 15), sum[k], mirrorToo, ti == tj);
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
	int tile;   // 64
	int splits;
	int tilesM, tilesN;
};

// Tiles and reduction splits of a product.  One tile size: 64 x 64 with slices of 32 -- two of its workgroups share a
// compute unit (two waves per SIMD), which a 128 x 128 tile's 512 registers per lane do not allow, and that beats the large
// tile's better ratio of arithmetic to LDS traffic everywhere (4096^3: 49-52 against 46-48 TFLOP/s; a symmetric order-4609
// factor over 4096 positions: 1.9 against 2.75 ms).  Splits, each rule from a sweep on the box: a grid far below the chip
// splits down to 256 reduction steps per split; a deep reduction on a grid of less than two rounds of workgroups splits in
// two to four (order-2305 factors: 2.46 -> 2.0 ms and 0.64 -> 0.53 ms; order 1153: 1.32 -> 0.67 ms; 4609 x 512 x 4609:
// 0.67 -> 0.51 ms).
static DgemmPlan plan_dgemm(long M, long N, long K, int flags, bool pairOperand = false)
{
	(void)pairOperand;
	DgemmPlan p;
	const int cus = device_compute_units() > 0 ? device_compute_units() : 256;
	p.tile = 64;
	p.tilesM = (int)((M + p.tile - 1) / p.tile);
	p.tilesN = (int)((N + p.tile - 1) / p.tile);
	const long live = (flags & kDgMirror) ? (long)p.tilesM * (p.tilesM + 1) / 2 : (long)p.tilesM * p.tilesN;
	long splits = 1;
	if (2 * live < cus) {
		splits = (2 * cus + live - 1) / live;
		const long deepest = K / 256 > 0 ? K / 256 : 1;
		if (splits > deepest) splits = deepest;
		if (splits > 512) splits = 512;
	} else if (K >= 2048 && live < 4 * cus) {
		splits = (6 * cus + live / 2) / live;
		if (splits > 4) splits = 4;
		while (splits > 1 && K / splits < 1024) splits--;
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

template <int T, int BK, int KA, int KB, int AKC, int BKC>
static int launch_dgemm_layout(const DgemmArgs &g, const DgemmPlan &p, dim3 grid)
{
	constexpr size_t perOperand = (BK * (T + 16) > T * (BK + 1)) ? BK * (T + 16) : T * (BK + 1);
	constexpr size_t ldsBytes = (size_t)4 * perOperand * sizeof(double);
	static bool attributeSet = false; // dynamic LDS above 64 KB has to be allowed once per kernel
	if (!attributeSet) {
		FITRE_HIP_TRY(hipFuncSetAttribute((const void *)dgemm_kernel<T, T, BK, KA, KB, AKC, BKC>, hipFuncAttributeMaxDynamicSharedMemorySize,
		                                  (int)ldsBytes));
		attributeSet = true;
	}
	dgemm_kernel<T, T, BK, KA, KB, AKC, BKC><<<grid, 256, ldsBytes, stream()>>>(g);
	if (p.splits > 1) dgemm_reduce_kernel<T, T><<<dim3(grid.x, (T / 32) * (T / 32) * 4 / kDgReduceElements), 256, 0, stream()>>>(g);
	return FITRE_OK;
}

// Operands of one kind on both sides (the products of the inverse, the factor products) get a kernel per layout pair;
// the mixed products keep the layout as a run-time value.
template <int T, int BK, int KA, int KB>
static int launch_dgemm_kinds(const DgemmArgs &g, const DgemmPlan &p, dim3 grid)
{
	if constexpr (KA == KB && KA != FITRE_MAT_SYM_PAIR) {
		if (g.aKContig && g.bKContig) return launch_dgemm_layout<T, BK, KA, KB, 1, 1>(g, p, grid);
		if (g.aKContig) return launch_dgemm_layout<T, BK, KA, KB, 1, 0>(g, p, grid);
		if (g.bKContig) return launch_dgemm_layout<T, BK, KA, KB, 0, 1>(g, p, grid);
		return launch_dgemm_layout<T, BK, KA, KB, 0, 0>(g, p, grid);
	} else {
		return launch_dgemm_layout<T, BK, KA, KB, -1, -1>(g, p, grid);
	}
}

template <int KA, int KB>
static int launch_dgemm_tiles(const DgemmArgs &g, const DgemmPlan &p, dim3 grid)
{
	// slices of 32: the products at the bottom of the inverse's recursion (reduction 64) then have all their loads in flight at once
	return launch_dgemm_kinds<64, 32, KA, KB>(g, p, grid);
}

// the operand pairs the library's products have (either order: the kernel may work on the transposed problem)
static int launch_dgemm(const DgemmArgs &g, const DgemmPlan &p, dim3 grid)
{
	constexpr int F32 = FITRE_MAT_F32, F64 = FITRE_MAT_F64, PAIR = FITRE_MAT_SYM_PAIR;
	const int ka = g.A.kind, kb = g.B.kind;
	if (ka == F32 && kb == F32) return launch_dgemm_tiles<F32, F32>(g, p, grid);
	if (ka == F64 && kb == F64) return launch_dgemm_tiles<F64, F64>(g, p, grid);
	if (ka == F32 && kb == F64) return launch_dgemm_tiles<F32, F64>(g, p, grid);
	if (ka == F64 && kb == F32) return launch_dgemm_tiles<F64, F32>(g, p, grid);
	if (ka == F32 && kb == PAIR) return launch_dgemm_tiles<F32, PAIR>(g, p, grid);
	if (ka == PAIR && kb == F32) return launch_dgemm_tiles<PAIR, F32>(g, p, grid);
	if (ka == F64 && kb == PAIR) return launch_dgemm_tiles<F64, PAIR>(g, p, grid);
	if (ka == PAIR && kb == F64) return launch_dgemm_tiles<PAIR, F64>(g, p, grid);
	return fail(FITRE_E_UNSUPPORTED, "float64 product: no kernel for two float-pair operands");
}

size_t dgemm_workspace(long M, long N, long K, int flags)
{
	// the kernel may work on the transposed problem; the plan is symmetric in M and N
	const size_t a = dgemm_partial_bytes(plan_dgemm(M, N, K, flags, false)), b = dgemm_partial_bytes(plan_dgemm(M, N, K, flags, true));
	return dalign(a > b ? a : b) + dalign((size_t)(M > N ? M : N) * sizeof(float)) + 256;
}

// C(M x N) = alpha * A(M x K) * B(K x N) + beta * C (+ diagAdd on the diagonal), on the selected lane
struct DgemmLaunch {
	DgemmArgs g;
	DgemmPlan p;
	double flops;
	float *diagRemainder;
	int kernelClass;
};

static int dgemm_setup(long M, long N, long K, double alpha, DMat A, DMat B, double beta, DOut C, double diagAdd, int flags, int kernelClass,
                       void *ws, size_t wsBytes, DgemmLaunch *out)
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
		const long sa = C.addRs;
		C.addRs = C.addCs, C.addCs = sa;
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
	DgemmPlan p = plan_dgemm(M, N, K, flags, A.kind == FITRE_MAT_SYM_PAIR || B.kind == FITRE_MAT_SYM_PAIR);
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
	// byte offsets inside an operand are 32-bit
	auto extent_bytes = [](const DMat &m, long rows, long cols, long ones0, long ones1) {
		if (m.kind == FITRE_MAT_SYM_PAIR) return ((m.rs - 1) * m.cs + m.rs) * 4;
		const long r = rows - (ones0 >= 0 ? 1 : 0), c = cols - (ones1 >= 0 ? 1 : 0);
		return ((r - 1) * m.rs + (c - 1) * m.cs + 1) * (m.kind == FITRE_MAT_F64 ? 8 : 4);
	};
	const long bytesA = extent_bytes(A, M, K, A.onesRow, -1), bytesB = extent_bytes(B, K, N, -1, B.onesCol);
	FITRE_REQUIRE(bytesA > 0 && bytesB > 0 && bytesA < 4294967295l && bytesB < 4294967295l, "float64 product: an operand of 4 GiB or more");
	FITRE_REQUIRE(A.onesRow < 0 || A.onesRow == M - 1, "float64 product: the constant row must be the last one");
	FITRE_REQUIRE(B.onesCol < 0 || B.onesCol == N - 1, "float64 product: the constant column must be the last one");
	g.bytesA = (uint32_t)bytesA, g.bytesB = (uint32_t)bytesB;
	FITRE_REQUIRE(A.rs >= 0 && A.cs >= 0 && B.rs >= 0 && B.cs >= 0, "float64 product: negative stride");
	FITRE_REQUIRE(A.onesCol < 0 && B.onesRow < 0, "float64 product: a constant row / column along the reduction is not supported");
	out->g = g, out->p = p, out->diagRemainder = diagRemainder, out->kernelClass = kernelClass;
	out->flops = ((flags & kDgMirror) ? 1.0 : 2.0) * (double)M * (double)N * (double)K;
	return FITRE_OK;
}

static int dgemm_issue(const DgemmLaunch &l)
{
	const dim3 grid((unsigned)(l.p.tilesM * l.p.tilesN), (unsigned)l.p.splits);
	LaunchScope scope(l.kernelClass, l.flops);
	int rc = launch_dgemm(l.g, l.p, grid);
	if (rc) return rc;
	if (l.diagRemainder)
		pair_fold_diagonal_kernel<<<blocks_for(l.g.M, 256), 256, 0, stream()>>>((float *)l.g.C.p, l.g.C.cs, l.g.M, l.diagRemainder);
	return check_launch("float64 product");
}

// Two products that do not depend on each other: one launch when both are unsplit products of doubles on the small tile
// (the nodes at the lower levels of the inverse's recursion, which last about as long as a launch costs), else one
// after the other.
static int dgemm_issue_pair(const DgemmLaunch &a, const DgemmLaunch &b)
{
	const bool together = a.p.splits == 1 && b.p.splits == 1 && a.p.tile == 64 && b.p.tile == 64 && a.g.A.kind == FITRE_MAT_F64 &&
	                      a.g.B.kind == FITRE_MAT_F64 && b.g.A.kind == FITRE_MAT_F64 && b.g.B.kind == FITRE_MAT_F64 && !a.diagRemainder &&
	                      !b.diagRemainder;
	if (!together) {
		int rc = dgemm_issue(a);
		return rc ? rc : dgemm_issue(b);
	}
	constexpr int T = 64, BK = 32;
	constexpr size_t perOperand = (BK * (T + 16) > T * (BK + 1)) ? BK * (T + 16) : T * (BK + 1);
	constexpr size_t ldsBytes = (size_t)4 * perOperand * sizeof(double);
	static bool attributeSet = false;
	if (!attributeSet) {
		FITRE_HIP_TRY(hipFuncSetAttribute((const void *)dgemm_pair_kernel<T, T, BK, FITRE_MAT_F64, FITRE_MAT_F64>,
		                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
		attributeSet = true;
	}
	const int tiles1 = a.p.tilesM * a.p.tilesN, tiles2 = b.p.tilesM * b.p.tilesN;
	LaunchScope scope(a.kernelClass, a.flops + b.flops);
	dgemm_pair_kernel<T, T, BK, FITRE_MAT_F64, FITRE_MAT_F64><<<(unsigned)(tiles1 + tiles2), 256, ldsBytes, stream()>>>(a.g, b.g, tiles1);
	return check_launch("float64 product pair");
}

int dgemm(long M, long N, long K, double alpha, DMat A, DMat B, double beta, DOut C, double diagAdd, int flags, int kernelClass,
          void *ws, size_t wsBytes)
{
	DgemmLaunch l;
	int rc = dgemm_setup(M, N, K, alpha, A, B, beta, C, diagAdd, flags, kernelClass, ws, wsBytes, &l);
	return rc ? rc : dgemm_issue(l);
}

// ---- leaf of the inverse: a diagonal block of order <= 64, one workgroup, float64 in registers -----------------------
//
// One sweep of 64 steps, a barrier every four, does the Cholesky factorisation W = L L^T (right-looking) and the inverse of
// the factor together: the column operations that turn L^T into the identity (scale column j by 1 / l_jj, then column
// k -= column j * l_kj for k > j) turn the identity into Y = L^-T, and step j of them needs exactly column j of L, which
// step j of the factorisation has just produced.  Thread (i, q) = (lane, wave) keeps row i of the trailing matrix --
// W(i, k) for k = 4 t + q -- and column i of Y -- Y(r, i) for r = 4 t + q -- in registers, 16 doubles each; what a step
// needs from other threads: column j of W goes through LDS, four columns (a register of each wave) at a time, and is read
// back one row per lane, so that the entries a thread multiplies by are lanes of one register; column j of Y (rows r =
// 4 t + q) is lane j of the same wave's registers.  The steps are unrolled by template recursion, so that every
// register index, lane index and loop bound is a constant or wave-uniform.
constexpr int kDLeaf = 64;

__device__ __forceinline__ double rsqrt_f64(double a)
{
	double d = __builtin_amdgcn_rsq(a);
	d = d * (1.5 - 0.5 * a * d * d);
	return d * (1.5 - 0.5 * a * d * d);
}

// Step J.  Entries of a row right of the diagonal (k > i) are never read, so the trailing update runs over them
// unmasked; what has to be masked is folded into the multiplier (zero where a thread must not update), which keeps
// the step free of branches and of selects on loaded values.
// a double of another lane of the wave (the lane index is wave-uniform)
__device__ __forceinline__ double lane_value(double v, int lane)
{
	const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane), hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
	return __hiloint2double(hi, lo);
}

// Step S of panel JB (column J = 4 JB + S).  c[]: the panel's four columns, one row per lane, every thread updating
// them alike.  Entries of a row right of the diagonal (k > i) are never read, so the trailing update runs over them
// unmasked; what has to be masked is folded into the multiplier (zero where a thread must not update), which keeps
// the step free of branches and of selects on loaded values.
template <int JB, int S>
__device__ __forceinline__ void dleaf_step(double (&w)[16], double (&y)[16], double (&c)[4], double &dOwn, int &bad, int i, int q)
{
	constexpr int J = 4 * JB + S;
	const double li = c[S];
	const double ajj = lane_value(li, J);
	double lk[16 - JB], yr[JB + 1], lc[4];
#pragma unroll
	for (int t = JB + 1; t < 16; t++) lk[t - JB] = lane_value(li, 4 * t + q);
#pragma unroll
	for (int u = S + 1; u < 4; u++) lc[u] = lane_value(li, 4 * JB + u);
#pragma unroll
	for (int t = 0; t <= JB; t++) yr[t] = lane_value(y[t], J);
	if (!(ajj > 0.0) && bad == 0) bad = J + 1; // wave-uniform
	const double d = rsqrt_f64(ajj);
	const double m = li * (d * d);              // l_iJ / l_JJ
	const double mw = (i > J) ? m : 0.0;        // rows below the pivot row take the update
	if (i == J) dOwn = d;                       // column J of Y is final but for this factor (row J of X)
	// trailing matrix: W(i, k) -= l_iJ l_kJ for k > J: the rest of the panel first (the next pivot is in it)
#pragma unroll
	for (int u = S + 1; u < 4; u++) c[u] = __builtin_fma(-mw, lc[u], c[u]);
#pragma unroll
	for (int t = JB + 1; t < 16; t++) w[t] = __builtin_fma(-mw, lk[t - JB], w[t]);
	// Y: column i -= column J * l_iJ / l_JJ for i > J, rows r <= J
#pragma unroll
	for (int t = 0; t < JB; t++) y[t] = __builtin_fma(-mw, yr[t], y[t]);
	y[JB] = __builtin_fma((q <= S) ? -mw : 0.0, yr[JB], y[JB]);
	// the updates stay in this step: left to itself the compiler postpones them until a value is needed and keeps
	// the operands of every postponed step alive
#pragma unroll
	for (int t = JB + 1; t < 16; t++) asm volatile("" : "+v"(w[t]));
#pragma unroll
	for (int t = 0; t <= JB; t++) asm volatile("" : "+v"(y[t]));
}

// Panel JB: columns 4 JB .. 4 JB + 3 of the trailing matrix are register JB of the four waves; they go through LDS once
// (double-buffered by the parity of the panel) and every wave then runs the panel's four steps on its own.
template <int JB>
__device__ __forceinline__ void dleaf_panels(double (&w)[16], double (&y)[16], double &dOwn, int &bad, double *panel, int i, int q)
{
	double *pc = panel + (JB & 1) * 4 * kDLeaf;
	pc[q * kDLeaf + i] = w[JB];
	__syncthreads();
	double c[4];
#pragma unroll
	for (int u = 0; u < 4; u++) c[u] = pc[u * kDLeaf + i];
	dleaf_step<JB, 0>(w, y, c, dOwn, bad, i, q);
	dleaf_step<JB, 1>(w, y, c, dOwn, bad, i, q);
	dleaf_step<JB, 2>(w, y, c, dOwn, bad, i, q);
	dleaf_step<JB, 3>(w, y, c, dOwn, bad, i, q);
	if constexpr (JB + 1 < 16) dleaf_panels<JB + 1>(w, y, dOwn, bad, panel, i, q);
}

// the whole leaf: L is consumed column by column, Y = L^-T comes out; i = lane, q = wave (uniform); panel: 8 * kDLeaf doubles
__device__ __forceinline__ void dleaf_run(double (&w)[16], double (&y)[16], double *panel, int i, int q, int k0, int *info)
{
	double dOwn = 1.0;
	int bad = 0;
	dleaf_panels<0>(w, y, dOwn, bad, panel, i, q);
#pragma unroll
	for (int t = 0; t < 16; t++) y[t] *= dOwn;
	if (bad != 0 && i == 0 && q == 0) atomicCAS(info, 0, k0 + bad);
}

__global__ void __launch_bounds__(256) dchol_leaf_kernel(const double *W, long ld, int k0, int nn, double *X, int *info)
{
	__shared__ double Lcol[8 * kDLeaf];
	const int tid = threadIdx.x, i = tid & 63, q = __builtin_amdgcn_readfirstlane(tid >> 6);
	const double *blk = W + (size_t)k0 * ld + k0;
	double w[16], y[16];
#pragma unroll
	for (int t = 0; t < 16; t++) {
		const int c = 4 * t + q;
		double v = (i == c) ? 1.0 : 0.0; // beyond the block: identity, which factors to itself
		if (i < nn && c <= i) v = blk[(size_t)c * ld + i];
		w[t] = v;
		y[t] = (i == c) ? 1.0 : 0.0;
	}
	dleaf_run(w, y, Lcol, i, q, k0, info);
	// X(i, r) = Y(r, i) for r <= i
	double *xblk = X + (size_t)k0 * ld + k0;
	if (i < nn) {
#pragma unroll
		for (int t = 0; t < 16; t++) {
			const int r = 4 * t + q;
			if (r <= i) xblk[(size_t)r * ld + i] = y[t];
		}
	}
}

// ---- a node of two leaves as one launch -----------------------------------------------------------------------------
//
// The node of the recursion that joins two 64-order blocks (the second may be smaller) is two leaf factorisations and four
// 64 x 64 x 64 products, six dependent launches of 16 to 28 us each; here one workgroup does all of it without leaving
// the compute unit: leaf of A11 in registers, X11 to memory and to LDS; L21 = A21 X11^T, T2 = L21 X11 and L21 L21^T on the
// matrix pipes from LDS (a wave owns sixteen rows); leaf of A22 - L21 L21^T; X21 = -X22 T2.  Same arithmetic and the same
// order of every sum as the separate launches up to the blocking of the products.
constexpr int kNodeLd = kDLeaf + 1; // row stride of the 64 x 64 blocks in LDS (doubles)
constexpr int kNodeBlock = kDLeaf * kNodeLd;

// C = A * B (transposedB: C = A * B^T) for this wave's sixteen rows, all 64 columns; A, B, C are 64 x 64 blocks in LDS
template <bool TRANSPOSED_B>
__device__ __forceinline__ void node_product(const double *A, const double *B, v4d (&acc)[4], int wave, int lane)
{
	const int l16 = lane & 15, kq = lane >> 4;
#pragma unroll
	for (int nb = 0; nb < 4; nb++) acc[nb] = v4d{ 0.0, 0.0, 0.0, 0.0 };
#pragma unroll 4
	for (int kk = 0; kk < kDLeaf / 4; kk++) {
		const int k = 4 * kk + kq;
		const double a = A[(16 * wave + l16) * kNodeLd + k];
#pragma unroll
		for (int nb = 0; nb < 4; nb++) {
			const double b = TRANSPOSED_B ? B[(16 * nb + l16) * kNodeLd + k] : B[k * kNodeLd + 16 * nb + l16];
			acc[nb] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[nb], 0, 0, 0);
		}
	}
}

// register r of block nb holds C(16 wave + 4 r + lane / 16, 16 nb + lane % 16)
__device__ __forceinline__ void node_store_lds(double *C, const v4d (&acc)[4], int wave, int lane)
{
#pragma unroll
	for (int nb = 0; nb < 4; nb++)
#pragma unroll
		for (int r = 0; r < 4; r++) C[(16 * wave + 4 * r + (lane >> 4)) * kNodeLd + 16 * nb + (lane & 15)] = acc[nb][r];
}

__global__ void __launch_bounds__(256) dnode_pair_kernel(const double *W, long ld, int r0, int m, double *X, int *info)
{
	extern __shared__ double nodeLds[];
	double *Xs = nodeLds, *As = Xs + kNodeBlock, *Ls = As + kNodeBlock, *Ts = Ls + kNodeBlock; // X11 / X22, A21 / L21 L21^T, L21, T2
	__shared__ double Lcol[8 * kDLeaf];
	const int tid = threadIdx.x, i = tid & 63, q = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, wave = tid >> 6;
	const int r1 = r0 + kDLeaf;
	double w[16], y[16];
	// A21(i, k) = W(r1 + i, r0 + k): on its way while the first leaf runs
	double a21[16];
#pragma unroll
	for (int t = 0; t < 16; t++) a21[t] = i < m ? W[(size_t)(r0 + 4 * t + q) * ld + r1 + i] : 0.0;
	for (int pass = 0; pass < 2; pass++) {
		const int k0 = pass ? r1 : r0, nn = pass ? m : kDLeaf;
		const double *blk = W + (size_t)k0 * ld + k0;
#pragma unroll
		for (int t = 0; t < 16; t++) {
			const int c = 4 * t + q;
			double v = (i == c) ? 1.0 : 0.0; // beyond the block: identity, which factors to itself
			if (i < nn && c <= i) v = blk[(size_t)c * ld + i] - (pass ? As[i * kNodeLd + c] : 0.0);
			w[t] = v;
			y[t] = (i == c) ? 1.0 : 0.0;
		}
		dleaf_run(w, y, Lcol, i, q, k0, info);
		// X(i, r) = Y(r, i) for r <= i: to memory, and the whole block (zeros above the diagonal) to LDS
		double *xblk = X + (size_t)k0 * ld + k0;
#pragma unroll
		for (int t = 0; t < 16; t++) {
			const int r = 4 * t + q;
			if (i < nn && r <= i) xblk[(size_t)r * ld + i] = y[t];
			Xs[i * kNodeLd + r] = (i < nn && r < nn) ? y[t] : 0.0;
		}
		if (pass == 0) {
#pragma unroll
			for (int t = 0; t < 16; t++) As[i * kNodeLd + 4 * t + q] = a21[t];
			__syncthreads();
			v4d acc[4];
			node_product<true>(As, Xs, acc, wave, lane); // L21 = A21 X11^T
			node_store_lds(Ls, acc, wave, lane);
			__syncthreads();
			node_product<false>(Ls, Xs, acc, wave, lane); // T2 = L21 X11
			node_store_lds(Ts, acc, wave, lane);
			node_product<true>(Ls, Ls, acc, wave, lane); // L21 L21^T, which the second leaf takes off A22
			node_store_lds(As, acc, wave, lane);          // (A21 has been read by every wave: the barrier above)
			__syncthreads();
		}
	}
	__syncthreads();
	// X21 = -X22 T2, rows i < m, to X(r1 + i, r0 + j)
	v4d acc[4];
	node_product<false>(Xs, Ts, acc, wave, lane);
#pragma unroll
	for (int nb = 0; nb < 4; nb++)
#pragma unroll
		for (int r = 0; r < 4; r++) {
			const int row = 16 * wave + 4 * r + (lane >> 4), col = 16 * nb + (lane & 15);
			if (row < m) X[(size_t)(r0 + col) * ld + r1 + row] = -acc[nb][r];
		}
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
	if (blocks == 2) {
		constexpr size_t ldsBytes = sizeof(double) * 4 * kNodeBlock;
		static bool attributeSet = false;
		if (!attributeSet) {
			FITRE_HIP_TRY(hipFuncSetAttribute((const void *)dnode_pair_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
			attributeSet = true;
		}
		const int m = nn - kDLeaf;
		LaunchScope scope(KC, 2.0 * (2.0 * kDLeaf * (double)kDLeaf * kDLeaf / 3.0) + 8.0 * kDLeaf * (double)kDLeaf * m);
		dnode_pair_kernel<<<1, 256, ldsBytes, stream()>>>(r.W, n, r0, m, r.X, r.dInfo);
		return check_launch("dnode_pair_kernel");
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
	// A22 -= L21 L21^T and T2(m x n1) = L21 * X11 (B(k, j) = X11(k, j), zero for k < j): neither reads what the other writes
	DgemmLaunch update, inner;
	rc = dgemm_setup(m, m, n1, -1.0, dmat64(L21, 1, m), dmat64(L21, m, 1), 1.0, DOut{ A22, 1, n, FITRE_MAT_F64 }, 0.0, kDgMirror, KC, r.gws, r.gBytes,
	                 &update);
	if (rc) return rc;
	rc = dgemm_setup(m, n1, n1, 1.0, dmat64(L21, 1, m), dmat64(X11, 1, n), 0.0, DOut{ T2, 1, m, FITRE_MAT_F64 }, 0.0, kDgBLower, KC, r.gws, r.gBytes,
	                 &inner);
	if (rc) return rc;
	rc = dgemm_issue_pair(update, inner);
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

int fitre_hip_gemm_f64_add(long M, long N, long K, double alpha, const fitre_matrix *A, const fitre_matrix *B, double addScale,
                           const fitre_matrix *add, const fitre_matrix *C, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	DMat a, b;
	int rc = to_dmat(A, &a, "fitre_hip_gemm_f64_add");
	if (rc) return rc;
	rc = to_dmat(B, &b, "fitre_hip_gemm_f64_add");
	if (rc) return rc;
	FITRE_REQUIRE(C && C->data && add && add->data && add->kind == FITRE_MAT_F64, "fitre_hip_gemm_f64_add: null result or addend that is not of doubles");
	DOut c{ (void *)C->data, C->rowStride, C->colStride, C->kind };
	c.add = (const double *)add->data, c.addRs = add->rowStride, c.addCs = add->colStride, c.addScale = addScale;
	return dgemm(M, N, K, alpha, a, b, 0.0, c, 0.0, 0, FITRE_KC_FC_GEMM, ws, wsBytes);
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

// the first words of up to 40 arrays, four each, gathered into one array (what a host needs to tell the forms of stored
// inverses apart with one copy)
struct HeaderPointers {
	const uint32_t *p[40];
};
__global__ void gather_headers_kernel(HeaderPointers h, int count, uint32_t *out)
{
	const int t = blockIdx.x * blockDim.x + threadIdx.x;
	if (t < 4 * count) out[t] = h.p[t >> 2][t & 3];
}
struct HeaderWords {
	uint32_t w[16];
};
__global__ void write_header_kernel(uint32_t *dst, HeaderWords h, int count)
{
	if ((int)threadIdx.x < count) dst[threadIdx.x] = h.w[threadIdx.x];
}

int fitre_hip_gather_headers(const void *const *arrays, int count, void *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(arrays && out && count > 0 && count <= 40, "fitre_hip_gather_headers: bad argument");
	HeaderPointers h;
	for (int i = 0; i < count; i++) h.p[i] = (const uint32_t *)arrays[i];
	gather_headers_kernel<<<1, 256, 0, stream()>>>(h, count, (uint32_t *)out);
	return check_launch("gather_headers_kernel");
}

int fitre_hip_write_header(void *dst, const unsigned int *words, int count)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(dst && words && count > 0 && count <= 16, "fitre_hip_write_header: bad argument");
	HeaderWords h;
	for (int i = 0; i < count; i++) h.w[i] = words[i];
	write_header_kernel<<<1, 64, 0, stream()>>>((uint32_t *)dst, h, count);
	return check_launch("write_header_kernel");
}

// the dense double matrix a float pair stands for, 32 x 32 tiles: a tile and its mirror image are both read along their
// columns (coalesced) and meet in LDS
__global__ void __launch_bounds__(256) pair_decode_kernel(const float *P, long ld, int n, double *out, long ldo)
{
	__shared__ float U[32][33], V[32][33];
	const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
	const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
	for (int k = 0; k < 4; k++) {
		const int j = ty + 8 * k;
		U[j][tx] = (r0 + tx < n && c0 + j < n) ? P[(long)(c0 + j) * ld + r0 + tx] : 0.f; // P(r0 + tx, c0 + j)
		V[j][tx] = (c0 + tx < n && r0 + j < n) ? P[(long)(r0 + j) * ld + c0 + tx] : 0.f; // P(c0 + tx, r0 + j)
	}
	__syncthreads();
#pragma unroll
	for (int k = 0; k < 4; k++) {
		const int j = ty + 8 * k, r = r0 + tx, c = c0 + j;
		if (r >= n || c >= n) continue;
		const float here = U[j][tx], mirrored = V[tx][j]; // P(r, c), P(c, r)
		const int a = r < c ? r : c, b = r < c ? c : r;
		float hi = r <= c ? here : mirrored;
		uint32_t lo = __float_as_uint(r <= c ? mirrored : here);
		if (a == b) {
			lo = 0u;
			if (n >= 3) lo = __float_as_uint(P[(a + 1 < n) ? (long)a * ld + a + 1 : (long)(n - 1)]) << 16;
		} else if (n >= 3 && (b == a + 1 || (a == 0 && b == n - 1))) {
			lo &= 0xFFFF0000u;
		}
		out[(long)c * ldo + r] = (double)hi + (double)__uint_as_float(lo);
	}
}

int fitre_hip_pair_to_f64(const float *pairs, long ld, int n, double *out, long ldOut)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(pairs && out && n > 0 && ld >= n && ldOut >= n, "fitre_hip_pair_to_f64: bad argument");
	LaunchScope scope(FITRE_KC_BLAS1, 12.0 * (double)n * n);
	const unsigned tiles = (unsigned)((n + 31) / 32);
	pair_decode_kernel<<<dim3(tiles, tiles), 256, 0, stream()>>>(pairs, ld, n, out, ldOut);
	return check_launch("pair_decode_kernel");
}

int fitre_hip_widen_shift(const float *matrix, int n, double shift, double *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(matrix && out && n > 0, "fitre_hip_widen_shift: bad argument");
	widen_shift_kernel<<<blocks_for((long)n * n, 256, 8192), 256, 0, stream()>>>(matrix, out, n, shift);
	return check_launch("widen_shift_kernel");
}

} // extern "C"
