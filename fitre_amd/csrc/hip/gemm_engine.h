// fp32-MFMA tile engine shared by every dense contraction of the gradient path.
//
//   C[i][j] = sum_r A(i, r) * B(r, j),   0 <= i < I, 0 <= j < J, 0 <= r < R
//
// One workgroup of 256 threads (4 wave64 in a 2 x 2 arrangement) owns a BM x BN
// tile of C; each wave owns (BM/2) x (BN/2) of it as 32x32 accumulator blocks
// of v_mfma_f32_32x32x2_f32.  Operands are never materialised as matrices in
// memory: an "operand" object fetches its BK-deep slice straight from the
// tensors (plain strided matrix, implicit image patches, flipped weights) into
// registers, and the slice is then staged in LDS in [k][row] order, so that the
// 32 lanes feeding one MFMA operand read 32 consecutive words.  The next slice
// is fetched from global memory while the current one is being multiplied.
//
// j is the index that is contiguous in the output tensor, i the channel-like
// one; lanes of a wave map to j in the accumulator layout, which makes the
// final stores coalesced.  A third grid dimension cuts the reduction range
// (split-K); partial tiles then go to a workspace and are combined in a fixed
// order by splitk_reduce_kernel, so results do not depend on scheduling.
#pragma once
#include "common.h"

namespace fitre {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;

template <int BM_, int BN_, int BK_>
struct TileCfg {
	static constexpr int BM = BM_, BN = BN_, BK = BK_;
	static constexpr int WM = BM / 2, WN = BN / 2; // wave tile
	static constexpr int TM = WM / 32, TN = WN / 32; // 32x32 blocks per wave
	static constexpr int LDA = BM + 1, LDB = BN + 1; // odd strides: conflict-light for both access patterns
	static_assert(BM % 64 == 0 && BN % 64 == 0 && BK % 2 == 0, "tile shape");
	static_assert((BM * BK) % kGemmThreads == 0 && (BN * BK) % kGemmThreads == 0, "tile shape");
	static_assert(kGemmThreads % BK == 0, "BK must divide the workgroup");
};

// ---------------------------------------------------------------------------
// operands.  ROWS is BM or BN.  Every operand provides
//   init(params, row0, tid)      once per workgroup
//   load(k0, kend, regs)         global -> registers, zero outside the matrix
//   store(lds, regs)             registers -> LDS [k][row], row stride LD
// ---------------------------------------------------------------------------

// a strided matrix operand: rows along the non-reduction index
struct PlainParams {
	const float *p;
	long ld;
	int rows;
};

// element(row, k) = p[k * ld + row]   (contiguous along the non-reduction index)
template <int ROWS, int BK, int LD>
struct PlainRowContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int KSTEP = kGemmThreads / ROWS;
	typedef PlainParams Params;
	const float *p;
	long ld;
	int rowL, kL;
	bool rowOk;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		rowL = tid % ROWS;
		kL = tid / ROWS;
		rowOk = (row0 + rowL) < pr.rows;
		p = pr.p + (row0 + rowL);
		ld = pr.ld;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) {
			int k = k0 + kL + KSTEP * e;
			r[e] = (rowOk && k < kend) ? p[(size_t)k * ld] : 0.f;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[(kL + KSTEP * e) * LD + rowL] = r[e];
	}
};

// element(row, k) = p[row * ld + k]   (contiguous along the reduction index)
template <int ROWS, int BK, int LD>
struct PlainKContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	typedef PlainParams Params;
	const float *p;
	long ld;
	int rowL, kL, rowsLeft;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		kL = tid % BK;
		rowL = tid / BK;
		rowsLeft = pr.rows - row0;
		p = pr.p + (size_t)row0 * pr.ld;
		ld = pr.ld;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		int k = k0 + kL;
		bool kOk = k < kend;
#pragma unroll
		for (int e = 0; e < E; e++) {
			int row = rowL + RSTEP * e;
			r[e] = (kOk && row < rowsLeft) ? p[(size_t)row * ld + k] : 0.f;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[kL * LD + rowL + RSTEP * e] = r[e];
	}
};

// Geometry of an image-patch gather: positions m = (n, oa, ob) of an output grid
// outA x outB, taps (ta, tb) of a ksize x ksize window, source image srcA x srcB,
// source cell (oa*stride - pad + ta, ob*stride - pad + tb); cells outside the
// image read as zero.
struct PatchGeom {
	const float *src; // [channels][samples][srcA][srcB]
	int samples, srcA, srcB, outA, outB, ksize, stride, pad;
	int positions;      // samples * outA * outB
	int taps;           // ksize * ksize
	int patchLen;       // channels * taps
	long chanStride;    // samples * srcA * srcB
	FastDiv divOutB, divOutA, divTaps, divK;
};

// element(row = m, k = (c, ta, tb)) of the patch matrix; contiguous along m.
template <int ROWS, int BK, int LD>
struct PatchRowContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int KSTEP = kGemmThreads / ROWS;
	typedef PatchGeom Params;
	PatchGeom g; // copy of the kernel argument: stays in scalar registers
	int rowL, kL;
	int a0, b0;  // source cell of tap (0,0)
	int base;    // offset of that cell inside a channel plane (may be negative)
	bool rowOk;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		g = pr;
		rowL = tid % ROWS;
		kL = __builtin_amdgcn_readfirstlane(tid / ROWS); // the same for a whole wave (ROWS >= 64)
		uint32_t m = (uint32_t)(row0 + rowL);
		rowOk = m < (uint32_t)pr.positions;
		uint32_t q, ob, n, oa;
		pr.divOutB.divmod(m, q, ob);
		pr.divOutA.divmod(q, n, oa);
		a0 = (int)oa * pr.stride - pr.pad;
		b0 = (int)ob * pr.stride - pr.pad;
		base = (int)n * pr.srcA * pr.srcB + a0 * pr.srcB + b0;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) {
			int k = k0 + kL + KSTEP * e; // wave-uniform
			uint32_t c, tap, ta, tb;
			g.divTaps.divmod((uint32_t)k, c, tap);
			g.divK.divmod(tap, ta, tb);
			int a = a0 + (int)ta, b = b0 + (int)tb;
			bool ok = rowOk && k < kend && (unsigned)a < (unsigned)g.srcA && (unsigned)b < (unsigned)g.srcB;
			long off = (long)c * g.chanStride + base + (int)ta * g.srcB + (int)tb;
			r[e] = ok ? g.src[off] : 0.f;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[(kL + KSTEP * e) * LD + rowL] = r[e];
	}
};

// element(row = (c, ta, tb), k = m) of the transposed patch matrix; the reduction
// index m is the contiguous one.  Used for the weight gradient.
template <int ROWS, int BK, int LD>
struct PatchKContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	typedef PatchGeom Params;
	PatchGeom g;
	int rowL, kL;
	long rowOff[E]; // c*chanStride + ta*srcB + tb, or -1 for rows past the patch length
	int rowTap[E];  // ta << 16 | tb
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		g = pr;
		kL = tid % BK;
		rowL = tid / BK;
#pragma unroll
		for (int e = 0; e < E; e++) {
			uint32_t row = (uint32_t)(row0 + rowL + RSTEP * e);
			uint32_t c, tap, ta, tb;
			pr.divTaps.divmod(row, c, tap);
			pr.divK.divmod(tap, ta, tb);
			rowOff[e] = (row < (uint32_t)pr.patchLen) ? (long)c * pr.chanStride + (long)ta * pr.srcB + tb : -1;
			rowTap[e] = (int)((ta << 16) | tb);
		}
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		uint32_t m = (uint32_t)(k0 + kL);
		bool kOk = (int)m < kend;
		uint32_t q, ob, n, oa;
		g.divOutB.divmod(m, q, ob);
		g.divOutA.divmod(q, n, oa);
		int a0 = (int)oa * g.stride - g.pad, b0 = (int)ob * g.stride - g.pad;
		long base = (long)n * g.srcA * g.srcB + (long)a0 * g.srcB + b0;
#pragma unroll
		for (int e = 0; e < E; e++) {
			int a = a0 + (rowTap[e] >> 16), b = b0 + (rowTap[e] & 0xffff);
			bool ok = kOk && rowOff[e] >= 0 && (unsigned)a < (unsigned)g.srcA && (unsigned)b < (unsigned)g.srcB;
			r[e] = ok ? g.src[rowOff[e] + base] : 0.f;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[kL * LD + rowL + RSTEP * e] = r[e];
	}
};

// Weights as seen by the input gradient: element(row = ci, k = (o, ta, tb)) =
// w[o][ci][ksize-1-ta][ksize-1-tb]  (w is [Cout][Cin][k][k]).
struct FlipWeightParams {
	const float *w;
	int cin, taps;   // taps = ksize*ksize
	long outStride;  // cin * taps
	FastDiv divTaps;
};
template <int ROWS, int BK, int LD>
struct FlipWeightKContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	typedef FlipWeightParams Params;
	FlipWeightParams g;
	int rowL, kL, row0;
	__device__ __forceinline__ void init(const Params &pr, int r0, int tid)
	{
		g = pr;
		kL = tid % BK;
		rowL = tid / BK;
		row0 = r0;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		int k = k0 + kL;
		bool kOk = k < kend;
		uint32_t o, tap;
		g.divTaps.divmod((uint32_t)k, o, tap);
		long off = (long)o * g.outStride + (g.taps - 1 - (int)tap);
#pragma unroll
		for (int e = 0; e < E; e++) {
			int row = row0 + rowL + RSTEP * e;
			r[e] = (kOk && row < g.cin) ? g.w[off + (long)row * g.taps] : 0.f;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[kL * LD + rowL + RSTEP * e] = r[e];
	}
};

// ---------------------------------------------------------------------------
// output
// ---------------------------------------------------------------------------
struct OutParams {
	float *C;          // C[i * ldc + j]
	long ldc;
	long splitStride;  // distance between the partial results of two splits (0 when unsplit)
	const float *biasI; // added per i (may be null); ignored when split
	const float *biasJ; // added per j (may be null); ignored when split
	float alpha, beta;  // C = alpha * acc (+ bias) + beta * C; ignored when split
};

// ---------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------
template <class Cfg, class OpA, class OpB>
__global__ void __launch_bounds__(kGemmThreads)
mfma_gemm_kernel(const typename OpA::Params pa, const typename OpB::Params pb, const OutParams out, int I, int J, int R,
                 int kChunk)
{
	constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
	constexpr int TM = Cfg::TM, TN = Cfg::TN;
	__shared__ float As[BK * Cfg::LDA];
	__shared__ float Bs[BK * Cfg::LDB];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int i0 = blockIdx.y * BM, j0 = blockIdx.x * BN;
	const int kbeg = blockIdx.z * kChunk;
	const int kend = (kbeg + kChunk < R) ? kbeg + kChunk : R;

	OpA opA;
	OpB opB;
	opA.init(pa, i0, tid);
	opB.init(pb, j0, tid);

	v16f acc[TM][TN];
#pragma unroll
	for (int tm = 0; tm < TM; tm++)
#pragma unroll
		for (int tn = 0; tn < TN; tn++)
#pragma unroll
			for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.f;

	float ra[OpA::E], rb[OpB::E];
	opA.load(kbeg, kend, ra);
	opB.load(kbeg, kend, rb);

	const int wi = (wave >> 1) * Cfg::WM + (lane & 31);
	const int wj = (wave & 1) * Cfg::WN + (lane & 31);
	const int khalf = lane >> 5;

	for (int k0 = kbeg; k0 < kend; k0 += BK) {
		__syncthreads(); // everyone is done reading the previous slice
		opA.store(As, ra);
		opB.store(Bs, rb);
		__syncthreads();
		if (k0 + BK < kend) {
			opA.load(k0 + BK, kend, ra);
			opB.load(k0 + BK, kend, rb);
		}
#pragma unroll
		for (int kk = 0; kk < BK / 2; kk++) {
			const int krow = 2 * kk + khalf;
			float a[TM], b[TN];
#pragma unroll
			for (int tm = 0; tm < TM; tm++) a[tm] = As[krow * Cfg::LDA + wi + tm * 32];
#pragma unroll
			for (int tn = 0; tn < TN; tn++) b[tn] = Bs[krow * Cfg::LDB + wj + tn * 32];
#pragma unroll
			for (int tm = 0; tm < TM; tm++)
#pragma unroll
				for (int tn = 0; tn < TN; tn++)
					acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm], b[tn], acc[tm][tn], 0, 0, 0);
		}
	}

	// accumulator layout of the 32x32 block: register v of lane l holds
	// row 8*(v/4) + 4*(l/32) + v%4, column l%32.
	const bool split = out.splitStride != 0;
	float *C = out.C + (size_t)blockIdx.z * out.splitStride;
#pragma unroll
	for (int tm = 0; tm < TM; tm++) {
#pragma unroll
		for (int tn = 0; tn < TN; tn++) {
			const int j = j0 + (wave & 1) * Cfg::WN + tn * 32 + (lane & 31);
			if (j >= J) continue;
#pragma unroll
			for (int v = 0; v < 16; v++) {
				const int i = i0 + (wave >> 1) * Cfg::WM + tm * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
				if (i >= I) continue;
				float val = acc[tm][tn][v];
				float *dst = C + (size_t)i * out.ldc + j;
				if (!split) {
					val *= out.alpha;
					if (out.biasI) val += out.biasI[i];
					if (out.biasJ) val += out.biasJ[j];
					if (out.beta != 0.f) val += out.beta * *dst;
				}
				*dst = val;
			}
		}
	}
}

// C[i*ldc + j] = alpha * sum_s ws[s][i][j] (+bias) + beta*C, partials summed in split order.
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *ws, int splits, int I, int J, OutParams out)
{
	long total = (long)I * J;
	long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		int i = (int)(idx / J), j = (int)(idx - (long)i * J);
		double acc = 0.0;
		for (int s = 0; s < splits; s++) acc += (double)ws[(size_t)s * total + idx];
		float val = (float)acc * out.alpha;
		if (out.biasI) val += out.biasI[i];
		if (out.biasJ) val += out.biasJ[j];
		float *dst = out.C + (size_t)i * out.ldc + j;
		if (out.beta != 0.f) val += out.beta * *dst;
		*dst = val;
	}
}

// ---------------------------------------------------------------------------
// host-side planning
// ---------------------------------------------------------------------------
struct GemmPlan {
	int bm, bn;     // tile
	int splits;     // grid.z
	int kChunk;     // reduction indices per split (multiple of BK)
	size_t wsBytes; // workspace needed (0 when unsplit)
};

constexpr int kGemmBK = 16;

inline GemmPlan plan_gemm(long I, long J, long R)
{
	GemmPlan p;
	p.bm = (I <= 64) ? 64 : 128;
	p.bn = (J <= 64) ? 64 : 128;
	long tiles = ((I + p.bm - 1) / p.bm) * ((J + p.bn - 1) / p.bn);
	long want = (768 + tiles - 1) / tiles; // aim at three workgroups per compute unit
	long maxByDepth = R / (4 * kGemmBK);    // keep at least four slices per split
	if (maxByDepth < 1) maxByDepth = 1;
	long splits = want < maxByDepth ? want : maxByDepth;
	if (splits > 1024) splits = 1024;
	if (splits < 1) splits = 1;
	long chunk = (R + splits - 1) / splits;
	chunk = ((chunk + kGemmBK - 1) / kGemmBK) * kGemmBK;
	splits = (R + chunk - 1) / chunk;
	p.splits = (int)splits;
	p.kChunk = (int)chunk;
	p.wsBytes = (splits > 1) ? (size_t)splits * I * J * sizeof(float) : 0;
	return p;
}

// Shrinks the number of splits until the partial tiles fit the workspace the
// caller actually has; with too little for two splits the product runs unsplit.
inline GemmPlan fit_plan(GemmPlan p, long I, long J, long R, const void *ws, size_t wsBytes)
{
	if (p.splits <= 1) return p;
	size_t per = (size_t)I * J * sizeof(float);
	long fit = ws ? (long)(wsBytes / per) : 0;
	if (fit >= p.splits) return p;
	long splits = fit >= 2 ? fit : 1;
	long chunk = (R + splits - 1) / splits;
	chunk = ((chunk + kGemmBK - 1) / kGemmBK) * kGemmBK;
	splits = (R + chunk - 1) / chunk;
	p.splits = (int)splits;
	p.kChunk = (int)chunk;
	p.wsBytes = (splits > 1) ? (size_t)splits * per : 0;
	return p;
}

template <template <int, int, int> class OpA, template <int, int, int> class OpB, int BM, int BN>
static int launch_tile(const typename OpA<BM, kGemmBK, BM + 1>::Params &pa, const typename OpB<BN, kGemmBK, BN + 1>::Params &pb,
                       const OutParams &out, int I, int J, int R, const GemmPlan &plan, void *ws, int kernelClass, double flops)
{
	typedef TileCfg<BM, BN, kGemmBK> Cfg;
	constexpr int tileId = (BM == 64 ? (BN == 64 ? 1 : 2) : (BN == 64 ? 3 : 4));
	typedef OpA<BM, kGemmBK, Cfg::LDA> A;
	typedef OpB<BN, kGemmBK, Cfg::LDB> B;
	dim3 grid((J + BN - 1) / BN, (I + BM - 1) / BM, plan.splits);
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "gemm grid %u x %u x %u too large", grid.x, grid.y, grid.z);
	if (plan.splits > 1) {
		OutParams part = out;
		part.C = (float *)ws;
		part.ldc = J;
		part.splitStride = (long)I * J;
		{
			LaunchScope scope(kernelClass, flops, tileId);
			mfma_gemm_kernel<Cfg, A, B><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, part, I, J, R, plan.kChunk);
		}
		OutParams fin = out;
		fin.splitStride = 0;
		LaunchScope scope(FITRE_KC_SPLITK_REDUCE, 4.0 * (double)I * J * (plan.splits + 1));
		splitk_reduce_kernel<<<blocks_for((long)I * J, 256, 4096), 256, 0, stream()>>>((const float *)ws, plan.splits, I, J, fin);
	} else {
		OutParams direct = out;
		direct.splitStride = 0;
		LaunchScope scope(kernelClass, flops, tileId);
		mfma_gemm_kernel<Cfg, A, B><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, direct, I, J, R, plan.kChunk);
	}
	return check_launch("mfma_gemm_kernel");
}

// Picks the tile instantiation the plan names.
template <template <int, int, int> class OpA, template <int, int, int> class OpB, class PA, class PB>
static int launch_gemm(const PA &pa, const PB &pb, const OutParams &out, int I, int J, int R, const GemmPlan &ideal, void *ws,
                       size_t wsBytes, int kernelClass, double flops)
{
	const GemmPlan plan = fit_plan(ideal, I, J, R, ws, wsBytes);
	if (plan.wsBytes > 0) {
		if (!ws || (((uintptr_t)ws) & 3)) return fail(FITRE_E_WORKSPACE, "split-K workspace is null or misaligned");
		if (wsBytes < plan.wsBytes)
			return fail(FITRE_E_WORKSPACE, "split-K workspace of %zu bytes is smaller than the %zu required", wsBytes, plan.wsBytes);
	}
	if (plan.bm == 128 && plan.bn == 128) return launch_tile<OpA, OpB, 128, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	if (plan.bm == 64 && plan.bn == 128) return launch_tile<OpA, OpB, 64, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	if (plan.bm == 128 && plan.bn == 64) return launch_tile<OpA, OpB, 128, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	return launch_tile<OpA, OpB, 64, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
}

} // namespace fitre
