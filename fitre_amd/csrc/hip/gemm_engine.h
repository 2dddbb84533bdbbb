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

// WAVES_M x WAVES_N: how the four waves are arranged over the tile.  2 x 2 for the square tiles; 1 x 4 for
// the 96-row tile (three 32-row blocks per wave, no padding for 96-channel layers such as AlexNet's).
template <int BM_, int BN_, int BK_, int WAVES_M_ = 2, int WAVES_N_ = 2>
struct TileCfg {
	static constexpr int BM = BM_, BN = BN_, BK = BK_;
	static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
	static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N; // wave tile
	static constexpr int TM = WM / 32, TN = WN / 32; // 32x32 blocks per wave
	static_assert(WAVES_M * WAVES_N == 4, "four waves per workgroup");
	static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 2 == 0, "tile shape");
	static_assert((BM * BK) % kGemmThreads == 0 && (BN * BK) % kGemmThreads == 0, "tile shape");
	static_assert(kGemmThreads % BK == 0, "BK must divide the workgroup");
};

// Operands whose threads walk the rows in steps of 256 / BK (the reduction-contiguous ones) work for any row
// count that gives whole elements per thread, 96 included; they say so with `kAnyRows`.  The row-contiguous
// operands need 256 % ROWS == 0.
template <class T, class = void>
struct operand_any_rows { static constexpr bool value = false; };
template <class T>
struct operand_any_rows<T, decltype((void)T::kAnyRows)> { static constexpr bool value = T::kAnyRows; };

// ---------------------------------------------------------------------------
// operands.  ROWS is BM or BN.  Every operand provides
//   init(params, row0, tid)      once per workgroup
//   load(k0, kend, regs)         global -> registers, zero outside the matrix
//   store(lds, regs)             registers -> LDS [k][row], row stride LD
//
// Global reads go through a raw buffer resource: an element outside the matrix
// or the image gets the byte offset 0xFFFFFFFF, which the hardware range check
// answers with zero -- no branch and no 64-bit address arithmetic per element.
// Every tensor an operand reads must therefore be smaller than 4 GiB.
// ---------------------------------------------------------------------------

constexpr uint32_t kOutOfRange = 0xFFFFFFFFu;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float *p, uint32_t bytes)
{
	return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, bytes, 0x00020000);
}
__device__ __forceinline__ float buffer_load(__amdgpu_buffer_rsrc_t r, uint32_t byteOffset)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byteOffset, 0, 0));
}

// LDS row stride for a tile of ROWS rows: stores of the k-contiguous operands
// put 16 (BK = 16) or 32 (BK = 32) consecutive k of a few rows into one
// instruction; stride = 2 (resp. 1) mod 32 spreads them over all banks.  Reads
// (32 consecutive rows of one k) are conflict-free for any stride.
template <int ROWS, int BK>
struct LdsStride {
	static constexpr int value = ROWS + (BK == 16 ? 2 : 1);
};

// a strided matrix operand: rows along the non-reduction index
struct PlainParams {
	const float *p;
	uint32_t bytes; // extent of the matrix in memory
	int ld;
	int rows;
};

// element(row, k) = p[k * ld + row]   (contiguous along the non-reduction index)
template <int ROWS, int BK>
struct PlainRowContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int KSTEP = kGemmThreads / ROWS;
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	typedef PlainParams Params;
	__amdgpu_buffer_rsrc_t rsrc;
	int ld, rowL, kL, row;
	bool rowOk;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		rsrc = make_rsrc(pr.p, pr.bytes);
		rowL = tid % ROWS;
		kL = tid / ROWS;
		row = row0 + rowL;
		rowOk = row < pr.rows;
		ld = pr.ld;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) {
			int k = k0 + kL + KSTEP * e;
			uint32_t off = (rowOk & (k < kend)) ? 4u * (uint32_t)(k * ld + row) : kOutOfRange;
			r[e] = buffer_load(rsrc, off);
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[(kL + KSTEP * e) * LD + rowL] = r[e];
	}
};

// element(row, k) = p[row * ld + k]   (contiguous along the reduction index)
template <int ROWS, int BK>
struct PlainKContig {
	static constexpr bool kAnyRows = true;
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	typedef PlainParams Params;
	__amdgpu_buffer_rsrc_t rsrc;
	int rowL, kL;
	uint32_t rowOff[E]; // 4 * row * ld, or out of range
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		rsrc = make_rsrc(pr.p, pr.bytes);
		kL = tid % BK;
		rowL = tid / BK;
#pragma unroll
		for (int e = 0; e < E; e++) {
			int row = row0 + rowL + RSTEP * e;
			rowOff[e] = (row < pr.rows) ? 4u * (uint32_t)(row * pr.ld) : kOutOfRange;
		}
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		int k = k0 + kL;
		bool kOk = k < kend;
#pragma unroll
		for (int e = 0; e < E; e++) {
			uint32_t off = (kOk & (rowOff[e] != kOutOfRange)) ? rowOff[e] + 4u * (uint32_t)k : kOutOfRange;
			r[e] = buffer_load(rsrc, off);
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
	uint32_t bytes;   // extent of src
	int samples, srcA, srcB, outA, outB, ksize, stride, pad;
	int positions;   // samples * outA * outB
	int taps;        // ksize * ksize
	int patchLen;    // channels * taps
	int chanStride;  // samples * srcA * srcB
	float onesValue; // value of the constant row that PatchKContigOnes appends after the patch rows
	// Decode of the reduction index k = (c, ta, tb) for the operand whose k is uniform across a
	// wave: low word c*chanStride + ta*srcB + tb, high word ta << 16 | tb.  Entries are stored in
	// the order the waves consume them (see patch_table_slot) and read with scalar loads.
	const unsigned long long *ktable;
	FastDiv divOutB, divOutA, divTaps, divK;
};

// A wave of the row-contiguous patch operand handles, in every BK-deep slice, the indices
// k0 + kL + kstep*e (e = 0..BK/kstep-1); their table entries sit next to each other.
__host__ __device__ inline int patch_table_slot(int k, int bk, int kstep)
{
	int in = k % bk;
	return (k - in) + (in % kstep) * (bk / kstep) + in / kstep;
}

// fills PatchGeom::ktable for slices of depth bk read with stride kstep; `padded` entries
static __global__ void patch_table_kernel(unsigned long long *table, int padded, int patchLen, int chanStride, int srcB,
                                   FastDiv divTaps, FastDiv divK, int bk, int kstep)
{
	int k = blockIdx.x * blockDim.x + threadIdx.x;
	if (k >= padded) return;
	unsigned long long entry = 0;
	if (k < patchLen) {
		uint32_t c, tap, ta, tb;
		divTaps.divmod((uint32_t)k, c, tap);
		divK.divmod(tap, ta, tb);
		uint32_t off = (uint32_t)((int)c * chanStride + (int)ta * srcB + (int)tb);
		entry = ((unsigned long long)((ta << 16) | tb) << 32) | off;
	}
	table[patch_table_slot(k, bk, kstep)] = entry;
}

// element(row = m, k = (c, ta, tb)) of the patch matrix; contiguous along m.
template <int ROWS, int BK>
struct PatchRowContig {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int KSTEP = kGemmThreads / ROWS;
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	typedef PatchGeom Params;
	PatchGeom g; // copy of the kernel argument: stays in scalar registers
	__amdgpu_buffer_rsrc_t rsrc;
	int rowL, kL;
	int a0, b0;  // source cell of tap (0,0)
	int base;    // offset of that cell inside a channel plane (may be negative)
	bool rowOk;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		g = pr;
		rsrc = make_rsrc(pr.src, pr.bytes);
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
		// the E entries of this wave are contiguous and 8*E-byte aligned: one wide scalar load
		const unsigned long long *p =
		    (const unsigned long long *)__builtin_assume_aligned(g.ktable + (k0 + kL * E), 8 * E);
		unsigned long long t[E];
#pragma unroll
		for (int e = 0; e < E; e++) t[e] = p[e];
#pragma unroll
		for (int e = 0; e < E; e++) {
			int k = k0 + kL + KSTEP * e; // wave-uniform
			int tap = (int)(t[e] >> 32), kOff = (int)(uint32_t)t[e];
			int a = a0 + (tap >> 16), b = b0 + (tap & 0xffff);
			bool ok = rowOk & (k < kend) & ((unsigned)a < (unsigned)g.srcA) & ((unsigned)b < (unsigned)g.srcB);
			r[e] = buffer_load(rsrc, ok ? 4u * (uint32_t)(base + kOff) : kOutOfRange);
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[(kL + KSTEP * e) * LD + rowL] = r[e];
	}
};

// element(row = (c, ta, tb), k = m) of the transposed patch matrix; the reduction
// index m is the contiguous one.  Used for the weight gradient and the Kronecker factors.
// ONES: row patchLen is a constant row (onesValue at every position) -- the bias column
// of the augmented patch matrix.
template <int ROWS, int BK, bool ONES>
struct PatchKContigT {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	typedef PatchGeom Params;
	PatchGeom g;
	__amdgpu_buffer_rsrc_t rsrc;
	int rowL, kL;
	int rowOff[E]; // c*chanStride + ta*srcB + tb, or -1 for rows past the patch length
	int rowTap[E]; // ta << 16 | tb
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		g = pr;
		rsrc = make_rsrc(pr.src, pr.bytes);
		kL = tid % BK;
		rowL = tid / BK;
#pragma unroll
		for (int e = 0; e < E; e++) {
			uint32_t row = (uint32_t)(row0 + rowL + RSTEP * e);
			uint32_t c, tap, ta, tb;
			pr.divTaps.divmod(row, c, tap);
			pr.divK.divmod(tap, ta, tb);
			rowOff[e] = (row < (uint32_t)pr.patchLen) ? (int)c * pr.chanStride + (int)ta * pr.srcB + (int)tb : -1;
			if (ONES && row == (uint32_t)pr.patchLen) rowOff[e] = -2;
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
		int base = (int)n * g.srcA * g.srcB + a0 * g.srcB + b0;
#pragma unroll
		for (int e = 0; e < E; e++) {
			int a = a0 + (rowTap[e] >> 16), b = b0 + (rowTap[e] & 0xffff);
			bool ok = kOk & (rowOff[e] >= 0) & ((unsigned)a < (unsigned)g.srcA) & ((unsigned)b < (unsigned)g.srcB);
			r[e] = buffer_load(rsrc, ok ? 4u * (uint32_t)(rowOff[e] + base) : kOutOfRange);
			if (ONES) r[e] = (kOk & (rowOff[e] == -2)) ? g.onesValue : r[e];
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int e = 0; e < E; e++) lds[kL * LD + rowL + RSTEP * e] = r[e];
	}
};
template <int ROWS, int BK> using PatchKContig = PatchKContigT<ROWS, BK, false>;
template <int ROWS, int BK> using PatchKContigOnes = PatchKContigT<ROWS, BK, true>;

// Weights as seen by the input gradient: element(row = ci, k = (o, ta, tb)) =
// w[o][ci][ksize-1-ta][ksize-1-tb]  (w is [Cout][Cin][k][k]).
struct FlipWeightParams {
	const float *w;
	uint32_t bytes;
	int cin, taps;  // taps = ksize*ksize
	int outStride;  // cin * taps
	FastDiv divTaps;
};
template <int ROWS, int BK>
struct FlipWeightKContig {
	static constexpr bool kAnyRows = true;
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int RSTEP = kGemmThreads / BK;
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	typedef FlipWeightParams Params;
	FlipWeightParams g;
	__amdgpu_buffer_rsrc_t rsrc;
	int rowL, kL;
	int rowOff[E]; // row * taps, or -1
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		g = pr;
		rsrc = make_rsrc(pr.w, pr.bytes);
		kL = tid % BK;
		rowL = tid / BK;
#pragma unroll
		for (int e = 0; e < E; e++) {
			int row = row0 + rowL + RSTEP * e;
			rowOff[e] = (row < pr.cin) ? row * pr.taps : -1;
		}
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		int k = k0 + kL;
		bool kOk = k < kend;
		uint32_t o, tap;
		g.divTaps.divmod((uint32_t)k, o, tap);
		int off = (int)o * g.outStride + (g.taps - 1 - (int)tap);
#pragma unroll
		for (int e = 0; e < E; e++)
			r[e] = buffer_load(rsrc, (kOk & (rowOff[e] >= 0)) ? 4u * (uint32_t)(off + rowOff[e]) : kOutOfRange);
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
	// Symmetric product (both operands are the same matrix, I == J): tiles entirely below the
	// diagonal are skipped, elements with j < i are not stored and every stored element with
	// j > i is also written to C[j][i].  With split-K the mirroring happens in the reduction.
	int mirror;
	// Bit mask of kTri*: operands that are zero on one side of the diagonal in the reduction index.
	int triK;
	// Non-zero: rows come in groups of four that are interleaved with the columns in memory -- element (i, j)
	// lives at C[(i / 4) * quadLd + 4 * j + i % 4] (a [C][N][2][2] tensor with i = (c, cell), j = n; quadLd = 4 J).
	// A lane's four consecutive rows then form one 16-byte group.  Applies to split partials as well (each a
	// permutation of I x J elements, I % 4 == 0); bias, beta and mirror are not used with it.
	long quadLd;
	// Non-zero tapRows: both operands are patch rows in tap-major order (rows t * tapRows .. of tap t = (ta, tb) of a
	// tapKs x tapKs window, stride 1, padding tapPad) over the reduction index (cell of the tapOutA x tapOutB output map,
	// image), cells row by row, tapImages images per cell.  Row (t, c) is zero at the cells whose tap falls outside the
	// tapSrcA x tapSrcB image, so the reduction of a tile (one tap on each side: tapRows is a multiple of the tile) runs
	// from the first to the last cell at which both taps are inside; a pair of taps that never are gives a zero tile.
	int tapRows, tapImages, tapKs, tapPad, tapOutA, tapOutB, tapSrcA, tapSrcB;
};

// first and one-past-last reduction index of the cells at which taps t1 and t2 both fall inside the image (lo >= hi: none)
__host__ __device__ inline void tap_pair_range(const OutParams &o, int t1, int t2, int &lo, int &hi)
{
	const int a1 = t1 / o.tapKs - o.tapPad, b1 = t1 % o.tapKs - o.tapPad; // source cell = output cell + (a, b)
	const int a2 = t2 / o.tapKs - o.tapPad, b2 = t2 % o.tapKs - o.tapPad;
	const int amin = a1 < a2 ? a1 : a2, amax = a1 > a2 ? a1 : a2;
	const int bmin = b1 < b2 ? b1 : b2, bmax = b1 > b2 ? b1 : b2;
	int alo = -amin > 0 ? -amin : 0, ahi = o.tapSrcA - 1 - amax;
	int blo = -bmin > 0 ? -bmin : 0, bhi = o.tapSrcB - 1 - bmax;
	if (ahi > o.tapOutA - 1) ahi = o.tapOutA - 1;
	if (bhi > o.tapOutB - 1) bhi = o.tapOutB - 1;
	if (alo > ahi || blo > bhi) {
		lo = hi = 0;
		return;
	}
	lo = (alo * o.tapOutB + blo) * o.tapImages;
	hi = (ahi * o.tapOutB + bhi + 1) * o.tapImages;
}
// both operands: element (row, k) is zero for k < row, so the reduction of a tile starts at the larger of its first rows
constexpr int kTriBoth = 1;
constexpr int kTriAFromRow = 2; // operand A: element (i, k) is zero for k < i
constexpr int kTriAToRow = 4;   // operand A: element (i, k) is zero for k > i
constexpr int kTriBToRow = 8;   // operand B: element (j, k) is zero for k > j

// ---------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------
// One workgroup's tile of reduction range `split` (the body of both kernels below).
// As, Bs: the workgroup's LDS for one reduction slice of each operand (BK * OpA::LD resp. BK * OpB::LD floats)
template <class Cfg, class OpA, class OpB>
__device__ __forceinline__ void gemm_tile(const typename OpA::Params &pa, const typename OpB::Params &pb, const OutParams &out,
                                          int I, int J, int R, int kChunk, int splitIndex, float *As, float *Bs)
{
	constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
	constexpr int TM = Cfg::TM, TN = Cfg::TN;
	constexpr int LDA = OpA::LD, LDB = OpB::LD;

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int i0 = blockIdx.y * BM, j0 = blockIdx.x * BN;
	int kbeg = splitIndex * kChunk;
	int kend = (kbeg + kChunk < R) ? kbeg + kChunk : R;
	if (out.mirror && j0 + BN <= i0) return; // the mirror tile produces these elements
	// triangular operands: the part of the reduction range in which an operand of this tile is all zero is skipped
	// (a split whose whole range falls there writes a zero partial tile)
	if (out.triK & kTriBoth) {
		const int first = ((i0 > j0) ? i0 : j0) & ~(BK - 1);
		kbeg = (kbeg > first) ? kbeg : first;
	}
	if (out.triK & kTriAFromRow) {
		const int first = i0 & ~(BK - 1);
		kbeg = (kbeg > first) ? kbeg : first;
	}
	if (out.triK & kTriAToRow) kend = (kend < i0 + BM) ? kend : i0 + BM;
	if (out.triK & kTriBToRow) kend = (kend < j0 + BN) ? kend : j0 + BN;
	if (out.tapRows) {
		int lo, hi;
		tap_pair_range(out, i0 / out.tapRows, j0 / out.tapRows, lo, hi);
		lo &= ~(BK - 1);
		kbeg = (kbeg > lo) ? kbeg : lo;
		kend = (kend < hi) ? kend : hi;
	}

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

	const int khalf = lane >> 5;
	const int waveM = wave / Cfg::WAVES_N, waveN = wave % Cfg::WAVES_N;
	const float *aRd = As + khalf * LDA + waveM * Cfg::WM + (lane & 31);
	const float *bRd = Bs + khalf * LDB + waveN * Cfg::WN + (lane & 31);

	for (int k0 = kbeg; k0 < kend; k0 += BK) {
		__syncthreads(); // everyone is done reading the previous slice
		opA.store(As, ra);
		opB.store(Bs, rb);
		__syncthreads();
		if (k0 + BK < kend) {
			opA.load(k0 + BK, kend, ra);
			opB.load(k0 + BK, kend, rb);
		}
		// the fragments of step kk+1 are read from LDS while the MFMAs of step kk run
		float a[2][TM], b[2][TN];
#pragma unroll
		for (int tm = 0; tm < TM; tm++) a[0][tm] = aRd[tm * 32];
#pragma unroll
		for (int tn = 0; tn < TN; tn++) b[0][tn] = bRd[tn * 32];
#pragma unroll
		for (int kk = 0; kk < BK / 2; kk++) {
			const int cur = kk & 1, nxt = cur ^ 1;
			if (kk + 1 < BK / 2) {
#pragma unroll
				for (int tm = 0; tm < TM; tm++) a[nxt][tm] = aRd[(2 * kk + 2) * LDA + tm * 32];
#pragma unroll
				for (int tn = 0; tn < TN; tn++) b[nxt][tn] = bRd[(2 * kk + 2) * LDB + tn * 32];
			}
#pragma unroll
			for (int tm = 0; tm < TM; tm++)
#pragma unroll
				for (int tn = 0; tn < TN; tn++)
					acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][tm], b[cur][tn], acc[tm][tn], 0, 0, 0);
			// issue order: the LDS reads of the next step go out right behind the first MFMAs
			// of this one, so that their latency is covered by the 64-cycle matrix operations
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
			__builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
			__builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
			__builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
		}
	}

	// accumulator layout of the 32x32 block: register v of lane l holds
	// row 8*(v/4) + 4*(l/32) + v%4, column l%32.
	const bool split = out.splitStride != 0;
	float *C = out.C + (size_t)splitIndex * out.splitStride;
#pragma unroll
	for (int tm = 0; tm < TM; tm++) {
#pragma unroll
		for (int tn = 0; tn < TN; tn++) {
			const int j = j0 + waveN * Cfg::WN + tn * 32 + (lane & 31);
			if (j >= J) continue;
#pragma unroll
			for (int v = 0; v < 16; v++) {
				const int i = i0 + waveM * Cfg::WM + tm * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
				if (i >= I) continue;
				if (out.mirror && j < i) continue;
				float val = acc[tm][tn][v];
				float *dst = out.quadLd ? C + (size_t)(i >> 2) * out.quadLd + 4 * (size_t)j + (i & 3) : C + (size_t)i * out.ldc + j;
				if (!split) {
					val *= out.alpha;
					if (out.biasI) val += out.biasI[i];
					if (out.biasJ) val += out.biasJ[j];
					if (out.beta != 0.f) val += out.beta * *dst;
					if (out.mirror && j > i) C[(size_t)j * out.ldc + i] = val; // bias and beta are not used with mirror
				}
				*dst = val;
			}
		}
	}
}

template <class Cfg, class OpA, class OpB>
__global__ void __launch_bounds__(kGemmThreads)
mfma_gemm_kernel(const typename OpA::Params pa, const typename OpB::Params pb, const OutParams out, int I, int J, int R,
                 int kChunk)
{
	__shared__ float As[Cfg::BK * OpA::LD];
	__shared__ float Bs[Cfg::BK * OpB::LD];
	gemm_tile<Cfg, OpA, OpB>(pa, pb, out, I, J, R, kChunk, blockIdx.z, As, Bs);
}

// `batch` independent products of one shape in one launch: grid.z = batch * splits; problem b reads its operands
// aStride / bStride elements behind problem b-1's and writes cStride elements behind (plain operands only).
template <class Cfg, class OpA, class OpB>
__global__ void __launch_bounds__(kGemmThreads)
mfma_gemm_batched_kernel(typename OpA::Params pa, typename OpB::Params pb, OutParams out, int I, int J, int R, int kChunk,
                         int splits, long aStride, long bStride, long cStride)
{
	const int batch = blockIdx.z / splits, split = blockIdx.z - batch * splits;
	pa.p += (size_t)batch * aStride;
	pb.p += (size_t)batch * bStride;
	out.C += (size_t)batch * cStride;
	__shared__ float As[Cfg::BK * OpA::LD];
	__shared__ float Bs[Cfg::BK * OpB::LD];
	gemm_tile<Cfg, OpA, OpB>(pa, pb, out, I, J, R, kChunk, split, As, Bs);
}

// Two unsplit batched products of different operand kinds in one launch (products that do not depend on each other
// and would each leave most of the chip idle, or its last round of workgroups): blockIdx.z = which * batch + problem.
// The grid covers the larger tile count of the two; a workgroup outside its product's tiles leaves at once.
struct PairSide {
	PlainParams pa, pb;
	OutParams out;
	int I, J, R;
	int tilesI, tilesJ;
	long aStride, bStride, cStride;
};

template <class Cfg, class OpA1, class OpB1, class OpA2, class OpB2>
__global__ void __launch_bounds__(kGemmThreads)
mfma_gemm_pair_kernel(PairSide first, PairSide second, int batch)
{
	constexpr int LA = OpA1::LD > OpA2::LD ? OpA1::LD : OpA2::LD;
	constexpr int LB = OpB1::LD > OpB2::LD ? OpB1::LD : OpB2::LD;
	__shared__ float As[Cfg::BK * LA];
	__shared__ float Bs[Cfg::BK * LB];
	const bool isSecond = (int)blockIdx.z >= batch; // uniform over the workgroup
	const int problem = isSecond ? blockIdx.z - batch : blockIdx.z;
	if (!isSecond) {
		if ((int)blockIdx.y >= first.tilesI || (int)blockIdx.x >= first.tilesJ) return;
		first.pa.p += (size_t)problem * first.aStride;
		first.pb.p += (size_t)problem * first.bStride;
		first.out.C += (size_t)problem * first.cStride;
		const int kChunk = (first.R + Cfg::BK - 1) / Cfg::BK * Cfg::BK;
		gemm_tile<Cfg, OpA1, OpB1>(first.pa, first.pb, first.out, first.I, first.J, first.R, kChunk, 0, As, Bs);
	} else {
		if ((int)blockIdx.y >= second.tilesI || (int)blockIdx.x >= second.tilesJ) return;
		second.pa.p += (size_t)problem * second.aStride;
		second.pb.p += (size_t)problem * second.bStride;
		second.out.C += (size_t)problem * second.cStride;
		const int kChunk = (second.R + Cfg::BK - 1) / Cfg::BK * Cfg::BK;
		gemm_tile<Cfg, OpA2, OpB2>(second.pa, second.pb, second.out, second.I, second.J, second.R, kChunk, 0, As, Bs);
	}
}

// C[i*ldc + j] = alpha * sum_s ws[s][i][j] (+bias) + beta*C, partials summed in split order.
// VEC = 4: four consecutive j per thread with 16-byte reads (J % 4 == 0, aligned workspace).
template <int VEC>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *ws, int splits, int I, int J, OutParams out, long wsBatchStride = 0, long cBatchStride = 0)
{
	FITRE_RAISE_WAVE_PRIORITY();
	ws += (size_t)blockIdx.y * wsBatchStride; // blockIdx.y: problem of a batch (0 otherwise)
	out.C += (size_t)blockIdx.y * cBatchStride;
	const long total = (long)I * J;
	const long groups = total / VEC;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long gidx = (long)blockIdx.x * blockDim.x + threadIdx.x; gidx < groups; gidx += stride) {
		const long idx = gidx * VEC;
		const int i = (int)(idx / J), j = (int)(idx - (long)i * J);
		double acc[VEC];
#pragma unroll
		for (int v = 0; v < VEC; v++) acc[v] = 0.0;
		const float *p = ws + idx;
		int s = 0;
		for (; s + 4 <= splits; s += 4) { // four independent reads in flight
			float part[4][VEC];
#pragma unroll
			for (int u = 0; u < 4; u++) {
				if constexpr (VEC == 4) {
					float4 t = *reinterpret_cast<const float4 *>(p + (size_t)(s + u) * total);
					part[u][0] = t.x, part[u][1] = t.y, part[u][2] = t.z, part[u][3] = t.w;
				} else {
					part[u][0] = p[(size_t)(s + u) * total];
				}
			}
#pragma unroll
			for (int u = 0; u < 4; u++)
#pragma unroll
				for (int v = 0; v < VEC; v++) acc[v] += (double)part[u][v];
		}
		for (; s < splits; s++) {
			if constexpr (VEC == 4) {
				float4 t = *reinterpret_cast<const float4 *>(p + (size_t)s * total);
				acc[0] += (double)t.x, acc[1] += (double)t.y, acc[2] += (double)t.z, acc[3] += (double)t.w;
			} else {
				acc[0] += (double)p[(size_t)s * total];
			}
		}
#pragma unroll
		for (int v = 0; v < VEC; v++) {
			if (out.mirror && j + v < i) continue; // no partials below the diagonal
			float val = (float)acc[v] * out.alpha;
			if (out.biasI) val += out.biasI[i];
			if (out.biasJ) val += out.biasJ[j + v];
			float *dst = out.C + (size_t)i * out.ldc + j + v;
			if (out.beta != 0.f) val += out.beta * *dst;
			*dst = val;
			if (out.mirror && j + v > i) out.C[(size_t)(j + v) * out.ldc + i] = val;
		}
	}
}

// The same sum for a SMALL output with MANY partials (a weight gradient of a thin layer): a
// workgroup owns 16 output groups, its 16 phases each add every 16th partial, and the phases are
// combined in a fixed order -- the parallelism comes from the partials, not from the output.
template <int VEC>
__global__ void __launch_bounds__(256)
splitk_reduce_wide_kernel(const float *ws, int splits, int I, int J, OutParams out, long wsBatchStride = 0, long cBatchStride = 0)
{
	FITRE_RAISE_WAVE_PRIORITY();
	ws += (size_t)blockIdx.y * wsBatchStride;
	out.C += (size_t)blockIdx.y * cBatchStride;
	__shared__ double part[16][16 * VEC + 1];
	const long total = (long)I * J;
	const long groups = total / VEC;
	const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
	const long gidx = (long)blockIdx.x * 16 + tx;
	double acc[VEC];
#pragma unroll
	for (int v = 0; v < VEC; v++) acc[v] = 0.0;
	if (gidx < groups) {
		const float *p = ws + gidx * VEC;
		for (int s = ty; s < splits; s += 16) {
			if constexpr (VEC == 4) {
				float4 t = *reinterpret_cast<const float4 *>(p + (size_t)s * total);
				acc[0] += (double)t.x, acc[1] += (double)t.y, acc[2] += (double)t.z, acc[3] += (double)t.w;
			} else {
				acc[0] += (double)p[(size_t)s * total];
			}
		}
	}
#pragma unroll
	for (int v = 0; v < VEC; v++) part[ty][tx * VEC + v] = acc[v];
	__syncthreads();
	if (ty == 0 && gidx < groups) {
		const long idx = gidx * VEC;
		const int i = (int)(idx / J), j = (int)(idx - (long)i * J);
#pragma unroll
		for (int v = 0; v < VEC; v++) {
			if (out.mirror && j + v < i) continue;
			double sum = 0.0;
#pragma unroll
			for (int q = 0; q < 16; q++) sum += part[q][tx * VEC + v];
			float val = (float)sum * out.alpha;
			if (out.biasI) val += out.biasI[i];
			if (out.biasJ) val += out.biasJ[j + v];
			float *dst = out.C + (size_t)i * out.ldc + j + v;
			if (out.beta != 0.f) val += out.beta * *dst;
			*dst = val;
			if (out.mirror && j + v > i) out.C[(size_t)(j + v) * out.ldc + i] = val;
		}
	}
}

// Sums `splits` partial I x J matrices from ws into fin (alpha, beta and biases applied once).
static inline void launch_splitk_reduce(const float *ws, int splits, int I, int J, const OutParams &fin, int batch = 1,
                                        long wsBatchStride = 0, long cBatchStride = 0)
{
	LaunchScope scope(FITRE_KC_SPLITK_REDUCE, 4.0 * (double)I * J * (splits + 1) * batch);
	const bool vec = (J % 4 == 0) && ((((uintptr_t)ws) & 15) == 0) && (wsBatchStride % 4 == 0);
	const long groups = (long)I * J / (vec ? 4 : 1);
	const bool wide = splits >= 32 && groups <= 64 * 1024; // too few outputs to fill the chip one thread each
	if (wide) {
		const dim3 blocks((unsigned)((groups + 15) / 16), (unsigned)batch);
		if (vec) splitk_reduce_wide_kernel<4><<<blocks, 256, 0, stream()>>>(ws, splits, I, J, fin, wsBatchStride, cBatchStride);
		else splitk_reduce_wide_kernel<1><<<blocks, 256, 0, stream()>>>(ws, splits, I, J, fin, wsBatchStride, cBatchStride);
	} else {
		const dim3 blocks(blocks_for(groups, 256, 8192), (unsigned)batch);
		if (vec) splitk_reduce_kernel<4><<<blocks, 256, 0, stream()>>>(ws, splits, I, J, fin, wsBatchStride, cBatchStride);
		else splitk_reduce_kernel<1><<<blocks, 256, 0, stream()>>>(ws, splits, I, J, fin, wsBatchStride, cBatchStride);
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
	int bk;         // depth of a reduction slice (kGemmBK; kGemmDeepBK for small batched products)
	double estimateUs;
};

constexpr int kGemmBK = 16;
constexpr int kGemmDeepBK = 64;

// Estimated duration (microseconds) of a product cut into `splits` reduction ranges.
// Workgroups are spread evenly over the compute units; a compute unit runs up to three of
// them at once, and the more it holds the better the matrix pipes stay fed.  A split
// product pays for writing and re-reading its partial tiles.
inline double estimate_us(long tiles, int bm, int bn, long I, long J, long R, long splits, long cus, long *chunkOut,
                          long *splitsOut)
{
	long chunk = (R + splits - 1) / splits;
	chunk = ((chunk + kGemmBK - 1) / kGemmBK) * kGemmBK;
	long s = (R + chunk - 1) / chunk;
	long groups = tiles * s;
	// one k-step of a bm x bn tile keeps the four matrix pipes of a compute unit busy for this long
	double stepUs = (double)(bm / 32) * (bn / 32) * (kGemmBK / 2) * 64.0 / 4.0 / 2400.0;
	// Workgroups run in rounds of three per compute unit; a round that is not full leaves the pipes less well fed,
	// and one behind full rounds worse still (measured on symmetric products of order 1152 and 2304: 684 workgroups
	// beat 1197, which beat 855).
	const double perGroup = (double)(chunk / kGemmBK) * stepUs;
	const long full = groups / (3 * cus), rest = groups - full * 3 * cus;
	const long perCu = (rest + cus - 1) / cus;
	double t = (double)full * 3.0 * perGroup / 0.80 + 3.0;
	if (perCu >= 3) t += 3.0 * perGroup / 0.80;
	else if (perCu == 2) t += 2.0 * perGroup / 0.62;
	else if (perCu == 1) t += perGroup / (full > 0 ? 0.40 : 0.52);
	if (s > 1) t += 8.0 + (double)(s + 1) * (double)I * (double)J * 4.0 / 3.0e6; // second launch; ~3 TB/s, bytes -> us
	*chunkOut = chunk;
	*splitsOut = s;
	return t;
}

// mirror: a symmetric product (I == J) that only computes the tiles on and above the diagonal
// rows96: the row operand can feed a 96-row tile (operand_any_rows): used when it saves a quarter of a 128-row tile
inline GemmPlan plan_gemm_search(long I, long J, long R, bool mirror, long cus, bool rows96 = false)
{
	GemmPlan p;
	p.bm = (I <= 64) ? 64 : 128;
	p.bn = (J <= 64) ? 64 : 128;
	if (rows96 && !mirror && I > 64 && I <= 96 && p.bn == 128) p.bm = 96;
	long tiles = ((I + p.bm - 1) / p.bm) * ((J + p.bn - 1) / p.bn);
	if (mirror) {
		long t = (I + p.bm - 1) / p.bm;
		tiles = t * (t + 1) / 2;
	}
	long maxSplits = R / (2 * kGemmBK); // at least two slices per split
	if (maxSplits > 1024) maxSplits = 1024;
	if (maxSplits < 1) maxSplits = 1;
	double best = 1e30;
	long bestChunk = ((R + kGemmBK - 1) / kGemmBK) * kGemmBK, bestSplits = 1;
	for (long s = 1; s <= maxSplits; s++) {
		long chunk, eff;
		double t = estimate_us(tiles, p.bm, p.bn, I, J, R, s, cus, &chunk, &eff);
		if (t < best) {
			best = t;
			bestChunk = chunk;
			bestSplits = eff;
		}
	}
	p.splits = (int)bestSplits;
	p.kChunk = (int)bestChunk;
	p.wsBytes = (bestSplits > 1) ? (size_t)bestSplits * I * J * sizeof(float) : 0;
	p.bk = kGemmBK;
	p.estimateUs = best;
	return p;
}

// The search above walks up to 1024 split counts; a layer asks for the same plan on every call
// (and once more per workspace query), so the results are kept in a small table.  The plan is
// made for the compute units of the lane the product will be launched on.
inline GemmPlan plan_gemm(long I, long J, long R, bool mirror = false, int cus = 0, bool rows96 = false)
{
	struct Entry {
		long I, J, R;
		bool mirror;
		int cus;
		bool rows96;
		GemmPlan plan;
	};
	if (cus <= 0) cus = lane_compute_units();
	constexpr int kEntries = 128;
	static Entry table[kEntries];
	static int used = 0, next = 0;
	for (int i = 0; i < used; i++)
		if (table[i].I == I && table[i].J == J && table[i].R == R && table[i].mirror == mirror && table[i].cus == cus &&
		    table[i].rows96 == rows96)
			return table[i].plan;
	Entry e{ I, J, R, mirror, cus, rows96, plan_gemm_search(I, J, R, mirror, cus, rows96) };
	table[next] = e;
	next = (next + 1) % kEntries;
	if (used < kEntries) used++;
	return e.plan;
}

// Workspace that covers the plan of every lane (a size query does not know the lane of the launch).
inline size_t plan_gemm_workspace(long I, long J, long R, bool mirror = false, bool rows96 = false)
{
	size_t a = plan_gemm(I, J, R, mirror, device_compute_units(), rows96).wsBytes;
	size_t b = plan_gemm(I, J, R, mirror, lane_compute_units_min(), rows96).wsBytes;
	return a > b ? a : b;
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

template <template <int, int> class OpA, template <int, int> class OpB, int BM, int BN>
static int launch_tile(const typename OpA<BM, kGemmBK>::Params &pa, const typename OpB<BN, kGemmBK>::Params &pb,
                       const OutParams &out, int I, int J, int R, const GemmPlan &plan, void *ws, int kernelClass, double flops)
{
	typedef TileCfg<BM, BN, kGemmBK, (BM == 96 ? 1 : 2), (BM == 96 ? 4 : 2)> Cfg;
	constexpr int tileId = (BM == 96 ? 5 : (BM == 64 ? (BN == 64 ? 1 : 2) : (BN == 64 ? 3 : 4)));
	typedef OpA<BM, kGemmBK> A;
	typedef OpB<BN, kGemmBK> B;
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
		launch_splitk_reduce((const float *)ws, plan.splits, I, J, fin);
	} else {
		OutParams direct = out;
		direct.splitStride = 0;
		LaunchScope scope(kernelClass, flops, tileId);
		mfma_gemm_kernel<Cfg, A, B><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, direct, I, J, R, plan.kChunk);
	}
	return check_launch("mfma_gemm_kernel");
}

// Picks the tile instantiation the plan names.
template <template <int, int> class OpA, template <int, int> class OpB, class PA, class PB>
static int launch_gemm(const PA &pa, const PB &pb, const OutParams &out, int I, int J, int R, const GemmPlan &ideal, void *ws,
                       size_t wsBytes, int kernelClass, double flops)
{
	const GemmPlan plan = fit_plan(ideal, I, J, R, ws, wsBytes);
	if (plan.wsBytes > 0) {
		if (!ws || (((uintptr_t)ws) & 3)) return fail(FITRE_E_WORKSPACE, "split-K workspace is null or misaligned");
		if (wsBytes < plan.wsBytes)
			return fail(FITRE_E_WORKSPACE, "split-K workspace of %zu bytes is smaller than the %zu required", wsBytes, plan.wsBytes);
	}
	if (plan.bm == 96) {
		if constexpr (operand_any_rows<OpA<96, kGemmBK>>::value)
			return launch_tile<OpA, OpB, 96, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
		else
			return fail(FITRE_E_UNSUPPORTED, "a 96-row tile needs a reduction-contiguous row operand");
	}
	if (plan.bm == 128 && plan.bn == 128) return launch_tile<OpA, OpB, 128, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	if (plan.bm == 64 && plan.bn == 128) return launch_tile<OpA, OpB, 64, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	if (plan.bm == 128 && plan.bn == 64) return launch_tile<OpA, OpB, 128, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
	return launch_tile<OpA, OpB, 64, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops);
}

// A product whose output is a handful of tiles and whose reduction is short spends its time waiting for one global
// load per reduction slice: with slices of sixteen a 128 x 128 x 128 product lasts 8-12 us, split or not.  Such
// products run unsplit on 64 x 64 tiles with slices of sixty-four (four times fewer dependent loads, sixteen elements
// per thread and operand in flight).  `groups`: tiles of all problems of the launch.
inline bool deep_slice_plan(long I, long J, long R, bool mirror, int batch, long cus, const GemmPlan &standard, GemmPlan *deep)
{
	// one problem: up to 384 x 384 results; side by side, two or more problems bring enough 64 x 64 tiles for the chip up
	// to order 1280 (measured on halves of order 576 and 1152 of three matrices: 36 -> 22 us and 106 -> 85 us per product
	// with its reduction)
	const long limit = batch >= 2 ? 1280 : 384;
	if (I > limit || J > limit || R > (batch >= 2 ? 1280 : 1024)) return false;
	long ti = (I + 63) / 64, tj = (J + 63) / 64;
	long tiles = mirror ? ti * (ti + 1) / 2 : ti * tj;
	long rounds = (tiles * batch + 3 * cus - 1) / (3 * cus);
	long steps = (R + kGemmDeepBK - 1) / kGemmDeepBK;
	double estimate = (double)rounds * (double)steps * 1.6 + 3.0;
	if (estimate >= standard.estimateUs) return false;
	deep->bm = deep->bn = 64;
	deep->splits = 1;
	deep->kChunk = (int)(steps * kGemmDeepBK);
	deep->wsBytes = 0;
	deep->bk = kGemmDeepBK;
	deep->estimateUs = estimate;
	return true;
}

// ---- batched products of plain operands ------------------------------------------------------------------------
struct BatchStrides {
	int batch;
	long a, b, c; // elements between the operands / results of consecutive problems
	long ws;      // floats between their split-K workspaces
};

template <template <int, int> class OpA, template <int, int> class OpB, int BM, int BN, int BK = kGemmBK>
static int launch_tile_batched(const PlainParams &pa, const PlainParams &pb, const OutParams &out, int I, int J, int R,
                               const GemmPlan &plan, void *ws, int kernelClass, double flops, const BatchStrides &bs)
{
	typedef TileCfg<BM, BN, BK> Cfg;
	constexpr int tileId = (BM == 64 ? (BN == 64 ? 1 : 2) : (BN == 64 ? 3 : 4));
	typedef OpA<BM, BK> A;
	typedef OpB<BN, BK> B;
	dim3 grid((J + BN - 1) / BN, (I + BM - 1) / BM, plan.splits * bs.batch);
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "gemm grid %u x %u x %u too large", grid.x, grid.y, grid.z);
	if (plan.splits > 1) {
		OutParams part = out;
		part.C = (float *)ws;
		part.ldc = J;
		part.splitStride = (long)I * J;
		{
			LaunchScope scope(kernelClass, flops * bs.batch, tileId);
			mfma_gemm_batched_kernel<Cfg, A, B><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, part, I, J, R, plan.kChunk, plan.splits, bs.a,
			                                                                        bs.b, bs.ws);
		}
		OutParams fin = out;
		fin.splitStride = 0;
		launch_splitk_reduce((const float *)ws, plan.splits, I, J, fin, bs.batch, bs.ws, bs.c);
	} else {
		OutParams direct = out;
		direct.splitStride = 0;
		LaunchScope scope(kernelClass, flops * bs.batch, tileId);
		mfma_gemm_batched_kernel<Cfg, A, B><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, direct, I, J, R, plan.kChunk, 1, bs.a, bs.b, bs.c);
	}
	return check_launch("mfma_gemm_batched_kernel");
}

// wsBytes: the workspace of ONE problem (problem b's starts bs.ws floats behind problem b-1's)
template <template <int, int> class OpA, template <int, int> class OpB>
static int launch_gemm_batched(const PlainParams &pa, const PlainParams &pb, const OutParams &out, int I, int J, int R,
                               const GemmPlan &ideal, void *ws, size_t wsBytes, int kernelClass, double flops, const BatchStrides &bs)
{
	const GemmPlan plan = fit_plan(ideal, I, J, R, ws, wsBytes);
	if (plan.wsBytes > 0) {
		if (!ws || (((uintptr_t)ws) & 3)) return fail(FITRE_E_WORKSPACE, "split-K workspace is null or misaligned");
		if (wsBytes < plan.wsBytes)
			return fail(FITRE_E_WORKSPACE, "split-K workspace of %zu bytes is smaller than the %zu required", wsBytes, plan.wsBytes);
	}
	if (plan.bk == kGemmDeepBK) return launch_tile_batched<OpA, OpB, 64, 64, kGemmDeepBK>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, bs);
	if (plan.bm == 128 && plan.bn == 128)
		return launch_tile_batched<OpA, OpB, 128, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, bs);
	if (plan.bm == 64 && plan.bn == 128) return launch_tile_batched<OpA, OpB, 64, 128>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, bs);
	if (plan.bm == 128 && plan.bn == 64) return launch_tile_batched<OpA, OpB, 128, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, bs);
	return launch_tile_batched<OpA, OpB, 64, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, bs);
}

} // namespace fitre
