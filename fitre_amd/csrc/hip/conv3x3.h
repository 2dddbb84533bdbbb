// 3x3 / stride 1 / pad 1 convolutions on the fp32 MFMA pipes, written around the
// one property the general tile engine cannot use: the nine taps of a window read
// the SAME image data, only shifted.
//
// Forward and input gradient ("position-contiguous" products):
//     out[i][m] = sum_{c, ta, tb} Wsel(i, c, ta, tb) * src[c][m + (ta-1)*B + (tb-1)]      (zero outside the image)
//   i = output channel of the product, c = reduction channel, m = (n, a, b) flat position.
//   A workgroup owns 128 channels x 128 positions.  The reduction runs in blocks of CB
//   channels: the block's raw source window (128 positions plus B+1 cells on either
//   side, per channel) and the block's 9*CB weights per output channel are staged in LDS
//   ONCE, with wide contiguous global loads, and then feed 9*CB/2 MFMA steps: for every tap
//   the B fragment is the same LDS window read at a shifted address, zeroed at the image
//   border by AND-ing with a per-lane bit mask.  Per MFMA this needs ~6x fewer global load
//   instructions and almost no address arithmetic compared with gathering every
//   (channel, tap) slice separately, and a barrier pair every 18*CB MFMAs per wave.
//
// Weight gradient ("reduction over positions"):
//     dW[o][c][ta][tb] = sum_m delta[o][m] * src[c][m + (ta-1)*B + (tb-1)]
//   A workgroup of twelve waves owns 128 output channels x 32 input channels x all nine taps:
//   each wave keeps three 32x32 accumulator blocks (the taps of one window row).  A stage brings
//   64 positions of delta (128 rows) and of the source (32 rows, plus the halo) into LDS; every
//   MFMA step then reads one delta fragment and three shifted source fragments.
//
// The code avoids everything the compiler turns into control flow, private memory or vector
// arithmetic in the hot loops: no conditional loads or stores (invalid cells go to an
// out-of-range buffer offset, resp. a dummy LDS word), image borders as zero words in the LDS
// layout instead of per-element tests, per-thread staging offsets computed once, staging
// registers as plain float arrays filled by unrolled loops.
#pragma once
#include "gemm_engine.h"

namespace fitre {

constexpr int kC3Tile = 128; // positions (and output channels) per workgroup tile

struct Conv3x3Params {
	const float *src;   // [Cred][N][A][B]
	const float *w;     // [Cout][Cin][3][3]
	// A sum of two products of one shape in one launch (the R operator's conv(z, V) + conv(R{z}, W) and its like): the
	// reduction runs over the first pair (src, w) and then over the second; for the weight gradient `w2` is the second
	// delta.  Null for a single product.
	const float *src2, *w2;
	uint32_t srcBytes, wBytes;
	int I;              // output channels of this product
	int cred;           // reduction channels of ONE pair
	int J;              // positions N*A*B
	int A, B;
	int perSplit;       // channel blocks (position-contiguous) or position stages (weight gradient) per split
	FastDiv divB, divA; // position -> (n, a, b)
};

// Index of flat position m = (n, a, b) in the zero-padded layout: every image row is followed by
// one zero cell and every image by one zero row, so that a window tap that leaves the image on
// any side lands on a zero:  (n*(A+1) + a)*(B+1) + b.  `m` is taken one image late (callers add
// 2*A*B) so that positions a little before the tensor map consistently too.
__device__ __forceinline__ uint32_t padded_index(const Conv3x3Params &p, uint32_t m)
{
	uint32_t q, b, n, a;
	p.divB.divmod(m, q, b);
	p.divA.divmod(q, n, a);
	return (n * (uint32_t)(p.A + 1) + a) * (uint32_t)(p.B + 1) + b;
}

// offset that marks a 16-byte group as out of range for all four of its words
constexpr uint32_t kGroupOutOfRange = 0xFFFFFFF0u;

// ---------------------------------------------------------------------------------
// position-contiguous product (forward: DX = false, input gradient: DX = true)
// CB reduction channels per block; MAXB = widest image row the window is sized for.
//
// The source window of a block sits in LDS in the zero-padded layout above, so the B fragment
// of tap (ta, tb) is the lane's own cell address plus (ta-1)*(B+1) + (tb-1): no border test in
// the MFMA loop.  Which LDS word a staged cell goes to, which global offsets a thread loads and
// where they are stored do not depend on the channel block: all of it is computed once, and a
// block only moves the (uniform) base of the buffer resources.
// ---------------------------------------------------------------------------------
// IT = channel rows per workgroup tile (128, or 64 for products with at most 64 output channels).
template <int CB, bool DX, int MAXB, int IT>
struct C3Pos {
	static constexpr int TM = IT / 64, TN = 2;
	// weights in LDS.  forward: IT rows (output channel) x CB*9, odd row stride.
	// input gradient: CB rows (reduction channel) x IT*9 weights of the tile's channels.
	static constexpr int A_LD = DX ? (IT * 9 + 4) : (CB * 9 + 1);
	static constexpr int A_FLOATS = DX ? CB * A_LD : IT * A_LD;
	static constexpr int WQ = DX ? (IT * 9 / 4) : (CB * 9 / 4); // 4-float groups per LDS row
	static constexpr int WROWS = DX ? CB : IT;
	static constexpr int WGROUPS = WROWS * WQ;
	static constexpr int WE = (WGROUPS + kGemmThreads - 1) / kGemmThreads; // groups per thread
	static constexpr int A_DUMMY = A_FLOATS;                               // four spare words for threads without a group
	// flat cells staged per channel: 128 positions plus B+1 on either side
	static constexpr int CELLS_MAX = kC3Tile + 2 * (MAXB + 1);
	// the same cells in the padded layout (the host checks that the shape fits)
	static constexpr int PAD_MAX = MAXB <= 32 ? 384 : 512;
	static constexpr int WIN_LD = PAD_MAX + 1; // odd channel stride
	static constexpr int B_FLOATS = CB * WIN_LD + 1;
	static constexpr int B_DUMMY = CB * WIN_LD;
	// window staging: each wave owns CB/4 channels, lanes walk the cells 64 at a time
	static constexpr int CH_PER_WAVE = CB / 4;
	static constexpr int XI = (CELLS_MAX + 63) / 64;
	static constexpr int SE = CH_PER_WAVE * XI;
	static_assert(CB % 4 == 0, "CB must be a multiple of the wave count");
};

// words of the padded window a tile needs: what lies before the tile's first position
// (B+1 cells, at most two row ends and two image ends) ...
__host__ __device__ inline int c3_pad_before(int B) { return 3 * (B + 1) + 2; }
// ... plus 128 + B+1 positions forward with every row end and image end they can cross
inline int c3_pad_window(int A, int B)
{
	const int span = kC3Tile - 1 + B + 1;
	const int rowEnds = (span + B - 1) / B, imageEnds = (span + A * B - 1) / (A * B);
	return c3_pad_before(B) + span + rowEnds + imageEnds * (B + 1) + 2;
}

template <int CB, bool DX, bool VECW, int MAXB, int IT>
__global__ void __launch_bounds__(kGemmThreads)
conv3x3_pos_kernel(const Conv3x3Params p, const OutParams out)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	typedef C3Pos<CB, DX, MAXB, IT> K;
	constexpr int TM = K::TM, TN = K::TN;
	__shared__ __attribute__((aligned(16))) float As[K::A_FLOATS + 4];
	__shared__ float Bs[K::B_FLOATS];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int i0 = blockIdx.y * IT, j0 = blockIdx.x * kC3Tile;
	const int halo = p.B + 1;
	const int win = kC3Tile + 2 * halo;
	const int plane = p.J; // floats per channel of src
	const int cbHalf = p.cred / CB;                      // channel blocks of one (src, w) pair
	const int cbTotal = p.src2 ? 2 * cbHalf : cbHalf;
	const int cbBeg = blockIdx.z * p.perSplit;
	const int cbEnd = (cbBeg + p.perSplit < cbTotal) ? cbBeg + p.perSplit : cbTotal;
	const int rowLen = DX ? p.I * 9 : p.cred * 9;
	const uint32_t late = (uint32_t)(2 * p.A * p.B);              // see padded_index; covers the B+1 cells before position 0
	const uint32_t ref = padded_index(p, (uint32_t)j0 + late);    // the tile's first position
	const int before = c3_pad_before(p.B);

	// the padded window starts out all zero; staging only ever writes the cells of real positions
	for (int i = tid; i < K::B_FLOATS; i += kGemmThreads) Bs[i] = 0.f;

	// ---- what this thread stages, the same for every channel block -------------------------
	// weights: 16-byte groups idx = tid + 256*e of the block's WROWS x WQ group matrix
	uint32_t wOff[K::WE]; // byte offset inside the block's weights
	int wLds[K::WE];
#pragma unroll
	for (int e = 0; e < K::WE; e++) {
		const int idx = tid + kGemmThreads * e;
		const int row = idx / K::WQ, qd = idx - row * K::WQ;
		const bool has = idx < K::WGROUPS;
		// forward: row = output channel, w[(i0+row)*cred*9 + c0*9 + 4*qd ..]
		// input gradient: row = reduction channel, w[(c0+row)*I*9 + i0*9 + 4*qd ..]
		// Rows or columns past the tensor's extent only feed accumulator rows that are never stored:
		// they may read any valid address (vector loads) or be answered with zero (buffer loads).
		const int rowG = DX ? row : (i0 + row);
		const int colG = DX ? (i0 * 9 + 4 * qd) : (4 * qd);
		const bool inside = has & (DX ? (colG + 3 < rowLen) : (rowG < p.I));
		const uint32_t off = 4u * (uint32_t)(rowG * rowLen + colG);
		wOff[e] = VECW ? (inside ? off : 0u) : (has ? off : kGroupOutOfRange);
		wLds[e] = has ? row * K::A_LD + 4 * qd : K::A_DUMMY;
	}
	// window cells x = lane + 64*xi of CH_PER_WAVE channels
	uint32_t sOff[K::SE]; // byte offset inside the block's channels
	int sLds[K::SE];
#pragma unroll
	for (int e = 0; e < K::SE; e++) {
		const int c = wave * K::CH_PER_WAVE + e / K::XI, x = lane + 64 * (e % K::XI);
		const int m = j0 - halo + x; // flat position inside the channel plane
		const bool has = x < win;
		const bool inside = has & (m >= 0) & (m < plane);
		sOff[e] = inside ? 4u * (uint32_t)(c * plane + m) : kOutOfRange;
		const int cell = (int)(padded_index(p, (uint32_t)m + late) - ref) + before;
		sLds[e] = has ? c * K::WIN_LD + cell : K::B_DUMMY;
	}

	float wreg[K::WE * 4];
	float sreg[K::SE];

	v16f acc[TM][TN];
#pragma unroll
	for (int tm = 0; tm < TM; tm++)
#pragma unroll
		for (int tn = 0; tn < TN; tn++)
#pragma unroll
			for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.f;

	// fragment base addresses; the channel pair, the tap column and (A side) the tap are
	// compile-time offsets from these
	const int rowA = (wave >> 1) * (IT / 2) + l32; // channel row inside the tile (+32 for tm = 1)
	const float *aBase = DX ? (As + khalf * K::A_LD + rowA * 9) : (As + rowA * K::A_LD + khalf * 9);
	constexpr int aTmStep = DX ? 32 * 9 : 32 * K::A_LD;
	constexpr int aCpStep = DX ? 2 * K::A_LD : 18;
	const float *bRow[TN][3]; // per tap row: the lane's cell one row up / same row / one row down, one column left
#pragma unroll
	for (int tn = 0; tn < TN; tn++) {
		const uint32_t m = (uint32_t)(j0 + (wave & 1) * 64 + tn * 32 + l32);
		const int cell = (int)(padded_index(p, m + late) - ref) + before;
#pragma unroll
		for (int r = 0; r < 3; r++) bRow[tn][r] = Bs + khalf * K::WIN_LD + cell + (r - 1) * (p.B + 1) - 1;
	}

// global -> registers for channel block CBI (a macro: the register arrays must stay registers)
#define C3_LOAD_BLOCK(CBI)                                                                                            \
	{                                                                                                                 \
		const bool second_ = (CBI) >= cbHalf; /* uniform: the block belongs to the second pair */                    \
		const int c0_ = ((CBI) - (second_ ? cbHalf : 0)) * CB;                                                        \
		const float *wSel = second_ ? p.w2 : p.w, *sSel = second_ ? p.src2 : p.src;                                   \
		const size_t wShift = DX ? (size_t)c0_ * rowLen : (size_t)c0_ * 9; /* floats, uniform */                      \
		if constexpr (VECW) {                                                                                         \
			const char *wBlk = reinterpret_cast<const char *>(wSel + wShift);                                         \
			_Pragma("unroll") for (int e = 0; e < K::WE; e++)                                                         \
			{                                                                                                         \
				const float4 v4 = *reinterpret_cast<const float4 *>(wBlk + wOff[e]);                                  \
				wreg[4 * e + 0] = v4.x, wreg[4 * e + 1] = v4.y, wreg[4 * e + 2] = v4.z, wreg[4 * e + 3] = v4.w;       \
			}                                                                                                         \
		} else {                                                                                                      \
			const __amdgpu_buffer_rsrc_t wRs = make_rsrc(wSel + wShift, p.wBytes - (uint32_t)(4 * wShift));           \
			_Pragma("unroll") for (int e = 0; e < K::WE; e++)                                                         \
			{                                                                                                         \
				wreg[4 * e + 0] = buffer_load(wRs, wOff[e]);                                                          \
				wreg[4 * e + 1] = buffer_load(wRs, wOff[e] + 4u);                                                     \
				wreg[4 * e + 2] = buffer_load(wRs, wOff[e] + 8u);                                                     \
				wreg[4 * e + 3] = buffer_load(wRs, wOff[e] + 12u);                                                    \
			}                                                                                                         \
		}                                                                                                             \
		const size_t sShift = (size_t)c0_ * plane;                                                                    \
		const __amdgpu_buffer_rsrc_t sRs = make_rsrc(sSel + sShift, p.srcBytes - (uint32_t)(4 * sShift));            \
		_Pragma("unroll") for (int e = 0; e < K::SE; e++) sreg[e] = buffer_load(sRs, sOff[e]);                        \
	}

	if (cbBeg < cbEnd) C3_LOAD_BLOCK(cbBeg);

	for (int cb = cbBeg; cb < cbEnd; cb++) {
		__syncthreads();
#pragma unroll
		for (int e = 0; e < K::WE; e++) {
			float *dst = As + wLds[e];
			if constexpr (DX) { // A_LD is a multiple of four
				*reinterpret_cast<float4 *>(dst) = make_float4(wreg[4 * e], wreg[4 * e + 1], wreg[4 * e + 2], wreg[4 * e + 3]);
			} else {
				dst[0] = wreg[4 * e], dst[1] = wreg[4 * e + 1], dst[2] = wreg[4 * e + 2], dst[3] = wreg[4 * e + 3];
			}
		}
#pragma unroll
		for (int e = 0; e < K::SE; e++) Bs[sLds[e]] = sreg[e];
		__syncthreads();
		if (cb + 1 < cbEnd) C3_LOAD_BLOCK(cb + 1);

		// 9 * CB/2 MFMA steps, step = (tap, channel pair); the fragments of step+1 are read
		// from LDS while the MFMAs of the current step run
		constexpr int STEPS = 9 * (CB / 2);
		float a[2][TM], b[2][TN];
#pragma unroll
		for (int tm = 0; tm < TM; tm++) a[0][tm] = aBase[tm * aTmStep + (DX ? 8 : 0)];
#pragma unroll
		for (int tn = 0; tn < TN; tn++) b[0][tn] = bRow[tn][0][0];
#pragma unroll
		for (int step = 0; step < STEPS; step++) {
			const int cur = step & 1, nxt = cur ^ 1;
			if (step + 1 < STEPS) {
				const int tapN = (step + 1) / (CB / 2), cpN = (step + 1) % (CB / 2);
				const int aTapN = DX ? (8 - tapN) : tapN;
#pragma unroll
				for (int tm = 0; tm < TM; tm++) a[nxt][tm] = aBase[tm * aTmStep + cpN * aCpStep + aTapN];
#pragma unroll
				for (int tn = 0; tn < TN; tn++) b[nxt][tn] = bRow[tn][tapN / 3][cpN * 2 * K::WIN_LD + tapN % 3];
			}
#pragma unroll
			for (int tm = 0; tm < TM; tm++)
#pragma unroll
				for (int tn = 0; tn < TN; tn++)
					acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][tm], b[cur][tn], acc[tm][tn], 0, 0, 0);
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       // first MFMA
			__builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0); // LDS reads of the next step
			__builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);
		}
	}
#undef C3_LOAD_BLOCK

	// ---- store (accumulator layout as in mfma_gemm_kernel) ---------------------------------
	const bool split = out.splitStride != 0;
	float *C = out.C + (size_t)blockIdx.z * out.splitStride;
#pragma unroll
	for (int tm = 0; tm < TM; tm++) {
#pragma unroll
		for (int tn = 0; tn < TN; tn++) {
			const int j = j0 + (wave & 1) * 64 + tn * 32 + l32;
			if (j >= p.J) continue;
#pragma unroll
			for (int v = 0; v < 16; v++) {
				const int i = i0 + (wave >> 1) * (IT / 2) + tm * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
				if (i >= p.I) continue;
				float val = acc[tm][tn][v];
				if (!split && out.biasI) val += out.biasI[i];
				C[(size_t)i * out.ldc + j] = val;
			}
		}
	}
}

// ---------------------------------------------------------------------------------
// weight gradient
// ---------------------------------------------------------------------------------
constexpr int kC3DwThreads = 768;          // 12 waves: (output-channel block 0..3) x (tap row 0..2)
constexpr int kC3Stage = 64;               // positions per LDS stage
constexpr int kC3DwCin = 32;               // input channels per workgroup
constexpr int kC3DeltaLd = kC3Stage + 1;   // odd row stride of the delta stage

// One workgroup per compute unit: 128 output channels x 32 input channels x 9 taps, i.e. 36
// accumulator blocks of 32x32, three per wave (the three taps of one window row).  Twelve waves
// keep three wavefronts on every SIMD while the accumulators of the whole chip -- the volume a
// split reduction has to write out and sum again -- stay at half of what two four-wave
// workgroups per compute unit would hold.  LDS stages are double buffered: one barrier per
// stage, and the next stage is written half way through the current one.
//
// Border handling costs two vector instructions per MFMA step:
//   * the source stage keeps every image row followed by one zero word ("row pads"), so the
//     taps one column left / right of the row ends read zeros; the word of flat window cell r
//     is r + (bs + r) / B with bs = column of the window's first cell;
//   * taps one row up / down are invalid on the first / last row of an image; that depends on
//     the position only, i.e. on the reduction index, so the mask is applied to the delta
//     fragment (one AND per step) with a per-position mask table;
//   * the padded word of a position comes from a second table (one add per step).
// Requires positions % 64 == 0 (no partial stage).
// MAXB: widest image row this instantiation's source window holds: 16 (for 2 <= B <= 16) or 32
template <bool VECD, int MAXB>
__global__ void __launch_bounds__(kC3DwThreads)
conv3x3_dw_kernel(const Conv3x3Params p, const float *delta, uint32_t deltaBytes, const OutParams out)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	constexpr int T = kC3DwThreads;
	constexpr int CELLS_MAX = kC3Stage + 2 * (MAXB + 1);               // flat window cells per channel
	constexpr int XP_MAX = CELLS_MAX + (CELLS_MAX + MAXB - 2) / MAXB + 1; // with row pads (largest at B = MAXB)
	constexpr int XP_LD = XP_MAX + 1 - (XP_MAX & 1);                    // odd row stride
	constexpr int X_DUMMY = kC3DwCin * XP_LD;                           // swallows stores that have no target
	constexpr int D_DUMMY = kC3Tile * kC3DeltaLd;
	constexpr int DGROUPS = kC3Tile * kC3Stage / 4;                     // 4-float groups of delta per stage
	constexpr int DE = (DGROUPS + T - 1) / T;
	// source window staging: a thread keeps ONE cell of the window and takes it from XCP channels apart
	// in every pass, so where a cell comes from and where it goes differ between passes by constants
	// only (few live registers: this kernel leaves room for a bandwidth kernel's waves beside its own)
	constexpr int XG = (MAXB == 16) ? 128 : 192; // threads per channel in a pass (>= cells of the window)
	constexpr int XCP = T / XG;                  // channels per pass
	constexpr int XE = (kC3DwCin + XCP - 1) / XCP;
	static_assert(XG >= CELLS_MAX && T % XG == 0, "one thread per window cell");
	static_assert(T % (kC3Stage / 4) == 0, "a thread keeps its column group in every round");
	static_assert(MAXB == 16 || MAXB == 32, "row-pad bound: taken at B = MAXB it covers 2 <= B <= 16 resp. 1 <= B <= 32");
	__shared__ float Ds[2][D_DUMMY + 4];
	__shared__ float Xs[2][X_DUMMY + 1];
	__shared__ int Pk[2][kC3Stage];          // padded word of position k of the stage
	__shared__ uint32_t Mk[2][3][kC3Stage];  // per tap row: all ones where the tap row is inside the image

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int ob = wave & 3, ta = wave >> 2; // output-channel block, tap row
	// Workgroups are dealt to the eight XCDs (each with its own L2) round-robin by launch index.
	// Renumber them so that an XCD holds consecutive indices, input-channel tile fastest and split
	// slowest: the workgroups that read the same range of positions -- the same delta rows and the
	// same input rows -- then share an L2 instead of fetching them once per XCD.
	int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
	{
		const unsigned groups = gridDim.x * gridDim.y * gridDim.z;
		const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
		// XCD x receives launch indices x, x + 8, ...: groups / 8 of them, one more on the first groups % 8
		const unsigned xcd = lin & 7u, each = groups >> 3, extra = groups & 7u;
		const unsigned logical = xcd * each + (xcd < extra ? xcd : extra) + (lin >> 3);
		const unsigned tiles = gridDim.x * gridDim.y;
		bz = (int)(logical / tiles);
		const unsigned rem = logical - (unsigned)bz * tiles;
		by = (int)(rem / gridDim.x);
		bx = (int)(rem - (unsigned)by * gridDim.x);
	}
	const int c0 = bx * kC3DwCin, o0 = by * kC3Tile;
	const int halo = p.B + 1;
	const int win = kC3Stage + 2 * halo;
	const int plane = p.J;
	const int stagesHalf = p.J / kC3Stage;                       // stages of one (src, delta) pair
	const int stagesTotal = p.src2 ? 2 * stagesHalf : stagesHalf; // a second pair continues the reduction
	const int stBeg = bz * p.perSplit;
	const int stEnd = (stBeg + p.perSplit < stagesTotal) ? stBeg + p.perSplit : stagesTotal;
	const bool movingRows = (kC3Stage % p.B) != 0; // else every stage window starts in the same column

	// the row pads must read as zero: with fixed rows they are never written after this
	for (int i = tid; i < 2 * (X_DUMMY + 1); i += T) (&Xs[0][0])[i] = 0.f;

	// ---- what this thread stages ------------------------------------------------------------
	const int dCol = 4 * (tid % (kC3Stage / 4)); // first position of its delta groups inside the stage
	uint32_t dOff[DE];                           // byte offset of the group at stage 0
	int dLds[DE];
#pragma unroll
	for (int e = 0; e < DE; e++) {
		const int idx = tid + T * e;
		const int row = idx / (kC3Stage / 4);
		const bool has = idx < DGROUPS;
		const bool inside = has & ((o0 + row) < p.I);
		// rows past the tensor feed accumulator rows that are never stored
		const uint32_t off = 4u * (uint32_t)((o0 + row) * plane + dCol);
		dOff[e] = VECD ? (inside ? off : 4u * (uint32_t)dCol) : (inside ? off : kGroupOutOfRange);
		dLds[e] = has ? row * kC3DeltaLd + dCol : D_DUMMY;
	}
	const int xr = tid % XG, xcg = tid / XG; // the thread's window cell (first cell = stage start - halo) and first channel
	const bool xHas = xr < win;
	float dreg[DE * 4];
	float xreg[XE];
	int xWord = X_DUMMY; // LDS word of the cell in channel xcg; bit 31: the cell ends an image row (the next word is a row pad)
	int pkReg = 0;
	uint32_t mkReg0 = 0, mkReg2 = 0;

// global -> registers for stage ST, and where its cells go in LDS
#define C3_LOAD_STAGE(ST)                                                                                             \
	{                                                                                                                 \
		const bool second_ = (ST) >= stagesHalf; /* uniform: the stage belongs to the second pair */                 \
		const int m0_ = ((ST) - (second_ ? stagesHalf : 0)) * kC3Stage;                                               \
		const float *dSel = second_ ? p.w2 : delta;                                                                   \
		const __amdgpu_buffer_rsrc_t xRs = second_ ? srcRs2 : srcRs;                                                  \
		if constexpr (VECD) {                                                                                         \
			const char *dBlk = reinterpret_cast<const char *>(dSel + m0_);                                            \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				const float4 v4 = *reinterpret_cast<const float4 *>(dBlk + dOff[e]);                                  \
				dreg[4 * e + 0] = v4.x, dreg[4 * e + 1] = v4.y, dreg[4 * e + 2] = v4.z, dreg[4 * e + 3] = v4.w;       \
			}                                                                                                         \
		} else {                                                                                                      \
			const __amdgpu_buffer_rsrc_t dRs = make_rsrc(dSel + m0_, deltaBytes - 4u * (uint32_t)m0_);                \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				dreg[4 * e + 0] = buffer_load(dRs, dOff[e]);                                                          \
				dreg[4 * e + 1] = buffer_load(dRs, dOff[e] + 4u);                                                     \
				dreg[4 * e + 2] = buffer_load(dRs, dOff[e] + 8u);                                                     \
				dreg[4 * e + 3] = buffer_load(dRs, dOff[e] + 12u);                                                    \
			}                                                                                                         \
		}                                                                                                             \
		/* column of the window's first cell; the bias keeps the dividend non-negative */                             \
		const uint32_t bs_ = (uint32_t)(m0_ + halo * (p.B - 1)) - p.divB.quot((uint32_t)(m0_ + halo * (p.B - 1))) * (uint32_t)p.B; \
		{                                                                                                             \
			const int m = m0_ - halo + xr;                                                                            \
			const bool okm = xHas & ((unsigned)m < (unsigned)plane);                                                  \
			_Pragma("unroll") for (int e = 0; e < XE; e++)                                                            \
			{                                                                                                         \
				const int c = xcg + XCP * e;                                                                          \
				const bool ok = okm & (c < kC3DwCin) & ((c0 + c) < p.cred);                                           \
				xreg[e] = buffer_load(xRs, ok ? 4u * (uint32_t)((c0 + c) * plane + m) : kOutOfRange);                 \
			}                                                                                                         \
			if (movingRows | ((ST) == stBeg)) {                                                                       \
				uint32_t q_, b_;                                                                                      \
				p.divB.divmod(bs_ + (uint32_t)xr, q_, b_);                                                            \
				const int word = xcg * XP_LD + xr + (int)q_;                                                          \
				const int end = (b_ == (uint32_t)(p.B - 1)) ? (int)0x80000000 : 0;                                    \
				xWord = xHas ? (word | end) : X_DUMMY;                                                                \
			}                                                                                                         \
		}                                                                                                             \
		if (tid < kC3Stage) {                                                                                         \
			uint32_t q_, b_, n_, a_;                                                                                  \
			p.divB.divmod((uint32_t)(m0_ + tid), q_, b_);                                                             \
			p.divA.divmod(q_, n_, a_);                                                                                \
			pkReg = halo + tid + (int)p.divB.quot(bs_ + (uint32_t)(halo + tid));                                      \
			mkReg0 = (a_ != 0u) ? 0xFFFFFFFFu : 0u;                                                                   \
			mkReg2 = (a_ != (uint32_t)(p.A - 1)) ? 0xFFFFFFFFu : 0u;                                                  \
		}                                                                                                             \
	}

#define C3_STORE_STAGE(BUF)                                                                                           \
	{                                                                                                                 \
		_Pragma("unroll") for (int e = 0; e < DE; e++)                                                                \
		{                                                                                                             \
			float *dst = Ds[BUF] + dLds[e];                                                                           \
			dst[0] = dreg[4 * e], dst[1] = dreg[4 * e + 1], dst[2] = dreg[4 * e + 2], dst[3] = dreg[4 * e + 3];       \
		}                                                                                                             \
		_Pragma("unroll") for (int e = 0; e < XE; e++)                                                                \
		{                                                                                                             \
			const bool has = xHas & ((xcg + XCP * e) < kC3DwCin);                                                     \
			Xs[BUF][has ? (xWord & 0x7FFFFFFF) + e * XCP * XP_LD : X_DUMMY] = xreg[e];                                \
		}                                                                                                             \
		if (movingRows) { /* the row pads move with the stage: rewrite them */                                        \
			_Pragma("unroll") for (int e = 0; e < XE; e++)                                                            \
			{                                                                                                         \
				const bool has = (xWord < 0) & ((xcg + XCP * e) < kC3DwCin);                                          \
				Xs[BUF][has ? (xWord & 0x7FFFFFFF) + e * XCP * XP_LD + 1 : X_DUMMY] = 0.f;                            \
			}                                                                                                         \
		}                                                                                                             \
		if (tid < kC3Stage) {                                                                                         \
			Pk[BUF][tid] = pkReg;                                                                                     \
			Mk[BUF][0][tid] = mkReg0;                                                                                 \
			Mk[BUF][1][tid] = 0xFFFFFFFFu;                                                                            \
			Mk[BUF][2][tid] = mkReg2;                                                                                 \
		}                                                                                                             \
	}

	const __amdgpu_buffer_rsrc_t srcRs = make_rsrc(p.src, p.srcBytes);
	const __amdgpu_buffer_rsrc_t srcRs2 = make_rsrc(p.src2 ? p.src2 : p.src, p.srcBytes);

	v16f acc[3];
#pragma unroll
	for (int t = 0; t < 3; t++)
#pragma unroll
		for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

	const int aOff = (ob * 32 + l32) * kC3DeltaLd + khalf;
	const int bOff = l32 * XP_LD + (ta - 1) * (p.B + 1) - 1; // tap (ta, 0) relative to the position's word; +1, +2 for the other two

	__syncthreads(); // the zero fill above
	if (stBeg < stEnd) {
		C3_LOAD_STAGE(stBeg);
		C3_STORE_STAGE(0);
	}
	__syncthreads();
	for (int st = stBeg; st < stEnd; st++) {
		const int buf = (st - stBeg) & 1;
		const bool more = st + 1 < stEnd;
		if (more) C3_LOAD_STAGE(st + 1);

		// 32 MFMA steps of two positions.  Tables are read two steps ahead, fragments one step ahead.
		const float *aBase = Ds[buf] + aOff;
		const float *bBase = Xs[buf] + bOff;
		const int *pBase = Pk[buf] + khalf;
		const uint32_t *mBase = Mk[buf][ta] + khalf;
		constexpr int STEPS = kC3Stage / 2;
		int tp[3];
		uint32_t tm[3];
		float fa[2], fb[2][3];
		tp[0] = pBase[0], tm[0] = mBase[0];
		tp[1] = pBase[2], tm[1] = mBase[2];
		fa[0] = aBase[0];
#pragma unroll
		for (int tb = 0; tb < 3; tb++) fb[0][tb] = bBase[tp[0] + tb];
#pragma unroll
		for (int s = 0; s < STEPS; s++) {
			const int cur = s & 1, nxt = cur ^ 1;
			if (s + 2 < STEPS) {
				tp[(s + 2) % 3] = pBase[2 * (s + 2)];
				tm[(s + 2) % 3] = mBase[2 * (s + 2)];
			}
			if (s + 1 < STEPS) {
				const float *q = bBase + tp[(s + 1) % 3];
				fa[nxt] = aBase[2 * (s + 1)];
#pragma unroll
				for (int tb = 0; tb < 3; tb++) fb[nxt][tb] = q[tb];
			}
			const float am = __int_as_float(__float_as_int(fa[cur]) & (int)tm[s % 3]);
#pragma unroll
			for (int tb = 0; tb < 3; tb++) acc[tb] = __builtin_amdgcn_mfma_f32_32x32x2f32(am, fb[cur][tb], acc[tb], 0, 0, 0);
			__builtin_amdgcn_sched_group_barrier(0x002, 2, 0); // the mask and the next address
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
			__builtin_amdgcn_sched_group_barrier(0x100, 6, 0); // LDS reads for the next two steps
			__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
			if (s == STEPS / 2 && more) C3_STORE_STAGE(buf ^ 1); // the other buffer was released by the last barrier
		}
		__syncthreads();
	}
#undef C3_LOAD_STAGE
#undef C3_STORE_STAGE

	// ---- store: dW[o][c][tap].  A wave holds taps (ta, 0..2) of 32 output x 32 input channels, i.e.
	// runs of three words; the three waves of an output-channel block go through LDS together so that
	// global memory sees whole rows of 32*9 consecutive words. --------------------------------------
	float *C = out.C + (size_t)bz * out.splitStride;
	float *stage = &Ds[0][0];
	constexpr int ROW = kC3DwCin * 9, ROW_LD = ROW + 1;
	static_assert(32 * ROW_LD <= 2 * (D_DUMMY + 4), "the output stage must fit the delta buffers");
	const int validCols = ((p.cred - c0 < kC3DwCin) ? (p.cred - c0) : kC3DwCin) * 9;
	for (int r = 0; r < 4; r++) {
		if (r > 0) __syncthreads(); // the copy of the previous block is done
		if (ob == r) {
#pragma unroll
			for (int v = 0; v < 16; v++) {
				float *dst = stage + (8 * (v / 4) + 4 * khalf + (v % 4)) * ROW_LD + l32 * 9 + ta * 3;
#pragma unroll
				for (int tb = 0; tb < 3; tb++) dst[tb] = acc[tb][v];
			}
		}
		__syncthreads();
		for (int i = tid; i < 32 * ROW; i += T) {
			const int row = i / ROW, col = i - row * ROW;
			const int o = o0 + r * 32 + row;
			if ((o < p.I) & (col < validCols)) C[(size_t)o * out.ldc + c0 * 9 + col] = stage[row * ROW_LD + col];
		}
	}
}

// ---------------------------------------------------------------------------------
// weight gradient of a layer with very few input channels (the first layer: Cin = 3)
// ---------------------------------------------------------------------------------
// With Cin*9 <= 32 the whole patch index (c, ta, tb) fits the 32 columns of ONE accumulator block,
// so the product is a plain  dW[64 x 27] = delta[64 x M] * patch[M x 27]  whose cost is reading
// delta once (HBM-bound, not MFMA-bound).  A workgroup walks chunks of 128 positions = whole image
// rows: delta goes through LDS as [channel][position]; the layer input as a window of R + 2 rows
// with a zero column on either side and zero rows above / below the image, so that the patch
// element of lane k = (c, ta, tb) at position (row r, column b) of the chunk is the word
// c*plane + (r + ta)*(B + 2) + b + tb: no border test.  Four waves take 32 positions each and are
// summed through LDS at the end; every workgroup leaves one partial 64 x 27 block (split layout
// of the general engine: combined by splitk_reduce_kernel).
// Requires B a power of two, 2 <= B <= 128, (A*B) % 128 == 0 or 128 % (A*B) == 0 -- here:
// A % (128 / B) == 0 --, Cin <= 3, Cout <= 64.
constexpr int kThinChunk = 128;
constexpr int kThinDeltaLd = kThinChunk + 1;
constexpr int kThinXPlane = 400; // words per input channel of the window: (R + 2) * (B + 2) <= 396

struct ThinDwParams {
	const float *x;     // [Cin][N][A][B]
	const float *delta; // [Cout][N][A][B]
	int cin, cout;
	int A, B, logB;
	int plane;          // N*A*B
	int chunks;         // plane / 128
	int perGroup;       // chunks per workgroup
};

__global__ void __launch_bounds__(kGemmThreads)
conv3x3_dw_thin_kernel(const ThinDwParams p, float *partial)
{
	__shared__ float Ds[2][64 * kThinDeltaLd];
	__shared__ float Xs[2][3 * kThinXPlane];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int R = kThinChunk >> p.logB;  // image rows per chunk
	const int rowLd = p.B + 2;
	const int imageCells = p.A * p.B;
	const int qBeg = blockIdx.x * p.perGroup;
	const int qEnd = (qBeg + p.perGroup < p.chunks) ? qBeg + p.perGroup : p.chunks;

	// this lane's patch column k = (c, ta, tb); columns past Cin*9 repeat the last one and are never stored
	const int K = p.cin * 9;
	const int k = (l32 < K) ? l32 : K - 1;
	const int kc = k / 9, kt = k - kc * 9, kta = kt / 3, ktb = kt - kta * 3;
	const int xBase = kc * kThinXPlane + kta * rowLd + ktb;

	// staging: delta 64 x 128 as 2048 groups of four, eight per thread; the window cell by cell
	constexpr int DE = 64 * kThinChunk / 4 / kGemmThreads;
	float4 dreg[DE];
	constexpr int XE = (3 * kThinXPlane + kGemmThreads - 1) / kGemmThreads;
	float xreg[XE];
	const int winCells = (R + 2) * rowLd;
	// which window cell each of this thread's XE words is does not depend on the chunk: worked out once
	// (three divisions by run-time values per word)
	int xRow[XE], xSrc[XE], xDst[XE]; // window row, channel and column offset in x (< 0: a border cell), word in Xs (< 0: none)
#pragma unroll
	for (int e = 0; e < XE; e++) {
		const int w = tid + kGemmThreads * e;
		const int c = w / winCells, cell = w - c * winCells;
		const int r = cell / rowLd, col = cell - r * rowLd;
		xRow[e] = r;
		xSrc[e] = (c < p.cin && col >= 1 && col <= p.B) ? c * p.plane + col - 1 : -1; // -1: a border column or no channel
		xDst[e] = (c < 3) ? c * kThinXPlane + cell : -1;
	}

	auto load_chunk = [&](int q) {
		const int m0 = q * kThinChunk;
#pragma unroll
		for (int e = 0; e < DE; e++) {
			const int g = tid + kGemmThreads * e;
			const int o = g / (kThinChunk / 4), c4 = g - o * (kThinChunk / 4);
			dreg[e] = (o < p.cout) ? *reinterpret_cast<const float4 *>(p.delta + (size_t)o * p.plane + m0 + 4 * c4)
			                       : make_float4(0.f, 0.f, 0.f, 0.f);
		}
		const int n = m0 / imageCells;
		const int a0 = (m0 - n * imageCells) >> p.logB; // first image row of the chunk
		const int imageBase = n * imageCells;
#pragma unroll
		for (int e = 0; e < XE; e++) {
			const int a = a0 - 1 + xRow[e];
			const bool ok = (xSrc[e] >= 0) & ((unsigned)a < (unsigned)p.A);
			xreg[e] = ok ? p.x[(size_t)xSrc[e] + (size_t)imageBase + a * p.B] : 0.f;
		}
	};
	auto store_chunk = [&](int buf) {
#pragma unroll
		for (int e = 0; e < DE; e++) {
			const int g = tid + kGemmThreads * e;
			const int o = g / (kThinChunk / 4), c4 = g - o * (kThinChunk / 4);
			float *dst = Ds[buf] + o * kThinDeltaLd + 4 * c4;
			dst[0] = dreg[e].x, dst[1] = dreg[e].y, dst[2] = dreg[e].z, dst[3] = dreg[e].w;
		}
#pragma unroll
		for (int e = 0; e < XE; e++)
			if (xDst[e] >= 0) Xs[buf][xDst[e]] = xreg[e];
	};

	v16f acc0, acc1;
#pragma unroll
	for (int v = 0; v < 16; v++) acc0[v] = 0.f, acc1[v] = 0.f;

	if (qBeg < qEnd) {
		load_chunk(qBeg);
		store_chunk(0);
	}
	__syncthreads();
	for (int q = qBeg; q < qEnd; q++) {
		const int buf = (q - qBeg) & 1;
		const bool more = q + 1 < qEnd;
		if (more) load_chunk(q + 1);
		const float *dA = Ds[buf] + l32 * kThinDeltaLd + wave * 32 + khalf;
		const float *dB = dA + 32 * kThinDeltaLd;
#pragma unroll
		for (int st = 0; st < 16; st++) {
			const int pos = wave * 32 + 2 * st + khalf; // position inside the chunk
			const int r = pos >> p.logB, b = pos & (p.B - 1);
			const float bv = Xs[buf][xBase + r * rowLd + b];
			acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(dA[2 * st], bv, acc0, 0, 0, 0);
			acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(dB[2 * st], bv, acc1, 0, 0, 0);
		}
		if (more) store_chunk(buf ^ 1);
		__syncthreads();
	}

	// sum the four waves through LDS (the delta buffers are free now), then one coalesced store
	float *red = &Ds[0][0]; // [wave][64][33]
	static_assert(4 * 64 * 33 <= 2 * 64 * kThinDeltaLd, "the wave partials fit the delta buffers");
#pragma unroll
	for (int v = 0; v < 16; v++) {
		const int row = 8 * (v / 4) + 4 * khalf + (v % 4);
		red[(wave * 64 + row) * 33 + l32] = acc0[v];
		red[(wave * 64 + 32 + row) * 33 + l32] = acc1[v];
	}
	__syncthreads();
	float *out = partial + (size_t)blockIdx.x * p.cout * K;
	for (int i = tid; i < p.cout * K; i += kGemmThreads) {
		const int o = i / K, kk = i - o * K;
		out[i] = (red[(0 * 64 + o) * 33 + kk] + red[(1 * 64 + o) * 33 + kk]) + (red[(2 * 64 + o) * 33 + kk] + red[(3 * 64 + o) * 33 + kk]);
	}
}

} // namespace fitre
