// 3x3 / stride 1 / pad 1 convolution gradients on 4 x 4 maps without the padding's share of the arithmetic.
//
// On a 4 x 4 map 44 of the 16 x 9 = 144 (cell, tap) pairs of an image reach outside it.  The nine-tap kernels
// of conv3x3.h multiply those with zeros: their MFMA blocks hold consecutive flat positions, i.e. two whole
// images, so every block has live cells for every tap.  Here a block's 32 columns (input gradient) or its
// reduction pairs (weight gradient) are the SAME cell of different images: a (cell, tap) pair is then live or
// dead for the whole block, the dead ones are left out at compile time, and the matrix pipes do 100 / 144 of
// the work (the layers of VGG-11 with 4 x 4 maps hold 40 % of a backward pass's matrix time).  No border
// masks, pads or halo are needed: a tap that is issued always reads a cell of the same image.
#pragma once
#include "conv3x3.h"

namespace fitre {

constexpr int kCellMap = 4;                   // map extent
constexpr int kCells = kCellMap * kCellMap;   // cells per image
constexpr int kCellStageImages = kC3Stage / kCells; // images per weight-gradient stage (64 positions)

__host__ __device__ constexpr bool cell_tap_live(int cell, int tap)
{
	const int a = cell / kCellMap + tap / 3 - 1, b = cell % kCellMap + tap % 3 - 1;
	return a >= 0 && a < kCellMap && b >= 0 && b < kCellMap;
}
__host__ __device__ constexpr int cell_tap_source(int cell, int tap) { return cell + (tap / 3 - 1) * kCellMap + (tap % 3 - 1); }
// the k-th live tap of a cell, or -1
__host__ __device__ constexpr int cell_nth_live_tap(int cell, int k)
{
	for (int tap = 0; tap < 9; tap++)
		if (cell_tap_live(cell, tap) && k-- == 0) return tap;
	return -1;
}

// ---------------------------------------------------------------------------------
// weight gradient: dW[o][c][tap] = sum over images and live cells of delta[o][n][cell] * src[c][n][cell + tap shift]
// ---------------------------------------------------------------------------------
// Geometry of conv3x3_dw_kernel: twelve waves own 128 output channels x 32 input channels x nine taps, a stage
// is 64 positions = four images.  A reduction pair of an MFMA step is one cell of two neighbouring images, so
// delta and source sit in LDS as they sit in memory, [channel][image][cell] with an odd row stride.  The nine
// taps have 9 (corner taps), 12 (edge taps) and 16 (centre) live cells; the three waves of an output-channel
// block take tap groups of equal weight -- {centre, two opposite corners} = 34, {two edges, a corner} = 33 twice.
__device__ constexpr int kCellTapGroups[3][3] = { { 4, 0, 8 }, { 1, 3, 2 }, { 5, 7, 6 } };

template <int TG>
__device__ __forceinline__ void cell_dw_steps(const float *aBase, const float *bBase, v16f (&acc)[3])
{
#pragma unroll
	for (int ip = 0; ip < kCellStageImages / 2; ip++) {
#pragma unroll
		for (int cell = 0; cell < kCells; cell++) {
			const bool any = cell_tap_live(cell, kCellTapGroups[TG][0]) || cell_tap_live(cell, kCellTapGroups[TG][1]) ||
			                 cell_tap_live(cell, kCellTapGroups[TG][2]);
			if (!any) continue;
			const float fa = aBase[ip * 2 * kCells + cell];
#pragma unroll
			for (int j = 0; j < 3; j++) {
				const int tap = kCellTapGroups[TG][j];
				if (cell_tap_live(cell, tap)) {
					const float fb = bBase[ip * 2 * kCells + cell_tap_source(cell, tap)];
					acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc[j], 0, 0, 0);
				}
			}
		}
	}
}

template <bool VEC>
__global__ void __launch_bounds__(kC3DwThreads)
conv3x3_dw_cell_kernel(const Conv3x3Params p, const float *delta, uint32_t deltaBytes, const OutParams out)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	constexpr int T = kC3DwThreads;
	constexpr int LD = kC3Stage + 1; // odd row stride of both stages
	constexpr int D_DUMMY = kC3Tile * LD, X_DUMMY = kC3DwCin * LD;
	constexpr int DGROUPS = kC3Tile * kC3Stage / 4; // 4-float groups of delta per stage
	constexpr int DE = (DGROUPS + T - 1) / T;
	constexpr int XGROUPS = kC3DwCin * kC3Stage / 4; // 512: one per thread of the first eight waves
	static_assert(XGROUPS <= T, "one source group per thread");
	__shared__ float Ds[2][D_DUMMY + 4];
	__shared__ float Xs[2][X_DUMMY + 4];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int ob = wave & 3, tg = wave >> 2; // output-channel block, tap group
	// workgroups renumbered so that an XCD (its own L2) holds consecutive indices, as in conv3x3_dw_kernel
	int bx, by, bz;
	{
		const unsigned groups = gridDim.x * gridDim.y * gridDim.z;
		const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
		const unsigned xcd = lin & 7u, each = groups >> 3, extra = groups & 7u;
		const unsigned logical = xcd * each + (xcd < extra ? xcd : extra) + (lin >> 3);
		const unsigned tiles = gridDim.x * gridDim.y;
		bz = (int)(logical / tiles);
		const unsigned rem = logical - (unsigned)bz * tiles;
		by = (int)(rem / gridDim.x);
		bx = (int)(rem - (unsigned)by * gridDim.x);
	}
	const int c0 = bx * kC3DwCin, o0 = by * kC3Tile;
	const int plane = p.J;
	const int stagesHalf = p.J / kC3Stage;
	const int stagesTotal = p.src2 ? 2 * stagesHalf : stagesHalf; // a second (source, delta) pair continues the reduction
	const int stBeg = bz * p.perSplit;
	const int stEnd = (stBeg + p.perSplit < stagesTotal) ? stBeg + p.perSplit : stagesTotal;

	// ---- what this thread stages ------------------------------------------------------------
	const int dCol = 4 * (tid % (kC3Stage / 4));
	uint32_t dOff[DE];
	int dLds[DE];
#pragma unroll
	for (int e = 0; e < DE; e++) {
		const int idx = tid + T * e;
		const int row = idx / (kC3Stage / 4);
		const bool has = idx < DGROUPS;
		const bool inside = has & ((o0 + row) < p.I);
		// rows past the tensor feed accumulator rows that are never stored
		const uint32_t off = 4u * (uint32_t)((o0 + row) * plane + dCol);
		dOff[e] = VEC ? (inside ? off : 4u * (uint32_t)dCol) : (inside ? off : kGroupOutOfRange);
		dLds[e] = has ? row * LD + dCol : D_DUMMY;
	}
	const int xRow = tid / (kC3Stage / 4);
	const bool xHas = tid < XGROUPS;
	const bool xInside = xHas & ((c0 + xRow) < p.cred);
	const uint32_t xOff = VEC ? (xInside ? 4u * (uint32_t)((c0 + xRow) * plane + dCol) : 4u * (uint32_t)dCol)
	                          : (xInside ? 4u * (uint32_t)((c0 + xRow) * plane + dCol) : kGroupOutOfRange);
	const int xLds = xHas ? xRow * LD + dCol : X_DUMMY;
	float dreg[DE * 4];
	float xreg[4];

#define CELL_LOAD_STAGE(ST)                                                                                           \
	{                                                                                                                 \
		const bool second_ = (ST) >= stagesHalf; /* uniform */                                                        \
		const int m0_ = ((ST) - (second_ ? stagesHalf : 0)) * kC3Stage;                                               \
		const float *dSel = second_ ? p.w2 : delta;                                                                   \
		const float *xSel = second_ ? p.src2 : p.src;                                                                 \
		if constexpr (VEC) {                                                                                          \
			const char *dBlk = reinterpret_cast<const char *>(dSel + m0_);                                            \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				const float4 v4 = *reinterpret_cast<const float4 *>(dBlk + dOff[e]);                                  \
				dreg[4 * e + 0] = v4.x, dreg[4 * e + 1] = v4.y, dreg[4 * e + 2] = v4.z, dreg[4 * e + 3] = v4.w;       \
			}                                                                                                         \
			const float4 x4 = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(xSel + m0_) + xOff);   \
			xreg[0] = xInside ? x4.x : 0.f, xreg[1] = xInside ? x4.y : 0.f;                                           \
			xreg[2] = xInside ? x4.z : 0.f, xreg[3] = xInside ? x4.w : 0.f;                                           \
		} else {                                                                                                      \
			const __amdgpu_buffer_rsrc_t dRs = make_rsrc(dSel + m0_, deltaBytes - 4u * (uint32_t)m0_);                \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				dreg[4 * e + 0] = buffer_load(dRs, dOff[e]);                                                          \
				dreg[4 * e + 1] = buffer_load(dRs, dOff[e] + 4u);                                                     \
				dreg[4 * e + 2] = buffer_load(dRs, dOff[e] + 8u);                                                     \
				dreg[4 * e + 3] = buffer_load(dRs, dOff[e] + 12u);                                                    \
			}                                                                                                         \
			const __amdgpu_buffer_rsrc_t xRs = make_rsrc(xSel + m0_, p.srcBytes - 4u * (uint32_t)m0_);                \
			xreg[0] = buffer_load(xRs, xOff), xreg[1] = buffer_load(xRs, xOff + 4u);                                  \
			xreg[2] = buffer_load(xRs, xOff + 8u), xreg[3] = buffer_load(xRs, xOff + 12u);                            \
		}                                                                                                             \
	}

#define CELL_STORE_STAGE(BUF)                                                                                         \
	{                                                                                                                 \
		_Pragma("unroll") for (int e = 0; e < DE; e++)                                                                \
		{                                                                                                             \
			float *dst = Ds[BUF] + dLds[e];                                                                           \
			dst[0] = dreg[4 * e], dst[1] = dreg[4 * e + 1], dst[2] = dreg[4 * e + 2], dst[3] = dreg[4 * e + 3];       \
		}                                                                                                             \
		float *xd = Xs[BUF] + xLds;                                                                                   \
		xd[0] = xreg[0], xd[1] = xreg[1], xd[2] = xreg[2], xd[3] = xreg[3];                                           \
	}

	v16f acc[3];
#pragma unroll
	for (int t = 0; t < 3; t++)
#pragma unroll
		for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

	// fragment of lane (l32, khalf) for cell q of image pair ip: row l32, word (2 * ip + khalf) * 16 + q
	const int aOff = (ob * 32 + l32) * LD + khalf * kCells;
	const int bOff = l32 * LD + khalf * kCells;

	if (stBeg < stEnd) {
		CELL_LOAD_STAGE(stBeg);
		CELL_STORE_STAGE(0);
	}
	__syncthreads();
	for (int st = stBeg; st < stEnd; st++) {
		const int buf = (st - stBeg) & 1;
		const bool more = st + 1 < stEnd;
		if (more) CELL_LOAD_STAGE(st + 1);
		const float *aBase = Ds[buf] + aOff;
		const float *bBase = Xs[buf] + bOff;
		if (tg == 0) cell_dw_steps<0>(aBase, bBase, acc);
		else if (tg == 1) cell_dw_steps<1>(aBase, bBase, acc);
		else cell_dw_steps<2>(aBase, bBase, acc);
		if (more) CELL_STORE_STAGE(buf ^ 1); // the other buffer was released by the last barrier
		__syncthreads();
	}
#undef CELL_LOAD_STAGE
#undef CELL_STORE_STAGE

	// ---- store: dW[o][c][tap], through LDS so that global memory sees whole rows of 32 * 9 consecutive words ----
	float *C = out.C + (size_t)bz * out.splitStride;
	float *stage = &Ds[0][0];
	constexpr int ROW = kC3DwCin * 9, ROW_LD = ROW + 1;
	static_assert(32 * ROW_LD <= 2 * (D_DUMMY + 4), "the output stage must fit the delta buffers");
	const int validCols = ((p.cred - c0 < kC3DwCin) ? (p.cred - c0) : kC3DwCin) * 9;
	const int tap0 = kCellTapGroups[tg][0], tap1 = kCellTapGroups[tg][1], tap2 = kCellTapGroups[tg][2];
	for (int r = 0; r < 4; r++) {
		if (r > 0) __syncthreads(); // the copy of the previous block is done
		if (ob == r) {
#pragma unroll
			for (int v = 0; v < 16; v++) {
				float *dst = stage + (8 * (v / 4) + 4 * khalf + (v % 4)) * ROW_LD + l32 * 9;
				dst[tap0] = acc[0][v], dst[tap1] = acc[1][v], dst[tap2] = acc[2][v];
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
// weight gradient on 8 x 8 maps: the same idea with a stage of 64 positions = the upper or the lower half (four
// rows) of TWO neighbouring images.  92 of the 576 (cell, tap) pairs of an image are dead (16 %); a stage has 242
// live ones of 288.  The source stage holds the half's four rows and the row above / below it that lies inside
// the image (five rows of eight cells per image), so no tap that is issued leaves it.  Tap groups {centre, two
// opposite corners}, {down, up, up-right}, {left, right, down-left}: 81 / 77 / 84 live pairs on an upper half,
// 81 / 84 / 77 on a lower one, against 96 steps of the nine-tap kernel.
// ---------------------------------------------------------------------------------
// The 32 cells of a stage are unrolled; left alone the compiler hoists their LDS reads until the kernel holds 166
// registers, and three waves of 166 fill a SIMD's register file: nothing else can then run beside this kernel, and
// the bandwidth-bound kernels of the other lane wait for its last workgroup.  A scheduling barrier every four cells
// keeps it to 149 registers at the same speed (109.9 us alone either way); the pass is 1.5 % shorter.
#ifndef FITRE_CELL8_CHUNK
#define FITRE_CELL8_CHUNK 4
#endif
constexpr int kCell8Map = 8;
constexpr int kCell8Half = 32;                 // cells of half a map
constexpr int kCell8SrcCells = 5 * kCell8Map;  // source cells per image and half
__device__ constexpr int kCell8TapGroups[3][3] = { { 4, 0, 8 }, { 7, 1, 2 }, { 3, 5, 6 } };

// LOWER: the stage is the lower half (rows 4..7; the source rows are 3..7), else the upper (rows 0..3; source 0..4)
template <int TG, bool LOWER>
__device__ __forceinline__ void cell8_dw_steps(const float *aBase, const float *bBase, v16f (&acc)[3])
{
#pragma unroll
	for (int cell = 0; cell < kCell8Half; cell++) {
		const int a = cell / kCell8Map + (LOWER ? 4 : 0), b = cell % kCell8Map; // row and column in the image
		bool live[3] = { false, false, false };
		int src[3] = { 0, 0, 0 };
#pragma unroll
		for (int j = 0; j < 3; j++) {
			const int tap = kCell8TapGroups[TG][j];
			const int sa = a + tap / 3 - 1, sb = b + tap % 3 - 1;
			live[j] = sa >= 0 && sa < kCell8Map && sb >= 0 && sb < kCell8Map;
			src[j] = (sa - (LOWER ? 3 : 0)) * kCell8Map + sb; // word inside the image's five source rows
		}
#if FITRE_CELL8_CHUNK > 0
		if (cell % FITRE_CELL8_CHUNK == 0 && cell > 0) __builtin_amdgcn_sched_barrier(0);
#endif
		if (!(live[0] || live[1] || live[2])) continue;
		const float fa = aBase[cell];
#pragma unroll
		for (int j = 0; j < 3; j++)
			if (live[j]) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, bBase[src[j]], acc[j], 0, 0, 0);
	}
}

template <bool VEC>
__global__ void __launch_bounds__(kC3DwThreads)
conv3x3_dw_cell8_kernel(const Conv3x3Params p, const float *delta, uint32_t deltaBytes, const OutParams out)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	constexpr int T = kC3DwThreads;
	constexpr int D_LD = kC3Stage + 1;              // delta: [row][image of the pair][32 cells], odd stride
	constexpr int X_LD = 2 * kCell8SrcCells + 1;    // source: [row][image of the pair][40 cells], odd stride
	constexpr int D_DUMMY = kC3Tile * D_LD, X_DUMMY = kC3DwCin * X_LD;
	constexpr int DGROUPS = kC3Tile * kC3Stage / 4; // 16-byte groups of delta per stage
	constexpr int DE = (DGROUPS + T - 1) / T;
	constexpr int XGROUPS = kC3DwCin * 2 * kCell8SrcCells / 4; // 640: one per thread of the first ten waves
	static_assert(XGROUPS <= T, "one source group per thread");
	constexpr int IMG = kCell8Map * kCell8Map;
	__shared__ float Ds[2][D_DUMMY + 4];
	__shared__ float Xs[2][X_DUMMY + 4];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int ob = wave & 3, tg = wave >> 2; // output-channel block, tap group
	// workgroups renumbered so that an XCD (its own L2) holds consecutive indices, as in conv3x3_dw_kernel
	int bx, by, bz;
	{
		const unsigned groups = gridDim.x * gridDim.y * gridDim.z;
		const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
		const unsigned xcd = lin & 7u, each = groups >> 3, extra = groups & 7u;
		const unsigned logical = xcd * each + (xcd < extra ? xcd : extra) + (lin >> 3);
		const unsigned tiles = gridDim.x * gridDim.y;
		bz = (int)(logical / tiles);
		const unsigned rem = logical - (unsigned)bz * tiles;
		by = (int)(rem / gridDim.x);
		bx = (int)(rem - (unsigned)by * gridDim.x);
	}
	const int c0 = bx * kC3DwCin, o0 = by * kC3Tile;
	const int plane = p.J;
	const int stagesHalf = p.J / kC3Stage; // stage st: image pair st / 2, half st % 2
	const int stagesTotal = p.src2 ? 2 * stagesHalf : stagesHalf;
	const int stBeg = bz * p.perSplit;
	const int stEnd = (stBeg + p.perSplit < stagesTotal) ? stBeg + p.perSplit : stagesTotal;

	// ---- what this thread stages: offsets relative to the first cell of the stage's image pair -----------------
	uint32_t dOff[DE]; // without the half's 32 cells
	int dLds[DE];
#pragma unroll
	for (int e = 0; e < DE; e++) {
		const int idx = tid + T * e;
		const int row = idx / (kC3Stage / 4), g = idx - row * (kC3Stage / 4); // g: 0..15 = image of the pair x 8 groups
		const int img = g / 8, cg = 4 * (g - img * 8);
		const bool has = idx < DGROUPS;
		const bool inside = has & ((o0 + row) < p.I);
		const uint32_t off = 4u * (uint32_t)((o0 + row) * plane + img * IMG + cg);
		// rows past the tensor feed accumulator rows that are never stored
		dOff[e] = VEC ? (inside ? off : 4u * (uint32_t)(img * IMG + cg)) : (inside ? off : kGroupOutOfRange);
		dLds[e] = has ? row * D_LD + img * kCell8Half + cg : D_DUMMY;
	}
	// source: group tid of [32 rows][2 images][10 groups of four cells = five image rows]
	const int xRow = tid / (2 * kCell8SrcCells / 4), xg = tid - xRow * (2 * kCell8SrcCells / 4);
	const int xImg = xg / (kCell8SrcCells / 4), xCg = 4 * (xg - xImg * (kCell8SrcCells / 4));
	const bool xHas = tid < XGROUPS;
	const bool xInside = xHas & ((c0 + xRow) < p.cred);
	const uint32_t xOffRaw = 4u * (uint32_t)((c0 + xRow) * plane + xImg * IMG + xCg); // plus the first source row of the half
	const uint32_t xOff = VEC ? (xInside ? xOffRaw : 4u * (uint32_t)(xImg * IMG + xCg)) : (xInside ? xOffRaw : kGroupOutOfRange);
	const int xLds = xHas ? xRow * X_LD + xImg * kCell8SrcCells + xCg : X_DUMMY;
	float dreg[DE * 4];
	float xreg[4];

#define CELL8_LOAD_STAGE(ST)                                                                                          \
	{                                                                                                                 \
		const bool second_ = (ST) >= stagesHalf; /* uniform */                                                        \
		const int s_ = (ST) - (second_ ? stagesHalf : 0);                                                             \
		const int pair0_ = (s_ >> 1) * 2 * IMG;            /* first cell of the image pair */                         \
		const int dBase_ = pair0_ + (s_ & 1) * kCell8Half;  /* the half's first cell */                               \
		const int xBase_ = pair0_ + (s_ & 1) * 3 * kCell8Map; /* its first source row: 0 or 3 */                      \
		const float *dSel = second_ ? p.w2 : delta;                                                                   \
		const float *xSel = second_ ? p.src2 : p.src;                                                                 \
		if constexpr (VEC) {                                                                                          \
			const char *dBlk = reinterpret_cast<const char *>(dSel + dBase_);                                         \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				const float4 v4 = *reinterpret_cast<const float4 *>(dBlk + dOff[e]);                                  \
				dreg[4 * e + 0] = v4.x, dreg[4 * e + 1] = v4.y, dreg[4 * e + 2] = v4.z, dreg[4 * e + 3] = v4.w;       \
			}                                                                                                         \
			const float4 x4 = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(xSel + xBase_) + xOff); \
			xreg[0] = xInside ? x4.x : 0.f, xreg[1] = xInside ? x4.y : 0.f;                                           \
			xreg[2] = xInside ? x4.z : 0.f, xreg[3] = xInside ? x4.w : 0.f;                                           \
		} else {                                                                                                      \
			const __amdgpu_buffer_rsrc_t dRs = make_rsrc(dSel + dBase_, deltaBytes - 4u * (uint32_t)dBase_);          \
			_Pragma("unroll") for (int e = 0; e < DE; e++)                                                            \
			{                                                                                                         \
				dreg[4 * e + 0] = buffer_load(dRs, dOff[e]);                                                          \
				dreg[4 * e + 1] = buffer_load(dRs, dOff[e] + 4u);                                                     \
				dreg[4 * e + 2] = buffer_load(dRs, dOff[e] + 8u);                                                     \
				dreg[4 * e + 3] = buffer_load(dRs, dOff[e] + 12u);                                                    \
			}                                                                                                         \
			const __amdgpu_buffer_rsrc_t xRs = make_rsrc(xSel + xBase_, p.srcBytes - 4u * (uint32_t)xBase_);          \
			xreg[0] = buffer_load(xRs, xOff), xreg[1] = buffer_load(xRs, xOff + 4u);                                  \
			xreg[2] = buffer_load(xRs, xOff + 8u), xreg[3] = buffer_load(xRs, xOff + 12u);                            \
		}                                                                                                             \
	}

#define CELL8_STORE_STAGE(BUF)                                                                                        \
	{                                                                                                                 \
		_Pragma("unroll") for (int e = 0; e < DE; e++)                                                                \
		{                                                                                                             \
			float *dst = Ds[BUF] + dLds[e];                                                                           \
			dst[0] = dreg[4 * e], dst[1] = dreg[4 * e + 1], dst[2] = dreg[4 * e + 2], dst[3] = dreg[4 * e + 3];       \
		}                                                                                                             \
		float *xd = Xs[BUF] + xLds;                                                                                   \
		xd[0] = xreg[0], xd[1] = xreg[1], xd[2] = xreg[2], xd[3] = xreg[3];                                           \
	}

	v16f acc[3];
#pragma unroll
	for (int t = 0; t < 3; t++)
#pragma unroll
		for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

	// fragment of lane (l32, khalf): row l32, image khalf of the pair
	const int aOff = (ob * 32 + l32) * D_LD + khalf * kCell8Half;
	const int bOff = l32 * X_LD + khalf * kCell8SrcCells;

	if (stBeg < stEnd) {
		CELL8_LOAD_STAGE(stBeg);
		CELL8_STORE_STAGE(0);
	}
	__syncthreads();
	for (int st = stBeg; st < stEnd; st++) {
		const int buf = (st - stBeg) & 1;
		const bool more = st + 1 < stEnd;
		if (more) CELL8_LOAD_STAGE(st + 1);
		const float *aBase = Ds[buf] + aOff;
		const float *bBase = Xs[buf] + bOff;
		const bool lower = (st & 1) != 0; // stagesHalf is even, so this holds for the second pair as well
		if (!lower) {
			if (tg == 0) cell8_dw_steps<0, false>(aBase, bBase, acc);
			else if (tg == 1) cell8_dw_steps<1, false>(aBase, bBase, acc);
			else cell8_dw_steps<2, false>(aBase, bBase, acc);
		} else {
			if (tg == 0) cell8_dw_steps<0, true>(aBase, bBase, acc);
			else if (tg == 1) cell8_dw_steps<1, true>(aBase, bBase, acc);
			else cell8_dw_steps<2, true>(aBase, bBase, acc);
		}
		if (more) CELL8_STORE_STAGE(buf ^ 1); // the other buffer was released by the last barrier
		__syncthreads();
	}
#undef CELL8_LOAD_STAGE
#undef CELL8_STORE_STAGE

	// ---- store: dW[o][c][tap], through LDS so that global memory sees whole rows of 32 * 9 consecutive words ----
	float *C = out.C + (size_t)bz * out.splitStride;
	float *stage = &Ds[0][0];
	constexpr int ROW = kC3DwCin * 9, ROW_LD = ROW + 1;
	static_assert(32 * ROW_LD <= 2 * (D_DUMMY + 4), "the output stage must fit the delta buffers");
	const int validCols = ((p.cred - c0 < kC3DwCin) ? (p.cred - c0) : kC3DwCin) * 9;
	const int tap0 = kCell8TapGroups[tg][0], tap1 = kCell8TapGroups[tg][1], tap2 = kCell8TapGroups[tg][2];
	for (int r = 0; r < 4; r++) {
		if (r > 0) __syncthreads(); // the copy of the previous block is done
		if (ob == r) {
#pragma unroll
			for (int v = 0; v < 16; v++) {
				float *dst = stage + (8 * (v / 4) + 4 * khalf + (v % 4)) * ROW_LD + l32 * 9;
				dst[tap0] = acc[0][v], dst[tap1] = acc[1][v], dst[tap2] = acc[2][v];
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
// input gradient (and any position-contiguous product with the DX weight layout):
//     out[i][n][cell] = sum over c and live taps of W[c][i][8 - tap] * src[c][n][cell + tap shift]
// ---------------------------------------------------------------------------------
// A workgroup owns 32 channels x 32 images x the 16 cells; an MFMA block is 32 channels x 32 images of ONE cell.
// Each of the four waves owns a quadrant of the map -- a corner, two edge cells and a centre cell: 25 live taps,
// the same for every quadrant -- i.e. four accumulator blocks, and per reduction pair reads the nine taps'
// weight fragments and the nine source cells around its quadrant for 25 MFMAs.  The source block sits in LDS as
// [channel][cell][image] (images contiguous: a fragment is 32 consecutive words), the weights as in
// conv3x3_pos_kernel's input-gradient form: CB rows (reduction channel) of the tile's IT * 9 weights.  The result
// leaves through LDS as whole 64-byte images ([row][image][cell]).  Requires samples % 32 == 0, cred % CB == 0.
constexpr int kCellImages = 32; // images per workgroup tile
constexpr int kCellIT = 32;     // channel rows per workgroup tile
constexpr int kCellCB = 8;      // reduction channels per LDS block

// the MFMAs of one reduction block for the wave that owns quadrant (QA, QB)
// A_PAIR: words between the weight fragments of two reduction pairs; FLIP: the weight of tap t is stored at 8 - t
template <int QA, int QB, int A_PAIR, bool FLIP, int B_LD>
__device__ __forceinline__ void cell_dx_block(const float *aBase, const float *bBase, v16f (&acc)[2][2])
{
	constexpr int CELL_LD = kCellImages + 1;
#pragma unroll
	for (int cp = 0; cp < kCellCB / 2; cp++) {
		const float *aPair = aBase + cp * A_PAIR, *bPair = bBase + cp * 2 * B_LD;
		float a[9], b[kCells];
#pragma unroll
		for (int tap = 0; tap < 9; tap++) a[tap] = aPair[FLIP ? 8 - tap : tap];
#pragma unroll
		for (int q = 0; q < kCells; q++) {
			const int qa = q / kCellMap, qb = q % kCellMap;
			const bool used = qa >= 2 * QA - 1 && qa <= 2 * QA + 2 && qb >= 2 * QB - 1 && qb <= 2 * QB + 2;
			b[q] = used ? bPair[q * CELL_LD] : 0.f;
		}
		// the four cells take turns, so that consecutive MFMAs do not wait for each other's accumulator
#pragma unroll
		for (int k = 0; k < 9; k++)
#pragma unroll
			for (int da = 0; da < 2; da++)
#pragma unroll
				for (int db = 0; db < 2; db++) {
					const int cell = (2 * QA + da) * kCellMap + 2 * QB + db;
					const int tap = cell_nth_live_tap(cell, k);
					if (tap < 0) continue;
					acc[da][db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tap], b[cell_tap_source(cell, tap)], acc[da][db], 0, 0, 0);
				}
	}
}

// DX = false: the forward product, out[i][n][cell] = bias[i] + sum over c and live taps of W[i][c][tap] * src[c][n][cell + tap
// shift]; its weights sit in LDS as IT rows (output channel) of the block's CB * 9 weights, odd row stride.
template <bool DX, bool VECW>
__global__ void __launch_bounds__(kGemmThreads, 2)
conv3x3_cell_dx_kernel(const Conv3x3Params p, const OutParams out)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	constexpr int IT = kCellIT, CB = kCellCB;
	constexpr int A_LD = DX ? (IT * 9 + 4) : (CB * 9 + 1); // input gradient: a multiple of four (16-byte stores)
	constexpr int A_FLOATS = DX ? CB * A_LD : IT * A_LD, A_DUMMY = A_FLOATS;
	constexpr int WQ = DX ? (IT * 9 / 4) : (CB * 9 / 4);   // 16-byte groups per LDS row
	constexpr int WGROUPS = (DX ? CB : IT) * WQ;           // 16-byte groups of weights per block
	constexpr int WE = (WGROUPS + kGemmThreads - 1) / kGemmThreads;
	constexpr int CELL_LD = kCellImages + 1;             // images of one cell, odd stride
	constexpr int B_LD = kCells * CELL_LD + 1;           // per reduction channel
	constexpr int B_FLOATS = CB * B_LD;
	constexpr int SGROUPS = CB * kCellImages * kCells / 4; // 16-byte groups of the source block
	constexpr int SE = SGROUPS / kGemmThreads;
	static_assert(SGROUPS % kGemmThreads == 0, "whole rounds of source groups");
	constexpr int IMG_LD = kCells + 1, ROW_LD = kCellImages * IMG_LD; // the output stage: [row][image][cell]
	constexpr int OUT_ROWS = 8;                                       // rows per round of the output stage
	constexpr int LDS_FLOATS = (A_FLOATS + 4 + B_FLOATS) > OUT_ROWS * ROW_LD ? (A_FLOATS + 4 + B_FLOATS) : OUT_ROWS * ROW_LD;
	__shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
	float *As = lds, *Bs = lds + A_FLOATS + 4;

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int i0 = blockIdx.y * IT, n0 = blockIdx.x * kCellImages;
	const int plane = p.J;
	const int cbHalf = p.cred / CB;                    // channel blocks of one (src, w) pair
	const int cbTotal = p.src2 ? 2 * cbHalf : cbHalf; // a second pair continues the reduction
	const int cbBeg = blockIdx.z * p.perSplit;
	const int cbEnd = (cbBeg + p.perSplit < cbTotal) ? cbBeg + p.perSplit : cbTotal;
	const int rowLen = DX ? p.I * 9 : p.cred * 9;

	// ---- what this thread stages, the same for every channel block -------------------------
	uint32_t wOff[WE];
	int wLds[WE];
#pragma unroll
	for (int e = 0; e < WE; e++) {
		const int idx = tid + kGemmThreads * e;
		const int row = idx / WQ, qd = idx - row * WQ;
		const bool has = idx < WGROUPS;
		// input gradient: row = reduction channel, w[(c0 + row) * I * 9 + i0 * 9 + 4 * qd ..]
		// forward:        row = output channel,    w[(i0 + row) * cred * 9 + c0 * 9 + 4 * qd ..]
		const int rowG = DX ? row : (i0 + row);
		const int colG = DX ? (i0 * 9 + 4 * qd) : (4 * qd);
		const bool inside = has & (DX ? (colG + 3 < rowLen) : (rowG < p.I));
		const uint32_t off = 4u * (uint32_t)(rowG * rowLen + colG);
		// rows or columns past the tensor only feed accumulator rows that are never stored
		wOff[e] = VECW ? (inside ? off : 0u) : (inside ? off : kGroupOutOfRange);
		wLds[e] = has ? row * A_LD + 4 * qd : A_DUMMY;
	}
	// source: group g = tid + 256 * e of the block's CB x (32 images x 16 cells) floats; a group is four cells of an image
	uint32_t sOff[SE];
	int sLds[SE];
#pragma unroll
	for (int e = 0; e < SE; e++) {
		const int g = tid + kGemmThreads * e;
		const int c = g / (kCellImages * kCells / 4), r = g - c * (kCellImages * kCells / 4);
		const int img = r / (kCells / 4), q0 = 4 * (r - img * (kCells / 4));
		sOff[e] = 4u * (uint32_t)(c * plane + (n0 + img) * kCells + q0);
		sLds[e] = c * B_LD + q0 * CELL_LD + img;
	}
	float wreg[WE * 4];
	float sreg[SE * 4];

	v16f acc[2][2];
#pragma unroll
	for (int x = 0; x < 4; x++)
#pragma unroll
		for (int v = 0; v < 16; v++) acc[x >> 1][x & 1][v] = 0.f;

	const float *aBase = DX ? (As + khalf * A_LD + l32 * 9) : (As + l32 * A_LD + khalf * 9);
	constexpr int A_PAIR = DX ? 2 * A_LD : 18;
	const float *bBase = Bs + khalf * B_LD + l32;

#define CELL_LOAD_BLOCK(CBI)                                                                                          \
	{                                                                                                                 \
		const bool second_ = (CBI) >= cbHalf; /* uniform: the block belongs to the second pair */                    \
		const int c0_ = ((CBI) - (second_ ? cbHalf : 0)) * CB;                                                        \
		const float *wSel = second_ ? p.w2 : p.w, *sSel = second_ ? p.src2 : p.src;                                   \
		const size_t wShift = DX ? (size_t)c0_ * rowLen : (size_t)c0_ * 9; /* floats, uniform */                      \
		if constexpr (VECW) {                                                                                         \
			const char *wBlk = reinterpret_cast<const char *>(wSel + wShift);                                         \
			_Pragma("unroll") for (int e = 0; e < WE; e++)                                                            \
			{                                                                                                         \
				const float4 v4 = *reinterpret_cast<const float4 *>(wBlk + wOff[e]);                                  \
				wreg[4 * e + 0] = v4.x, wreg[4 * e + 1] = v4.y, wreg[4 * e + 2] = v4.z, wreg[4 * e + 3] = v4.w;       \
			}                                                                                                         \
		} else {                                                                                                      \
			const __amdgpu_buffer_rsrc_t wRs = make_rsrc(wSel + wShift, p.wBytes - (uint32_t)(4 * wShift));            \
			_Pragma("unroll") for (int e = 0; e < WE; e++)                                                            \
			{                                                                                                         \
				wreg[4 * e + 0] = buffer_load(wRs, wOff[e]);                                                          \
				wreg[4 * e + 1] = buffer_load(wRs, wOff[e] + 4u);                                                     \
				wreg[4 * e + 2] = buffer_load(wRs, wOff[e] + 8u);                                                     \
				wreg[4 * e + 3] = buffer_load(wRs, wOff[e] + 12u);                                                    \
			}                                                                                                         \
		}                                                                                                             \
		const size_t sShift = (size_t)c0_ * plane;                                                                    \
		const __amdgpu_buffer_rsrc_t sRs = make_rsrc(sSel + sShift, p.srcBytes - (uint32_t)(4 * sShift));           \
		_Pragma("unroll") for (int e = 0; e < SE; e++)                                                                \
		{                                                                                                             \
			sreg[4 * e + 0] = buffer_load(sRs, sOff[e]);                                                              \
			sreg[4 * e + 1] = buffer_load(sRs, sOff[e] + 4u);                                                         \
			sreg[4 * e + 2] = buffer_load(sRs, sOff[e] + 8u);                                                         \
			sreg[4 * e + 3] = buffer_load(sRs, sOff[e] + 12u);                                                        \
		}                                                                                                             \
	}

	if (cbBeg < cbEnd) CELL_LOAD_BLOCK(cbBeg);
	for (int cb = cbBeg; cb < cbEnd; cb++) {
		__syncthreads();
#pragma unroll
		for (int e = 0; e < WE; e++) {
			float *dst = As + wLds[e];
			if constexpr (DX) {
				*reinterpret_cast<float4 *>(dst) = make_float4(wreg[4 * e], wreg[4 * e + 1], wreg[4 * e + 2], wreg[4 * e + 3]);
			} else {
				dst[0] = wreg[4 * e], dst[1] = wreg[4 * e + 1], dst[2] = wreg[4 * e + 2], dst[3] = wreg[4 * e + 3];
			}
		}
#pragma unroll
		for (int e = 0; e < SE; e++) {
			float *dst = Bs + sLds[e];
			dst[0] = sreg[4 * e], dst[CELL_LD] = sreg[4 * e + 1], dst[2 * CELL_LD] = sreg[4 * e + 2], dst[3 * CELL_LD] = sreg[4 * e + 3];
		}
		__syncthreads();
		if (cb + 1 < cbEnd) CELL_LOAD_BLOCK(cb + 1);
		if (wave == 0) cell_dx_block<0, 0, A_PAIR, DX, B_LD>(aBase, bBase, acc);
		else if (wave == 1) cell_dx_block<0, 1, A_PAIR, DX, B_LD>(aBase, bBase, acc);
		else if (wave == 2) cell_dx_block<1, 0, A_PAIR, DX, B_LD>(aBase, bBase, acc);
		else cell_dx_block<1, 1, A_PAIR, DX, B_LD>(aBase, bBase, acc);
	}
#undef CELL_LOAD_BLOCK

	// ---- store: out[i][(n0 + image) * 16 + cell].  A row of the tile is 32 images x 16 cells = 2 KB of consecutive
	// words, but a lane holds one cell of one image: eight rows at a time go through LDS and leave as 16-byte
	// groups of whole rows. ------------------------------------------------------------------------------------
	float *C = out.C + (size_t)blockIdx.z * out.splitStride;
	const bool split = out.splitStride != 0;
	const int QA = wave >> 1, QB = wave & 1;
	float *stage = lds;
#pragma unroll
	for (int vg = 0; vg < 4; vg++) {
		__syncthreads(); // the previous round has left (first round: the last block's fragments are read)
#pragma unroll
		for (int da = 0; da < 2; da++)
#pragma unroll
			for (int db = 0; db < 2; db++) {
				const int cell = (2 * QA + da) * kCellMap + 2 * QB + db;
#pragma unroll
				for (int vv = 0; vv < 4; vv++) stage[(4 * khalf + vv) * ROW_LD + l32 * IMG_LD + cell] = acc[da][db][4 * vg + vv];
			}
		__syncthreads();
#pragma unroll
		for (int k = 0; k < OUT_ROWS * kCellImages * kCells / 4 / kGemmThreads; k++) {
			const int f = tid + kGemmThreads * k; // 16-byte group of the round
			const int row = f / (kCellImages * kCells / 4), g = f - row * (kCellImages * kCells / 4);
			const int img = g / (kCells / 4), cell0 = 4 * (g - img * (kCells / 4));
			const int i = i0 + 8 * vg + row;
			const float *src = stage + row * ROW_LD + img * IMG_LD + cell0;
			float4 val = make_float4(src[0], src[1], src[2], src[3]);
			if (i < p.I) {
				if (!split && out.biasI) {
					const float bi = out.biasI[i];
					val.x += bi, val.y += bi, val.z += bi, val.w += bi;
				}
				*reinterpret_cast<float4 *>(C + (size_t)i * out.ldc + (size_t)(n0 + img) * kCells + cell0) = val;
			}
		}
	}
}

} // namespace fitre
