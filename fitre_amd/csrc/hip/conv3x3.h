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
// The code avoids everything the compiler turns into control flow or private memory in
// the hot loops: no conditional loads or stores (invalid cells go to an out-of-range
// buffer offset, resp. a dummy LDS word), border zeroing with v_bfe/v_and instead of a
// select, staging registers as plain float arrays filled by unrolled loops.
#pragma once
#include "gemm_engine.h"

namespace fitre {

constexpr int kC3Tile = 128; // positions (and output channels) per workgroup tile

struct Conv3x3Params {
	const float *src;   // [Cred][N][A][B]
	const float *w;     // [Cout][Cin][3][3]
	uint32_t srcBytes, wBytes;
	int I;              // output channels of this product
	int cred;           // reduction channels
	int J;              // positions N*A*B
	int A, B;
	int perSplit;       // channel blocks (position-contiguous) or position stages (weight gradient) per split
	FastDiv divB, divA; // position -> (n, a, b)
};

// nine border bits of flat position m: bit ta*3+tb is set when (a+ta-1, b+tb-1) is inside the image
__device__ __forceinline__ uint32_t border_bits(const Conv3x3Params &p, uint32_t m)
{
	uint32_t q, b, n, a;
	p.divB.divmod(m, q, b);
	p.divA.divmod(q, n, a);
	uint32_t bits = 0;
#pragma unroll
	for (int ta = 0; ta < 3; ta++)
#pragma unroll
		for (int tb = 0; tb < 3; tb++) {
			int aa = (int)a + ta - 1, bb = (int)b + tb - 1;
			bool ok = ((int)m < p.J) & ((unsigned)aa < (unsigned)p.A) & ((unsigned)bb < (unsigned)p.B);
			bits |= ok ? (1u << (ta * 3 + tb)) : 0u;
		}
	return bits;
}

// value if bit `tap` of bits is set, +0.0f otherwise: sign-extending 1-bit field extract, then AND
__device__ __forceinline__ float keep_if(float value, uint32_t bits, int tap)
{
	int m = __builtin_amdgcn_sbfe((int)bits, tap, 1); // 0 or -1
	return __int_as_float(__float_as_int(value) & m);
}

// ---------------------------------------------------------------------------------
// position-contiguous product (forward: DX = false, input gradient: DX = true)
// CB reduction channels per block; MAXB = widest image row the window is sized for.
// ---------------------------------------------------------------------------------
// IT = channel rows per workgroup tile (128, or 64 for products with at most 64 output channels).
template <int CB, bool DX, int MAXB, int IT>
struct C3Pos {
	static constexpr int TM = IT / 64, TN = 2;
	// weights in LDS.  forward: 128 rows (output channel) x CB*9, odd row stride.
	// input gradient: CB rows (reduction channel) x 128*9 weights of the tile's channels.
	static constexpr int A_LD = DX ? (IT * 9 + 4) : (CB * 9 + 1);
	static constexpr int A_FLOATS = DX ? CB * A_LD : IT * A_LD;
	static constexpr int WQ = DX ? (IT * 9 / 4) : (CB * 9 / 4); // 4-float groups per LDS row
	static constexpr int WROWS = DX ? CB : IT;
	static constexpr int WGROUPS = WROWS * WQ;
	static constexpr int WE = (WGROUPS + kGemmThreads - 1) / kGemmThreads; // groups per thread
	static constexpr bool WEXACT = WGROUPS % kGemmThreads == 0;            // else the last round is partial
	static constexpr int A_DUMMY = A_FLOATS;                               // four spare words for the idle threads of that round
	// source window in LDS: CB channels x (128 + 2*(B+1)) cells, odd channel stride; one spare
	// word at the end swallows the writes of threads that have no cell
	static constexpr int WIN_MAX = kC3Tile + 2 * (MAXB + 1);
	static constexpr int WIN_LD = WIN_MAX + 1 - (WIN_MAX & 1); // odd
	static constexpr int B_FLOATS = CB * WIN_LD + 1;
	static constexpr int B_DUMMY = CB * WIN_LD;
	// window staging: each wave owns CB/4 channels, lanes walk the cells 64 at a time
	static constexpr int CH_PER_WAVE = CB / 4;
	static constexpr int XI = (WIN_MAX + 63) / 64;
	static constexpr int SE = CH_PER_WAVE * XI;
	static_assert(CB % 4 == 0, "CB must be a multiple of the wave count");
};

template <int CB, bool DX, bool VECW, int MAXB, int IT>
__global__ void __launch_bounds__(kGemmThreads)
conv3x3_pos_kernel(const Conv3x3Params p, const OutParams out)
{
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
	const int cbTotal = p.cred / CB;
	const int cbBeg = blockIdx.z * p.perSplit;
	const int cbEnd = (cbBeg + p.perSplit < cbTotal) ? cbBeg + p.perSplit : cbTotal;

	const __amdgpu_buffer_rsrc_t srcRs = make_rsrc(p.src, p.srcBytes);
	const __amdgpu_buffer_rsrc_t wRs = make_rsrc(p.w, p.wBytes);

	uint32_t bits[TN];
#pragma unroll
	for (int tn = 0; tn < TN; tn++) bits[tn] = border_bits(p, (uint32_t)(j0 + (wave & 1) * 64 + tn * 32 + l32));

	float wreg[K::WE * 4];
	float sreg[K::SE];
	const int rowLen = DX ? p.I * 9 : p.cred * 9;

	v16f acc[TM][TN];
#pragma unroll
	for (int tm = 0; tm < TM; tm++)
#pragma unroll
		for (int tn = 0; tn < TN; tn++)
#pragma unroll
			for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.f;

	// fragment base addresses; the channel pair (2*cp + khalf) and the tap are added per step
	const int rowA = (wave >> 1) * (IT / 2) + l32; // channel row inside the tile (+32 for tm = 1)
	const float *aBase = DX ? (As + khalf * K::A_LD + rowA * 9) : (As + rowA * K::A_LD + khalf * 9);
	constexpr int aTmStep = DX ? 32 * 9 : 32 * K::A_LD;
	constexpr int aCpStep = DX ? 2 * K::A_LD : 18;
	const float *bBase = Bs + khalf * K::WIN_LD + halo + (wave & 1) * 64 + l32;

// global -> registers for channel block CBI (a macro: the register arrays must stay registers)
#define C3_LOAD_BLOCK(CBI)                                                                                            \
	{                                                                                                                 \
		const int c0_ = (CBI) * CB;                                                                                   \
		_Pragma("unroll") for (int e = 0; e < K::WE; e++)                                                             \
		{                                                                                                             \
			const int idx = tid + kGemmThreads * e;                                                                   \
			const int row = idx / K::WQ, qd = idx - row * K::WQ;                                                      \
			/* forward: row = output channel, w[(i0+row)*cred*9 + c0*9 + 4*qd ..]                                    \
			   input gradient: row = reduction channel, w[(c0+row)*I*9 + i0*9 + 4*qd ..] */                           \
			const int rowG = DX ? (c0_ + row) : (i0 + row);                                                           \
			const int colG = DX ? (i0 * 9 + 4 * qd) : (c0_ * 9 + 4 * qd);                                             \
			const bool ok = (DX ? (colG < rowLen) : (rowG < p.I)) & (K::WEXACT | (idx < K::WGROUPS));                 \
			if constexpr (VECW) {                                                                                     \
				/* rows / columns past the tensor are clamped to element 0: their products land in                   \
				   accumulator rows that are never stored */                                                          \
				const float4 v4 = *reinterpret_cast<const float4 *>(p.w + (ok ? rowG * rowLen + colG : 0));           \
				wreg[4 * e + 0] = v4.x, wreg[4 * e + 1] = v4.y, wreg[4 * e + 2] = v4.z, wreg[4 * e + 3] = v4.w;       \
			} else {                                                                                                  \
				const uint32_t off = ok ? 4u * (uint32_t)(rowG * rowLen + colG) : kOutOfRange;                        \
				wreg[4 * e + 0] = buffer_load(wRs, off);                                                              \
				wreg[4 * e + 1] = buffer_load(wRs, ok ? off + 4u : kOutOfRange);                                      \
				wreg[4 * e + 2] = buffer_load(wRs, ok ? off + 8u : kOutOfRange);                                      \
				wreg[4 * e + 3] = buffer_load(wRs, ok ? off + 12u : kOutOfRange);                                     \
			}                                                                                                         \
		}                                                                                                             \
		_Pragma("unroll") for (int e = 0; e < K::SE; e++)                                                             \
		{                                                                                                             \
			const int c = wave * K::CH_PER_WAVE + e / K::XI, x = lane + 64 * (e % K::XI);                             \
			const int m = j0 - halo + x; /* flat position inside the channel plane */                                 \
			const bool ok = (x < win) & (m >= 0) & (m < plane);                                                       \
			sreg[e] = buffer_load(srcRs, ok ? 4u * (uint32_t)((c0_ + c) * plane + m) : kOutOfRange);                  \
		}                                                                                                             \
	}

	if (cbBeg < cbEnd) C3_LOAD_BLOCK(cbBeg);

	for (int cb = cbBeg; cb < cbEnd; cb++) {
		__syncthreads();
#pragma unroll
		for (int e = 0; e < K::WE; e++) {
			const int idx = tid + kGemmThreads * e;
			const int row = idx / K::WQ, qd = idx - row * K::WQ;
			float *dst = As + ((K::WEXACT | (idx < K::WGROUPS)) ? row * K::A_LD + 4 * qd : K::A_DUMMY);
			if constexpr (DX) { // A_LD is a multiple of four
				*reinterpret_cast<float4 *>(dst) = make_float4(wreg[4 * e], wreg[4 * e + 1], wreg[4 * e + 2], wreg[4 * e + 3]);
			} else {
				dst[0] = wreg[4 * e], dst[1] = wreg[4 * e + 1], dst[2] = wreg[4 * e + 2], dst[3] = wreg[4 * e + 3];
			}
		}
#pragma unroll
		for (int e = 0; e < K::SE; e++) {
			const int c = wave * K::CH_PER_WAVE + e / K::XI, x = lane + 64 * (e % K::XI);
			Bs[(x < win) ? c * K::WIN_LD + x : K::B_DUMMY] = sreg[e];
		}
		__syncthreads();
		if (cb + 1 < cbEnd) C3_LOAD_BLOCK(cb + 1);

		// 9 * CB/2 MFMA steps, step = (tap, channel pair); the fragments of step+1 are read
		// from LDS while the MFMAs of the current step run
		constexpr int STEPS = 9 * (CB / 2);
		float a[2][TM], b[2][TN];
#pragma unroll
		for (int tm = 0; tm < TM; tm++) a[0][tm] = aBase[tm * aTmStep + (DX ? 8 : 0)];
#pragma unroll
		for (int tn = 0; tn < TN; tn++) b[0][tn] = bBase[tn * 32 - p.B - 1];
#pragma unroll
		for (int step = 0; step < STEPS; step++) {
			const int cur = step & 1, nxt = cur ^ 1;
			const int tap = step / (CB / 2);
			float bm[TN];
#pragma unroll
			for (int tn = 0; tn < TN; tn++) bm[tn] = keep_if(b[cur][tn], bits[tn], tap);
			if (step + 1 < STEPS) {
				const int tapN = (step + 1) / (CB / 2), cpN = (step + 1) % (CB / 2);
				const int shiftN = (tapN / 3 - 1) * p.B + (tapN % 3 - 1);
				const int aTapN = DX ? (8 - tapN) : tapN;
#pragma unroll
				for (int tm = 0; tm < TM; tm++) a[nxt][tm] = aBase[tm * aTmStep + cpN * aCpStep + aTapN];
#pragma unroll
				for (int tn = 0; tn < TN; tn++) b[nxt][tn] = bBase[cpN * 2 * K::WIN_LD + tn * 32 + shiftN];
			}
#pragma unroll
			for (int tm = 0; tm < TM; tm++)
#pragma unroll
				for (int tn = 0; tn < TN; tn++)
					acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][tm], bm[tn], acc[tm][tn], 0, 0, 0);
			__builtin_amdgcn_sched_group_barrier(0x002, 2 * TN, 0);  // border masking of this step
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
// workgroups per compute unit would hold.  LDS stages are double buffered: one barrier per stage.
// MAXB: widest image row this instantiation's source window holds (32 or 64)
template <bool VECD, int MAXB>
__global__ void __launch_bounds__(kC3DwThreads)
conv3x3_dw_kernel(const Conv3x3Params p, const float *delta, uint32_t deltaBytes, const OutParams out)
{
	constexpr int T = kC3DwThreads;
	constexpr int WIN_MAX = kC3Stage + 2 * (MAXB + 1);
	constexpr int SRC_LD = WIN_MAX + 1 - (WIN_MAX & 1); // odd row stride of the source stage
	constexpr int X_DUMMY = kC3DwCin * SRC_LD;          // swallows the stores of threads without a cell
	constexpr int D_DUMMY = kC3Tile * kC3DeltaLd;
	constexpr int DGROUPS = kC3Tile * kC3Stage / 4;     // 4-float groups of delta per stage
	constexpr int DE = (DGROUPS + T - 1) / T;
	constexpr int XE = (kC3DwCin * WIN_MAX + T - 1) / T;
	static_assert(T % (kC3Stage / 4) == 0, "a thread keeps its column group in every round");
	__shared__ float Ds[2][D_DUMMY + 4];
	__shared__ float Xs[2][X_DUMMY + 1];
	__shared__ uint32_t Ms[2][kC3Stage];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int khalf = lane >> 5, l32 = lane & 31;
	const int ob = wave & 3, ta = wave >> 2; // output-channel block, tap row
	const int c0 = blockIdx.x * kC3DwCin, o0 = blockIdx.y * kC3Tile;
	const int halo = p.B + 1;
	const int win = kC3Stage + 2 * halo;
	const int plane = p.J;
	const int stagesTotal = (p.J + kC3Stage - 1) / kC3Stage;
	const int stBeg = blockIdx.z * p.perSplit;
	const int stEnd = (stBeg + p.perSplit < stagesTotal) ? stBeg + p.perSplit : stagesTotal;

	const __amdgpu_buffer_rsrc_t srcRs = make_rsrc(p.src, p.srcBytes);
	const __amdgpu_buffer_rsrc_t dRs = make_rsrc(delta, deltaBytes);

	// what this thread stages, fixed for all stages
	const int dCol = 4 * (tid % (kC3Stage / 4)); // first position of its delta groups inside the stage
	int dRowOff[DE];                             // (o0 + row) * plane, or -1 for no group / row past the tensor
	int dLds[DE];
#pragma unroll
	for (int e = 0; e < DE; e++) {
		const int idx = tid + T * e;
		const int row = idx / (kC3Stage / 4);
		const bool has = idx < DGROUPS;
		dRowOff[e] = (has & ((o0 + row) < p.I)) ? (o0 + row) * plane : -1;
		dLds[e] = has ? row * kC3DeltaLd + dCol : D_DUMMY;
	}
	int xChanOff[XE]; // (c0 + c) * plane, or -1
	int xRel[XE];     // cell position relative to the first position of the stage
	int xLds[XE];
#pragma unroll
	for (int e = 0; e < XE; e++) {
		const int idx = tid + T * e;
		const int c = idx / win, x = idx - c * win;
		const bool has = c < kC3DwCin;
		xChanOff[e] = (has & ((c0 + c) < p.cred)) ? (c0 + c) * plane : -1;
		xRel[e] = x - halo;
		xLds[e] = has ? c * SRC_LD + x : X_DUMMY;
	}

	float dreg[DE * 4];
	float xreg[XE];
	uint32_t mreg = 0;

#define C3_LOAD_STAGE(ST)                                                                                             \
	{                                                                                                                 \
		const int m0_ = (ST) * kC3Stage;                                                                              \
		_Pragma("unroll") for (int e = 0; e < DE; e++)                                                                \
		{                                                                                                             \
			const int m = m0_ + dCol;                                                                                 \
			if constexpr (VECD) { /* plane % 4 == 0: a group is inside the row or past its end as a whole */          \
				const bool ok = (dRowOff[e] >= 0) & (m < plane);                                                      \
				const float4 v4 = *reinterpret_cast<const float4 *>(delta + (ok ? dRowOff[e] + m : 0));               \
				dreg[4 * e + 0] = ok ? v4.x : 0.f, dreg[4 * e + 1] = ok ? v4.y : 0.f;                                 \
				dreg[4 * e + 2] = ok ? v4.z : 0.f, dreg[4 * e + 3] = ok ? v4.w : 0.f;                                 \
			} else {                                                                                                  \
				const bool rowOk = dRowOff[e] >= 0;                                                                   \
				const uint32_t off = 4u * (uint32_t)(dRowOff[e] + m);                                                 \
				dreg[4 * e + 0] = buffer_load(dRs, (rowOk & (m + 0 < plane)) ? off : kOutOfRange);                    \
				dreg[4 * e + 1] = buffer_load(dRs, (rowOk & (m + 1 < plane)) ? off + 4u : kOutOfRange);               \
				dreg[4 * e + 2] = buffer_load(dRs, (rowOk & (m + 2 < plane)) ? off + 8u : kOutOfRange);               \
				dreg[4 * e + 3] = buffer_load(dRs, (rowOk & (m + 3 < plane)) ? off + 12u : kOutOfRange);              \
			}                                                                                                         \
		}                                                                                                             \
		_Pragma("unroll") for (int e = 0; e < XE; e++)                                                                \
		{                                                                                                             \
			const int m = m0_ + xRel[e];                                                                              \
			const bool ok = (xChanOff[e] >= 0) & (m >= 0) & (m < plane);                                              \
			xreg[e] = buffer_load(srcRs, ok ? 4u * (uint32_t)(xChanOff[e] + m) : kOutOfRange);                        \
		}                                                                                                             \
		if (tid < kC3Stage) mreg = border_bits(p, (uint32_t)(m0_ + tid));                                             \
	}

#define C3_STORE_STAGE(BUF)                                                                                           \
	{                                                                                                                 \
		_Pragma("unroll") for (int e = 0; e < DE; e++)                                                                \
		{                                                                                                             \
			float *dst = Ds[BUF] + dLds[e];                                                                           \
			dst[0] = dreg[4 * e], dst[1] = dreg[4 * e + 1], dst[2] = dreg[4 * e + 2], dst[3] = dreg[4 * e + 3];       \
		}                                                                                                             \
		_Pragma("unroll") for (int e = 0; e < XE; e++) Xs[BUF][xLds[e]] = xreg[e];                                    \
		if (tid < kC3Stage) Ms[BUF][tid] = mreg;                                                                      \
	}

	v16f acc[3];
#pragma unroll
	for (int t = 0; t < 3; t++)
#pragma unroll
		for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

	const int aOff = (ob * 32 + l32) * kC3DeltaLd + khalf;
	const int bOff = l32 * SRC_LD + halo + khalf + (ta - 1) * p.B - 1; // tap (ta, 0); +1, +2 for the other two
	const int tap0 = ta * 3;

	if (stBeg < stEnd) {
		C3_LOAD_STAGE(stBeg);
		C3_STORE_STAGE(0);
	}
	__syncthreads();
	for (int st = stBeg; st < stEnd; st++) {
		const int buf = (st - stBeg) & 1;
		if (st + 1 < stEnd) C3_LOAD_STAGE(st + 1);

		// 32 MFMA steps of two positions; per step one delta fragment, the border bits of the two
		// positions and three shifted source fragments, read one step ahead
		const float *aBase = Ds[buf] + aOff;
		const float *bBase = Xs[buf] + bOff;
		const uint32_t *mBase = Ms[buf] + khalf;
		float fa[2], fb[2][3];
		uint32_t fbits[2];
		fa[0] = aBase[0];
		fbits[0] = mBase[0];
#pragma unroll
		for (int tb = 0; tb < 3; tb++) fb[0][tb] = bBase[tb];
#pragma unroll
		for (int s = 0; s < kC3Stage / 2; s++) {
			const int cur = s & 1, nxt = cur ^ 1;
			float bm[3];
#pragma unroll
			for (int tb = 0; tb < 3; tb++) bm[tb] = keep_if(fb[cur][tb], fbits[cur], tap0 + tb);
			if (s + 1 < kC3Stage / 2) {
				fa[nxt] = aBase[2 * (s + 1)];
				fbits[nxt] = mBase[2 * (s + 1)];
#pragma unroll
				for (int tb = 0; tb < 3; tb++) fb[nxt][tb] = bBase[2 * (s + 1) + tb];
			}
#pragma unroll
			for (int tb = 0; tb < 3; tb++) acc[tb] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur], bm[tb], acc[tb], 0, 0, 0);
			__builtin_amdgcn_sched_group_barrier(0x002, 6, 0); // border masking of this step
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
			__builtin_amdgcn_sched_group_barrier(0x100, 5, 0); // LDS reads of the next step
			__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
		}
		if (st + 1 < stEnd) C3_STORE_STAGE(buf ^ 1);
		__syncthreads();
	}
#undef C3_LOAD_STAGE
#undef C3_STORE_STAGE

	// ---- store: dW[o][c][tap]; this wave holds taps (ta, 0..2) of 32 output x 32 input channels ----
	float *C = out.C + (size_t)blockIdx.z * out.splitStride;
	const int c = c0 + l32;
	if (c < p.cred) {
#pragma unroll
		for (int v = 0; v < 16; v++) {
			const int o = o0 + ob * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
			if (o >= p.I) continue;
			float *dst = C + (size_t)o * out.ldc + c * 9 + tap0;
#pragma unroll
			for (int tb = 0; tb < 3; tb++) dst[tb] = acc[tb][v];
		}
	}
}

} // namespace fitre
