// Convolution gradients of layers with very few channels (LeNet: 3 -> 6 and 6 -> 16 with 5 x 5 windows).
//
// With six or sixteen output channels a 32 x 32 MFMA block is a tenth to a half full and the tile engine's
// 64-row tiles a tenth: such layers are bound by launch and load latency there, not by arithmetic (two
// GFLOP per pass at batch 1024).  Here both gradients are computed with ordinary vector multiply-adds by
// workgroups that keep one image at a time in LDS:
//
//   input gradient   one thread per (input channel, four neighbouring cells of a row) with the channel uniform over
//                    a wave: the image's delta (all output channels, zero border) in LDS, read in 16-byte groups,
//                    the weights through scalar loads;
//   weight gradient  one thread per (patch index k = (ci, ta, tb), position slice), Cout accumulators in
//                    registers; per position one LDS read of the input cell and Cout / 4 broadcast 16-byte
//                    reads of delta (stored [position][channel]); a patch index of constant one yields the bias
//                    gradient in the same loop; slices are added in a fixed order, every workgroup leaves one
//                    partial Cout x (K + 1) block and a reduction sums the blocks in workgroup order -- the
//                    result does not depend on scheduling.
#pragma once
#include "conv_common.h"

namespace fitre {

constexpr int kThinMaxChannels = 16; // accumulators a thread holds
constexpr int kThinLdsFloats = 12288; // 48 KB of staging per workgroup

struct ThinConvParams {
	const float *x;     // [Cin][N][inA][inB]   (weight gradient)
	const float *delta; // [Cout][N][outA][outB]
	const float *w;     // [Cout][Cin][k][k]     (input gradient)
	int cin, cout, samples, inA, inB, outA, outB, ksize, stride, pad;
	int imagesPerGroup;
	int ciPerGroup; // input gradient: input channels per workgroup
	int parts, rowsPerUnit, unitsPerGroup; // weight gradient: bands of output rows per image, rows per band, units per workgroup
	int xRowWords;                         // weight gradient: words per row of the bordered input in LDS
	FastDiv divInB, divOutB, divK, divKK, divCells, divOcells;
	FastDiv divPlane, divPB; // input gradient: bordered delta plane and its row length
	FastDiv divGroups;       // input gradient: groups of four cells per image row
	FastDiv divPBx;          // weight gradient: row length of the bordered input
	FastDiv divXPlane[2], divDPos[2]; // weight gradient: bordered input plane / positions of a full band [0] and of an image's last band [1]
};

// ---- input gradient (stride 1): dx[ci][n][a][b] = sum_co sum_taps W[co][ci][ta][tb] * delta[co][n][a - ta + p][b - tb + p]
// One workgroup per (image, group of input channels).  The image's delta (all output channels) sits in LDS with a
// zero border of k - 1 - p cells, so that no tap needs a bounds check, in rows padded to a multiple of four words.
// A thread owns FOUR neighbouring cells of a row (columns 4g .. 4g + 3): the k + 3 delta words a window row needs
// for them are two aligned 16-byte reads (k = 5) that feed 4 k multiply-adds -- a quarter of the LDS traffic of a
// thread per cell, which is what bounds this kernel.  A wave works on ONE input channel at a time, so the weights
// W[co][ci][.] come through scalar loads and a multiply-add takes a scalar operand.
// KS: window extent known at compile time (the tap loops are unrolled), 0: any
constexpr int kThinDxCells = 4; // cells of a row per thread
__host__ __device__ inline int thin_dx_row_words(int inB, int ks) { return (((inB + 3) & ~3) + ks - 1 + 3) & ~3; }

//
// FOLD: the layer below ends in a 2 x 2 / stride 2 max pool (no padding) behind an activation, and this gradient is taken
// on through both in the same launch (functions/cnn_backward.cu:560-640 does them as steps of their own): a thread's four
// cells are four windows of the map below, two rows of eight cells, which it routes and scales exactly as
// maxpool2_backward_kernel does -- the first largest cell of a window in memory order takes the gradient, then times
// f'(.).  inB is even, so a pair of windows is one 16-byte group of each row.
struct ThinPoolFold {
	const float *zIn;  // the activation's input where its derivative needs it, else null
	const float *zAct; // the activation's output = the pool's input, [Cin][N][2 inA][2 inB]
	float *dxPool;     // gradient at the pool's input, or null
	float *dxAct;      // gradient at the activation's input
	int actFun;
};

template <int KS, bool FOLD>
__global__ void __launch_bounds__(256)
thin_input_grad_kernel(const ThinConvParams p, const float *__restrict__ w, const float *__restrict__ delta, float *__restrict__ dx,
                       const ThinPoolFold fold)
{
	extern __shared__ __align__(16) float thin_lds[];
	const int tid = threadIdx.x;
	const int ks = KS > 0 ? KS : p.ksize;
	const int cells = p.inA * p.inB, ocells = p.outA * p.outB, taps = ks * ks;
	const int border = ks - 1 - p.pad;
	const int PB = thin_dx_row_words(p.inB, ks), plane = (p.inA + ks - 1) * PB;
	const int n = blockIdx.x;
	const size_t oplane = (size_t)p.samples * ocells, iplane = (size_t)p.samples * cells;
	// delta with its border, eight loads of a thread in flight at a time
	const int total = p.cout * plane;
	for (int base = tid; base < total; base += 256 * 8) {
		float v[8];
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int i = base + 256 * u;
			uint32_t co, q, r, c;
			p.divPlane.divmod((uint32_t)(i < total ? i : 0), co, q);
			p.divPB.divmod(q, r, c);
			const int oa = (int)r - border, ob = (int)c - border;
			const bool ok = (i < total) & ((unsigned)oa < (unsigned)p.outA) & ((unsigned)ob < (unsigned)p.outB);
			v[u] = ok ? delta[(size_t)co * oplane + (size_t)n * ocells + oa * p.outB + ob] : 0.f;
		}
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int i = base + 256 * u;
			if (i < total) thin_lds[i] = v[u];
		}
	}
	__syncthreads();
	const int lane = tid & 63, wave = tid >> 6;
	const int groups = (p.inB + kThinDxCells - 1) / kThinDxCells; // column groups of a row
	const int items = p.inA * groups;                              // threads' worth of work per input channel
	const int chunks = (items + 63) / 64, chunk = (items + chunks - 1) / chunks; // items per wave, evenly
	const int ci0 = blockIdx.y * p.ciPerGroup;
	const int ciN = (p.cin - ci0 < p.ciPerGroup) ? p.cin - ci0 : p.ciPerGroup;
	for (int task = wave; task < ciN * chunks; task += 4) {
		const int ci = __builtin_amdgcn_readfirstlane(ci0 + task / chunks);
		const int part = task % chunks;
		const int item = part * chunk + lane;
		const bool live = lane < chunk && item < items;
		uint32_t a, g;
		p.divGroups.divmod((uint32_t)(live ? item : 0), a, g);
		const int b0 = kThinDxCells * (int)g;
		// delta[a - ta + p][b - tb + p] is the bordered cell [a + (k - 1 - ta)][b + (k - 1 - tb)]
		const float *d0 = thin_lds + (int)a * PB + b0;
		const float *wci = w + (size_t)ci * taps;
		// the map below, on its way while the sums run
		const int bigB = 2 * p.inB;
		const size_t below = ((size_t)ci * p.samples + n) * (size_t)(4 * cells) + (size_t)(2 * (int)a) * bigB + 2 * b0;
		float4 zo[2][2], zi[2][2];
		if constexpr (FOLD) {
#pragma unroll
			for (int h = 0; h < 2; h++)
#pragma unroll
				for (int r = 0; r < 2; r++) {
					zo[h][r] = make_float4(0.f, 0.f, 0.f, 0.f);
					if (live && b0 + 2 * h < p.inB) zo[h][r] = *reinterpret_cast<const float4 *>(fold.zAct + below + (size_t)r * bigB + 4 * h);
					zi[h][r] = zo[h][r];
					if (fold.zIn && live && b0 + 2 * h < p.inB) zi[h][r] = *reinterpret_cast<const float4 *>(fold.zIn + below + (size_t)r * bigB + 4 * h);
				}
		}
		float acc[kThinDxCells] = { 0.f, 0.f, 0.f, 0.f };
		for (int co = 0; co < p.cout; co++) {
			const float *wk = wci + (size_t)co * p.cin * taps;
			const float *dco = d0 + co * plane;
			if constexpr (KS > 0) {
				constexpr int WORDS = (KS + kThinDxCells - 1 + 3) & ~3; // delta words of a window row, in whole 16-byte groups
#pragma unroll
				for (int ta = 0; ta < KS; ta++) {
					const float4 *drow = reinterpret_cast<const float4 *>(dco + (KS - 1 - ta) * PB);
					float d[WORDS];
#pragma unroll
					for (int q = 0; q < WORDS / 4; q++) {
						const float4 v4 = drow[q];
						d[4 * q] = v4.x, d[4 * q + 1] = v4.y, d[4 * q + 2] = v4.z, d[4 * q + 3] = v4.w;
					}
#pragma unroll
					for (int tb = 0; tb < KS; tb++) {
						const float wv = wk[ta * KS + tb];
#pragma unroll
						for (int jj = 0; jj < kThinDxCells; jj++) acc[jj] = fmaf(wv, d[jj + KS - 1 - tb], acc[jj]);
					}
				}
			} else {
				for (int ta = 0; ta < ks; ta++)
					for (int tb = 0; tb < ks; tb++) {
						const float wv = wk[ta * ks + tb];
						const float *dd = dco + (ks - 1 - ta) * PB + (ks - 1 - tb);
#pragma unroll
						for (int jj = 0; jj < kThinDxCells; jj++) acc[jj] = fmaf(wv, dd[jj], acc[jj]);
					}
			}
		}
		if (live) {
			float *out = dx + (size_t)ci * iplane + (size_t)n * cells + (int)a * p.inB + b0;
#pragma unroll
			for (int jj = 0; jj < kThinDxCells; jj++)
				if (b0 + jj < p.inB) out[jj] = acc[jj];
			if constexpr (FOLD) {
#pragma unroll
				for (int h = 0; h < 2; h++) {
					if (b0 + 2 * h >= p.inB) continue;
					const float4 r0 = zo[h][0], r1 = zo[h][1];
					float4 g0 = make_float4(0.f, 0.f, 0.f, 0.f), g1 = g0;
					int arg = scan2x2(r0.x, r0.y, r1.x, r1.y);
					if (arg == 0) g0.x = acc[2 * h];
					else if (arg == 1) g0.y = acc[2 * h];
					else if (arg == 2) g1.x = acc[2 * h];
					else if (arg == 3) g1.y = acc[2 * h];
					arg = scan2x2(r0.z, r0.w, r1.z, r1.w);
					if (arg == 0) g0.z = acc[2 * h + 1];
					else if (arg == 1) g0.w = acc[2 * h + 1];
					else if (arg == 2) g1.z = acc[2 * h + 1];
					else if (arg == 3) g1.w = acc[2 * h + 1];
					const size_t at = below + 4 * h;
					if (fold.dxPool) {
						*reinterpret_cast<float4 *>(fold.dxPool + at) = g0;
						*reinterpret_cast<float4 *>(fold.dxPool + at + bigB) = g1;
					}
					const float4 i0 = zi[h][0], i1 = zi[h][1];
					g0.x *= act_derivative(fold.actFun, i0.x, r0.x);
					g0.y *= act_derivative(fold.actFun, i0.y, r0.y);
					g0.z *= act_derivative(fold.actFun, i0.z, r0.z);
					g0.w *= act_derivative(fold.actFun, i0.w, r0.w);
					g1.x *= act_derivative(fold.actFun, i1.x, r1.x);
					g1.y *= act_derivative(fold.actFun, i1.y, r1.y);
					g1.z *= act_derivative(fold.actFun, i1.z, r1.z);
					g1.w *= act_derivative(fold.actFun, i1.w, r1.w);
					*reinterpret_cast<float4 *>(fold.dxAct + at) = g0;
					*reinterpret_cast<float4 *>(fold.dxAct + at + bigB) = g1;
				}
			}
		}
	}
}

// ---- weight gradient: dW[co][k] = sum over positions of delta[co][position] * patch[position][k], and with the
// patch extended by a constant one (index k = K) the bias gradient db[co] = sum of delta[co][.] comes out of the
// same loop (functions/cnn_backward.cu:662-689 takes it with a ones-vector product of its own).
// blockDim = 512: thread (k, slice), slices = 512 / (K + 1).  A workgroup walks its units (image, band of output
// rows) one at a time.  LDS: [x rows of the band, zero border of `pad` cells | delta of the band as
// [position][COUT]]; afterwards the slice sums.
template <int COUT>
__global__ void __launch_bounds__(512)
thin_weight_grad_kernel(const ThinConvParams p, const float *__restrict__ x, const float *__restrict__ delta, float *__restrict__ partial)
{
	extern __shared__ __align__(16) float thin_lds[];
	const int tid = threadIdx.x;
	const int K = p.cin * p.ksize * p.ksize, K1 = K + 1;
	const int cells = p.inA * p.inB, ocells = p.outA * p.outB;
	const int slices = 512 / K1; // >= 1 (host checks K + 1 <= 512)
	const int PBx = p.xRowWords; // >= inB + 2 * pad, chosen so that the lanes' patch offsets spread over the LDS banks
	const int xRowsMax = (p.rowsPerUnit - 1) * p.stride + p.ksize;
	float *xs = thin_lds;
	float *ds = thin_lds + ((p.cin * xRowsMax * PBx + 3) & ~3);
	const int k = tid % K1, slice = tid / K1;
	const bool live = slice < slices, ones = k == K;
	uint32_t ci, tap, ta, tb;
	p.divKK.divmod((uint32_t)(ones ? 0 : k), ci, tap);
	p.divK.divmod(tap, ta, tb);
	float acc[COUT];
#pragma unroll
	for (int c = 0; c < COUT; c++) acc[c] = 0.f;
	const size_t oplane = (size_t)p.samples * ocells, iplane = (size_t)p.samples * cells;
	const int units = p.samples * p.parts;
	const int u0 = blockIdx.x * p.unitsPerGroup;
	const int u1 = (u0 + p.unitsPerGroup < units) ? u0 + p.unitsPerGroup : units;
	for (int unit = u0; unit < u1; unit++) {
		const int n = unit / p.parts, part = unit - n * p.parts;
		const int oa0 = part * p.rowsPerUnit;
		const int rows = (p.outA - oa0 < p.rowsPerUnit) ? p.outA - oa0 : p.rowsPerUnit;
		const int xRows = (rows - 1) * p.stride + p.ksize;
		const int a0 = oa0 * p.stride - p.pad; // input row of the band's first bordered row
		__syncthreads(); // the previous unit's readers are done
		// eight loads of a thread in flight at a time
		const int xPlane = xRows * PBx, xTotal = p.cin * xPlane, dPos = rows * p.outB, dTotal = COUT * dPos;
		const FastDiv divXPlane = p.divXPlane[rows == p.rowsPerUnit ? 0 : 1], divDPos = p.divDPos[rows == p.rowsPerUnit ? 0 : 1];
		for (int base = tid; base < xTotal; base += 512 * 8) {
			float v[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int i = base + 512 * u;
				uint32_t c, q, r, col;
				divXPlane.divmod((uint32_t)(i < xTotal ? i : 0), c, q);
				p.divPBx.divmod(q, r, col);
				const int a = a0 + (int)r, b = (int)col - p.pad;
				const bool ok = (i < xTotal) & ((unsigned)a < (unsigned)p.inA) & ((unsigned)b < (unsigned)p.inB);
				v[u] = ok ? x[(size_t)c * iplane + (size_t)n * cells + a * p.inB + b] : 0.f;
			}
#pragma unroll
			for (int u = 0; u < 8; u++)
				if (base + 512 * u < xTotal) xs[base + 512 * u] = v[u];
		}
		for (int base = tid; base < dTotal; base += 512 * 8) {
			float v[8];
			uint32_t c[8], q[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int i = base + 512 * u; // reads contiguous along the positions of a channel
				divDPos.divmod((uint32_t)(i < dTotal ? i : 0), c[u], q[u]);
				v[u] = (i < dTotal && (int)c[u] < p.cout) ? delta[(size_t)c[u] * oplane + (size_t)n * ocells + oa0 * p.outB + q[u]] : 0.f;
			}
#pragma unroll
			for (int u = 0; u < 8; u++)
				if (base + 512 * u < dTotal) ds[q[u] * COUT + c[u]] = v[u];
		}
		__syncthreads();
		if (live) {
			// A slice takes a run of consecutive positions, row segment by row segment: position (r, ob) of the band
			// reads the bordered cell [r * stride + ta][ob * stride + tb], so inside a segment both operands advance
			// by constants.
			const int run = (dPos + slices - 1) / slices;
			int q = slice * run;
			const int qEnd = (q + run < dPos) ? q + run : dPos;
			uint32_t r = 0, ob = 0;
			p.divOutB.divmod((uint32_t)(q < dPos ? q : 0), r, ob);
			const float *xrow = xs + ((int)ci * xRows + (int)ta + (int)r * p.stride) * PBx + (int)tb;
			while (q < qEnd) {
				int segEnd = q + (p.outB - (int)ob);
				segEnd = segEnd < qEnd ? segEnd : qEnd;
				const float *xp = xrow + (int)ob * p.stride;
				const float4 *dq = reinterpret_cast<const float4 *>(ds + q * COUT);
				for (; q < segEnd; q++) {
					const float xv = ones ? 1.f : *xp;
					xp += p.stride;
#pragma unroll
					for (int g = 0; g < COUT / 4; g++) {
						const float4 d = dq[g];
						acc[4 * g] = fmaf(d.x, xv, acc[4 * g]);
						acc[4 * g + 1] = fmaf(d.y, xv, acc[4 * g + 1]);
						acc[4 * g + 2] = fmaf(d.z, xv, acc[4 * g + 2]);
						acc[4 * g + 3] = fmaf(d.w, xv, acc[4 * g + 3]);
					}
					dq += COUT / 4;
				}
				ob = 0;
				xrow += p.stride * PBx;
			}
		}
	}
	// slices of one k are added in slice order; the sums go out as one Cout x (K + 1) block per workgroup
	__syncthreads();
	float *red = thin_lds; // [slice][k][COUT]
	if (live) {
#pragma unroll
		for (int c = 0; c < COUT; c++) red[(slice * K1 + k) * COUT + c] = acc[c];
	}
	__syncthreads();
	float *out = partial + (size_t)blockIdx.x * p.cout * K1;
	for (int i = tid; i < p.cout * K1; i += 512) {
		const int c = i / K1, kk = i - c * K1;
		float s = 0.f;
		for (int sl = 0; sl < slices; sl++) s += red[(sl * K1 + kk) * COUT + c];
		out[i] = s;
	}
}

// dW[c][k] (k < K) and db[c] (k = K) = sum over the workgroups' blocks, in workgroup order: sixteen phases each add
// every sixteenth block in double precision and are combined in phase order.
struct ThinReduceJob {
	const float *partial;
	int groups, cout, K;
	float *dW, *db;
};
__device__ __forceinline__ void thin_dw_reduce_block(const float *partial, int groups, int cout, int K, float *dW, float *db, int block)
{
	__shared__ double part[16][17];
	const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
	const int total = cout * (K + 1);
	const int idx = block * 16 + tx;
	double acc = 0.0;
	if (idx < total)
		for (int s = ty; s < groups; s += 16) acc += (double)partial[(size_t)s * total + idx];
	part[ty][tx] = acc;
	__syncthreads();
	if (ty == 0 && idx < total) {
		double sum = 0.0;
#pragma unroll
		for (int q = 0; q < 16; q++) sum += part[q][tx];
		const int c = idx / (K + 1), kk = idx - c * (K + 1);
		if (kk < K) dW[(size_t)c * K + kk] = (float)sum;
		else if (db) db[c] = (float)sum;
	}
}
__global__ void __launch_bounds__(256) thin_dw_reduce_kernel(const float *partial, int groups, int cout, int K, float *dW, float *db)
{
	thin_dw_reduce_block(partial, groups, cout, K, dW, db, blockIdx.x);
}
// The reductions of several layers in one launch (each workgroup finds its layer by its index): the same sums in the
// same order as one launch per layer.
constexpr int kThinReduceJobs = 4;
struct ThinReduceBatch {
	ThinReduceJob job[kThinReduceJobs];
	int first[kThinReduceJobs + 1]; // first workgroup of each job
	int jobs;
};
__global__ void __launch_bounds__(256) thin_dw_reduce_batch_kernel(const ThinReduceBatch b)
{
	const int block = blockIdx.x;
	// constant indices only: a run-time index into the argument block would copy it to scratch memory
	if (b.jobs > 3 && block >= b.first[3]) thin_dw_reduce_block(b.job[3].partial, b.job[3].groups, b.job[3].cout, b.job[3].K, b.job[3].dW, b.job[3].db, block - b.first[3]);
	else if (b.jobs > 2 && block >= b.first[2]) thin_dw_reduce_block(b.job[2].partial, b.job[2].groups, b.job[2].cout, b.job[2].K, b.job[2].dW, b.job[2].db, block - b.first[2]);
	else if (b.jobs > 1 && block >= b.first[1]) thin_dw_reduce_block(b.job[1].partial, b.job[1].groups, b.job[1].cout, b.job[1].K, b.job[1].dW, b.job[1].db, block - b.first[1]);
	else thin_dw_reduce_block(b.job[0].partial, b.job[0].groups, b.job[0].cout, b.job[0].K, b.job[0].dW, b.job[0].db, block);
}

// Words per row of the weight gradient's bordered input in LDS.  The lanes of a wave are consecutive patch indices
// (tb fastest, then ta): they read words tb + ta * row apart, so a row length that is a multiple of 32 puts all of
// a window's rows on the same banks (LeNet's first layer: 32-wide images, 15 lanes per bank).  The row is padded
// until the window's k * k offsets cover as many different banks as they can.
static inline int thin_dw_row_words(const fitre_conv_shape *s)
{
	const int base = s->inB + 2 * s->padding, k = s->ksize;
	int best = base, bestBanks = -1;
	for (int row = base; row < base + 32; row++) {
		unsigned used = 0;
		for (int ta = 0; ta < k; ta++)
			for (int tb = 0; tb < k; tb++) used |= 1u << ((tb + ta * row) & 31);
		const int banks = __builtin_popcount(used);
		if (banks > bestBanks) bestBanks = banks, best = row;
		if (banks == (k * k < 32 ? k * k : 32)) break;
	}
	return best;
}

static inline ThinConvParams thin_params(const fitre_conv_shape *s)
{
	ThinConvParams p;
	p.x = p.delta = p.w = nullptr;
	p.cin = s->inChannels, p.cout = s->outChannels, p.samples = s->samples;
	p.inA = s->inA, p.inB = s->inB, p.outA = s->outA, p.outB = s->outB;
	p.ksize = s->ksize, p.stride = s->stride, p.pad = s->padding;
	p.imagesPerGroup = 1;
	p.ciPerGroup = 1;
	p.parts = 1, p.rowsPerUnit = s->outA, p.unitsPerGroup = 1;
	p.xRowWords = thin_dw_row_words(s);
	p.divPBx = FastDiv((uint32_t)p.xRowWords);
	p.divPB = FastDiv((uint32_t)thin_dx_row_words(s->inB, s->ksize));
	p.divPlane = FastDiv((uint32_t)((s->inA + s->ksize - 1) * thin_dx_row_words(s->inB, s->ksize)));
	p.divGroups = FastDiv((uint32_t)((s->inB + 3) / 4));
	p.divInB = FastDiv((uint32_t)s->inB);
	p.divOutB = FastDiv((uint32_t)s->outB);
	p.divK = FastDiv((uint32_t)s->ksize);
	p.divKK = FastDiv((uint32_t)(s->ksize * s->ksize));
	p.divCells = FastDiv((uint32_t)(s->inA * s->inB));
	p.divOcells = FastDiv((uint32_t)(s->outA * s->outB));
	return p;
}

// ---- input gradient --------------------------------------------------------------------------------------------
constexpr int kThinDxLdsFloats = 15360; // 60 KB: the bordered delta of one image
static inline int thin_dx_lds_floats(const fitre_conv_shape *s)
{
	return s->outChannels * (s->inA + s->ksize - 1) * thin_dx_row_words(s->inB, s->ksize);
}
static inline bool thin_dx_eligible(const fitre_conv_shape *s)
{
	return s->stride == 1 && s->padding <= s->ksize - 1 && s->inChannels <= kThinMaxChannels && s->outChannels <= 32 &&
	       s->ksize <= 7 && s->inChannels * s->outChannels <= 256 && thin_dx_lds_floats(s) <= kThinDxLdsFloats;
}
// the pool / activation fold on top: whole 16-byte groups of the map below
static inline bool thin_dx_fold_eligible(const fitre_conv_shape *s) { return thin_dx_eligible(s) && s->inB % 2 == 0; }
static int launch_thin_dx(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, const ThinPoolFold *fold = nullptr)
{
	ThinConvParams p = thin_params(s);
	// enough workgroups for two per compute unit where the batch alone does not give them
	int groupsY = (2 * device_compute_units() + s->samples - 1) / s->samples;
	if (groupsY > s->inChannels) groupsY = s->inChannels;
	if (groupsY < 1) groupsY = 1;
	p.ciPerGroup = (s->inChannels + groupsY - 1) / groupsY;
	groupsY = (s->inChannels + p.ciPerGroup - 1) / p.ciPerGroup;
	const dim3 grid((unsigned)s->samples, (unsigned)groupsY);
	const size_t lds = sizeof(float) * (size_t)thin_dx_lds_floats(s);
	LaunchScope scope(FITRE_KC_CONV_DX, conv_flops(s), 0);
	if (fold) {
		if (s->ksize == 5) thin_input_grad_kernel<5, true><<<grid, 256, lds, stream()>>>(p, w, delta, dx, *fold);
		else if (s->ksize == 3) thin_input_grad_kernel<3, true><<<grid, 256, lds, stream()>>>(p, w, delta, dx, *fold);
		else thin_input_grad_kernel<0, true><<<grid, 256, lds, stream()>>>(p, w, delta, dx, *fold);
	} else {
		const ThinPoolFold none{};
		if (s->ksize == 5) thin_input_grad_kernel<5, false><<<grid, 256, lds, stream()>>>(p, w, delta, dx, none);
		else if (s->ksize == 3) thin_input_grad_kernel<3, false><<<grid, 256, lds, stream()>>>(p, w, delta, dx, none);
		else thin_input_grad_kernel<0, false><<<grid, 256, lds, stream()>>>(p, w, delta, dx, none);
	}
	return check_launch("thin_input_grad_kernel");
}

// ---- weight gradient -------------------------------------------------------------------------------------------
static inline int thin_dw_pad(int cout) { return cout <= 8 ? 8 : 16; }
struct ThinDwPlan {
	int parts, rowsPerUnit, unitsPerGroup, groups;
};
// One workgroup per compute unit where the batch gives that many images; below that the images are cut into bands
// of output rows (at least four rows each).
static inline ThinDwPlan thin_dw_plan(const fitre_conv_shape *s)
{
	const int target = device_compute_units();
	ThinDwPlan pl;
	pl.parts = (target + s->samples - 1) / s->samples;
	if (pl.parts > s->outA / 4) pl.parts = s->outA / 4;
	if (pl.parts < 1) pl.parts = 1;
	pl.rowsPerUnit = (s->outA + pl.parts - 1) / pl.parts;
	pl.parts = (s->outA + pl.rowsPerUnit - 1) / pl.rowsPerUnit;
	const long units = (long)s->samples * pl.parts;
	long groups = 2L * target < units ? 2L * target : units;
	pl.unitsPerGroup = (int)((units + groups - 1) / groups);
	pl.groups = (int)((units + pl.unitsPerGroup - 1) / pl.unitsPerGroup);
	return pl;
}
static inline size_t thin_dw_lds_floats(const fitre_conv_shape *s)
{
	const ThinDwPlan pl = thin_dw_plan(s);
	const int K1 = s->inChannels * s->ksize * s->ksize + 1, cp = thin_dw_pad(s->outChannels);
	const int xRows = (pl.rowsPerUnit - 1) * s->stride + s->ksize;
	const size_t stage = (size_t)((s->inChannels * xRows * thin_dw_row_words(s) + 3) & ~3) + (size_t)pl.rowsPerUnit * s->outB * cp;
	const size_t red = (size_t)(512 / K1) * K1 * cp;
	return stage > red ? stage : red;
}
static inline bool thin_dw_general_eligible(const fitre_conv_shape *s)
{
	const int K = s->inChannels * s->ksize * s->ksize;
	return s->outChannels <= kThinMaxChannels && K < 512 && K >= 16 && thin_dw_lds_floats(s) <= (size_t)kThinLdsFloats;
}
// sized for the largest number of workgroups any batch size gets, so that a buffer laid out for a model's full
// batch also serves its partial batches
static inline size_t thin_dw_general_workspace(const fitre_conv_shape *s)
{
	return sizeof(float) * 2 * (size_t)device_compute_units() * s->outChannels * (s->inChannels * s->ksize * s->ksize + 1);
}
// Reductions held back so that several layers' share one launch (fitre_hip_thin_reduce_defer / _flush)
static bool g_thin_reduce_deferred = false;
static ThinReduceBatch g_thin_reduce = {};
static double g_thin_reduce_bytes = 0.0;
static int thin_reduce_flush()
{
	if (g_thin_reduce.jobs == 0) return FITRE_OK;
	{
		LaunchScope scope(FITRE_KC_SPLITK_REDUCE, g_thin_reduce_bytes);
		if (g_thin_reduce.jobs == 1) {
			const ThinReduceJob &j = g_thin_reduce.job[0];
			thin_dw_reduce_kernel<<<(unsigned)g_thin_reduce.first[1], 256, 0, stream()>>>(j.partial, j.groups, j.cout, j.K, j.dW, j.db);
		} else {
			thin_dw_reduce_batch_kernel<<<(unsigned)g_thin_reduce.first[g_thin_reduce.jobs], 256, 0, stream()>>>(g_thin_reduce);
		}
	}
	g_thin_reduce.jobs = 0;
	g_thin_reduce.first[0] = 0;
	g_thin_reduce_bytes = 0.0;
	return check_launch("thin_dw_reduce_batch_kernel");
}

// db may be null
static int launch_thin_dw_general(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, float *db, void *ws)
{
	ThinConvParams p = thin_params(s);
	const ThinDwPlan pl = thin_dw_plan(s);
	p.parts = pl.parts, p.rowsPerUnit = pl.rowsPerUnit, p.unitsPerGroup = pl.unitsPerGroup;
	const int lastRows = s->outA - (pl.parts - 1) * pl.rowsPerUnit;
	const int bandRows[2] = { pl.rowsPerUnit, lastRows };
	for (int i = 0; i < 2; i++) {
		p.divXPlane[i] = FastDiv((uint32_t)(((bandRows[i] - 1) * s->stride + s->ksize) * p.xRowWords));
		p.divDPos[i] = FastDiv((uint32_t)(bandRows[i] * s->outB));
	}
	const int K = s->inChannels * s->ksize * s->ksize;
	const size_t lds = sizeof(float) * thin_dw_lds_floats(s);
	{
		LaunchScope scope(FITRE_KC_CONV_DW, conv_flops(s), 0);
		if (thin_dw_pad(s->outChannels) == 8) thin_weight_grad_kernel<8><<<pl.groups, 512, lds, stream()>>>(p, x, delta, (float *)ws);
		else thin_weight_grad_kernel<16><<<pl.groups, 512, lds, stream()>>>(p, x, delta, (float *)ws);
	}
	const ThinReduceJob job{ (const float *)ws, pl.groups, s->outChannels, K, dW, db };
	if (g_thin_reduce_deferred) {
		// the caller keeps this workspace untouched until fitre_hip_thin_reduce_flush()
		if (g_thin_reduce.jobs == kThinReduceJobs) {
			const int rc = thin_reduce_flush();
			if (rc) return rc;
		}
		const int j = g_thin_reduce.jobs++;
		g_thin_reduce.job[j] = job;
		g_thin_reduce.first[j + 1] = g_thin_reduce.first[j] + (s->outChannels * (K + 1) + 15) / 16;
		g_thin_reduce_bytes += 4.0 * (double)s->outChannels * (K + 1) * (pl.groups + 1);
		return check_launch("thin_weight_grad_kernel");
	}
	{
		const int total = s->outChannels * (K + 1);
		LaunchScope scope(FITRE_KC_SPLITK_REDUCE, 4.0 * (double)total * (pl.groups + 1));
		thin_dw_reduce_kernel<<<(total + 15) / 16, 256, 0, stream()>>>(job.partial, job.groups, job.cout, job.K, job.dW, job.db);
	}
	return check_launch("thin_weight_grad_kernel");
}

} // namespace fitre
