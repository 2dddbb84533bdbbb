// 3x3 / stride 1 / padding 1 convolutions on 2 x 2 maps as dense products.
//
// On a 2 x 2 map every output cell's window covers the whole map: of the nine taps of a window only
// four fall inside the image (16 of the 36 (tap, cell) pairs of a map), the rest multiply padding.
// Written with cell indices instead of taps the convolution is a dense linear map per image,
//
//   y[(co, ab)][n] = sum over (ci, a'b')  Weff[(co, ab)][(ci, a'b')] * x[(ci, a'b')][n],
//   Weff[(co, ab)][(ci, a'b')] = W[co][ci][a' - a + 1][b' - b + 1]        (ab = 2a + b, a'b' = 2a' + b'),
//
// with no structural zeros left, so its two gradients are plain products on the tile engine at
// 16/36 of the multiply-adds of the nine-tap form:
//
//   input gradient   dx[(ci, a'b')][n]        = sum over (co, ab)  Weff[(co, ab)][(ci, a'b')] * delta[(co, ab)][n]
//   weight gradient  dWeff[(co, ab)][(ci, a'b')] = sum over n      delta[(co, ab)][n] * x[(ci, a'b')][n]
//                    dW[co][ci][ta][tb] = sum of the (at most four) dWeff entries whose cells differ by the tap.
//
// The tensors stay in the [C][N][2][2] layout: operands read it in place ("quad" operands: four
// consecutive rows or reduction indices are the four cells of one map), and the input gradient's
// tile stores put a lane's four rows -- the four cells of a map -- into one 16-byte group.
#pragma once
#include "conv_common.h"

namespace fitre {

struct QuadParams {
	const float *p;
	uint32_t bytes;  // extent of the tensor
	int groupStride; // floats between consecutive channels: 4 * samples
	int rows;
};

typedef float quad4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ quad4f buffer_load4(__amdgpu_buffer_rsrc_t r, uint32_t byteOffset)
{
	return __builtin_bit_cast(quad4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byteOffset, 0, 0));
}

// element(row = (c, q), k = n) = p[c * groupStride + 4 * k + q].  A thread moves 16-byte groups: the four rows
// of one channel at one k; the groups of a channel over the k of a slice are contiguous in memory, and the
// lanes of a wave run along them.  The tensor must be 16-byte aligned.
template <int ROWS, int BK>
struct QuadRowOp {
	static constexpr int E = ROWS * BK / kGemmThreads; // floats per thread
	static constexpr int G = E / 4;                     // 16-byte groups per thread
	static constexpr int CSTEP = kGemmThreads / BK;     // channels between a thread's groups
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	static_assert(E % 4 == 0, "a thread moves whole groups");
	typedef QuadParams Params;
	__amdgpu_buffer_rsrc_t rsrc;
	int kL, cL;
	uint32_t grpOff[G]; // float offset of channel (row0 / 4 + cL + CSTEP * g), or out of range
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		rsrc = make_rsrc(pr.p, pr.bytes);
		kL = tid % BK;
		cL = tid / BK;
#pragma unroll
		for (int g = 0; g < G; g++) {
			const int row = row0 + 4 * (cL + CSTEP * g);
			grpOff[g] = (row < pr.rows) ? (uint32_t)((row >> 2) * pr.groupStride) : kOutOfRange; // rows % 4 == 0
		}
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
		const int k = k0 + kL;
#pragma unroll
		for (int g = 0; g < G; g++) {
			const uint32_t off = ((grpOff[g] != kOutOfRange) & (k < kend)) ? 4u * (grpOff[g] + 4u * (uint32_t)k) : kOutOfRange;
			const quad4f v = (off != kOutOfRange) ? buffer_load4(rsrc, off) : quad4f{ 0.f, 0.f, 0.f, 0.f };
			r[4 * g] = v.x, r[4 * g + 1] = v.y, r[4 * g + 2] = v.z, r[4 * g + 3] = v.w;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int g = 0; g < G; g++)
#pragma unroll
			for (int q = 0; q < 4; q++) lds[kL * LD + 4 * (cL + CSTEP * g) + q] = r[4 * g + q];
	}
};

// element(row = n, k = (c, q)) = p[c * groupStride + 4 * row + q].  A thread moves 16-byte groups: one row at
// the four k of one channel; the lanes of a wave run along the rows, whose groups are contiguous in memory.
template <int ROWS, int BK>
struct QuadKOp {
	static constexpr int E = ROWS * BK / kGemmThreads;
	static constexpr int G = E / 4;
	static constexpr int CSTEP = kGemmThreads / ROWS; // channels between a thread's groups
	static constexpr int LD = LdsStride<ROWS, BK>::value;
	static_assert(E % 4 == 0 && BK % 4 == 0, "a thread moves whole groups");
	typedef QuadParams Params;
	__amdgpu_buffer_rsrc_t rsrc;
	int rowL, cL, groupStride;
	uint32_t rowOff;
	bool rowOk;
	__device__ __forceinline__ void init(const Params &pr, int row0, int tid)
	{
		rsrc = make_rsrc(pr.p, pr.bytes);
		rowL = tid % ROWS;
		cL = tid / ROWS;
		const int row = row0 + rowL;
		rowOk = row < pr.rows;
		rowOff = 4u * (uint32_t)row;
		groupStride = pr.groupStride;
	}
	__device__ __forceinline__ void load(int k0, int kend, float (&r)[E]) const
	{
#pragma unroll
		for (int g = 0; g < G; g++) {
			const int k = k0 + 4 * (cL + CSTEP * g); // first of the channel's four reduction indices (kend % 4 == 0)
			const bool ok = rowOk & (k < kend);
			const quad4f v = ok ? buffer_load4(rsrc, 4u * ((uint32_t)((k >> 2) * groupStride) + rowOff)) : quad4f{ 0.f, 0.f, 0.f, 0.f };
			r[4 * g] = v.x, r[4 * g + 1] = v.y, r[4 * g + 2] = v.z, r[4 * g + 3] = v.w;
		}
	}
	__device__ __forceinline__ void store(float *lds, const float (&r)[E]) const
	{
#pragma unroll
		for (int g = 0; g < G; g++)
#pragma unroll
			for (int q = 0; q < 4; q++) lds[(4 * (cL + CSTEP * g) + q) * LD + rowL] = r[4 * g + q];
	}
};

// tap index 3 * ta + tb that links output cell ab to input cell a'b' (always inside the window on a 2 x 2 map)
__host__ __device__ inline int quad_tap(int ab, int apbp)
{
	const int a = ab >> 1, b = ab & 1, ap = apbp >> 1, bp = apbp & 1;
	return 3 * (ap - a + 1) + (bp - b + 1);
}

// Weff[(co, ab)][(ci, a'b')] from W[co][ci][3][3]: one thread per (co, ci), lanes along ci
__global__ void __launch_bounds__(256) quad_weff_build_kernel(const float *w, int cin, int cout, float *weff)
{
	const int ci = blockIdx.x * blockDim.x + threadIdx.x, co = blockIdx.y;
	if (ci >= cin) return;
	float t[9];
	const float *src = w + ((size_t)co * cin + ci) * 9;
#pragma unroll
	for (int k = 0; k < 9; k++) t[k] = src[k];
#pragma unroll
	for (int ab = 0; ab < 4; ab++) {
		float4 v = make_float4(t[quad_tap(ab, 0)], t[quad_tap(ab, 1)], t[quad_tap(ab, 2)], t[quad_tap(ab, 3)]);
		*reinterpret_cast<float4 *>(weff + ((size_t)(co * 4 + ab) * cin + ci) * 4) = v;
	}
}

// dW[co][ci][3][3] from dWeff[(co, ab)][(ci, a'b')]: the entries of one tap are added in the order of ab
__global__ void __launch_bounds__(256) quad_fold_kernel(const float *dweff, int cin, int cout, float *dW)
{
	const int ci = blockIdx.x * blockDim.x + threadIdx.x, co = blockIdx.y;
	if (ci >= cin) return;
	float e[4][4];
#pragma unroll
	for (int ab = 0; ab < 4; ab++) {
		const float4 v = *reinterpret_cast<const float4 *>(dweff + ((size_t)(co * 4 + ab) * cin + ci) * 4);
		e[ab][0] = v.x, e[ab][1] = v.y, e[ab][2] = v.z, e[ab][3] = v.w;
	}
	float t[9];
#pragma unroll
	for (int k = 0; k < 9; k++) t[k] = 0.f;
#pragma unroll
	for (int ab = 0; ab < 4; ab++)
#pragma unroll
		for (int q = 0; q < 4; q++) t[quad_tap(ab, q)] += e[ab][q];
	float *dst = dW + ((size_t)co * cin + ci) * 9;
#pragma unroll
	for (int k = 0; k < 9; k++) dst[k] = t[k];
}

static inline bool quad_eligible(const fitre_conv_shape *s)
{
	return s->ksize == 3 && s->stride == 1 && s->padding == 1 && s->inA == 2 && s->inB == 2 && s->outA == 2 && s->outB == 2 &&
	       s->inChannels >= 64 && s->outChannels >= 64 && s->inChannels % 4 == 0 && s->samples >= 32 &&
	       (double)s->inChannels * s->outChannels * 16.0 < 1.0e9;
}

static inline size_t quad_weff_bytes(const fitre_conv_shape *s)
{
	return sizeof(float) * 16 * (size_t)s->inChannels * s->outChannels; // a multiple of 256 bytes
}

// 64 x 64 tiles; as many reduction ranges as give about four workgroups per compute unit (forceSplits > 0: that many)
static inline GemmPlan quad_plan(int I, int J, int R, int forceSplits = 0)
{
	GemmPlan p;
	p.bm = p.bn = 64;
	const long tiles = (long)((I + 63) / 64) * ((J + 63) / 64);
	long splits = forceSplits > 0 ? forceSplits : (4L * device_compute_units() + tiles / 2) / tiles;
	if (splits > R / 128) splits = R / 128; // at least 128 reduction indices per range
	if (splits < 1) splits = 1;
	p.bk = (R / splits >= 256 && splits == 1) ? 64 : 32;
	long chunk = (R + splits - 1) / splits;
	chunk = ((chunk + p.bk - 1) / p.bk) * p.bk;
	p.splits = (int)((R + chunk - 1) / chunk);
	p.kChunk = (int)chunk;
	p.wsBytes = p.splits > 1 ? (size_t)p.splits * I * J * sizeof(float) : 0;
	p.estimateUs = 0.0;
	return p;
}

// input gradient: I = 4 Cin, J = samples, R = 4 Cout
static inline size_t quad_input_grad_workspace(const fitre_conv_shape *s)
{
	return quad_weff_bytes(s) + quad_plan(4 * s->inChannels, s->samples, 4 * s->outChannels).wsBytes;
}
// weight gradient: I = 4 Cout, J = 4 Cin, R = samples
static inline size_t quad_weight_grad_workspace(const fitre_conv_shape *s)
{
	return quad_weff_bytes(s) + quad_plan(4 * s->outChannels, 4 * s->inChannels, s->samples).wsBytes;
}

// One tile launch of the engine with the split partials left in `ws` when leftSplits is given
// (they are stored in the layout of the result, so a consumer can add them slab by slab).
template <template <int, int> class OpA, template <int, int> class OpB, int BM, int BN, int BK, class PA, class PB>
static int quad_launch_tile(const PA &pa, const PB &pb, const OutParams &out, int I, int J, int R, const GemmPlan &plan, void *ws,
                            int kernelClass, double flops, int *leftSplits)
{
	typedef TileCfg<BM, BN, BK> Cfg;
	dim3 grid((J + BN - 1) / BN, (I + BM - 1) / BM, plan.splits);
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "gemm grid %u x %u x %u too large", grid.x, grid.y, grid.z);
	OutParams part = out;
	part.splitStride = 0;
	if (plan.splits > 1) {
		part.C = (float *)ws;
		part.splitStride = (long)I * J;
		if (!out.quadLd) part.ldc = J;
	}
	{
		LaunchScope scope(kernelClass, flops, 6);
		mfma_gemm_kernel<Cfg, OpA<BM, BK>, OpB<BN, BK>><<<grid, kGemmThreads, 0, stream()>>>(pa, pb, part, I, J, R, plan.kChunk);
	}
	if (leftSplits) *leftSplits = plan.splits;
	if (plan.splits > 1 && !leftSplits) {
		OutParams fin = out;
		fin.splitStride = 0;
		if (out.quadLd) {
			// the partials are already in the result's layout: a flat sum
			fin.quadLd = 0;
			fin.ldc = (long)I * J;
			launch_splitk_reduce((const float *)ws, plan.splits, 1, I * J, fin);
		} else {
			launch_splitk_reduce((const float *)ws, plan.splits, I, J, fin);
		}
	}
	return check_launch("mfma_gemm_kernel (2x2 maps)");
}

template <template <int, int> class OpA, template <int, int> class OpB, class PA, class PB>
static int quad_launch(const PA &pa, const PB &pb, const OutParams &out, int I, int J, int R, void *ws, size_t wsBytes, int kernelClass,
                       double flops, int *leftSplits)
{
	// Both products are small (2 GFLOP at the benchmark's shapes) and latency-bound on the engine's usual plan;
	// measured sweep (512 x 512 channels, 256 images): 64 x 64 tiles with about four workgroups per compute unit,
	// deep reduction slices: weight gradient 46 -> 36 us (unsplit, slices of 64), input gradient 43 -> 40 us
	// (eight splits, slices of 32).
	const GemmPlan ideal = quad_plan(I, J, R);
	GemmPlan plan = ideal;
	if (plan.splits > 1 && (!ws || wsBytes < plan.wsBytes)) plan = quad_plan(I, J, R, 1); // no room for partials: unsplit
	if (plan.wsBytes > 0 && (!ws || (((uintptr_t)ws) & 15) || wsBytes < plan.wsBytes))
		return fail(FITRE_E_WORKSPACE, "split-K workspace of %zu bytes is null, misaligned or smaller than the %zu required", wsBytes,
		            plan.wsBytes);
	if (plan.bk == 64) return quad_launch_tile<OpA, OpB, 64, 64, 64>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, leftSplits);
	if (plan.bk == 32) return quad_launch_tile<OpA, OpB, 64, 64, 32>(pa, pb, out, I, J, R, plan, ws, kernelClass, flops, leftSplits);
	return fail(FITRE_E_UNSUPPORTED, "no tile %d x %d x %d", plan.bm, plan.bn, plan.bk);
}

// Weff from W (what the input gradient multiplies by); `weff` holds quad_weff_bytes(s)
static int quad_prepare_weights(const fitre_conv_shape *s, const float *w, float *weff)
{
	const int cin = s->inChannels, cout = s->outChannels;
	LaunchScope scope(FITRE_KC_PERMUTE, 4.0 * 25.0 * (double)cin * cout);
	quad_weff_build_kernel<<<dim3((cin + 255) / 256, cout), 256, 0, stream()>>>(w, cin, cout, weff);
	return check_launch("quad_weff_build_kernel");
}

// dx[ci][n][a'b'] from delta[co][n][ab] and W.  prepared: Weff built beforehand (quad_prepare_weights), or null:
// then it is built here at the head of ws, which is laid out [Weff | split partials].
static int quad_input_grad(const fitre_conv_shape *s, const float *delta, const float *w, const float *prepared, float *dx, void *ws,
                           size_t wsBytes, int *leftSplits, float **partials)
{
	const int cin = s->inChannels, cout = s->outChannels, N = s->samples;
	const size_t weffBytes = quad_weff_bytes(s);
	const float *weff = prepared;
	float *rest = (float *)ws;
	size_t restBytes = wsBytes;
	if (!prepared) {
		if (!ws || (((uintptr_t)ws) & 15) || wsBytes < weffBytes)
			return fail(FITRE_E_WORKSPACE, "2x2-map input gradient: workspace of %zu bytes is null, misaligned or smaller than the %zu required",
			            wsBytes, quad_input_grad_workspace(s));
		int rc = quad_prepare_weights(s, w, (float *)ws);
		if (rc) return rc;
		weff = (const float *)ws;
		rest = (float *)((char *)ws + weffBytes);
		restBytes = wsBytes - weffBytes;
	}
	const int I = 4 * cin, J = N, R = 4 * cout;
	PlainParams pa{ weff, (uint32_t)weffBytes, I, I };
	QuadParams pb{ delta, (uint32_t)((size_t)cout * N * 4 * sizeof(float)), 4 * N, J };
	OutParams out{ dx, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	out.quadLd = 4L * J;
	if (partials) *partials = rest;
	return quad_launch<PlainRowContig, QuadKOp>(pa, pb, out, I, J, R, rest, restBytes, FITRE_KC_CONV_DX, conv_flops(s), leftSplits);
}

// dW[co][ci][3][3] from x[ci][n][a'b'] and delta[co][n][ab].  ws: [dWeff | split partials].
// x2 / delta2: a second (input, delta) pair whose product is added before the fold (the R operator's sums of two products)
static int quad_weight_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws, size_t wsBytes,
                            const float *x2 = nullptr, const float *delta2 = nullptr)
{
	const int cin = s->inChannels, cout = s->outChannels, N = s->samples;
	const size_t weffBytes = quad_weff_bytes(s);
	if (!ws || (((uintptr_t)ws) & 15) || wsBytes < weffBytes)
		return fail(FITRE_E_WORKSPACE, "2x2-map weight gradient: workspace of %zu bytes is null, misaligned or smaller than the %zu required",
		            wsBytes, quad_weight_grad_workspace(s));
	float *dweff = (float *)ws;
	float *rest = (float *)((char *)ws + weffBytes);
	const int I = 4 * cout, J = 4 * cin, R = N;
	QuadParams pa{ delta, (uint32_t)((size_t)cout * N * 4 * sizeof(float)), 4 * N, I };
	QuadParams pb{ x, (uint32_t)((size_t)cin * N * 4 * sizeof(float)), 4 * N, J };
	OutParams out{ dweff, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	int rc = quad_launch<QuadRowOp, QuadRowOp>(pa, pb, out, I, J, R, rest, wsBytes - weffBytes, FITRE_KC_CONV_DW, conv_flops(s), nullptr);
	if (rc) return rc;
	if (x2) {
		pa.p = delta2, pb.p = x2;
		out.beta = 1.f;
		rc = quad_launch<QuadRowOp, QuadRowOp>(pa, pb, out, I, J, R, rest, wsBytes - weffBytes, FITRE_KC_CONV_DW, conv_flops(s), nullptr);
		if (rc) return rc;
	}
	{
		LaunchScope scope(FITRE_KC_PERMUTE, 4.0 * 25.0 * (double)cin * cout);
		quad_fold_kernel<<<dim3((cin + 255) / 256, cout), 256, 0, stream()>>>(dweff, cin, cout, dW);
	}
	return check_launch("quad_fold_kernel");
}

} // namespace fitre
