// Convolution forward / weight gradient / input gradient and the general
// column-major GEMM, all on the fp32-MFMA tile engine.
#include <stdlib.h>
#include "conv3x3.h"
#include "conv_cell.h"
#include "conv_common.h"
#include "conv_quad.h"
#include "conv_thin.h"
#include "linear_small.h"
#include "linear_tail.h"
#include "linear_skinny.h"

namespace fitre {

// Device table of the patch decode, owned by the layer and grown on demand; every use is
// ordered on the layer's stream.
static unsigned long long *g_ktables[kMaxLanes] = {}; // one per lane
static int g_ktable_caps[kMaxLanes] = {};

void conv_gemm_release()
{
	for (int i = 0; i < kMaxLanes; i++) {
		if (g_ktables[i]) (void)hipFree(g_ktables[i]);
		g_ktables[i] = nullptr, g_ktable_caps[i] = 0;
	}
}

// bn = tile extent along the positions, which fixes how the waves stride through a slice
static int attach_patch_table(PatchGeom &g, int bn)
{
	const int kstep = kGemmThreads / bn;
	const int padded = ((g.patchLen + kGemmBK - 1) / kGemmBK) * kGemmBK;
	unsigned long long *&g_ktable = g_ktables[lane()];
	int &g_ktable_cap = g_ktable_caps[lane()];
	if (padded > g_ktable_cap) {
		FITRE_HIP_TRY(hipStreamSynchronize(stream()));
		if (g_ktable) FITRE_HIP_TRY(hipFree(g_ktable));
		g_ktable = nullptr;
		g_ktable_cap = 0;
		int cap = padded < 16384 ? 16384 : padded;
		FITRE_HIP_TRY(hipMalloc((void **)&g_ktable, sizeof(unsigned long long) * (size_t)cap));
		g_ktable_cap = cap;
	}
	patch_table_kernel<<<(padded + 255) / 256, 256, 0, stream()>>>(g_ktable, padded, g.patchLen, g.chanStride, g.srcB,
	                                                             g.divTaps, g.divK, kGemmBK, kstep);
	g.ktable = g_ktable;
	return check_launch("patch_table_kernel");
}


// ---- 3x3 / stride 1 / pad 1 fast paths -------------------------------------------------------
constexpr int kC3CB = 8; // reduction channels per LDS block of the position-contiguous kernels

struct BlockPlan {
	int splits, perSplit;
	size_t wsBytes;
};

// Splits a reduction of nBlocks equal blocks (blockUs microseconds of matrix-pipe time each) over
// workgroups so that the compute units are evenly loaded; same cost model as plan_gemm.
static BlockPlan plan_blocks_search(long tiles, long nBlocks, double blockUs, int residentPerCu, long I, long J, long cus)
{
	BlockPlan best{ 1, (int)nBlocks, 0 };
	double bestT = 1e30;
	for (long s = 1; s <= nBlocks && s <= 1024; s++) {
		long per = (nBlocks + s - 1) / s;
		long eff = (nBlocks + per - 1) / per;
		long groups = tiles * eff;
		long perCu = (groups + cus - 1) / cus;
		double e = perCu >= residentPerCu ? 0.85 : (perCu * 2 >= residentPerCu + 1 ? 0.72 : 0.55);
		double t = (double)perCu * (double)per * blockUs / e + 3.0;
		if (eff > 1) t += 4.0 + (double)(eff + 1) * (double)I * (double)J * 4.0 / 3.0e6;
		if (t < bestT) {
			bestT = t;
			best.splits = (int)eff;
			best.perSplit = (int)per;
			best.wsBytes = eff > 1 ? (size_t)eff * I * J * sizeof(float) : 0;
		}
	}
	return best;
}

// memo of the search (a layer asks for the same plan on every call)
static BlockPlan plan_blocks(long tiles, long nBlocks, double blockUs, int residentPerCu, long I, long J, int cus)
{
	struct Entry {
		long tiles, nBlocks, I, J;
		double blockUs;
		int resident, cus;
		BlockPlan plan;
	};
	constexpr int kEntries = 64;
	static Entry table[kEntries];
	static int used = 0, next = 0;
	for (int i = 0; i < used; i++) {
		const Entry &e = table[i];
		if (e.tiles == tiles && e.nBlocks == nBlocks && e.I == I && e.J == J && e.blockUs == blockUs && e.resident == residentPerCu &&
		    e.cus == cus)
			return e.plan;
	}
	Entry e{ tiles,         nBlocks, I, J, blockUs, residentPerCu,
		     cus,           plan_blocks_search(tiles, nBlocks, blockUs, residentPerCu, I, J, cus) };
	table[next] = e;
	next = (next + 1) % kEntries;
	if (used < kEntries) used++;
	return e.plan;
}

static BlockPlan fit_blocks(BlockPlan p, long nBlocks, long I, long J, const void *ws, size_t wsBytes)
{
	if (p.splits <= 1) return p;
	size_t per = (size_t)I * J * sizeof(float);
	long fit = ws ? (long)(wsBytes / per) : 0;
	if (fit >= p.splits) return p;
	long s = fit >= 2 ? fit : 1;
	p.perSplit = (int)((nBlocks + s - 1) / s);
	p.splits = (int)((nBlocks + p.perSplit - 1) / p.perSplit);
	p.wsBytes = p.splits > 1 ? (size_t)p.splits * per : 0;
	return p;
}

static bool c3_geometry(const fitre_conv_shape *s)
{
	return s->ksize == 3 && s->stride == 1 && s->padding == 1 && s->inB <= 64 && s->outA == s->inA && s->outB == s->inB;
}
// forward: reduce over Cin; input gradient: reduce over Cout
static bool c3_pos_eligible(const fitre_conv_shape *s, bool dx)
{
	int cred = dx ? s->outChannels : s->inChannels;
	return c3_geometry(s) && cred % kC3CB == 0 && c3_pad_window(s->inA, s->inB) <= (s->inB <= 32 ? 384 : 512);
}
static bool c3_dw_eligible(const fitre_conv_shape *s)
{
	return c3_geometry(s) && s->inChannels >= 16 && s->outChannels >= 32 && s->inB <= 32 &&
	       ((long)s->samples * s->inA * s->inB) % kC3Stage == 0;
}

// cus: compute units of the lane the kernel is launched on (0 = the selected lane)
// pairs = 2: a sum of two products of this shape in one launch (twice the reduction)
// 4 x 4 maps: the kernels of conv_cell.h, which leave out the taps that fall outside the image
static bool cell_geometry(const fitre_conv_shape *s) { return c3_geometry(s) && s->inA == kCellMap && s->inB == kCellMap; }
// 8 x 8 maps: the weight gradient's stage is half a map of two images
static bool cell8_geometry(const fitre_conv_shape *s) { return c3_geometry(s) && s->inA == kCell8Map && s->inB == kCell8Map && s->samples % 2 == 0; }
// the position-contiguous products on 4 x 4 maps in the cell form: whole tiles of 32 images (a second (source,
// weights) pair continues the reduction)
static bool cell_pos_eligible(const fitre_conv_shape *s, bool dx)
{
	return cell_geometry(s) && s->samples % kCellImages == 0 && (dx ? s->outChannels : s->inChannels) % kCellCB == 0;
}
static BlockPlan c3_pos_plan(const fitre_conv_shape *s, bool dx, int cus = 0, int pairs = 1)
{
	if (cus <= 0) cus = lane_compute_units();
	long I = dx ? s->inChannels : s->outChannels, J = (long)s->samples * s->inA * s->inB;
	long cred = dx ? s->outChannels : s->inChannels;
	if (cell_pos_eligible(s, dx)) {
		const long tiles = ((I + kCellIT - 1) / kCellIT) * (s->samples / kCellImages);
		const double blockUs = (kCellCB / 2.0) * 25.0 * 64.0 / 2400.0; // reduction pairs x MFMAs per wave and pair x 64 cycles
		return plan_blocks(tiles, pairs * cred / kCellCB, blockUs, 2, I, J, cus);
	}
	long it = I <= 64 ? 64 : kC3Tile;
	long tiles = ((I + it - 1) / it) * ((J + kC3Tile - 1) / kC3Tile);
	double blockUs = (9.0 * kC3CB / 2.0) * (it / 32.0) * 64.0 / 2400.0; // MFMA steps x blocks per wave x 64 cycles
	return plan_blocks(tiles, pairs * cred / kC3CB, blockUs, it == 64 ? 3 : 2, I, J, cus);
}
// cus == 0: the units fitre_hip_weight_grad_share leaves these kernels (all of the lane's, or three quarters where the
// caller runs them beside a chain of other kernels)
static BlockPlan c3_dw_plan(const fitre_conv_shape *s, int cus = 0, int pairs = 1)
{
	if (cus <= 0) cus = weight_grad_units();
	long J = (long)s->samples * s->inA * s->inB;
	long tiles = ((s->inChannels + kC3DwCin - 1) / kC3DwCin) * ((s->outChannels + kC3Tile - 1) / kC3Tile);
	double stageUs = (kC3Stage / 2.0) * 9.0 * 64.0 / 2400.0; // three waves per SIMD, three MFMAs per step each
	if (cell_geometry(s)) stageUs *= 100.0 / 144.0;
	if (cell8_geometry(s)) stageUs *= 84.0 / 96.0;
	return plan_blocks(tiles, pairs * ((J + kC3Stage - 1) / kC3Stage), stageUs, 1, s->outChannels, (long)s->inChannels * 9, cus);
}
static size_t c3_pos_workspace(const fitre_conv_shape *s, bool dx, int pairs = 1)
{
	size_t a = c3_pos_plan(s, dx, device_compute_units(), pairs).wsBytes, b = c3_pos_plan(s, dx, lane_compute_units_min(), pairs).wsBytes;
	return a > b ? a : b;
}
static size_t c3_dw_workspace(const fitre_conv_shape *s, int pairs = 1)
{
	size_t a = c3_dw_plan(s, device_compute_units(), pairs).wsBytes, b = c3_dw_plan(s, lane_compute_units_min(), pairs).wsBytes;
	a = a > b ? a : b;
	for (int eighths = 4; eighths < 8; eighths++) {
		const size_t c = c3_dw_plan(s, share_of_units(lane_compute_units_min(), eighths), pairs).wsBytes;
		a = a > c ? a : c;
	}
	return a;
}

// leftSplits (may be null): when the product is split, skip the reduction launch, leave the partial
// results in ws and report their number there (the caller's consumer sums them)
template <bool DX>
static int launch_c3_pos(const fitre_conv_shape *s, const float *src, const float *w, const float *bias, float *outPtr, void *ws,
                         size_t wsBytes, int *leftSplits = nullptr, const float *src2 = nullptr, const float *w2 = nullptr)
{
	const int I = DX ? s->inChannels : s->outChannels, cred = DX ? s->outChannels : s->inChannels;
	const int J = s->samples * s->inA * s->inB;
	const int pairs = src2 ? 2 : 1;
	BlockPlan plan = fit_blocks(c3_pos_plan(s, DX, 0, pairs), pairs * cred / kC3CB, I, J, ws, wsBytes);
	if (plan.wsBytes > 0 && (((uintptr_t)ws) & 3)) return fail(FITRE_E_WORKSPACE, "split workspace is misaligned");
	Conv3x3Params p;
	p.src = src;
	p.w = w;
	p.src2 = src2;
	p.w2 = w2;
	p.srcBytes = (uint32_t)((size_t)cred * J * sizeof(float));
	p.wBytes = (uint32_t)((size_t)s->outChannels * s->inChannels * 9 * sizeof(float));
	p.I = I;
	p.cred = cred;
	p.J = J;
	p.A = s->inA;
	p.B = s->inB;
	p.perSplit = plan.perSplit;
	p.divB = FastDiv((uint32_t)s->inB);
	p.divA = FastDiv((uint32_t)s->inA);
	OutParams out{ outPtr, (long)J, 0, bias, nullptr, 1.f, 0.f };
	OutParams part = out;
	if (plan.splits > 1) {
		part.C = (float *)ws;
		part.splitStride = (long)I * J;
	}
	const bool vecw = ((((uintptr_t)w) & 15) == 0) && (!w2 || (((uintptr_t)w2) & 15) == 0) && (DX ? (I % 4 == 0) : true);
	// (the cell kernel stores 16-byte groups; a plan made for it also fits the nine-tap kernel: same block size)
	if (cell_pos_eligible(s, DX) && (((uintptr_t)part.C) & 15) == 0) {
		dim3 grid((unsigned)(s->samples / kCellImages), (unsigned)((I + kCellIT - 1) / kCellIT), (unsigned)plan.splits);
		if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "conv3x3 grid too large");
		{
			LaunchScope scope(DX ? FITRE_KC_CONV_DX : FITRE_KC_CONV_FWD, pairs * conv_flops(s), 7);
			if (vecw) conv3x3_cell_dx_kernel<DX, true><<<grid, kGemmThreads, 0, stream()>>>(p, part);
			else conv3x3_cell_dx_kernel<DX, false><<<grid, kGemmThreads, 0, stream()>>>(p, part);
		}
		if (leftSplits) *leftSplits = plan.splits;
		if (plan.splits > 1 && !leftSplits) launch_splitk_reduce((const float *)ws, plan.splits, I, J, out);
		return check_launch("conv3x3_cell_dx_kernel");
	}
	const int it = I <= 64 ? 64 : kC3Tile;
	dim3 grid((J + kC3Tile - 1) / kC3Tile, (I + it - 1) / it, plan.splits);
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "conv3x3 grid too large");
	{
		LaunchScope scope(DX ? FITRE_KC_CONV_DX : FITRE_KC_CONV_FWD, pairs * conv_flops(s), it == 64 ? 2 : 4);
		const bool narrow = s->inB <= 32;
#define C3_LAUNCH(V, MB, IT_) conv3x3_pos_kernel<kC3CB, DX, V, MB, IT_><<<grid, kGemmThreads, 0, stream()>>>(p, part)
		if (it == 64) {
			if (vecw && narrow) C3_LAUNCH(true, 32, 64);
			else if (vecw) C3_LAUNCH(true, 64, 64);
			else if (narrow) C3_LAUNCH(false, 32, 64);
			else C3_LAUNCH(false, 64, 64);
		} else {
			if (vecw && narrow) C3_LAUNCH(true, 32, 128);
			else if (vecw) C3_LAUNCH(true, 64, 128);
			else if (narrow) C3_LAUNCH(false, 32, 128);
			else C3_LAUNCH(false, 64, 128);
		}
#undef C3_LAUNCH
	}
	if (leftSplits) *leftSplits = plan.splits;
	if (plan.splits > 1 && !leftSplits) launch_splitk_reduce((const float *)ws, plan.splits, I, J, out);
	return check_launch("conv3x3_pos_kernel");
}

// x2 / delta2 (may be null): a second (input, delta) pair whose product is added to the first one's
static int launch_c3_dw(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws, size_t wsBytes,
                        const float *x2 = nullptr, const float *delta2 = nullptr)
{
	const int I = s->outChannels, cin = s->inChannels, K = cin * 9;
	const int J = s->samples * s->inA * s->inB;
	const int pairs = x2 ? 2 : 1;
	const int stages = pairs * ((J + kC3Stage - 1) / kC3Stage);
	BlockPlan plan = fit_blocks(c3_dw_plan(s, 0, pairs), stages, I, K, ws, wsBytes);
	if (plan.wsBytes > 0 && (((uintptr_t)ws) & 3)) return fail(FITRE_E_WORKSPACE, "split workspace is misaligned");
	Conv3x3Params p;
	p.src2 = x2;
	p.w2 = delta2;
	p.src = x;
	p.w = nullptr;
	p.srcBytes = (uint32_t)((size_t)cin * J * sizeof(float));
	p.wBytes = 0;
	p.I = I;
	p.cred = cin;
	p.J = J;
	p.A = s->inA;
	p.B = s->inB;
	p.perSplit = plan.perSplit;
	p.divB = FastDiv((uint32_t)s->inB);
	p.divA = FastDiv((uint32_t)s->inA);
	OutParams out{ dW, (long)K, 0, nullptr, nullptr, 1.f, 0.f };
	OutParams part = out;
	if (plan.splits > 1) {
		part.C = (float *)ws;
		part.splitStride = (long)I * K;
	}
	const uint32_t deltaBytes = (uint32_t)((size_t)I * J * sizeof(float));
	const bool vecd = ((((uintptr_t)delta) & 15) == 0) && (!delta2 || (((uintptr_t)delta2) & 15) == 0) && (J % 4 == 0);
	dim3 grid((cin + kC3DwCin - 1) / kC3DwCin, (I + kC3Tile - 1) / kC3Tile, plan.splits);
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "conv3x3 grid too large");
	{
		LaunchScope scope(FITRE_KC_CONV_DW, pairs * conv_flops(s),
		                  cell_geometry(s) ? 7 : (cell8_geometry(s) ? 8 : 4));
		const bool narrow = s->inB >= 2 && s->inB <= 16;
		const bool vecx = vecd && ((((uintptr_t)x) & 15) == 0) && (!x2 || (((uintptr_t)x2) & 15) == 0);
		if (cell8_geometry(s)) { // whole pairs of images (eligibility)
			if (vecx) conv3x3_dw_cell8_kernel<true><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
			else conv3x3_dw_cell8_kernel<false><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
		} else if (cell_geometry(s)) { // J is a multiple of 64 (eligibility): whole stages of four images
			if (vecx) conv3x3_dw_cell_kernel<true><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
			else conv3x3_dw_cell_kernel<false><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
		} else if (vecd && narrow)
			conv3x3_dw_kernel<true, 16><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
		else if (vecd)
			conv3x3_dw_kernel<true, 32><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
		else if (narrow)
			conv3x3_dw_kernel<false, 16><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
		else
			conv3x3_dw_kernel<false, 32><<<grid, kC3DwThreads, 0, stream()>>>(p, delta, deltaBytes, part);
	}
	if (plan.splits > 1) launch_splitk_reduce((const float *)ws, plan.splits, I, K, out);
	return check_launch("conv3x3_dw_kernel");
}

// ---- 3x3 weight gradient with very few input channels (first layer) ----------------------------
static bool thin_dw_eligible(const fitre_conv_shape *s)
{
	if (!c3_geometry(s) || s->inChannels > 3 || s->outChannels > 64) return false;
	const int B = s->inB;
	if (B < 2 || B > 128 || (B & (B - 1)) != 0) return false;
	const int rows = kThinChunk / B; // image rows per chunk
	return rows >= 1 && s->inA % rows == 0 && (rows + 2) * (B + 2) <= kThinXPlane;
}
static int thin_dw_groups(const fitre_conv_shape *s, int *perGroup)
{
	const long chunks = (long)s->samples * s->inA * s->inB / kThinChunk;
	long groups = device_compute_units(); // measured: one workgroup per compute unit (28.8 us with the reduction; two: 33.0)
	if (groups > chunks) groups = chunks;
	const long per = (chunks + groups - 1) / groups;
	*perGroup = (int)per;
	return (int)((chunks + per - 1) / per);
}
static size_t thin_dw_workspace(const fitre_conv_shape *s)
{
	int per;
	return (size_t)thin_dw_groups(s, &per) * s->outChannels * s->inChannels * 9 * sizeof(float);
}
static int launch_thin_dw(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws)
{
	ThinDwParams p;
	p.x = x, p.delta = delta;
	p.cin = s->inChannels, p.cout = s->outChannels;
	p.A = s->inA, p.B = s->inB;
	p.logB = 0;
	while ((1 << p.logB) < s->inB) p.logB++;
	p.plane = s->samples * s->inA * s->inB;
	p.chunks = p.plane / kThinChunk;
	const int groups = thin_dw_groups(s, &p.perGroup);
	const int K = s->inChannels * 9;
	{
		LaunchScope scope(FITRE_KC_CONV_DW, conv_flops(s), 1);
		conv3x3_dw_thin_kernel<<<groups, kGemmThreads, 0, stream()>>>(p, (float *)ws);
	}
	OutParams out{ dW, (long)K, 0, nullptr, nullptr, 1.f, 0.f };
	launch_splitk_reduce((const float *)ws, groups, s->outChannels, K, out);
	return check_launch("conv3x3_dw_thin_kernel");
}

// the dense form of a 3x3 convolution on 2 x 2 maps, when the caller's workspace holds what it needs
// (the full size the *_workspace() query reports; with less the nine-tap kernels run)
static bool quad_usable(const fitre_conv_shape *s, const void *ws, size_t wsBytes, size_t need)
{
	return quad_eligible(s) && ws && ((((uintptr_t)ws) & 15) == 0) && wsBytes >= need;
}

size_t gemm_ex_workspace(int M, int N, int K, int flags)
{
	if (M <= 0 || N <= 0 || K <= 0) return 0;
	return plan_gemm_workspace(N, M, K, (flags & kGemmMirror) != 0);
}

int gemm_ex(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb,
            float beta, float *C, int ldc, const float *bias, int flags, int kernelClass, void *ws, size_t wsBytes)
{
	FITRE_REQUIRE(A && B && C, "fitre_hip_gemm: null pointer");
	FITRE_REQUIRE(M > 0 && N > 0 && K > 0, "fitre_hip_gemm: non-positive shape %d x %d x %d", M, N, K);
	FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "fitre_hip_gemm: bad transpose flags");
	FITRE_REQUIRE(lda >= (transA ? K : M) && ldb >= (transB ? N : K) && ldc >= M, "fitre_hip_gemm: leading dimension too small");
	const size_t aElems = (size_t)lda * (transA ? M : K), bElems = (size_t)ldb * (transB ? K : N);
	FITRE_REQUIRE(aElems < ((size_t)1 << 30) && bElems < ((size_t)1 << 30), "fitre_hip_gemm: an operand exceeds 2^30 elements");
	const int I = N, J = M, R = K;
	GemmPlan plan = plan_gemm(I, J, R, (flags & kGemmMirror) != 0);
	OutParams out{ C, (long)ldc, 0, nullptr, bias, alpha, beta, (flags & kGemmMirror) ? 1 : 0, (flags & kGemmTriK) ? 1 : 0 };
	FITRE_REQUIRE(!(flags & kGemmMirror) || M == N, "gemm: a mirrored product must be square");
	const double flops = 2.0 * (double)M * N * K;
	// engine A(i = n, k): op(B)(k, n).  transB == 0: B[n*ldb + k] (contiguous along k); else B[k*ldb + n]
	// engine B(j = m, k): op(A)(m, k).  transA == 0: A[k*lda + m] (contiguous along m); else A[m*lda + k]
	PlainParams bk{ B, (uint32_t)(bElems * sizeof(float)), ldb, I };
	PlainParams br = bk;
	PlainParams ar{ A, (uint32_t)(aElems * sizeof(float)), lda, J };
	PlainParams ak = ar;
	if (!transB && !transA) return launch_gemm<PlainKContig, PlainRowContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops);
	if (!transB && transA) return launch_gemm<PlainKContig, PlainKContig>(bk, ak, out, I, J, R, plan, ws, wsBytes, kernelClass, flops);
	if (transB && !transA) return launch_gemm<PlainRowContig, PlainRowContig>(br, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops);
	return launch_gemm<PlainRowContig, PlainKContig>(br, ak, out, I, J, R, plan, ws, wsBytes, kernelClass, flops);
}


// the plan of a batched product (engine shape I = N, J = M, R = K)
static GemmPlan batched_plan(int batch, int I, int J, int R, int flags)
{
	// every problem of the batch gets its share of the compute units
	int cus = lane_compute_units() / batch;
	if (cus < 1) cus = 1;
	GemmPlan plan = plan_gemm(I, J, R, (flags & kGemmMirror) != 0, cus);
	GemmPlan deep;
	if (deep_slice_plan(I, J, R, (flags & kGemmMirror) != 0, batch, lane_compute_units(), plan, &deep)) plan = deep;
	// Side by side, the problems of a batch fill the chip with their tiles alone once there are three workgroups per compute
	// unit: the partial tiles of a split and their reduction then cost more than the split gains (measured on three
	// matrices of order 2304: 0.03 ms per product).
	if (plan.bk == kGemmBK && plan.splits > 1) {
		long ti = (I + plan.bm - 1) / plan.bm, tj = (J + plan.bn - 1) / plan.bn;
		long tiles = (flags & kGemmMirror) ? ti * (ti + 1) / 2 : ti * tj;
		if (tiles * batch >= 3L * lane_compute_units()) {
			plan.splits = 1;
			plan.kChunk = (R + kGemmBK - 1) / kGemmBK * kGemmBK;
			plan.wsBytes = 0;
		}
	}
	return plan;
}

static int batched_check(const char *who, int batch, int transA, int transB, int M, int N, int K, const float *A, int lda, const float *B,
                         int ldb, const float *C, int ldc, int flags, long wsStrideBytes)
{
	FITRE_REQUIRE(A && B && C, "%s: null pointer", who);
	FITRE_REQUIRE(batch >= 1 && batch <= 64, "%s: batch of %d", who, batch);
	FITRE_REQUIRE(M > 0 && N > 0 && K > 0, "%s: non-positive shape %d x %d x %d", who, M, N, K);
	FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "%s: bad transpose flags", who);
	FITRE_REQUIRE(lda >= (transA ? K : M) && ldb >= (transB ? N : K) && ldc >= M, "%s: leading dimension too small", who);
	FITRE_REQUIRE(wsStrideBytes % 4 == 0, "%s: workspace stride must be a multiple of 4 bytes", who);
	const size_t aElems = (size_t)lda * (transA ? M : K), bElems = (size_t)ldb * (transB ? K : N);
	FITRE_REQUIRE(aElems < ((size_t)1 << 30) && bElems < ((size_t)1 << 30), "%s: an operand exceeds 2^30 elements", who);
	FITRE_REQUIRE(!(flags & kGemmMirror) || M == N, "%s: a mirrored product must be square", who);
	return FITRE_OK;
}

static int batched_tri_bits(int flags)
{
	// engine operand A is op(B), engine operand B is op(A) (see gemm_ex)
	return ((flags & kGemmTriK) ? kTriBoth : 0) | ((flags & kGemmBLowerTri) ? kTriAFromRow : 0) |
	       ((flags & kGemmBUpperTri) ? kTriAToRow : 0) | ((flags & kGemmALowerTri) ? kTriBToRow : 0);
}

int gemm_ex_batched(int batch, int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, long strideA,
                    const float *B, int ldb, long strideB, float beta, float *C, int ldc, long strideC, int flags, int kernelClass,
                    void *ws, size_t wsBytes, long wsStrideBytes)
{
	int rc = batched_check("gemm_ex_batched", batch, transA, transB, M, N, K, A, lda, B, ldb, C, ldc, flags, wsStrideBytes);
	if (rc) return rc;
	const size_t aElems = (size_t)lda * (transA ? M : K), bElems = (size_t)ldb * (transB ? K : N);
	const int I = N, J = M, R = K;
	const GemmPlan plan = batched_plan(batch, I, J, R, flags);
	OutParams out{ C, (long)ldc, 0, nullptr, nullptr, alpha, beta, (flags & kGemmMirror) ? 1 : 0, batched_tri_bits(flags) };
	const double flops = 2.0 * (double)M * N * K;
	PlainParams bk{ B, (uint32_t)(bElems * sizeof(float)), ldb, I };
	PlainParams ar{ A, (uint32_t)(aElems * sizeof(float)), lda, J };
	const BatchStrides bs{ batch, strideB, strideA, strideC, wsStrideBytes / 4 };
	if (!transB && !transA) return launch_gemm_batched<PlainKContig, PlainRowContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops, bs);
	if (!transB && transA) return launch_gemm_batched<PlainKContig, PlainKContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops, bs);
	if (transB && !transA) return launch_gemm_batched<PlainRowContig, PlainRowContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops, bs);
	return launch_gemm_batched<PlainRowContig, PlainKContig>(bk, ar, out, I, J, R, plan, ws, wsBytes, kernelClass, flops, bs);
}

static PairSide pair_side(const BatchedProduct &g, int bm, int bn)
{
	const size_t aElems = (size_t)g.lda * (g.transA ? g.M : g.K), bElems = (size_t)g.ldb * (g.transB ? g.K : g.N);
	PairSide s;
	s.I = g.N, s.J = g.M, s.R = g.K;
	s.pa = PlainParams{ g.B, (uint32_t)(bElems * sizeof(float)), g.ldb, s.I };
	s.pb = PlainParams{ g.A, (uint32_t)(aElems * sizeof(float)), g.lda, s.J };
	s.out = OutParams{ g.C, (long)g.ldc, 0, nullptr, nullptr, g.alpha, g.beta, (g.flags & kGemmMirror) ? 1 : 0, batched_tri_bits(g.flags) };
	s.tilesI = (s.I + bm - 1) / bm, s.tilesJ = (s.J + bn - 1) / bn;
	s.aStride = g.strideB, s.bStride = g.strideA, s.cStride = g.strideC;
	return s;
}

template <class Cfg>
static int launch_pair(int batch, const PairSide &a, const PairSide &b, int kernelClass, double flops, int tileId)
{
	// the pair the inverse of a matrix needs: op(A) plain on both sides, op(B) transposed in the first product only
	typedef PlainRowContig<Cfg::BM, Cfg::BK> RowsA;
	typedef PlainKContig<Cfg::BM, Cfg::BK> DepthA;
	typedef PlainRowContig<Cfg::BN, Cfg::BK> RowsB;
	const dim3 grid((unsigned)(a.tilesJ > b.tilesJ ? a.tilesJ : b.tilesJ), (unsigned)(a.tilesI > b.tilesI ? a.tilesI : b.tilesI),
	                (unsigned)(2 * batch));
	if (grid.y > 65535 || grid.z > 65535) return fail(FITRE_E_UNSUPPORTED, "gemm grid %u x %u x %u too large", grid.x, grid.y, grid.z);
	LaunchScope scope(kernelClass, flops, tileId);
	mfma_gemm_pair_kernel<Cfg, RowsA, RowsB, DepthA, RowsB><<<grid, kGemmThreads, 0, stream()>>>(a, b, batch);
	return check_launch("mfma_gemm_pair_kernel");
}

int gemm_pair_batched(int batch, const BatchedProduct &f, const BatchedProduct &g, int kernelClass, void *ws, size_t wsBytes,
                      long wsStrideBytes)
{
	int rc = batched_check("gemm_pair_batched", batch, f.transA, f.transB, f.M, f.N, f.K, f.A, f.lda, f.B, f.ldb, f.C, f.ldc, f.flags, wsStrideBytes);
	if (rc) return rc;
	rc = batched_check("gemm_pair_batched", batch, g.transA, g.transB, g.M, g.N, g.K, g.A, g.lda, g.B, g.ldb, g.C, g.ldc, g.flags, wsStrideBytes);
	if (rc) return rc;
	const GemmPlan pf = batched_plan(batch, f.N, f.M, f.K, f.flags), pg = batched_plan(batch, g.N, g.M, g.K, g.flags);
	// one launch where both run unsplit on the deep 64 x 64 tile (every node of the inverse's recursion below order 1280
	// resp. 384); larger products each fill the chip, or split their reduction, and are queued one after the other
	const bool oneLaunch = pf.splits == 1 && pg.splits == 1 && pf.bk == kGemmDeepBK && pg.bk == kGemmDeepBK && pf.bm == 64 && pf.bn == 64 &&
	                       pg.bm == 64 && pg.bn == 64 && !f.transA && f.transB && !g.transA && !g.transB;
	if (!oneLaunch) {
		rc = gemm_ex_batched(batch, f.transA, f.transB, f.M, f.N, f.K, f.alpha, f.A, f.lda, f.strideA, f.B, f.ldb, f.strideB, f.beta, f.C, f.ldc,
		                     f.strideC, f.flags, kernelClass, ws, wsBytes, wsStrideBytes);
		if (rc) return rc;
		return gemm_ex_batched(batch, g.transA, g.transB, g.M, g.N, g.K, g.alpha, g.A, g.lda, g.strideA, g.B, g.ldb, g.strideB, g.beta, g.C,
		                       g.ldc, g.strideC, g.flags, kernelClass, ws, wsBytes, wsStrideBytes);
	}
	const double flops = (2.0 * (double)f.M * f.N * f.K + 2.0 * (double)g.M * g.N * g.K) * batch;
	return launch_pair<TileCfg<64, 64, kGemmDeepBK> >(batch, pair_side(f, 64, 64), pair_side(g, 64, 64), kernelClass, flops, 1);
}


// C(MxN) = alpha*op(A)*op(B) + beta*C (+ bias per row), column-major, for products far below one engine tile: sixteen
// lanes share an output element, each takes every sixteenth reduction index, and their sums are combined by shuffles.
constexpr double kSmallProductWork = 8.0e6; // multiply-adds (LeNet's first linear layer at batch 128: 6.1e6, 20 -> 8 us)
__global__ void __launch_bounds__(256) small_product_kernel(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                                                            int lda, const float *B, int ldb, float beta, float *C, int ldc,
                                                            const float *bias)
{
	const int part = threadIdx.x & 15;
	const long o = (long)blockIdx.x * 16 + (threadIdx.x >> 4);
	const bool live = o < (long)M * N;
	const int n = live ? (int)(o / M) : 0, m = live ? (int)(o - (long)n * M) : 0;
	const float *a = transA ? A + (size_t)m * lda : A + m;
	const float *b = transB ? B + n : B + (size_t)n * ldb;
	const long aStep = transA ? 1 : lda, bStep = transB ? ldb : 1;
	float acc = 0.f;
	for (int k = part; k < K; k += 16) acc = fmaf(a[k * aStep], b[k * bStep], acc);
#pragma unroll
	for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 16);
	if (live && part == 0) {
		float v = alpha * acc;
		if (bias) v += bias[m];
		float *dst = C + (size_t)n * ldc + m;
		if (beta != 0.f) v += beta * *dst;
		*dst = v;
	}
}


} // namespace fitre

using namespace fitre;

extern "C" {

// ---- forward: I = Cout, J = positions, R = Cin*k*k ---------------------------
size_t fitre_hip_conv_forward_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	if (c3_pos_eligible(s, false)) return c3_pos_workspace(s, false);
	return plan_gemm_workspace(s->outChannels, (long)s->samples * s->outA * s->outB, (long)s->inChannels * s->ksize * s->ksize, false, true);
}

int fitre_hip_conv_forward(const fitre_conv_shape *s, const float *x, const float *w, const float *bias, float *y, void *ws,
                           size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_forward", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && w && y, "fitre_hip_conv_forward: null pointer");
	if (c3_pos_eligible(s, false)) return launch_c3_pos<false>(s, x, w, bias, y, ws, wsBytes);
	const int I = s->outChannels, J = s->samples * s->outA * s->outB, R = s->inChannels * s->ksize * s->ksize;
	GemmPlan plan = plan_gemm(I, J, R, false, 0, true);
	PlainParams pa{ w, (uint32_t)((size_t)I * R * sizeof(float)), R, I };
	PatchGeom pb = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	OutParams out{ y, (long)J, 0, bias, nullptr, 1.f, 0.f };
	rc = attach_patch_table(pb, plan.bn);
	if (rc) return rc;
	return launch_gemm<PlainKContig, PatchRowContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_FWD, conv_flops(s));
}

// ---- weight gradient: I = Cout, J = Cin*k*k, R = positions -------------------
size_t fitre_hip_conv_weight_grad_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	if (quad_eligible(s)) {
		const size_t q = quad_weight_grad_workspace(s), c = c3_dw_eligible(s) ? c3_dw_workspace(s) : 0;
		return q > c ? q : c;
	}
	if (c3_dw_eligible(s)) return c3_dw_workspace(s);
	size_t general = plan_gemm_workspace(s->outChannels, (long)s->inChannels * s->ksize * s->ksize, (long)s->samples * s->outA * s->outB, false, true);
	if (thin_dw_eligible(s) && thin_dw_workspace(s) > general) general = thin_dw_workspace(s);
	if (thin_dw_general_eligible(s) && thin_dw_general_workspace(s) > general) general = thin_dw_general_workspace(s);
	return general;
}

int fitre_hip_conv_weight_grad_runs_beside(const fitre_conv_shape *s)
{
	// Every weight gradient does by now.  Those on the general tile engine (5 x 5 and 11 x 11 windows) used to stay in line,
	// because beside the chain's matrix kernels both lost more than the overlap gained; with the chain's bandwidth kernels
	// finding room and priority beside a matrix kernel the balance has turned: AlexNet at batch 64 2.83 -> 2.69 ms.
	return s ? 1 : 0;
}

int fitre_hip_conv_weight_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_weight_grad", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && delta && dW, "fitre_hip_conv_weight_grad: null pointer");
	if (quad_usable(s, ws, wsBytes, quad_weight_grad_workspace(s)) && (((((uintptr_t)x) | ((uintptr_t)delta)) & 15) == 0))
		return quad_weight_grad(s, x, delta, dW, ws, wsBytes);
	if (c3_dw_eligible(s)) return launch_c3_dw(s, x, delta, dW, ws, wsBytes);
	if (thin_dw_eligible(s) && ws && wsBytes >= thin_dw_workspace(s) && ((((uintptr_t)delta) | ((uintptr_t)ws)) & 15) == 0)
		return launch_thin_dw(s, x, delta, dW, ws);
	if (thin_dw_general_eligible(s) && ws && wsBytes >= thin_dw_general_workspace(s) && ((((uintptr_t)ws) & 15) == 0))
		return launch_thin_dw_general(s, x, delta, dW, nullptr, ws);
	const int I = s->outChannels, J = s->inChannels * s->ksize * s->ksize, R = s->samples * s->outA * s->outB;
	GemmPlan plan = plan_gemm(I, J, R, false, 0, true);
	PlainParams pa{ delta, (uint32_t)((size_t)I * R * sizeof(float)), R, I };
	PatchGeom pb = make_patch_geom(x, s->inChannels, s->samples, s->inA, s->inB, s->outA, s->outB, s->ksize, s->stride, s->padding);
	OutParams out{ dW, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	return launch_gemm<PlainKContig, PatchKContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_DW, conv_flops(s));
}

// weight and bias gradient of a layer without batch norm: one pass over delta where the thin kernel applies
size_t fitre_hip_conv_weight_bias_grad_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	const size_t w = fitre_hip_conv_weight_grad_workspace(s);
	const size_t b = fitre_hip_channel_sum_workspace(s->outChannels, (long)s->samples * s->outA * s->outB);
	return w > b ? w : b;
}

int fitre_hip_conv_weight_bias_grad(const fitre_conv_shape *s, const float *x, const float *delta, float *dW, float *db, void *ws,
                                    size_t wsBytes)
{
	FITRE_NEED_INIT();
	if (!db) return fitre_hip_conv_weight_grad(s, x, delta, dW, ws, wsBytes);
	int rc = check_conv("fitre_hip_conv_weight_bias_grad", s);
	if (rc) return rc;
	FITRE_REQUIRE(x && delta && dW, "fitre_hip_conv_weight_bias_grad: null pointer");
	if (thin_dw_general_eligible(s) && ws && wsBytes >= thin_dw_general_workspace(s) && ((((uintptr_t)ws) & 15) == 0))
		return launch_thin_dw_general(s, x, delta, dW, db, ws);
	// the bias gradient first: it is done with the workspace before the weight gradient takes it
	rc = fitre_hip_channel_sum(delta, s->outChannels, (long)s->samples * s->outA * s->outB, db, ws, wsBytes);
	if (rc) return rc;
	return fitre_hip_conv_weight_grad(s, x, delta, dW, ws, wsBytes);
}

// ---- input gradient: I = Cin, J = input positions, R = Cout*k*k ----------------
size_t fitre_hip_conv_input_grad_workspace(const fitre_conv_shape *s)
{
	if (!s) return 0;
	if (quad_eligible(s)) {
		const size_t q = quad_input_grad_workspace(s), c = c3_pos_eligible(s, true) ? c3_pos_workspace(s, true) : 0;
		return q > c ? q : c;
	}
	if (c3_pos_eligible(s, true)) return c3_pos_workspace(s, true);
	return plan_gemm_workspace(s->inChannels, (long)s->samples * s->inA * s->inB, (long)s->outChannels * s->ksize * s->ksize, false, true);
}

int fitre_hip_conv_input_grad(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_input_grad", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && w && dx, "fitre_hip_conv_input_grad: null pointer");
	if (s->stride != 1)
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_input_grad: stride %d (only stride 1 is back-propagated through)", s->stride);
	FITRE_REQUIRE(s->padding < s->ksize, "fitre_hip_conv_input_grad: padding %d >= window %d", s->padding, s->ksize);
	if (quad_usable(s, ws, wsBytes, quad_input_grad_workspace(s)) && (((((uintptr_t)dx) | ((uintptr_t)delta) | ((uintptr_t)w)) & 15) == 0))
		return quad_input_grad(s, delta, w, nullptr, dx, ws, wsBytes, nullptr, nullptr);
	if (c3_pos_eligible(s, true)) return launch_c3_pos<true>(s, delta, w, nullptr, dx, ws, wsBytes);
	if (thin_dx_eligible(s)) return launch_thin_dx(s, delta, w, dx);
	const int I = s->inChannels, J = s->samples * s->inA * s->inB, R = s->outChannels * s->ksize * s->ksize;
	GemmPlan plan = plan_gemm(I, J, R, false, 0, true);
	FlipWeightParams pa;
	pa.w = w;
	pa.bytes = (uint32_t)((size_t)s->outChannels * s->inChannels * s->ksize * s->ksize * sizeof(float));
	pa.cin = s->inChannels;
	pa.taps = s->ksize * s->ksize;
	pa.outStride = s->inChannels * pa.taps;
	pa.divTaps = FastDiv((uint32_t)pa.taps);
	// a full correlation of delta with the flipped window: pad' = k - 1 - p
	PatchGeom pb = make_patch_geom(delta, s->outChannels, s->samples, s->outA, s->outB, s->inA, s->inB, s->ksize, 1,
	                               s->ksize - 1 - s->padding);
	OutParams out{ dx, (long)J, 0, nullptr, nullptr, 1.f, 0.f };
	rc = attach_patch_table(pb, plan.bn);
	if (rc) return rc;
	return launch_gemm<FlipWeightKContig, PatchRowContig>(pa, pb, out, I, J, R, plan, ws, wsBytes, FITRE_KC_CONV_DX, conv_flops(s));
}

// ---- the reductions of several small layers' weight gradients in one launch ----------------------------------------
int fitre_hip_thin_reduce_defer(int on)
{
	FITRE_NEED_INIT();
	if (!on) {
		const int rc = thin_reduce_flush();
		if (rc) return rc;
	}
	g_thin_reduce_deferred = (on != 0);
	return FITRE_OK;
}

size_t fitre_hip_thin_reduce_bytes(const fitre_conv_shape *s)
{
	if (!s || s->samples <= 0 || s->inChannels <= 0 || s->outChannels <= 0 || s->inA <= 0 || s->inB <= 0 || s->ksize <= 0 || s->stride <= 0) return 0;
	if (quad_eligible(s) || c3_dw_eligible(s) || thin_dw_eligible(s) || !thin_dw_general_eligible(s)) return 0;
	return (thin_dw_general_workspace(s) + 255) & ~(size_t)255;
}

int fitre_hip_thin_reduce_flush(void)
{
	FITRE_NEED_INIT();
	return thin_reduce_flush();
}

// ---- the input gradient taken on through the 2 x 2 max pool and the activation of the layer below ------------------
static bool input_grad_takes_thin(const fitre_conv_shape *s)
{
	return s->stride == 1 && s->padding < s->ksize && !quad_eligible(s) && !c3_pos_eligible(s, true) && thin_dx_eligible(s);
}

int fitre_hip_conv_input_grad_folds_pool(const fitre_conv_shape *s)
{
	if (!s || s->samples <= 0 || s->inChannels <= 0 || s->outChannels <= 0 || s->inA <= 0 || s->inB <= 0 || s->ksize <= 0 || s->stride != 1 ||
	    s->padding < 0 || s->outA != s->inA + 2 * s->padding - s->ksize + 1 || s->outB != s->inB + 2 * s->padding - s->ksize + 1 || s->outA <= 0 ||
	    s->outB <= 0)
		return 0;
	return (input_grad_takes_thin(s) && thin_dx_fold_eligible(s)) ? 1 : 0;
}

int fitre_hip_conv_input_grad_pool_act(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, int actFun, const float *z_in,
                                       const float *z_act, float *dxPool, float *dxAct, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_input_grad_pool_act", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && w && dx && z_act && dxAct, "fitre_hip_conv_input_grad_pool_act: null pointer");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_conv_input_grad_pool_act: unknown activation code %d", actFun);
	FITRE_REQUIRE(!act_needs_zin(actFun) || z_in, "fitre_hip_conv_input_grad_pool_act: activation %d needs z_in", actFun);
	const bool aligned = ((((uintptr_t)z_act) | ((uintptr_t)dxAct) | ((uintptr_t)dxPool) | ((uintptr_t)(act_needs_zin(actFun) ? z_in : nullptr))) & 15) == 0;
	if (fitre_hip_conv_input_grad_folds_pool(s) && aligned) {
		const ThinPoolFold fold{ act_needs_zin(actFun) ? z_in : nullptr, z_act, dxPool, dxAct, actFun };
		return launch_thin_dx(s, delta, w, dx, &fold);
	}
	// any other shape: the two steps one after the other
	rc = fitre_hip_conv_input_grad(s, delta, w, dx, ws, wsBytes);
	if (rc) return rc;
	return fitre_hip_pool_act_backward(MAX_POOL, actFun, dx, z_in, z_act, s->inChannels, s->samples, 2 * s->inA, 2 * s->inB, 2, 2, 0, s->inA, s->inB,
	                                   dxPool, dxAct);
}

// ---- sums of two products of one shape (the R operator's pairs) ---------------------------------------------------
int fitre_hip_conv_pair_supported(const fitre_conv_shape *s, int kind)
{
	if (!s) return 0;
	if (kind == 0) return c3_pos_eligible(s, false) ? 1 : 0;
	if (kind == 1) return (s->stride == 1 && c3_pos_eligible(s, true)) ? 1 : 0;
	if (kind == 2) return c3_dw_eligible(s) ? 1 : 0;
	return 0;
}

size_t fitre_hip_conv_pair_workspace(const fitre_conv_shape *s, int kind)
{
	if (!fitre_hip_conv_pair_supported(s, kind)) return 0;
	if (kind == 2) {
		const size_t nine = c3_dw_workspace(s, 2), dense = quad_eligible(s) ? quad_weight_grad_workspace(s) : 0;
		return nine > dense ? nine : dense;
	}
	return c3_pos_workspace(s, kind == 1, 2);
}

int fitre_hip_conv_forward_pair(const fitre_conv_shape *s, const float *x1, const float *w1, const float *x2, const float *w2,
                                const float *bias, float *y, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_forward_pair", s);
	if (rc) return rc;
	FITRE_REQUIRE(x1 && w1 && x2 && w2 && y, "fitre_hip_conv_forward_pair: null pointer");
	if (!c3_pos_eligible(s, false)) return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_forward_pair: only 3x3 windows with stride 1 and padding 1");
	return launch_c3_pos<false>(s, x1, w1, bias, y, ws, wsBytes, nullptr, x2, w2);
}

int fitre_hip_conv_input_grad_pair(const fitre_conv_shape *s, const float *delta1, const float *w1, const float *delta2,
                                   const float *w2, float *dx, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_input_grad_pair", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta1 && w1 && delta2 && w2 && dx, "fitre_hip_conv_input_grad_pair: null pointer");
	if (s->stride != 1 || !c3_pos_eligible(s, true))
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_input_grad_pair: only 3x3 windows with stride 1 and padding 1");
	return launch_c3_pos<true>(s, delta1, w1, nullptr, dx, ws, wsBytes, nullptr, delta2, w2);
}

int fitre_hip_conv_weight_grad_pair(const fitre_conv_shape *s, const float *x1, const float *delta1, const float *x2,
                                    const float *delta2, float *dW, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_weight_grad_pair", s);
	if (rc) return rc;
	FITRE_REQUIRE(x1 && delta1 && x2 && delta2 && dW, "fitre_hip_conv_weight_grad_pair: null pointer");
	if (!c3_dw_eligible(s)) return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_weight_grad_pair: shape outside the 3x3 weight-gradient kernel");
	// 2 x 2 maps: the two dense products into one buffer, folded once
	if (quad_usable(s, ws, wsBytes, quad_weight_grad_workspace(s)) &&
	    (((((uintptr_t)x1) | ((uintptr_t)delta1) | ((uintptr_t)x2) | ((uintptr_t)delta2)) & 15) == 0))
		return quad_weight_grad(s, x1, delta1, dW, ws, wsBytes, x2, delta2);
	return launch_c3_dw(s, x1, delta1, dW, ws, wsBytes, x2, delta2);
}

size_t fitre_hip_conv_input_grad_prepared_bytes(const fitre_conv_shape *s)
{
	return (s && quad_eligible(s)) ? quad_weff_bytes(s) : 0;
}

int fitre_hip_conv_input_grad_prepare(const fitre_conv_shape *s, const float *w, void *prepared, size_t preparedBytes)
{
	FITRE_NEED_INIT();
	int rc = check_conv("fitre_hip_conv_input_grad_prepare", s);
	if (rc) return rc;
	FITRE_REQUIRE(w && prepared, "fitre_hip_conv_input_grad_prepare: null pointer");
	if (!quad_eligible(s)) return fail(FITRE_E_UNSUPPORTED, "fitre_hip_conv_input_grad_prepare: nothing to prepare for this shape");
	if (preparedBytes < quad_weff_bytes(s) || (((uintptr_t)prepared) & 15))
		return fail(FITRE_E_WORKSPACE, "fitre_hip_conv_input_grad_prepare: buffer of %zu bytes is misaligned or smaller than the %zu required",
		            preparedBytes, quad_weff_bytes(s));
	return quad_prepare_weights(s, w, (float *)prepared);
}

int fitre_hip_conv_input_grad_split_prepared(const fitre_conv_shape *s, const float *delta, const float *w, const void *prepared,
                                             float *dx, void *ws, size_t wsBytes, fitre_split_view *view)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(view != nullptr, "fitre_hip_conv_input_grad_split: null view");
	view->base = dx;
	view->splits = 1;
	view->stride = 0;
	int rc = check_conv("fitre_hip_conv_input_grad_split", s);
	if (rc) return rc;
	FITRE_REQUIRE(delta && w && dx, "fitre_hip_conv_input_grad_split: null pointer");
	const bool aligned = (((((uintptr_t)dx) | ((uintptr_t)delta) | ((uintptr_t)w) | ((uintptr_t)ws) | ((uintptr_t)prepared)) & 15) == 0);
	if (quad_eligible(s) && aligned && ws &&
	    wsBytes >= (prepared ? quad_input_grad_workspace(s) - quad_weff_bytes(s) : quad_input_grad_workspace(s))) {
		int splits = 1;
		float *partials = nullptr;
		rc = quad_input_grad(s, delta, w, (const float *)prepared, dx, ws, wsBytes, &splits, &partials);
		if (rc) return rc;
		if (splits > 1) {
			view->base = partials;
			view->splits = splits;
			view->stride = (long)s->inChannels * s->samples * 4;
		}
		return FITRE_OK;
	}
	if (s->stride == 1 && s->padding < s->ksize && c3_pos_eligible(s, true)) {
		int splits = 1;
		rc = launch_c3_pos<true>(s, delta, w, nullptr, dx, ws, wsBytes, &splits);
		if (rc) return rc;
		if (splits > 1) {
			view->base = (float *)ws;
			view->splits = splits;
			view->stride = (long)s->inChannels * s->samples * s->inA * s->inB;
		}
		return FITRE_OK;
	}
	return fitre_hip_conv_input_grad(s, delta, w, dx, ws, wsBytes);
}

int fitre_hip_conv_input_grad_split(const fitre_conv_shape *s, const float *delta, const float *w, float *dx, void *ws,
                                    size_t wsBytes, fitre_split_view *view)
{
	return fitre_hip_conv_input_grad_split_prepared(s, delta, w, nullptr, dx, ws, wsBytes, view);
}

// ---- general column-major GEMM ---------------------------------------------------
// C(MxN) column-major is C[n*ldc + m]: engine i = n (column), j = m (row, contiguous).
// A operand of the engine (rows i = n) is op(B)^T, B operand (rows j = m) is op(A).
size_t fitre_hip_gemm_workspace(int M, int N, int K) { return gemm_ex_workspace(M, N, K, 0); }

int fitre_hip_gemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb,
                   float beta, float *C, int ldc, const float *bias, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	if (small_gemm_fits(M, N, K) && (long)M * N >= 256) {
		FITRE_REQUIRE(A && B && C, "fitre_hip_gemm: null pointer");
		FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "fitre_hip_gemm: bad transpose flags");
		FITRE_REQUIRE(lda >= (transA ? K : M) && ldb >= (transB ? N : K) && ldc >= M, "fitre_hip_gemm: leading dimension too small");
		SmallGemmParams p{};
		p.M = M, p.N = N, p.K = K;
		p.A = A, p.sAm = transA ? lda : 1, p.sAk = transA ? 1 : lda;
		p.B = B, p.sBk = transB ? ldb : 1, p.sBn = transB ? 1 : ldb;
		p.C = C, p.ldc = ldc, p.alpha = alpha, p.beta = beta, p.bias = bias;
		p.act = -1;
		return launch_small_gemm(p, FITRE_KC_FC_GEMM);
	}
	if (M > 0 && N > 0 && K > 0 && (double)M * N * K <= kSmallProductWork) {
		// a product this small (the output layer of a network: ten classes) does not fill one tile of the engine
		FITRE_REQUIRE(A && B && C, "fitre_hip_gemm: null pointer");
		FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "fitre_hip_gemm: bad transpose flags");
		FITRE_REQUIRE(lda >= (transA ? K : M) && ldb >= (transB ? N : K) && ldc >= M, "fitre_hip_gemm: leading dimension too small");
		const long outputs = (long)M * N;
		LaunchScope scope(FITRE_KC_FC_GEMM, 2.0 * (double)M * N * K, 0);
		small_product_kernel<<<(unsigned)((outputs + 15) / 16), 256, 0, stream()>>>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C,
		                                                                         ldc, bias);
		return check_launch("small_product_kernel");
	}
	return gemm_ex(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, bias, 0, FITRE_KC_FC_GEMM, ws, wsBytes);
}

// ---- backward products of a fully connected layer --------------------------------------------
int fitre_hip_linear_is_small(int in, int out, int n) { return small_gemm_fits(in, n, out) && small_gemm_fits(out, in, n); }

size_t fitre_hip_linear_weight_grad_workspace(int in, int out, int n)
{
	const size_t g = gemm_ex_workspace(out, in, n, 0);
	const size_t r = small_gemm_ranges_fit(out, in, n) ? small_gemm_ranges_workspace(out, in, n) : 0;
	return g > r ? g : r;
}

int fitre_hip_linear_input_grad(int in, int out, int n, const float *W, const float *delta, int actBelow, const float *zPre,
                                const float *zPost, int extA, int extB, float *result, float *staging, void *ws, size_t wsBytes,
                                float *deltaCopy)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in > 0 && out > 0 && n > 0, "fitre_hip_linear_input_grad: non-positive shape %d x %d, %d samples", out, in, n);
	FITRE_REQUIRE(W && delta && result && result != delta && result != deltaCopy, "fitre_hip_linear_input_grad: null or aliased pointer");
	const bool permute = extA > 0 || extB > 0;
	FITRE_REQUIRE(!permute || (extA > 0 && extB > 0 && in % (extA * extB) == 0),
	              "fitre_hip_linear_input_grad: %d inputs are not whole %d x %d maps", in, extA, extB);
	const bool derivative = actBelow != CNN_ACT_NONE && actBelow != ACT_LINEAR && actBelow >= 0;
	if (small_gemm_fits(in, n, out)) {
		SmallGemmParams p{};
		p.M = in, p.N = n, p.K = out;
		p.A = W, p.sAm = out, p.sAk = 1;
		p.B = delta, p.sBk = 1, p.sBn = out;
		p.C = result, p.ldc = in, p.alpha = 1.f, p.beta = 0.f;
		p.act = derivative ? actBelow : -1, p.zPre = zPre, p.zPost = zPost;
		p.extA = permute ? extA : 0, p.extB = permute ? extB : 0;
		p.copyB = (deltaCopy && deltaCopy != delta) ? deltaCopy : nullptr;
		return launch_small_gemm(p, FITRE_KC_FC_GEMM);
	}
	// the engine, then the steps of the epilogue one by one
	if (deltaCopy && deltaCopy != delta) {
		int rcCopy = fitre_hip_copy_d2d(deltaCopy, delta, sizeof(float) * (size_t)out * n);
		if (rcCopy) return rcCopy;
	}
	float *plain = permute ? staging : result;
	FITRE_REQUIRE(plain != nullptr && plain != delta, "fitre_hip_linear_input_grad: a product of this size needs the staging buffer");
	int rc = gemm_ex(1, 0, in, n, out, 1.f, W, out, delta, out, 0.f, plain, in, nullptr, 0, FITRE_KC_FC_GEMM, ws, wsBytes);
	if (rc) return rc;
	if (derivative) {
		rc = fitre_hip_activation_backward(actBelow, plain, zPre, zPost, plain, (long)in * n);
		if (rc) return rc;
	}
	if (permute) return fitre_hip_fc_to_conv(plain, in / (extA * extB), n, extA, extB, result);
	return FITRE_OK;
}

int fitre_hip_linear_weight_grad(int in, int out, int n, const float *delta, const float *zin, float *dW, float *db, void *ws,
                                 size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in > 0 && out > 0 && n > 0, "fitre_hip_linear_weight_grad: non-positive shape %d x %d, %d samples", out, in, n);
	FITRE_REQUIRE(delta && zin && dW, "fitre_hip_linear_weight_grad: null pointer");
	if (small_gemm_fits(out, in, n)) {
		SmallGemmParams p{};
		p.M = out, p.N = in, p.K = n;
		p.A = delta, p.sAm = 1, p.sAk = out;
		p.B = zin, p.sBk = in, p.sBn = 1;
		p.C = dW, p.ldc = out, p.alpha = 1.f, p.beta = 0.f;
		p.act = -1;
		p.rowSums = db;
		return launch_small_gemm(p, FITRE_KC_FC_GEMM);
	}
	if (small_gemm_ranges_fit(out, in, n) && ws && wsBytes >= small_gemm_ranges_workspace(out, in, n) && ((((uintptr_t)ws) & 3) == 0)) {
		SmallGemmParams p{};
		p.M = out, p.N = in, p.K = n;
		p.A = delta, p.sAm = 1, p.sAk = out;
		p.B = zin, p.sBk = in, p.sBn = 1;
		p.C = dW, p.ldc = out, p.alpha = 1.f, p.beta = 0.f;
		p.act = -1;
		p.rowSums = db;
		return launch_small_gemm_ranges(p, FITRE_KC_FC_GEMM, ws);
	}
	if (skinny_dw_fits(in, out, n)) {
		const int cus = device_compute_units() > 0 ? device_compute_units() : 256;
		return launch_skinny_dw(in, out, n, delta, zin, dW, db, cus);
	}
	int rc = gemm_ex(0, 1, out, in, n, 1.f, delta, out, zin, in, 0.f, dW, out, nullptr, 0, FITRE_KC_FC_GEMM, ws, wsBytes);
	if (rc || !db) return rc;
	return fitre_hip_row_sum(delta, out, n, db);
}

static int tail_samples(int n) { return n >= 512 ? kTailMaxSamples : 4; }
static bool tail_in_ranges(int n) { return n > kSmallGemmMaxK; }

// floats of LDS left for a workgroup's part of the lowest layer beside the two delta buffers and the upper layers
static long tail_low_floats(int layers, const fitre_fc_tail_layer *l, long upperLds)
{
	int maxDim = 1;
	for (int f = 0; f < layers; f++) {
		maxDim = l[f].in > maxDim ? l[f].in : maxDim;
		maxDim = l[f].out > maxDim ? l[f].out : maxDim;
	}
	return 160 * 1024 / 4 - 64 - 2L * kTailMaxSamples * (maxDim + 1) - upperLds;
}

int fitre_hip_fc_tail_fits(int layers, const fitre_fc_tail_layer *l, int n)
{
	if (!l || layers < 1 || layers > kTailMaxLayers || n < 1 || n > 65536) return 0;
	long upperLds = 0;
	for (int f = 0; f < layers; f++) {
		if (l[f].in < 1 || l[f].out < 1 || l[f].in > kTailMaxDim || l[f].out > kTailMaxDim) return 0;
		if (f > 0 && l[f].in != l[f - 1].out) return 0;
		if (!(tail_in_ranges(n) ? small_gemm_ranges_fit(l[f].out, l[f].in, n) : small_gemm_fits(l[f].out, l[f].in, n))) return 0;
		if (f > 0) upperLds += (long)l[f].in * (l[f].out + 1);
	}
	return upperLds <= kTailUpperLds && tail_low_floats(layers, l, upperLds) >= l[0].out + 1; // the layers above the lowest sit in LDS whole
}

size_t fitre_hip_fc_tail_workspace(int layers, const fitre_fc_tail_layer *l, int n)
{
	if (!fitre_hip_fc_tail_fits(layers, l, n)) return 0;
	size_t total = 256;
	if (tail_in_ranges(n))
		for (int f = 0; f < layers; f++) total += small_gemm_ranges_workspace(l[f].out, l[f].in, n);
	return total;
}

struct TailFold {
	int act;
	const float *zIn, *zAct;
	float *dxPool, *dxAct;
};
static int fc_tail_run(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA, int extB, float *features, void *ws,
                       size_t wsBytes, const TailFold *fold);

int fitre_hip_fc_tail_backward(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA, int extB, float *features,
                               void *ws, size_t wsBytes)
{
	return fc_tail_run(layers, l, n, delta, extA, extB, features, ws, wsBytes, nullptr);
}

int fitre_hip_fc_tail_backward_pool_act(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA, int extB, float *features,
                                        int actFun, const float *z_in, const float *z_act, float *dxPool, float *dxAct, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(extA > 0 && extB > 0, "fitre_hip_fc_tail_backward_pool_act: the lowest layer's inputs must be %d x %d maps", extA, extB);
	FITRE_REQUIRE(z_act && dxAct, "fitre_hip_fc_tail_backward_pool_act: null pointer");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_fc_tail_backward_pool_act: unknown activation code %d", actFun);
	FITRE_REQUIRE(!act_needs_zin(actFun) || z_in, "fitre_hip_fc_tail_backward_pool_act: activation %d needs z_in", actFun);
	const float *zi = act_needs_zin(actFun) ? z_in : nullptr;
	if (((((uintptr_t)z_act) | ((uintptr_t)dxAct) | ((uintptr_t)dxPool) | ((uintptr_t)zi)) & 7) == 0) {
		const TailFold fold{ actFun, zi, z_act, dxPool, dxAct };
		return fc_tail_run(layers, l, n, delta, extA, extB, features, ws, wsBytes, &fold);
	}
	int rc = fc_tail_run(layers, l, n, delta, extA, extB, features, ws, wsBytes, nullptr);
	if (rc) return rc;
	FITRE_REQUIRE(l[0].in % (extA * extB) == 0, "fitre_hip_fc_tail_backward_pool_act: %d inputs are not whole maps", l[0].in);
	return fitre_hip_pool_act_backward(MAX_POOL, actFun, features, z_in, z_act, l[0].in / (extA * extB), n, 2 * extA, 2 * extB, 2, 2, 0, extA, extB,
	                                   dxPool, dxAct);
}

static int fc_tail_run(int layers, const fitre_fc_tail_layer *l, int n, const float *delta, int extA, int extB, float *features, void *ws,
                       size_t wsBytes, const TailFold *fold)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(fitre_hip_fc_tail_fits(layers, l, n), "fitre_hip_fc_tail_backward: the layers do not fit (at most %d layers of at most %d units)",
	              kTailMaxLayers, kTailMaxDim);
	FITRE_REQUIRE(delta && features, "fitre_hip_fc_tail_backward: null pointer");
	const bool permute = extA > 0 || extB > 0;
	FITRE_REQUIRE(!permute || (extA > 0 && extB > 0 && l[0].in % (extA * extB) == 0),
	              "fitre_hip_fc_tail_backward: %d inputs are not whole %d x %d maps", l[0].in, extA, extB);
	const bool ranges = tail_in_ranges(n);
	const size_t need = fitre_hip_fc_tail_workspace(layers, l, n);
	if (ranges && (!ws || wsBytes < need || (((uintptr_t)ws) & 3) != 0))
		return fail(FITRE_E_WORKSPACE, "fitre_hip_fc_tail_backward: workspace of %zu bytes is smaller than the %zu required", wsBytes, need);
	FcTailParams p{};
	p.layers = layers, p.n = n, p.ns = tail_samples(n);
	p.extA = permute ? extA : 0, p.extB = permute ? extB : 0;
	p.delta = delta, p.features = features;
	p.foldAct = -2;
	if (fold) {
		p.foldAct = (fold->act == CNN_ACT_NONE || fold->act == ACT_LINEAR || fold->act < 0) ? -1 : fold->act;
		p.foldZIn = fold->zIn, p.foldZAct = fold->zAct, p.foldDxPool = fold->dxPool, p.foldDxAct = fold->dxAct;
		// which of its kernels fitre_hip_pool_act_backward would take for these maps: the one for rows of whole 16-byte
		// groups stores the gradient, the others add it to zero
		p.foldDirect = ((2 * extB) % 4 == 0 &&
		                ((((uintptr_t)fold->zAct) | ((uintptr_t)fold->dxAct) | ((uintptr_t)fold->dxPool) | ((uintptr_t)fold->zIn)) & 15) == 0 &&
		                (((uintptr_t)features) & 7) == 0)
		                   ? 1
		                   : 0;
	}
	int maxDim = 1, upperLds = 0;
	double chainFlops = 0.0;
	for (int f = 0; f < layers; f++) {
		FITRE_REQUIRE(l[f].W && l[f].zin && l[f].slot && l[f].dW && l[f].slot != delta, "fitre_hip_fc_tail_backward: null or aliased pointer in layer %d", f);
		const bool derivative = l[f].act != CNN_ACT_NONE && l[f].act != ACT_LINEAR && l[f].act >= 0;
		FITRE_REQUIRE(!derivative || (l[f].zPost && l[f].zPre), "fitre_hip_fc_tail_backward: layer %d has an activation but no z", f);
		FcTailLayer &d = p.l[f];
		d.in = l[f].in, d.out = l[f].out, d.act = l[f].act;
		d.W = l[f].W, d.zPre = l[f].zPre, d.zPost = l[f].zPost, d.slot = l[f].slot;
		d.outMagic = (unsigned)((1ull << 32) / (unsigned)d.out) + 1u;
		if (f > 0) d.ldsBase = upperLds, upperLds += d.in * (d.out + 1);
		maxDim = d.in > maxDim ? d.in : maxDim;
		maxDim = d.out > maxDim ? d.out : maxDim;
		chainFlops += 2.0 * (double)d.in * d.out * n;
	}
	p.maxDim = maxDim;
	const int groups = (n + p.ns - 1) / p.ns;
	// parts of the lowest layer: each fits its share of LDS, and together with the groups they fill the chip
	const int mostRows = (int)(tail_low_floats(layers, l, upperLds) / (l[0].out + 1));
	int parts = (l[0].in + mostRows - 1) / mostRows;
	const int cus = device_compute_units() > 0 ? device_compute_units() : 256;
	const int fill = (cus + groups - 1) / groups;
	parts = parts < fill ? fill : parts;
	parts = parts > l[0].in ? l[0].in : parts;
	p.partInputs = (l[0].in + parts - 1) / parts;
	if (p.partInputs > mostRows) p.partInputs = mostRows;
	parts = (l[0].in + p.partInputs - 1) / p.partInputs;
	p.lowBase = upperLds;
	const size_t ldsBytes = sizeof(float) * ((size_t)2 * kTailMaxSamples * (maxDim + 1) + upperLds + (size_t)p.partInputs * (l[0].out + 1) + 64);
	static bool attributeSet = false;
	if (!attributeSet) {
		FITRE_HIP_TRY(hipFuncSetAttribute((const void *)fc_tail_chain_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
		attributeSet = true;
	}
	{
		LaunchScope scope(FITRE_KC_FC_GEMM, chainFlops, 0);
		fc_tail_chain_kernel<<<dim3((unsigned)groups, (unsigned)parts), kTailThreads, ldsBytes, stream()>>>(p);
	}
	// every layer's delta * zin' and delta * 1
	SmallGemmBatch b{};
	SmallReduceBatch r{};
	b.count = r.count = layers;
	const int nRanges = ranges ? (n + kSmallRange - 1) / kSmallRange : 1;
	r.ranges = nRanges;
	float *part = (float *)ws;
	for (int f = 0; f < layers; f++) {
		SmallGemmParams &q = b.p[f];
		q.M = l[f].out, q.N = l[f].in, q.K = n;
		q.A = l[f].slot, q.sAm = 1, q.sAk = l[f].out;
		q.B = l[f].zin, q.sBk = l[f].in, q.sBn = 1;
		q.C = l[f].dW, q.ldc = l[f].out, q.alpha = 1.f, q.beta = 0.f;
		q.act = -1;
		q.rowSums = l[f].db;
		b.gridX[f] = (q.M + kSmallTile - 1) / kSmallTile, b.gridY[f] = (q.N + kSmallTile - 1) / kSmallTile;
		b.first[f + 1] = b.first[f] + b.gridX[f] * b.gridY[f] * nRanges;
		if (ranges) {
			q.kChunk = kSmallRange, q.partial = part;
			q.rowSums = l[f].db ? part : nullptr; // only its being non-null matters to the kernel in this mode
			r.M[f] = q.M, r.N[f] = q.N, r.partial[f] = part, r.C[f] = l[f].dW, r.rowSums[f] = l[f].db, r.alpha[f] = 1.f;
			r.first[f + 1] = r.first[f] + (long)q.M * q.N + q.M;
			part += (size_t)nRanges * ((size_t)q.M * q.N + q.M);
		}
	}
	{
		LaunchScope scope(FITRE_KC_FC_GEMM, chainFlops, 0);
		small_gemm_batch_kernel<<<(unsigned)b.first[layers], 256, 0, stream()>>>(b);
	}
	if (ranges) {
		LaunchScope scope(FITRE_KC_SPLITK_REDUCE, 4.0 * (double)r.first[layers] * (nRanges + 1));
		small_gemm_batch_reduce_kernel<<<(unsigned)((r.first[layers] + 255) / 256), 256, 0, stream()>>>(r);
	}
	return check_launch("fc_tail_chain_kernel");
}

} // extern "C"
