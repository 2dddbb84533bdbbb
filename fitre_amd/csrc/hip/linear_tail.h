// The backward pass of a whole tail of small fully connected layers in two launches (three at a large batch) instead of
// two per layer (LeNet's 400-120-84-10: six launches of 6-10 us each: functions/cnn_backward.cu:100-254 runs these steps
// layer by layer).
//
//   1. the chain of deltas.  It does not couple samples, so a workgroup owns a few samples and walks the layers top down
//      on its own: delta_f (after the activation derivative) into its dx slot and into LDS, delta_{f-1} = f'(.) .* (W_f'
//      delta_f) from weights staged in LDS.  The lowest layer has the most weights and nothing below it waits for
//      all of its outputs at once, so its inputs are cut into parts that different workgroups take (each repeats the
//      few thousand multiply-adds of the layers above).  A workgroup has sixteen waves, so that a wave's share of the
//      weight rows is a dozen loads, all in flight at once.  The result goes to the convolution layout.
//   2. every layer's weight and bias gradient, delta_f * zin_f' and delta_f * 1, as ONE launch of the small product
//      kernel over the blocks of all layers (a long batch is cut into ranges, added by a third launch in range order).
// The order of every sum is fixed by the shapes alone.
#pragma once
#include "gemm_engine.h"
#include "linear_small.h"

namespace fitre {

constexpr int kTailMaxLayers = 4;
constexpr int kTailMaxDim = 1024;   // inputs / outputs of a layer
constexpr int kTailMaxSamples = 8;  // samples of a group
constexpr int kTailThreads = 1024;  // sixteen waves: a wave's share of the weight rows is short enough for all its loads to be in flight
constexpr int kTailWaves = kTailThreads / 64;
constexpr int kTailUpperLds = 16384; // floats of LDS for the weights of the layers above the lowest

struct FcTailLayer {
	int in, out;
	int act;                   // this layer's activation
	unsigned outMagic;         // e / out == __umulhi(e, outMagic) for e < 2^20
	int ldsBase;               // where its weights sit in LDS as [input][out + 1] (layers above the lowest)
	const float *W;            // out x in, column-major
	const float *zPre, *zPost; // its output before / after the activation, out x n
	float *slot;               // receives delta (after the activation derivative), out x n
};

struct FcTailParams {
	int layers, n, ns;
	int extA, extB; // the lowest layer's inputs are whole extA x extB maps: its input gradient goes to [c][n][a][b]
	FcTailLayer l[kTailMaxLayers];
	const float *delta; // at the top layer's output, before its activation derivative
	float *features;
	int maxDim;
	int partInputs; // inputs of the lowest layer per blockIdx.y
	int lowBase;    // where the lowest layer's part sits in LDS
	// foldAct >= -1: the maps below end in an activation (-1: none) and a 2 x 2 / stride 2 max pool whose output the lowest
	// layer reads; its input gradient then goes on through both, exactly as maxpool_map_backward_kernel takes it (the first
	// largest cell of a window in memory order gets the gradient, then times f'(.)); foldAct == -2: no fold
	int foldAct;
	int foldDirect; // the gradient is stored as it is (else as 0 + gradient, the sum over the windows a cell is the maximum of)
	const float *foldZIn, *foldZAct; // [C][n][2 extA][2 extB]; foldZIn null where the derivative does not need it
	float *foldDxPool, *foldDxAct;   // foldDxPool may be null
};

__device__ __forceinline__ int tail_div(int e, int out, unsigned magic) { return out == 1 ? e : (int)__umulhi((unsigned)e, magic); }

// rows [row0, row0 + rows) of W (an input per row, its `out` output units contiguous) to LDS as [row][out + 1]: a wave
// moves whole rows, the lanes along a row
__device__ __forceinline__ void tail_stage_rows(const float *W, int out, int row0, int rows, float *dst, int wave, int lane)
{
	const int ldw = out + 1;
	for (int c0 = 0; c0 < out; c0 += 64) {
		const int col = c0 + lane;
		const bool ok = col < out;
		const float *src = W + (long)row0 * out + col;
#pragma unroll 8
		for (int r = wave; r < rows; r += kTailWaves) {
			const float v = ok ? src[(long)r * out] : 0.f;
			if (ok) dst[r * ldw + col] = v;
		}
	}
}

__global__ void __launch_bounds__(kTailThreads) fc_tail_chain_kernel(const FcTailParams p)
{
	extern __shared__ float lds[];
	const int ldd = p.maxDim + 1;
	float *dcur = lds, *dnext = lds + kTailMaxSamples * ldd, *wbuf = dnext + kTailMaxSamples * ldd;
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int s0 = blockIdx.x * p.ns;
	const int cnt = (p.n - s0 < p.ns) ? p.n - s0 : p.ns;
	const bool first = blockIdx.y == 0; // the workgroup that writes the slots of the layers above the lowest
	// every weight this workgroup multiplies by goes to LDS first: the layers above the lowest, whole, and its part of the lowest
	const FcTailLayer &low = p.l[0];
	const int pi0 = blockIdx.y * p.partInputs;
	const int pni = (low.in - pi0 < p.partInputs) ? low.in - pi0 : p.partInputs;
#pragma unroll
	for (int f = kTailMaxLayers - 1; f >= 1; f--)
		if (f < p.layers) tail_stage_rows(p.l[f].W, p.l[f].out, 0, p.l[f].in, wbuf + p.l[f].ldsBase, wave, lane);
	tail_stage_rows(low.W, low.out, pi0, pni, wbuf + p.lowBase, wave, lane);
	const int planeAB = p.extA * p.extB;
	// the layers top down; unrolled so that every index into the argument block is a constant
#pragma unroll
	for (int f = kTailMaxLayers - 1; f >= 0; f--) {
		if (f >= p.layers) continue;
		const FcTailLayer &lay = p.l[f];
		const FcTailLayer &under = p.l[f > 0 ? f - 1 : 0];
		const bool below = f > 0;
		if (f == p.layers - 1) { // delta at the top, times its activation derivative
			const bool derivative = lay.act != CNN_ACT_NONE && lay.act != ACT_LINEAR && lay.act >= 0;
			for (int e = tid; e < lay.out * cnt; e += kTailThreads) {
				const int s = tail_div(e, lay.out, lay.outMagic), o = e - s * lay.out;
				const long at = (long)(s0 + s) * lay.out + o;
				float v = p.delta[at];
				if (derivative) v = act_backward_value(lay.act, v, lay.zPre[at], lay.zPost[at]);
				dcur[s * ldd + o] = v;
				if (first) lay.slot[at] = v;
			}
		}
		const int in = lay.in, out = lay.out, ldw = out + 1;
		const bool derivative = below && under.act != CNN_ACT_NONE && under.act != ACT_LINEAR && under.act >= 0;
		const int i0 = below ? 0 : pi0, ni = below ? in : pni;
		const float *wl = wbuf + (below ? lay.ldsBase : p.lowBase);
		__syncthreads(); // dcur and the staged weights are complete; the layer above has been read
		// (i, s) = f'(.) * sum over o of W(o, i) delta(o, s)
		for (int e = tid; e < ni * cnt; e += kTailThreads) {
			const int s = e / ni, ii = e - s * ni;
			const int i = i0 + ii;
			const long at = (long)(s0 + s) * in + i;
			float zi = 0.f, zo = 0.f;
			if (derivative) zi = under.zPre[at], zo = under.zPost[at]; // on their way while the sum runs
			const float *w = wl + ii * ldw, *d = dcur + s * ldd;
			float acc = 0.f;
#pragma unroll 8
			for (int o = 0; o < out; o++) acc = fmaf(w[o], d[o], acc);
			if (below) {
				if (derivative) acc = act_backward_value(under.act, acc, zi, zo);
				dnext[s * ldd + i] = acc;
				if (first) under.slot[at] = acc;
			} else if (p.extA > 0) {
				const int c = i / planeAB, r = i - c * planeAB;
				const int b = r / p.extA, a = r - b * p.extA;
				p.features[(((long)c * p.n + (s0 + s)) * p.extA + a) * p.extB + b] = acc;
				if (p.foldAct != -2) {
					const int bigB = 2 * p.extB;
					const long at0 = (((long)c * p.n + (s0 + s)) * (2 * p.extA) + 2 * a) * bigB + 2 * b;
					const float2 r0 = *reinterpret_cast<const float2 *>(p.foldZAct + at0);
					const float2 r1 = *reinterpret_cast<const float2 *>(p.foldZAct + at0 + bigB);
					float2 i0 = r0, i1 = r1;
					if (p.foldZIn) {
						i0 = *reinterpret_cast<const float2 *>(p.foldZIn + at0);
						i1 = *reinterpret_cast<const float2 *>(p.foldZIn + at0 + bigB);
					}
					const int arg = scan2x2(r0.x, r0.y, r1.x, r1.y);
					const float g = p.foldDirect ? acc : 0.f + acc;
					float2 g0 = make_float2(arg == 0 ? g : 0.f, arg == 1 ? g : 0.f), g1 = make_float2(arg == 2 ? g : 0.f, arg == 3 ? g : 0.f);
					if (p.foldDxPool) {
						*reinterpret_cast<float2 *>(p.foldDxPool + at0) = g0;
						*reinterpret_cast<float2 *>(p.foldDxPool + at0 + bigB) = g1;
					}
					const int fa = p.foldAct < 0 ? CNN_ACT_NONE : p.foldAct;
					g0.x *= act_derivative(fa, i0.x, r0.x), g0.y *= act_derivative(fa, i0.y, r0.y);
					g1.x *= act_derivative(fa, i1.x, r1.x), g1.y *= act_derivative(fa, i1.y, r1.y);
					*reinterpret_cast<float2 *>(p.foldDxAct + at0) = g0;
					*reinterpret_cast<float2 *>(p.foldDxAct + at0 + bigB) = g1;
				}
			} else {
				p.features[at] = acc;
			}
		}
		float *t = dcur;
		dcur = dnext, dnext = t;
	}
}

} // namespace fitre
