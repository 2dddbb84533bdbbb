// Products of a fully connected layer that are far below one tile of the MFMA engine (LeNet's 400-120-84-10
// tail at batch 128: 0.1 to 6 million multiply-adds).  At that size a pass is bound by the number of launches,
// so the kernel here takes what the reference queues as separate steps into its epilogue:
//
//   input gradient   delta_below = f'(z_below) .* (W' * delta)        functions/cnn_backward.cu:250-254, then the
//                    activation step of the next loop iteration (:100-172), optionally stored in the
//                    convolution layout (the permutation at the boundary, :330-348)
//   weight gradient  dW = delta * z', db = delta * 1                  functions/cnn_backward.cu:189-197, :216-224
//
// One workgroup owns a 32 x 32 block of the result and walks the reduction in blocks of 64 through LDS; a thread
// holds 2 x 2 results.  The order of the additions is fixed by the shape alone.
#pragma once
#include "common.h"
#include "fitre_nn.h"

namespace fitre {

constexpr int kSmallTile = 32;
constexpr int kSmallDepth = 64; // reduction indices per block

struct SmallGemmParams {
	int M, N, K;
	const float *A; // op(A)(m, k) = A[m * sAm + k * sAk]
	long sAm, sAk;
	const float *B; // op(B)(k, n) = B[k * sBk + n * sBn]
	long sBk, sBn;
	float *C; // C(m, n) = C[n * ldc + m], or the convolution layout when extA > 0
	long ldc;
	float alpha, beta;
	const float *bias; // added per row m, or null
	int act;           // >= 0: the result is multiplied by f'(.) taken from zPre / zPost (laid out like C, leading dimension M)
	const float *zPre, *zPost;
	int extA, extB;  // > 0: row m = (c * extB + b) * extA + a goes to [c][n][a][b]
	float *rowSums;  // sum over k of op(A)(m, k) for every m, or null
	float *copyB;    // op(B) is also written here, in B's own layout, or null (the workgroups of the first block row do it)
	int kChunk;      // > 0: the reduction is cut into ranges of kChunk, one per blockIdx.z, whose raw sums go to `partial`
	float *partial;  // [range][N * M results, then M row sums] (no epilogue: small_gemm_reduce_kernel applies alpha and stores)
};

__device__ __forceinline__ float act_backward_value(int actFun, float d, float zi, float zo)
{
	switch (actFun) {
	case ACT_LOGISTIC: return d * zo * (1.f - zo);
	case ACT_TANH: return d * ((1.f + zo) * (1.f - zo));
	case CNN_ACT_SOFTPLUS: return d * (1.f / (1.f + expf(-zi)));
	case CNN_ACT_SWISH: {
		float t = 1.f / (1.f + expf(-zi));
		return d * (zo + t * (1.f - zo));
	}
	case CNN_ACT_RELU: return zo > 0.f ? d : 0.f;
	case CNN_ACT_ELU: return zo < 0.f ? d * (zo + 1.f) : d;
	default: return d;
	}
}

// one workgroup's block (bx, by) of the result over reduction range bz
__device__ __forceinline__ void small_gemm_block(const SmallGemmParams &p, const int bx, const int by, const int bz)
{
	__shared__ float As[kSmallDepth][kSmallTile + 1]; // [k][m]
	__shared__ float Bs[kSmallDepth][kSmallTile + 1]; // [k][n]
	const int tid = threadIdx.x;
	const int m0 = bx * kSmallTile, n0 = by * kSmallTile;
	const int tm = tid & 15, tn = tid >> 4;
	// loads run along whichever index is contiguous in memory; all of a block's loads are in flight together
	const bool aAlongM = p.sAm == 1, bAlongN = p.sBn == 1;
	constexpr int kPer = kSmallDepth * kSmallTile / 256; // elements of each operand a thread loads per block
	float acc00 = 0.f, acc01 = 0.f, acc10 = 0.f, acc11 = 0.f, rs0 = 0.f, rs1 = 0.f;
	const bool sums = p.rowSums != nullptr && by == 0 && tn == 0;
	const int kBeg = p.kChunk > 0 ? bz * p.kChunk : 0;
	const int kEnd = (p.kChunk > 0 && kBeg + p.kChunk < p.K) ? kBeg + p.kChunk : p.K;
	for (int k0 = kBeg; k0 < kEnd; k0 += kSmallDepth) {
		float av[kPer], bv[kPer];
#pragma unroll
		for (int i = 0; i < kPer; i++) {
			const int e = tid + 256 * i; // along the tile: e % 32; along the depth: e / 32 -- or the other way round
			const int am = aAlongM ? (e & 31) : e / kSmallDepth, ak = aAlongM ? (e >> 5) : e % kSmallDepth;
			const int bn = bAlongN ? (e & 31) : e / kSmallDepth, bk = bAlongN ? (e >> 5) : e % kSmallDepth;
			const bool aok = (m0 + am < p.M) & (k0 + ak < kEnd), bok = (n0 + bn < p.N) & (k0 + bk < kEnd);
			av[i] = aok ? p.A[(long)(m0 + am) * p.sAm + (long)(k0 + ak) * p.sAk] : 0.f;
			bv[i] = bok ? p.B[(long)(k0 + bk) * p.sBk + (long)(n0 + bn) * p.sBn] : 0.f;
			if (p.copyB != nullptr && bx == 0 && bok) p.copyB[(long)(k0 + bk) * p.sBk + (long)(n0 + bn) * p.sBn] = bv[i];
		}
		__syncthreads(); // the previous block's readers are done
#pragma unroll
		for (int i = 0; i < kPer; i++) {
			const int e = tid + 256 * i;
			const int am = aAlongM ? (e & 31) : e / kSmallDepth, ak = aAlongM ? (e >> 5) : e % kSmallDepth;
			const int bn = bAlongN ? (e & 31) : e / kSmallDepth, bk = bAlongN ? (e >> 5) : e % kSmallDepth;
			As[ak][am] = av[i];
			Bs[bk][bn] = bv[i];
		}
		__syncthreads();
		const int depth = (kEnd - k0 < kSmallDepth) ? kEnd - k0 : kSmallDepth;
		for (int k = 0; k < depth; k++) {
			const float a0 = As[k][tm], a1 = As[k][tm + 16], b0 = Bs[k][tn], b1 = Bs[k][tn + 16];
			acc00 = fmaf(a0, b0, acc00);
			acc10 = fmaf(a1, b0, acc10);
			acc01 = fmaf(a0, b1, acc01);
			acc11 = fmaf(a1, b1, acc11);
			if (sums) rs0 += a0, rs1 += a1;
		}
	}
	if (p.kChunk > 0) { // raw sums of this reduction range
		float *part = p.partial + (size_t)bz * ((size_t)p.M * p.N + p.M);
		if (sums) {
			if (m0 + tm < p.M) part[(size_t)p.M * p.N + m0 + tm] = rs0;
			if (m0 + tm + 16 < p.M) part[(size_t)p.M * p.N + m0 + tm + 16] = rs1;
		}
		auto put = [&](int m, int n, float acc) {
			if (m < p.M && n < p.N) part[(size_t)n * p.M + m] = acc;
		};
		put(m0 + tm, n0 + tn, acc00);
		put(m0 + tm + 16, n0 + tn, acc10);
		put(m0 + tm, n0 + tn + 16, acc01);
		put(m0 + tm + 16, n0 + tn + 16, acc11);
		return;
	}
	if (sums) {
		if (m0 + tm < p.M) p.rowSums[m0 + tm] = rs0;
		if (m0 + tm + 16 < p.M) p.rowSums[m0 + tm + 16] = rs1;
	}
	const int planeAB = p.extA * p.extB;
	auto store = [&](int m, int n, float acc) {
		if (m >= p.M || n >= p.N) return;
		float v = p.alpha * acc;
		if (p.bias) v += p.bias[m];
		if (p.act >= 0) {
			const long zi = (long)n * p.M + m;
			v = act_backward_value(p.act, v, p.zPre ? p.zPre[zi] : 0.f, p.zPost ? p.zPost[zi] : 0.f);
		}
		long dst = (long)n * p.ldc + m;
		if (p.extA > 0) {
			const int c = m / planeAB, r = m - c * planeAB;
			const int b = r / p.extA, a = r - b * p.extA;
			dst = (((long)c * p.N + n) * p.extA + a) * p.extB + b;
		}
		if (p.beta != 0.f) v += p.beta * p.C[dst];
		p.C[dst] = v;
	};
	store(m0 + tm, n0 + tn, acc00);
	store(m0 + tm + 16, n0 + tn, acc10);
	store(m0 + tm, n0 + tn + 16, acc01);
	store(m0 + tm + 16, n0 + tn + 16, acc11);
}

__global__ void __launch_bounds__(256) small_gemm_kernel(const SmallGemmParams p)
{
	small_gemm_block(p, (int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z);
}

// several independent products as one launch: the blocks of product j are blockIdx.x in [first[j], first[j + 1])
constexpr int kSmallBatch = 4;
struct SmallGemmBatch {
	int count;
	int first[kSmallBatch + 1];
	int gridX[kSmallBatch], gridY[kSmallBatch];
	SmallGemmParams p[kSmallBatch];
};
__global__ void __launch_bounds__(256) small_gemm_batch_kernel(const SmallGemmBatch b)
{
	const int block = (int)blockIdx.x;
	int j = 0;
	while (j + 1 < b.count && block >= b.first[j + 1]) j++;
	const int local = block - b.first[j];
	const int bx = local % b.gridX[j], rest = local / b.gridX[j];
	small_gemm_block(b.p[j], bx, rest % b.gridY[j], rest / b.gridY[j]);
}

// the second launch of a batch whose reductions were cut into ranges: every product's sums in range order, in double
struct SmallReduceBatch {
	int count, ranges;
	long first[kSmallBatch + 1]; // results (M * N + M) of the products before j
	int M[kSmallBatch], N[kSmallBatch];
	const float *partial[kSmallBatch];
	float *C[kSmallBatch], *rowSums[kSmallBatch];
	float alpha[kSmallBatch];
};
__global__ void __launch_bounds__(256) small_gemm_batch_reduce_kernel(const SmallReduceBatch b)
{
	const long at = (long)blockIdx.x * blockDim.x + threadIdx.x;
	if (at >= b.first[b.count]) return;
	int j = 0;
	while (j + 1 < b.count && at >= b.first[j + 1]) j++;
	const long i = at - b.first[j];
	const long mn = (long)b.M[j] * b.N[j], per = mn + b.M[j];
	const float *part = b.partial[j];
	double acc = 0.0;
	for (int r = 0; r < b.ranges; r++) acc += (double)part[(size_t)r * per + i];
	if (i < mn) b.C[j][i] = b.alpha[j] * (float)acc; // ldc == M
	else if (b.rowSums[j]) b.rowSums[j][i - mn] = (float)acc;
}

// C = alpha * (sum of the ranges' partial results, in range order, in double) and the row sums likewise
__global__ void __launch_bounds__(256) small_gemm_reduce_kernel(const float *partial, int ranges, int M, int N, float alpha, float *C,
                                                                long ldc, float *rowSums)
{
	const long per = (long)M * N + M;
	const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= per) return;
	double acc = 0.0;
	for (int r = 0; r < ranges; r++) acc += (double)partial[(size_t)r * per + i];
	if (i < (long)M * N) {
		const long n = i / M, m = i - n * M;
		C[n * ldc + m] = alpha * (float)acc;
	} else if (rowSums) {
		rowSums[i - (long)M * N] = (float)acc;
	}
}

// A product is "small" when it is below one wave of engine tiles and its reduction is short enough for one
// workgroup per result block to walk it alone.
constexpr double kSmallGemmWork = 3.2e7; // multiply-adds
constexpr int kSmallGemmMaxK = 512;
constexpr double kSmallGemmShortWork = 1.3e8; // the bound for reductions of at most two blocks (a wide, shallow product)
static inline bool small_gemm_fits(int M, int N, int K)
{
	if (M <= 0 || N <= 0 || K <= 0 || K > kSmallGemmMaxK) return false;
	return (double)M * N * K <= (K <= 2 * kSmallDepth ? kSmallGemmShortWork : kSmallGemmWork);
}

// A long reduction over a small result (the weight gradient of a small linear layer at a large batch): ranges of
// kSmallRange reduction indices go to different workgroups and a second launch adds their partial results.
constexpr int kSmallRange = 128;
constexpr int kSmallMaxRanges = 64;
static inline bool small_gemm_ranges_fit(int M, int N, int K)
{
	return M > 0 && N > 0 && K > kSmallGemmMaxK && K <= kSmallRange * kSmallMaxRanges && (long)M * N <= 65536 &&
	       (double)M * N * K <= 4.0e8;
}
static inline size_t small_gemm_ranges_workspace(int M, int N, int K)
{
	return sizeof(float) * (size_t)((K + kSmallRange - 1) / kSmallRange) * ((size_t)M * N + M);
}
// plain product + row sums only (no bias, activation, permutation, beta)
static inline int launch_small_gemm_ranges(SmallGemmParams p, int kernelClass, void *ws)
{
	const int ranges = (p.K + kSmallRange - 1) / kSmallRange;
	float *C = p.C, *rowSums = p.rowSums;
	const float alpha = p.alpha;
	p.kChunk = kSmallRange, p.partial = (float *)ws;
	p.rowSums = rowSums ? (float *)ws : nullptr; // only its being non-null matters to the kernel in this mode
	dim3 grid((unsigned)((p.M + kSmallTile - 1) / kSmallTile), (unsigned)((p.N + kSmallTile - 1) / kSmallTile), (unsigned)ranges);
	{
		LaunchScope scope(kernelClass, 2.0 * (double)p.M * p.N * p.K, 0);
		small_gemm_kernel<<<grid, 256, 0, stream()>>>(p);
	}
	const long per = (long)p.M * p.N + p.M;
	LaunchScope scope(FITRE_KC_SPLITK_REDUCE, 4.0 * (double)per * (ranges + 1));
	small_gemm_reduce_kernel<<<(unsigned)((per + 255) / 256), 256, 0, stream()>>>((const float *)ws, ranges, p.M, p.N, alpha, C, p.ldc, rowSums);
	return check_launch("small_gemm_kernel");
}

static inline int launch_small_gemm(const SmallGemmParams &p, int kernelClass)
{
	dim3 grid((unsigned)((p.M + kSmallTile - 1) / kSmallTile), (unsigned)((p.N + kSmallTile - 1) / kSmallTile));
	LaunchScope scope(kernelClass, 2.0 * (double)p.M * p.N * p.K, 0);
	small_gemm_kernel<<<grid, 256, 0, stream()>>>(p);
	return check_launch("small_gemm_kernel");
}

} // namespace fitre
