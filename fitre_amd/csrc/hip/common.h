// Shared plumbing of the gfx950 device layer: status reporting, the launch
// stream, per-class launch accounting, wave64 reductions and fast division.
#pragma once
#include <float.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "fitre_hip.h"
#include "fitre_nn.h"

namespace fitre {

constexpr int kWave = 64;

// ---- status -------------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
hipStream_t stream(); // the selected lane
// Column-major product C(MxN) = alpha*op(A)*op(B) + beta*C on the tile engine (defined with
// fitre_hip_gemm).  flags: kGemmMirror = the product is symmetric (M == N, same operand on
// both sides): compute the tiles on and above the diagonal and mirror them; kGemmTriK = both
// operands are zero where the reduction index is below their row / column index.
// kGemmBLowerTri / kGemmBUpperTri: op(B) (K x N) is zero above / below its diagonal; kGemmALowerTri: op(A) (M x K) is zero
// above its diagonal -- the reduction skips the zero part (batched products only).
constexpr int kGemmMirror = 1, kGemmTriK = 2, kGemmBLowerTri = 4, kGemmBUpperTri = 8, kGemmALowerTri = 16;
int gemm_ex(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb,
            float beta, float *C, int ldc, const float *bias, int flags, int kernelClass, void *ws, size_t wsBytes);
size_t gemm_ex_workspace(int M, int N, int K, int flags);
// `batch` such products of one shape in one launch (plus one reduction launch when split).  Problem b reads
// A + b*strideA, B + b*strideB, writes C + b*strideC and keeps its split-K partials in (char *)ws + b*wsStrideBytes;
// wsBytes is the workspace of ONE problem (gemm_ex_workspace).
int gemm_ex_batched(int batch, int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda, long strideA,
                    const float *B, int ldb, long strideB, float beta, float *C, int ldc, long strideC, int flags, int kernelClass,
                    void *ws, size_t wsBytes, long wsStrideBytes);
// One argument set of gemm_ex_batched; gemm_pair_batched queues two such products that do not depend on each other --
// as ONE launch when both are small enough to run unsplit on the deep 64 x 64 tile (a chain of dependent launches is then
// one launch shorter), as two launches otherwise.
struct BatchedProduct {
	int transA, transB, M, N, K;
	float alpha;
	const float *A;
	int lda;
	long strideA;
	const float *B;
	int ldb;
	long strideB;
	float beta;
	float *C;
	int ldc;
	long strideC;
	int flags;
};
int gemm_pair_batched(int batch, const BatchedProduct &first, const BatchedProduct &second, int kernelClass, void *ws, size_t wsBytes,
                      long wsStrideBytes);

// ---- float64 products (dense_f64.hip) -------------------------------------------------------
// A matrix operand: element (r, c) of floats or doubles at r * rs + c * cs; kind FITRE_MAT_SYM_PAIR: a symmetric
// matrix of order rs kept as a pair of floats per element in one dense float matrix with leading dimension cs (the
// rounded value on and above the diagonal, the remainder below it; see fitre_matrix in fitre_hip.h).
struct DMat {
	const void *p;
	long rs, cs;       // element (r, c) at r * rs + c * cs (pair of floats: order rs, column-major with leading dimension cs)
	int kind;          // FITRE_MAT_*
	long onesRow, onesCol; // floats only: a row / column that is not in memory and reads as onesValue (-1: none)
	double onesValue;
};

struct DOut {
	void *p;
	long rs, cs;
	int kind;
	// an optional third term of the result, addScale * add(i, j) (doubles; null: none)
	const double *add = nullptr;
	long addRs = 0, addCs = 0;
	double addScale = 0.0;
};
inline DMat dmat64(const double *p, long rs, long cs) { return DMat{ p, rs, cs, FITRE_MAT_F64, -1, -1, 0.0 }; }
inline DMat dmat32(const float *p, long rs, long cs) { return DMat{ p, rs, cs, FITRE_MAT_F32, -1, -1, 0.0 }; }
// kDgMirror: symmetric product (M == N, C = C^T): only the tiles on and above the diagonal are computed, the others
// mirrored.  Reduction ranges: A(i, k) is zero for k > i (kDgALower) / k < i (kDgAUpper), B(k, j) is zero for k < j
// (kDgBLower) / k > j (kDgBUpper).
constexpr int kDgMirror = 1, kDgALower = 2, kDgAUpper = 4, kDgBLower = 8, kDgBUpper = 16;
// C(M x N) = alpha * A(M x K) * B(K x N) + beta * C (+ C.addScale * C.add), plus diagAdd on the diagonal, accumulated in float64 on the
// matrix pipes; queued on the selected lane.  ws: dgemm_workspace bytes, 256-byte aligned (a smaller one costs splits).
int dgemm(long M, long N, long K, double alpha, DMat A, DMat B, double beta, DOut C, double diagAdd, int flags, int kernelClass,
          void *ws, size_t wsBytes);
size_t dgemm_workspace(long M, long N, long K, int flags);
// result = W^-1 for the symmetric positive definite W (n x n doubles, destroyed), stored dense with leading dimension
// n as `kind`; pivotInfo (device int): 0, or the 1-based index of the first non-positive pivot.
int dspd_inverse_run(double *W, int n, void *result, int kind, void *ws, size_t wsBytes, int *pivotInfo);
size_t dspd_inverse_workspace(int n);
constexpr int kMaxLanes = 4; // one hardware queue each
int lane();           // its index (0 .. kMaxLanes - 1)
int lane_compute_units();     // compute units a kernel launched on the selected lane can occupy
int lane_compute_units_min(); // the smallest such count over the lanes
int device_compute_units();
int weight_grad_units();      // compute units the 3 x 3 weight gradients are planned for (fitre_hip_weight_grad_share)
int share_of_units(int cus, int eighths); // that many eighths of `cus`, in whole groups of eight
bool ready();
int current_device();            // the device fitre_hip_init selected, -1 before
// Per-device set-up of the file that holds the batch-norm kernels (address of its static scratch
// array on the current device); called by fitre_hip_init with the device current.
int layers_device_setup(int device);
// Shutdown hooks of the files that keep device buffers between calls (loss scratch, reduction partials, patch
// decode tables): free them and forget their sizes, so that a later fitre_hip_init -- possibly on another device --
// starts clean.  Called by fitre_hip_shutdown after every lane has drained.
void layers_release();
void elementwise_release();
void conv_gemm_release();

#define FITRE_HIP_TRY(expr)                                                                          \
	do {                                                                                             \
		hipError_t e_ = (expr);                                                                      \
		if (e_ != hipSuccess)                                                                        \
			return ::fitre::fail(FITRE_E_DEVICE, "%s failed at %s:%d: %s", #expr, __FILE__,          \
			                     __LINE__, hipGetErrorString(e_));                                   \
	} while (0)

#define FITRE_REQUIRE(cond, ...)                                                                     \
	do {                                                                                             \
		if (!(cond)) return ::fitre::fail(FITRE_E_ARGUMENT, __VA_ARGS__);                            \
	} while (0)

#define FITRE_NEED_INIT()                                                                            \
	do {                                                                                             \
		if (!::fitre::ready())                                                                       \
			return ::fitre::fail(FITRE_E_DEVICE, "%s: fitre_hip_init has not been called", __func__); \
	} while (0)

// ---- wave priority of the bandwidth-bound kernels ---------------------------
// The short memory-bound kernels of the delta chain run beside chip-filling matrix kernels of the other
// lane, on the registers those leave free on every SIMD (the weight-gradient kernels are held to three waves of at
// most 152 registers for that).  Measured on the VGG-11 batch-256 backward pass: with the memory-bound waves at the
// top priority (FITRE_WAVE_PRIORITY=3) the pass is 1.5 % shorter than with none -- they issue a few instructions per
// 16 bytes and then wait for memory, so the matrix waves lose little, and the chain behind them moves on sooner; the
// matrix kernels' waves at 2 instead of 0 (FITRE_MATRIX_WAVE_PRIORITY) gain 0.4 %.  (While the largest
// weight-gradient kernel still filled the register file, the memory-bound kernels beside it only ran in its tail,
// and raising them cost 3 %.)
#ifndef FITRE_WAVE_PRIORITY
#define FITRE_WAVE_PRIORITY 3
#endif
#define FITRE_RAISE_WAVE_PRIORITY()                                                                  \
	do {                                                                                             \
		if (FITRE_WAVE_PRIORITY > 0) __builtin_amdgcn_s_setprio(FITRE_WAVE_PRIORITY);                \
	} while (0)

#ifndef FITRE_MATRIX_WAVE_PRIORITY
#define FITRE_MATRIX_WAVE_PRIORITY 2
#endif
#define FITRE_RAISE_MATRIX_WAVE_PRIORITY()                                                           \
	do {                                                                                             \
		if (FITRE_MATRIX_WAVE_PRIORITY > 0) __builtin_amdgcn_s_setprio(FITRE_MATRIX_WAVE_PRIORITY);  \
	} while (0)

// ---- activation functions: first and second derivative ------------------------
__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + expf(-x)); }
// f1 = f'(x), f2 = f''(x) from the activation's input zi and output zo (whichever the function needs)
__device__ __forceinline__ void act_derivatives(int actFun, float zi, float zo, float &f1, float &f2)
{
	switch (actFun) {
	case ACT_LOGISTIC: f1 = zo * (1.f - zo), f2 = f1 * (1.f - 2.f * zo); break;
	case ACT_TANH: f1 = (1.f + zo) * (1.f - zo), f2 = -2.f * zo * f1; break;
	case CNN_ACT_SOFTPLUS: {
		const float s = sigmoidf(zi);
		f1 = s, f2 = s * (1.f - s);
		break;
	}
	case CNN_ACT_SWISH: {
		const float s = sigmoidf(zi);
		f1 = zo + s * (1.f - zo), f2 = s * (1.f - s) * (2.f + zi * (1.f - 2.f * s));
		break;
	}
	case CNN_ACT_RELU: f1 = zo > 0.f ? 1.f : 0.f, f2 = 0.f; break;
	case CNN_ACT_ELU: f1 = zo < 0.f ? zo + 1.f : 1.f, f2 = zo < 0.f ? zo + 1.f : 0.f; break;
	default: f1 = 1.f, f2 = 0.f; break;
	}
}

// f'(x) alone, in the form the pooling / activation kernels multiply a gradient by
__device__ __forceinline__ float act_derivative(int actFun, float zi, float zo)
{
	switch (actFun) {
	case ACT_LOGISTIC: return zo * (1.f - zo);
	case ACT_TANH: return (1.f + zo) * (1.f - zo);
	case CNN_ACT_SOFTPLUS: return 1.f / (1.f + expf(-zi));
	case CNN_ACT_SWISH: {
		float t = 1.f / (1.f + expf(-zi));
		return zo + t * (1.f - zo);
	}
	case CNN_ACT_RELU: return zo > 0.f ? 1.f : 0.f;
	case CNN_ACT_ELU: return zo < 0.f ? zo + 1.f : 1.f;
	default: return 1.f;
	}
}

// strict-> scan of four values in order, starting below every finite float
__device__ __forceinline__ int scan2x2(float v0, float v1, float v2, float v3)
{
	float best = -FLT_MAX;
	int arg = -1;
	if (v0 > best) { best = v0; arg = 0; }
	if (v1 > best) { best = v1; arg = 1; }
	if (v2 > best) { best = v2; arg = 2; }
	if (v3 > best) { best = v3; arg = 3; }
	return arg;
}

static inline bool act_known(int actFun)
{
	switch (actFun) {
	case ACT_LOGISTIC:
	case ACT_TANH:
	case ACT_LINEAR:
	case CNN_ACT_NONE:
	case CNN_ACT_SOFTPLUS:
	case CNN_ACT_ELU:
	case CNN_ACT_RELU:
	case CNN_ACT_SWISH: return true;
	default: return false;
	}
}
static inline bool act_needs_zin(int actFun) { return actFun == CNN_ACT_SOFTPLUS || actFun == CNN_ACT_SWISH; }
static inline bool act_needs_zout(int actFun)
{
	return actFun == ACT_LOGISTIC || actFun == ACT_TANH || actFun == CNN_ACT_SWISH || actFun == CNN_ACT_RELU ||
	       actFun == CNN_ACT_ELU;
}


// ---- per-class launch accounting ------------------------------------------
// A LaunchScope brackets the launches made while it is alive with two events
// when accounting is on; otherwise it costs one branch.
struct LaunchScope {
	LaunchScope(int kernelClass, double work, int tile = 0);
	~LaunchScope();
	int slot;
};

int check_launch(const char *what);

// ---- integer division by a run-time constant ------------------------------
// q = n / d for 0 <= n < 2^31 via one 32x32->64 multiply.
struct FastDiv {
	uint32_t mul;
	uint32_t shiftm1; // ceil(log2 d) - 1 (0 for d <= 2)
	uint32_t div;
	__host__ __device__ FastDiv() : mul(0), shiftm1(0), div(1) {}
	__host__ __device__ explicit FastDiv(uint32_t d) : mul(0), shiftm1(0), div(d)
	{
		if (d <= 1) return;
		uint32_t l = 0;
		while ((1ull << l) < d) l++;
		shiftm1 = l - 1;
		mul = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
	}
	__device__ __forceinline__ uint32_t quot(uint32_t n) const
	{
		uint32_t t = __umulhi(n, mul);
		uint32_t q = (t + ((n - t) >> 1)) >> shiftm1;
		return (div == 1) ? n : q; // a select, not a branch
	}
	__device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const
	{
		q = quot(n);
		r = n - q * div;
	}
};

// ---- wave64 reductions ------------------------------------------------------
// Butterfly over the 64 lanes: DPP inside a row of 16 lanes, ds_swizzle across
// rows of a 32-lane half, one bpermute across halves.  Every lane ends with
// the total.
__device__ __forceinline__ int dpp_quad_xor1(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false); }
__device__ __forceinline__ int dpp_quad_xor2(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false); }
__device__ __forceinline__ int dpp_half_mirror(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false); }
__device__ __forceinline__ int dpp_row_mirror(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false); }
__device__ __forceinline__ int swz_xor16(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401F); }
__device__ __forceinline__ int xor32(int v) { return __shfl_xor(v, 32, 64); }

template <typename F>
__device__ __forceinline__ float wave_shuffle_f(float v, F f)
{
	return __int_as_float(f(__float_as_int(v)));
}
template <typename F>
__device__ __forceinline__ double wave_shuffle_d(double v, F f)
{
	int lo = __double2loint(v), hi = __double2hiint(v);
	return __hiloint2double(f(hi), f(lo));
}

__device__ __forceinline__ float wave_sum(float v)
{
	v += wave_shuffle_f(v, dpp_quad_xor1);
	v += wave_shuffle_f(v, dpp_quad_xor2);
	v += wave_shuffle_f(v, dpp_half_mirror);
	v += wave_shuffle_f(v, dpp_row_mirror);
	v += wave_shuffle_f(v, swz_xor16);
	v += wave_shuffle_f(v, xor32);
	return v;
}
__device__ __forceinline__ double wave_sum(double v)
{
	v += wave_shuffle_d(v, dpp_quad_xor1);
	v += wave_shuffle_d(v, dpp_quad_xor2);
	v += wave_shuffle_d(v, dpp_half_mirror);
	v += wave_shuffle_d(v, dpp_row_mirror);
	v += wave_shuffle_d(v, swz_xor16);
	v += wave_shuffle_d(v, xor32);
	return v;
}
__device__ __forceinline__ float wave_max(float v)
{
	v = fmaxf(v, wave_shuffle_f(v, dpp_quad_xor1));
	v = fmaxf(v, wave_shuffle_f(v, dpp_quad_xor2));
	v = fmaxf(v, wave_shuffle_f(v, dpp_half_mirror));
	v = fmaxf(v, wave_shuffle_f(v, dpp_row_mirror));
	v = fmaxf(v, wave_shuffle_f(v, swz_xor16));
	v = fmaxf(v, wave_shuffle_f(v, xor32));
	return v;
}

// Sum over a workgroup of BLOCK threads (BLOCK a multiple of 64, <= 1024);
// every thread gets the total.  lds must hold BLOCK/64 values of T.
template <int BLOCK, typename T>
__device__ __forceinline__ T block_sum(T v, T *lds)
{
	constexpr int WAVES = BLOCK / kWave;
	v = wave_sum(v);
	if constexpr (WAVES == 1) return v;
	const int wave = threadIdx.x / kWave;
	__syncthreads();
	if ((threadIdx.x % kWave) == 0) lds[wave] = v;
	__syncthreads();
	T total = lds[0];
#pragma unroll
	for (int w = 1; w < WAVES; w++) total += lds[w];
	return total;
}

// Three sums at once (two barriers instead of six); every thread gets the totals.
// lds must hold 3 * BLOCK/64 values of T.
template <int BLOCK, typename T>
__device__ __forceinline__ void block_sum3(T &a, T &b, T &c, T *lds)
{
	constexpr int WAVES = BLOCK / kWave;
	a = wave_sum(a);
	b = wave_sum(b);
	c = wave_sum(c);
	if constexpr (WAVES == 1) return;
	const int wave = threadIdx.x / kWave;
	__syncthreads();
	if ((threadIdx.x % kWave) == 0) {
		lds[3 * wave] = a;
		lds[3 * wave + 1] = b;
		lds[3 * wave + 2] = c;
	}
	__syncthreads();
	a = lds[0], b = lds[1], c = lds[2];
#pragma unroll
	for (int w = 1; w < WAVES; w++) {
		a += lds[3 * w];
		b += lds[3 * w + 1];
		c += lds[3 * w + 2];
	}
}

inline unsigned blocks_for(long n, int perBlock, unsigned cap = 1u << 20)
{
	long b = (n + perBlock - 1) / perBlock;
	if (b < 1) b = 1;
	if (b > (long)cap) b = cap;
	return (unsigned)b;
}

} // namespace fitre
