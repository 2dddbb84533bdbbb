// Bandwidth-bound elementwise kernels, level-1 helpers and scalar reductions.
// One templated grid-stride kernel per arity; 16-byte accesses whenever every
// pointer is 16-byte aligned, scalar accesses otherwise.
#include <math.h>
#include "common.h"
#include "fitre_nn.h"

namespace fitre {

constexpr int kEwBlock = 256;

template <typename T>
struct Vec;
template <>
struct Vec<float> {
	static constexpr int N = 1;
};
template <>
struct Vec<float4> {
	static constexpr int N = 4;
};

__device__ __forceinline__ float comp(const float &v, int) { return v; }
__device__ __forceinline__ float comp(const float4 &v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ __forceinline__ void setc(float &v, int, float x) { v = x; }
__device__ __forceinline__ void setc(float4 &v, int i, float x)
{
	if (i == 0) v.x = x;
	else if (i == 1) v.y = x;
	else if (i == 2) v.z = x;
	else v.w = x;
}

// out[i] = f(in0[i], in1[i], in2[i], in3[i]) for up to four inputs (unused ones alias in0).
template <typename V, int NIN, typename F>
__global__ void __launch_bounds__(kEwBlock) map_kernel(const V *a, const V *b, const V *c, const V *d, V *out, long nvec, F f)
{
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
		V va = a[i], vb = va, vc = va, vd = va, vo;
		if constexpr (NIN > 1) vb = b[i];
		if constexpr (NIN > 2) vc = c[i];
		if constexpr (NIN > 3) vd = d[i];
#pragma unroll
		for (int k = 0; k < Vec<V>::N; k++) setc(vo, k, f(comp(va, k), comp(vb, k), comp(vc, k), comp(vd, k)));
		out[i] = vo;
	}
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

template <int NIN, typename F>
static int launch_map(const char *name, int cls, const float *a, const float *b, const float *c, const float *d,
                      float *out, long n, F f)
{
	if (n == 0) return FITRE_OK;
	LaunchScope scope(cls, (double)(NIN + 1) * 4.0 * (double)n);
	bool vec = (n % 4 == 0) && aligned16(a) && aligned16(out) && (NIN < 2 || aligned16(b)) &&
	           (NIN < 3 || aligned16(c)) && (NIN < 4 || aligned16(d));
	if (vec) {
		long nv = n / 4;
		map_kernel<float4, NIN, F><<<blocks_for(nv, kEwBlock * 2, 8192), kEwBlock, 0, stream()>>>(
		    (const float4 *)a, (const float4 *)b, (const float4 *)c, (const float4 *)d, (float4 *)out, nv, f);
	} else {
		map_kernel<float, NIN, F><<<blocks_for(n, kEwBlock * 4, 8192), kEwBlock, 0, stream()>>>(a, b, c, d, out, n, f);
	}
	return check_launch(name);
}

// ---- functors ---------------------------------------------------------------
struct FAxpy { float alpha; __device__ float operator()(float x, float y, float, float) const { return y + alpha * x; } };
struct FScal { float alpha; __device__ float operator()(float x, float, float, float) const { return alpha * x; } };
struct FCopy { __device__ float operator()(float x, float, float, float) const { return x; } };
struct FMul { __device__ float operator()(float x, float y, float, float) const { return x * y; } };
struct FMulAdd2 { __device__ float operator()(float a, float b, float c, float d) const { return a * b + c * d; } };
struct FInvScale { float eps; __device__ float operator()(float x, float y, float, float) const { return x / (sqrtf(y) + eps); } };
struct FSqr { __device__ float operator()(float x, float, float, float) const { return x * x; } };
struct FSqrDecay { float decay; __device__ float operator()(float x, float y, float, float) const { return decay * x + (1.f - decay) * y * y; } };


// terms of the fully connected models' output heads (a = target y, b = network output or logit)
struct FScaledDiff { float scale; __device__ float operator()(float y, float z, float, float) const { return scale * (y - z); } };
struct FSquaredDiff { __device__ float operator()(float y, float z, float, float) const { return (y - z) * (y - z); } };
struct FLogisticLl { // y*x - log(1 + exp(x)), written as the reference does to stay finite for large |x|
	__device__ float operator()(float y, float x, float, float) const
	{
		const float ind = (x >= 0.f) ? 1.f : 0.f;
		return x * (y - ind) - logf(1.f + expf(x - 2.f * x * ind));
	}
};
struct FSoftmaxLl { __device__ float operator()(float y, float z, float, float) const { return y * logf(z); } };

// x[:, c] = exp(x[:, c]) / sum(exp(x[:, c])) for a column-major rows x cols matrix; one wave per column
__global__ void __launch_bounds__(256) column_softmax_kernel(float *x, int rows, int cols)
{
	const int lane = threadIdx.x & 63;
	const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
	if (c >= cols) return;
	float *p = x + (size_t)c * rows;
	float sum = 0.f;
	for (int r = lane; r < rows; r += 64) {
		const float e = expf(p[r]);
		p[r] = e;
		sum += e;
	}
	sum = wave_sum(sum);
	for (int r = lane; r < rows; r += 64) p[r] = p[r] / sum;
}

struct ActRelu { __device__ float operator()(float x, float, float, float) const { return x < 0.f ? 0.f : x; } };
struct ActSoftplus { __device__ float operator()(float x, float, float, float) const { return x < 20.f ? logf(1.f + expf(x)) : x; } };
struct ActElu { __device__ float operator()(float x, float, float, float) const { return x < 0.f ? (expf(x) - 1.f) : x; } };
struct ActSwish { __device__ float operator()(float x, float, float, float) const { return x / (1.f + expf(-x)); } };
struct ActLogistic { __device__ float operator()(float x, float, float, float) const { return sigmoidf(x); } };
struct ActTanh { __device__ float operator()(float x, float, float, float) const { return tanhf(x); } };

// backward functors take (delta, z_in, z_out)
struct DLogistic { __device__ float operator()(float d, float, float zo, float) const { return d * zo * (1.f - zo); } };
struct DTanh { __device__ float operator()(float d, float, float zo, float) const { return d * ((1.f + zo) * (1.f - zo)); } };
struct DSoftplus { __device__ float operator()(float d, float zi, float, float) const { return d * sigmoidf(zi); } };
struct DSwish { __device__ float operator()(float d, float zi, float zo, float) const { float t = sigmoidf(zi); return d * (zo + t * (1.f - zo)); } };
struct DRelu { __device__ float operator()(float d, float, float zo, float) const { return zo > 0.f ? d : 0.f; } };
struct DElu { __device__ float operator()(float d, float, float zo, float) const { return zo < 0.f ? d * (zo + 1.f) : d; } };

// ---- scalar reductions --------------------------------------------------------
enum RedOp { RED_SUM = 0, RED_DOT = 1, RED_SQR = 2, RED_ABS = 3, RED_ABSMAX = 4 };

template <int OP>
__global__ void __launch_bounds__(256) reduce_stage1(const float *x, const float *y, long n, double *partial)
{
	__shared__ double lds[4];
	double acc = 0.0;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
		float v = x[i];
		if constexpr (OP == RED_SUM) acc += (double)v;
		if constexpr (OP == RED_DOT) acc += (double)v * (double)y[i];
		if constexpr (OP == RED_SQR) acc += (double)v * (double)v;
		if constexpr (OP == RED_ABS) acc += (double)fabsf(v);
		if constexpr (OP == RED_ABSMAX) acc = fmax(acc, (double)fabsf(v));
	}
	if constexpr (OP == RED_ABSMAX) {
		float m = wave_max((float)acc);
		__shared__ float ldsm[4];
		if (threadIdx.x % kWave == 0) ldsm[threadIdx.x / kWave] = m;
		__syncthreads();
		if (threadIdx.x == 0) partial[blockIdx.x] = (double)fmaxf(fmaxf(ldsm[0], ldsm[1]), fmaxf(ldsm[2], ldsm[3]));
	} else {
		double t = block_sum<256>(acc, lds);
		if (threadIdx.x == 0) partial[blockIdx.x] = t;
	}
}

template <int OP>
__global__ void __launch_bounds__(256) reduce_stage2(const double *partial, int count, float *result)
{
	__shared__ double lds[4];
	double acc = 0.0;
	for (int i = threadIdx.x; i < count; i += 256) {
		if constexpr (OP == RED_ABSMAX) acc = fmax(acc, partial[i]);
		else acc += partial[i];
	}
	if constexpr (OP == RED_ABSMAX) {
		float m = wave_max((float)acc);
		__shared__ float ldsm[4];
		if (threadIdx.x % kWave == 0) ldsm[threadIdx.x / kWave] = m;
		__syncthreads();
		if (threadIdx.x == 0) result[0] = fmaxf(fmaxf(ldsm[0], ldsm[1]), fmaxf(ldsm[2], ldsm[3]));
	} else {
		double t = block_sum<256>(acc, lds);
		if (threadIdx.x == 0) result[0] = (OP == RED_SQR) ? (float)sqrt(t) : (float)t;
	}
}

constexpr int kRedBlocks = 1024;
static double *g_partials = nullptr; // kRedBlocks doubles + 1 float result slot
static float *g_host_result = nullptr;

void elementwise_release()
{
	if (g_partials) (void)hipFree(g_partials);
	if (g_host_result) (void)hipHostFree(g_host_result);
	g_partials = nullptr, g_host_result = nullptr;
}

static int ensure_reduce_buffers()
{
	if (g_partials) return FITRE_OK;
	FITRE_HIP_TRY(hipMalloc((void **)&g_partials, (kRedBlocks + 2) * sizeof(double)));
	FITRE_HIP_TRY(hipHostMalloc((void **)&g_host_result, 64, hipHostMallocDefault));
	return FITRE_OK;
}

template <int OP>
static int scalar_reduce(const char *name, int n, const float *x, const float *y, float *result)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(n >= 0 && x && result && (OP != RED_DOT || y), "%s: bad argument", name);
	if (n == 0) {
		*result = 0.f;
		return FITRE_OK;
	}
	int rc = ensure_reduce_buffers();
	if (rc) return rc;
	{
		LaunchScope scope(FITRE_KC_BLAS1, 4.0 * n * (OP == RED_DOT ? 2 : 1));
		unsigned blocks = blocks_for(n, 256 * 8, kRedBlocks);
		float *devResult = (float *)(g_partials + kRedBlocks);
		reduce_stage1<OP><<<blocks, 256, 0, stream()>>>(x, y, n, g_partials);
		reduce_stage2<OP><<<1, 256, 0, stream()>>>(g_partials, (int)blocks, devResult);
		rc = check_launch(name);
		if (rc) return rc;
		FITRE_HIP_TRY(hipMemcpyAsync(g_host_result, devResult, sizeof(float), hipMemcpyDeviceToHost, stream()));
	}
	FITRE_HIP_TRY(hipStreamSynchronize(stream()));
	*result = *g_host_result;
	return FITRE_OK;
}

// column-major rows x cols: out[i] = x[i] * y[i / rows]
__global__ void __launch_bounds__(256) col_scale_kernel(const float *x, int rows, long n, const float *y, float *out)
{
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = x[i] * y[i / rows];
}
// column-major rows x cols: mat[i] += vec[i % rows]
__global__ void __launch_bounds__(256) add_column_kernel(float *mat, int rows, long n, const float *vec)
{
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) mat[i] += vec[i % rows];
}
// [channels][perChannel]: x[c][i] += bias[c]
__global__ void __launch_bounds__(256) add_channel_bias_kernel(float *x, long perChannel, const float *bias)
{
	float b = bias[blockIdx.y];
	float *p = x + (size_t)blockIdx.y * perChannel;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < perChannel; i += stride) p[i] += b;
}
// out[r] = sum_c mat[r + c*rows]  (rows are the fast index).  A workgroup owns 16 rows; its 16
// column phases each add every 16th column in double, then the phases are combined in a fixed order.
__global__ void __launch_bounds__(256) row_sum_kernel(const float *mat, int rows, int cols, float *out)
{
	__shared__ double part[16][17];
	const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
	const int r = blockIdx.x * 16 + tx;
	double acc = 0.0;
	if (r < rows) {
		int c = ty;
		for (; c + 48 < cols; c += 64) { // four loads in flight
			float v0 = mat[(size_t)c * rows + r], v1 = mat[(size_t)(c + 16) * rows + r];
			float v2 = mat[(size_t)(c + 32) * rows + r], v3 = mat[(size_t)(c + 48) * rows + r];
			acc += (double)v0, acc += (double)v1, acc += (double)v2, acc += (double)v3;
		}
		for (; c < cols; c += 16) acc += (double)mat[(size_t)c * rows + r];
	}
	part[ty][tx] = acc;
	__syncthreads();
	if (ty == 0 && r < rows) {
		double total = 0.0;
#pragma unroll
		for (int q = 0; q < 16; q++) total += part[q][tx];
		out[r] = (float)total;
	}
}

// Counter-based generator: element g of the stream is a splitmix64 hash of seed and g, so the
// same (seed, position) gives the same number whatever the launch shape.  24 random bits make
// a float in (0, 1].
__host__ __device__ inline unsigned long long splitmix64(unsigned long long seed, unsigned long long g)
{
	unsigned long long z = seed + (g + 1ull) * 0x9E3779B97F4A7C15ull;
	z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
	z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
	return z ^ (z >> 31);
}
__device__ __forceinline__ float uniform_from(unsigned long long z) { return (float)((z >> 40) + 1ull) * (1.0f / 16777216.0f); }

__global__ void __launch_bounds__(256) random_uniform_kernel(float *out, long n, unsigned long long seed, unsigned long long first)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = uniform_from(splitmix64(seed, first + i));
}
// Box-Muller on consecutive pairs of the uniform stream
__global__ void __launch_bounds__(256) random_normal_kernel(float *out, long n, unsigned long long seed, unsigned long long first)
{
	const long pairs = (n + 1) / 2;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long j = (long)blockIdx.x * blockDim.x + threadIdx.x; j < pairs; j += stride) {
		const float u1 = uniform_from(splitmix64(seed, first + 2 * j)), u2 = uniform_from(splitmix64(seed, first + 2 * j + 1));
		const float r = sqrtf(-2.f * logf(u1));
		float sn, cs;
		sincosf(6.28318530717958647692f * u2, &sn, &cs);
		out[2 * j] = r * cs;
		if (2 * j + 1 < n) out[2 * j + 1] = r * sn;
	}
}
static unsigned long long g_rng_seed = 1234ull, g_rng_next = 0ull;

// out = rdelta * f'(.) + delta * f''(.) * rz_in: the directional derivative of delta * f'(.)
__global__ void __launch_bounds__(256) activation_rop_backward_kernel(int actFun, const float *rdelta, const float *delta,
                                                                       const float *z_in, const float *z_out, const float *rz_in,
                                                                       float *out, long n)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
		float f1, f2;
		act_derivatives(actFun, z_in ? z_in[i] : 0.f, z_out ? z_out[i] : 0.f, f1, f2);
		out[i] = rdelta[i] * f1 + delta[i] * f2 * rz_in[i];
	}
}

// The same, four elements per thread with 16-byte accesses.  SECOND false: the activation's second derivative is zero
// (ReLU, linear), so delta and rz_in are not read at all -- 12 instead of 24 bytes per element.  Tensors the activation
// does not use (z_in, z_out) may be null.
template <bool SECOND>
__global__ void __launch_bounds__(256) activation_rop_backward_vec_kernel(int actFun, const float *rdelta, const float *delta,
                                                                           const float *z_in, const float *z_out, const float *rz_in,
                                                                           float *out, long groups)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long g = (long)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
		const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
		const float4 rd = *reinterpret_cast<const float4 *>(rdelta + 4 * g);
		const float4 zi = z_in ? *reinterpret_cast<const float4 *>(z_in + 4 * g) : zero;
		const float4 zo = z_out ? *reinterpret_cast<const float4 *>(z_out + 4 * g) : zero;
		float4 d = zero, rz = zero;
		if constexpr (SECOND) {
			d = *reinterpret_cast<const float4 *>(delta + 4 * g);
			rz = *reinterpret_cast<const float4 *>(rz_in + 4 * g);
		}
		float4 r;
		float f1, f2;
		act_derivatives(actFun, zi.x, zo.x, f1, f2);
		r.x = SECOND ? rd.x * f1 + d.x * f2 * rz.x : rd.x * f1;
		act_derivatives(actFun, zi.y, zo.y, f1, f2);
		r.y = SECOND ? rd.y * f1 + d.y * f2 * rz.y : rd.y * f1;
		act_derivatives(actFun, zi.z, zo.z, f1, f2);
		r.z = SECOND ? rd.z * f1 + d.z * f2 * rz.z : rd.z * f1;
		act_derivatives(actFun, zi.w, zo.w, f1, f2);
		r.w = SECOND ? rd.w * f1 + d.w * f2 * rz.w : rd.w * f1;
		*reinterpret_cast<float4 *>(out + 4 * g) = r;
	}
}

// out = f'(z) rdz + rx g(z) dx with dx the delta BELOW the activation (dx = f'(z) dz, so f''(z) dz = g(z) dx):
// logistic f' = z (1 - z), g = 1 - 2 z; tanh f' = (1 + z)(1 - z), g = -2 z; linear f' = 1, g = 0.  rx == nullptr: first term only.
__global__ void __launch_bounds__(256) fc_rop_backward_kernel(int actFun, const float *z, const float *rdz, const float *rx,
                                                               const float *dx, float *out, long n)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
		const float zi = z ? z[i] : 0.f;
		float f1 = 1.f, g = 0.f;
		if (actFun == ACT_LOGISTIC) f1 = (1.f - zi) * zi, g = 1.f - 2.f * zi;
		else if (actFun == ACT_TANH) f1 = (1.f + zi) * (1.f - zi), g = -2.f * zi;
		float v = f1 * rdz[i];
		if (rx) v += rx[i] * g * dx[i];
		out[i] = v;
	}
}

// dst[c*ldd + r] = src[c*lds + r] for r < rows, c < cols
__global__ void __launch_bounds__(256) copy_2d_kernel(const float *src, long lds_, float *dst, long ldd, int rows, int cols)
{
	const long total = (long)rows * cols;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
		const long c = idx / rows, r = idx - c * rows;
		dst[c * ldd + r] = src[c * lds_ + r];
	}
}

// C(m x n) = alpha * op(A) + beta * op(B), column-major; one workgroup per 32 x 32 tile of C.  A transposed
// operand's tile is read along ITS contiguous index and turned in LDS (33-word rows: conflict-free), so every
// global access is coalesced.
__global__ void __launch_bounds__(256) geam_kernel(int transA, int transB, int m, int n, float alpha, const float *A, int lda, float beta,
                                                   const float *B, int ldb, float *C, int ldc)
{
	__shared__ float ta[32][33], tb[32][33];
	const int r0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
	const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // ty = 0..7
	// transposed operands: element (r, c) of op(X) is X[r * ld + c]: read with c contiguous
	if (A && transA)
		for (int q = ty; q < 32; q += 8) ta[q][tx] = (r0 + q < m && c0 + tx < n) ? A[(size_t)(r0 + q) * lda + c0 + tx] : 0.f;
	if (B && transB)
		for (int q = ty; q < 32; q += 8) tb[q][tx] = (r0 + q < m && c0 + tx < n) ? B[(size_t)(r0 + q) * ldb + c0 + tx] : 0.f;
	__syncthreads();
	for (int q = ty; q < 32; q += 8) {
		const int r = r0 + tx, c = c0 + q;
		if (r >= m || c >= n) continue;
		float v = 0.f;
		if (A) v += alpha * (transA ? ta[tx][q] : A[(size_t)c * lda + r]);
		if (B) v += beta * (transB ? tb[tx][q] : B[(size_t)c * ldb + r]);
		C[(size_t)c * ldc + r] = v;
	}
}

} // namespace fitre

using namespace fitre;

#define EW_CHECK(name, cond)                                                                         \
	FITRE_NEED_INIT();                                                                               \
	FITRE_REQUIRE(cond, "%s: null pointer or negative size", name)

extern "C" {

int fitre_hip_axpy(int n, float alpha, const float *x, float *y)
{
	EW_CHECK("fitre_hip_axpy", x && y && n >= 0);
	return launch_map<2>("axpy", FITRE_KC_BLAS1, x, y, nullptr, nullptr, y, n, FAxpy{ alpha });
}
int fitre_hip_scal(int n, float alpha, float *x)
{
	EW_CHECK("fitre_hip_scal", x && n >= 0);
	return launch_map<1>("scal", FITRE_KC_BLAS1, x, nullptr, nullptr, nullptr, x, n, FScal{ alpha });
}
// A copy far larger than the caches: every workgroup moves one contiguous 16 KiB piece, 64 bytes per lane in flight,
// around the caches in both directions (a 1 GiB copy: 0.77 of the 8 TB/s peak against 0.57 for the grid-stride form).
constexpr long kStreamCopyFloats = 16l << 20; // from 64 MiB per operand on
typedef float ew_f4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) stream_copy_kernel(const ew_f4 *a, ew_f4 *out, long nvec)
{
	const long base = (long)blockIdx.x * 1024 + threadIdx.x;
	ew_f4 r[4];
#pragma unroll
	for (int u = 0; u < 4; u++)
		if (base + u * 256 < nvec) r[u] = __builtin_nontemporal_load(a + base + u * 256);
#pragma unroll
	for (int u = 0; u < 4; u++)
		if (base + u * 256 < nvec) __builtin_nontemporal_store(r[u], out + base + u * 256);
}
int fitre_hip_copy(int n, const float *x, float *y)
{
	EW_CHECK("fitre_hip_copy", x && y && n >= 0);
	if (n >= kStreamCopyFloats && n % 4 == 0 && aligned16(x) && aligned16(y)) {
		LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)n);
		const long nv = n / 4;
		stream_copy_kernel<<<(unsigned)((nv + 1023) / 1024), 256, 0, stream()>>>((const ew_f4 *)x, (ew_f4 *)y, nv);
		return check_launch("copy");
	}
	return launch_map<1>("copy", FITRE_KC_BLAS1, x, nullptr, nullptr, nullptr, y, n, FCopy{});
}
int fitre_hip_dot(int n, const float *x, const float *y, float *result) { return scalar_reduce<RED_DOT>("fitre_hip_dot", n, x, y, result); }
int fitre_hip_nrm2(int n, const float *x, float *result) { return scalar_reduce<RED_SQR>("fitre_hip_nrm2", n, x, nullptr, result); }
int fitre_hip_asum(int n, const float *x, float *result) { return scalar_reduce<RED_ABS>("fitre_hip_asum", n, x, nullptr, result); }
int fitre_hip_norm_inf(int n, const float *x, float *result) { return scalar_reduce<RED_ABSMAX>("fitre_hip_norm_inf", n, x, nullptr, result); }
int fitre_hip_sum(int n, const float *x, float *result) { return scalar_reduce<RED_SUM>("fitre_hip_sum", n, x, nullptr, result); }

int fitre_hip_fill(float *x, long n, float value)
{
	EW_CHECK("fitre_hip_fill", x && n >= 0);
	// y = 0*x + value would read x; use a scaled copy of a constant instead
	struct FConst { float v; __device__ float operator()(float, float, float, float) const { return v; } };
	return launch_map<1>("fill", FITRE_KC_BLAS1, x, nullptr, nullptr, nullptr, x, n, FConst{ value });
}
int fitre_hip_hadamard(const float *x, float *y, long n)
{
	EW_CHECK("fitre_hip_hadamard", x && y && n >= 0);
	return launch_map<2>("hadamard", FITRE_KC_BLAS1, x, y, nullptr, nullptr, y, n, FMul{});
}
int fitre_hip_hadamard2(const float *m1, const float *m2, const float *m3, const float *m4, long n, float *out)
{
	EW_CHECK("fitre_hip_hadamard2", m1 && m2 && m3 && m4 && out && n >= 0);
	return launch_map<4>("hadamard2", FITRE_KC_BLAS1, m1, m2, m3, m4, out, n, FMulAdd2{});
}
int fitre_hip_elem_inv_scale(const float *x, const float *y, float eps, long n, float *out)
{
	EW_CHECK("fitre_hip_elem_inv_scale", x && y && out && n >= 0);
	return launch_map<2>("elem_inv_scale", FITRE_KC_BLAS1, x, y, nullptr, nullptr, out, n, FInvScale{ eps });
}
int fitre_hip_elem_sqr(const float *x, long n, float *out)
{
	EW_CHECK("fitre_hip_elem_sqr", x && out && n >= 0);
	return launch_map<1>("elem_sqr", FITRE_KC_BLAS1, x, nullptr, nullptr, nullptr, out, n, FSqr{});
}
int fitre_hip_elem_sqr_decay(const float *x, const float *y, float decay, long n, float *out)
{
	EW_CHECK("fitre_hip_elem_sqr_decay", x && y && out && n >= 0);
	return launch_map<2>("elem_sqr_decay", FITRE_KC_BLAS1, x, y, nullptr, nullptr, out, n, FSqrDecay{ decay });
}
int fitre_hip_mat_mat_scale(const float *x, const float *y, long n, float *out)
{
	EW_CHECK("fitre_hip_mat_mat_scale", x && y && out && n >= 0);
	return launch_map<2>("mat_mat_scale", FITRE_KC_BLAS1, x, y, nullptr, nullptr, out, n, FMul{});
}
int fitre_hip_mat_row_vec_scale(const float *x, int rows, int cols, const float *y, float *out)
{
	EW_CHECK("fitre_hip_mat_row_vec_scale", x && y && out && rows > 0 && cols > 0);
	long n = (long)rows * cols;
	LaunchScope scope(FITRE_KC_BLAS1, 8.0 * n);
	col_scale_kernel<<<blocks_for(n, 1024, 8192), 256, 0, stream()>>>(x, rows, n, y, out);
	return check_launch("col_scale_kernel");
}
int fitre_hip_add_column(float *mat, int rows, int cols, const float *vec)
{
	EW_CHECK("fitre_hip_add_column", mat && vec && rows > 0 && cols > 0);
	long n = (long)rows * cols;
	LaunchScope scope(FITRE_KC_BLAS1, 8.0 * n);
	add_column_kernel<<<blocks_for(n, 1024, 8192), 256, 0, stream()>>>(mat, rows, n, vec);
	return check_launch("add_column_kernel");
}
int fitre_hip_add_channel_bias(float *x, int channels, long perChannel, const float *bias)
{
	EW_CHECK("fitre_hip_add_channel_bias", x && bias && channels > 0 && perChannel > 0);
	FITRE_REQUIRE(channels <= 65535, "fitre_hip_add_channel_bias: %d channels exceed the grid limit", channels);
	LaunchScope scope(FITRE_KC_BLAS1, 8.0 * channels * perChannel);
	dim3 grid(blocks_for(perChannel, 1024, 1024), channels);
	add_channel_bias_kernel<<<grid, 256, 0, stream()>>>(x, perChannel, bias);
	return check_launch("add_channel_bias_kernel");
}
int fitre_hip_activation_rop_backward(int actFun, const float *rdelta, const float *delta, const float *z_in,
                                      const float *z_out, const float *rz_in, float *out, long n)
{
	EW_CHECK("fitre_hip_activation_rop_backward", rdelta && delta && rz_in && out && n >= 0);
	switch (actFun) {
	case ACT_LOGISTIC: case ACT_TANH: case CNN_ACT_RELU: case CNN_ACT_ELU:
		FITRE_REQUIRE(z_out, "fitre_hip_activation_rop_backward: activation %d needs z_out", actFun);
		break;
	case CNN_ACT_SOFTPLUS:
		FITRE_REQUIRE(z_in, "fitre_hip_activation_rop_backward: softplus needs z_in");
		break;
	case CNN_ACT_SWISH:
		FITRE_REQUIRE(z_in && z_out, "fitre_hip_activation_rop_backward: swish needs z_in and z_out");
		break;
	case ACT_LINEAR: case CNN_ACT_NONE: break;
	default: return fail(FITRE_E_UNSUPPORTED, "fitre_hip_activation_rop_backward: unknown activation code %d", actFun);
	}
	if (n == 0) return FITRE_OK;
	const bool usesZin = actFun == CNN_ACT_SOFTPLUS || actFun == CNN_ACT_SWISH;
	const bool usesZout = actFun == ACT_LOGISTIC || actFun == ACT_TANH || actFun == CNN_ACT_RELU || actFun == CNN_ACT_ELU || actFun == CNN_ACT_SWISH;
	const bool second = !(actFun == CNN_ACT_RELU || actFun == ACT_LINEAR || actFun == CNN_ACT_NONE);
	const uintptr_t bits = (uintptr_t)rdelta | (uintptr_t)out | (usesZin ? (uintptr_t)z_in : 0) | (usesZout ? (uintptr_t)z_out : 0) |
	                       (second ? ((uintptr_t)delta | (uintptr_t)rz_in) : 0);
	if (n % 4 == 0 && (bits & 15) == 0) {
		const long groups = n / 4;
		const double perElement = 8.0 + (usesZin ? 4.0 : 0.0) + (usesZout ? 4.0 : 0.0) + (second ? 8.0 : 0.0);
		LaunchScope scope(FITRE_KC_ACT_BWD, perElement * (double)n);
		if (second)
			activation_rop_backward_vec_kernel<true><<<blocks_for(groups, 512, 8192), 256, 0, stream()>>>(
			    actFun, rdelta, delta, usesZin ? z_in : nullptr, usesZout ? z_out : nullptr, rz_in, out, groups);
		else
			activation_rop_backward_vec_kernel<false><<<blocks_for(groups, 512, 8192), 256, 0, stream()>>>(
			    actFun, rdelta, delta, nullptr, usesZout ? z_out : nullptr, rz_in, out, groups);
		return check_launch("activation_rop_backward_vec_kernel");
	}
	LaunchScope scope(FITRE_KC_ACT_BWD, 24.0 * (double)n);
	activation_rop_backward_kernel<<<blocks_for(n, 1024, 8192), 256, 0, stream()>>>(actFun, rdelta, delta, z_in, z_out, rz_in, out, n);
	return check_launch("activation_rop_backward_kernel");
}

int fitre_hip_fc_rop_backward(int actFun, const float *z, const float *rdz, const float *rx, const float *dx, float *out, long n)
{
	EW_CHECK("fitre_hip_fc_rop_backward", rdz && out && n >= 0 && (rx == nullptr || dx != nullptr));
	if (actFun != ACT_LOGISTIC && actFun != ACT_TANH && actFun != ACT_LINEAR)
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_fc_rop_backward: activation code %d (logistic, tanh and linear only)", actFun);
	FITRE_REQUIRE(z || actFun == ACT_LINEAR, "fitre_hip_fc_rop_backward: activation %d needs z", actFun);
	if (n == 0) return FITRE_OK;
	LaunchScope scope(FITRE_KC_ACT_BWD, 20.0 * (double)n);
	fc_rop_backward_kernel<<<blocks_for(n, 1024, 8192), 256, 0, stream()>>>(actFun, z, rdz, rx, dx, out, n);
	return check_launch("fc_rop_backward_kernel");
}

int fitre_hip_column_softmax(float *x, int rows, int cols)
{
	EW_CHECK("fitre_hip_column_softmax", x && rows > 0 && cols > 0);
	LaunchScope scope(FITRE_KC_SOFTMAX, 8.0 * (double)rows * cols);
	column_softmax_kernel<<<(cols + 3) / 4, 256, 0, stream()>>>(x, rows, cols);
	return check_launch("column_softmax_kernel");
}

int fitre_hip_output_terms(int kind, const float *y, const float *z, long n, float scale, float *out)
{
	EW_CHECK("fitre_hip_output_terms", y && z && out && n >= 0);
	switch (kind) {
	case FITRE_TERM_SCALED_DIFFERENCE: return launch_map<2>("scaled_difference", FITRE_KC_SOFTMAX, y, z, nullptr, nullptr, out, n, FScaledDiff{ scale });
	case FITRE_TERM_SQUARED_DIFFERENCE: return launch_map<2>("squared_difference", FITRE_KC_SOFTMAX, y, z, nullptr, nullptr, out, n, FSquaredDiff{});
	case FITRE_TERM_LOGISTIC_LL: return launch_map<2>("logistic_ll", FITRE_KC_SOFTMAX, y, z, nullptr, nullptr, out, n, FLogisticLl{});
	case FITRE_TERM_SOFTMAX_LL: return launch_map<2>("softmax_ll", FITRE_KC_SOFTMAX, y, z, nullptr, nullptr, out, n, FSoftmaxLl{});
	default: return fail(FITRE_E_UNSUPPORTED, "fitre_hip_output_terms: unknown kind %d", kind);
	}
}

int fitre_hip_random_seed(unsigned long long seed)
{
	g_rng_seed = seed;
	g_rng_next = 0ull;
	return FITRE_OK;
}

int fitre_hip_random_uniform(float *out, long n)
{
	EW_CHECK("fitre_hip_random_uniform", out && n >= 0);
	if (n == 0) return FITRE_OK;
	LaunchScope scope(FITRE_KC_BLAS1, 4.0 * (double)n);
	random_uniform_kernel<<<blocks_for(n, 1024, 4096), 256, 0, stream()>>>(out, n, g_rng_seed, g_rng_next);
	g_rng_next += (unsigned long long)n;
	return check_launch("random_uniform_kernel");
}

int fitre_hip_random_normal(float *out, long n)
{
	EW_CHECK("fitre_hip_random_normal", out && n >= 0);
	if (n == 0) return FITRE_OK;
	LaunchScope scope(FITRE_KC_BLAS1, 4.0 * (double)n);
	random_normal_kernel<<<blocks_for((n + 1) / 2, 1024, 4096), 256, 0, stream()>>>(out, n, g_rng_seed, g_rng_next);
	g_rng_next += (unsigned long long)(2 * ((n + 1) / 2));
	return check_launch("random_normal_kernel");
}

int fitre_hip_geam(int transA, int transB, int m, int n, float alpha, const float *A, int lda, float beta, const float *B, int ldb,
                   float *C, int ldc)
{
	EW_CHECK("fitre_hip_geam", C && m > 0 && n > 0);
	FITRE_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "fitre_hip_geam: bad transpose flags");
	FITRE_REQUIRE(A || alpha == 0.f, "fitre_hip_geam: A is null with alpha != 0");
	FITRE_REQUIRE(B || beta == 0.f, "fitre_hip_geam: B is null with beta != 0");
	FITRE_REQUIRE(ldc >= m && (!A || lda >= (transA ? n : m)) && (!B || ldb >= (transB ? n : m)),
	              "fitre_hip_geam: leading dimension too small");
	// in-place use as cuBLAS allows it: C may be A (resp. B) only when that operand is not transposed and shares ldc
	FITRE_REQUIRE(!(C == A && (transA || lda != ldc)) && !(C == B && (transB || ldb != ldc)),
	              "fitre_hip_geam: in-place only for an untransposed operand with the same leading dimension");
	LaunchScope scope(FITRE_KC_BLAS1, 4.0 * (double)m * n * (1 + (A && alpha != 0.f ? 1 : 0) + (B && beta != 0.f ? 1 : 0)));
	dim3 grid((m + 31) / 32, (n + 31) / 32);
	geam_kernel<<<grid, 256, 0, stream()>>>(transA, transB, m, n, alpha, (alpha != 0.f) ? A : nullptr, lda, beta,
	                                        (beta != 0.f) ? B : nullptr, ldb, C, ldc);
	return check_launch("geam_kernel");
}

int fitre_hip_copy_2d(float *dst, long ldd, const float *src, long lds_, int rows, int cols)
{
	EW_CHECK("fitre_hip_copy_2d", dst && src && rows > 0 && cols > 0);
	FITRE_REQUIRE(ldd >= 1 && lds_ >= 1, "fitre_hip_copy_2d: non-positive leading dimension");
	LaunchScope scope(FITRE_KC_BLAS1, 8.0 * (double)rows * cols);
	copy_2d_kernel<<<blocks_for((long)rows * cols, 512, 8192), 256, 0, stream()>>>(src, lds_, dst, ldd, rows, cols);
	return check_launch("copy_2d_kernel");
}

int fitre_hip_row_sum(const float *mat, int rows, int cols, float *out)
{
	EW_CHECK("fitre_hip_row_sum", mat && out && rows > 0 && cols > 0);
	LaunchScope scope(FITRE_KC_BIAS_GRAD, 4.0 * rows * cols);
	row_sum_kernel<<<(rows + 15) / 16, 256, 0, stream()>>>(mat, rows, cols, out);
	return check_launch("row_sum_kernel");
}

int fitre_hip_activation_forward(int actFun, const float *in, float *out, long n)
{
	EW_CHECK("fitre_hip_activation_forward", in && out && n >= 0);
	const int cls = FITRE_KC_ACT_FWD;
	switch (actFun) {
	case CNN_ACT_RELU: return launch_map<1>("relu", cls, in, nullptr, nullptr, nullptr, out, n, ActRelu{});
	case CNN_ACT_SOFTPLUS: return launch_map<1>("softplus", cls, in, nullptr, nullptr, nullptr, out, n, ActSoftplus{});
	case CNN_ACT_ELU: return launch_map<1>("elu", cls, in, nullptr, nullptr, nullptr, out, n, ActElu{});
	case CNN_ACT_SWISH: return launch_map<1>("swish", cls, in, nullptr, nullptr, nullptr, out, n, ActSwish{});
	case ACT_LOGISTIC: return launch_map<1>("logistic", cls, in, nullptr, nullptr, nullptr, out, n, ActLogistic{});
	case ACT_TANH: return launch_map<1>("tanh", cls, in, nullptr, nullptr, nullptr, out, n, ActTanh{});
	case ACT_LINEAR:
	case CNN_ACT_NONE:
		if (in == out) return FITRE_OK;
		return launch_map<1>("copy", cls, in, nullptr, nullptr, nullptr, out, n, FCopy{});
	default: return fail(FITRE_E_UNSUPPORTED, "fitre_hip_activation_forward: unknown activation code %d", actFun);
	}
}

int fitre_hip_activation_backward(int actFun, const float *delta, const float *z_in, const float *z_out, float *out, long n)
{
	EW_CHECK("fitre_hip_activation_backward", delta && out && n >= 0);
	const int cls = FITRE_KC_ACT_BWD;
	switch (actFun) {
	case ACT_LOGISTIC:
		FITRE_REQUIRE(z_out, "activation backward (logistic): z_out is null");
		return launch_map<3>("dlogistic", cls, delta, z_out, z_out, nullptr, out, n, DLogistic{});
	case ACT_TANH:
		FITRE_REQUIRE(z_out, "activation backward (tanh): z_out is null");
		return launch_map<3>("dtanh", cls, delta, z_out, z_out, nullptr, out, n, DTanh{});
	case CNN_ACT_SOFTPLUS:
		FITRE_REQUIRE(z_in, "activation backward (softplus): z_in is null");
		return launch_map<2>("dsoftplus", cls, delta, z_in, nullptr, nullptr, out, n, DSoftplus{});
	case CNN_ACT_SWISH:
		FITRE_REQUIRE(z_in && z_out, "activation backward (swish): z_in or z_out is null");
		return launch_map<3>("dswish", cls, delta, z_in, z_out, nullptr, out, n, DSwish{});
	case CNN_ACT_RELU:
		FITRE_REQUIRE(z_out, "activation backward (relu): z_out is null");
		return launch_map<3>("drelu", cls, delta, z_out, z_out, nullptr, out, n, DRelu{});
	case CNN_ACT_ELU:
		FITRE_REQUIRE(z_out, "activation backward (elu): z_out is null");
		return launch_map<3>("delu", cls, delta, z_out, z_out, nullptr, out, n, DElu{});
	case ACT_LINEAR:
	case CNN_ACT_NONE:
		if (delta == out) return FITRE_OK;
		return launch_map<1>("copy", cls, delta, nullptr, nullptr, nullptr, out, n, FCopy{});
	default: return fail(FITRE_E_UNSUPPORTED, "fitre_hip_activation_backward: unknown activation code %d", actFun);
	}
}

} // extern "C"
