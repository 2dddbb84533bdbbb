// Bandwidth-bound layer kernels on [C][N][A][B] tensors: pooling, batch
// normalisation, per-channel sums, softmax cross entropy and the layout change
// at the convolution / fully-connected boundary.
#include <float.h>
#include <math.h>
#include "common.h"
#include "fitre_nn.h"

namespace fitre {

// =====================================================================
// pooling
// =====================================================================

struct PoolGeom {
	int inA, inB, outA, outB, ksize, stride, padding;
	FastDiv divOutB, divOutA, divInB, divInA;
};

static PoolGeom make_geom(int inA, int inB, int ksize, int stride, int padding, int outA, int outB)
{
	PoolGeom g;
	g.inA = inA;
	g.inB = inB;
	g.outA = outA;
	g.outB = outB;
	g.ksize = ksize;
	g.stride = stride;
	g.padding = padding;
	g.divOutB = FastDiv((uint32_t)outB);
	g.divOutA = FastDiv((uint32_t)outA);
	g.divInB = FastDiv((uint32_t)inB);
	g.divInA = FastDiv((uint32_t)inA);
	return g;
}

// First maximum of one window in memory order (A outer, B inner, strict >);
// returns the offset inside the map, or -1 for a window with no valid cell.
__device__ __forceinline__ int window_argmax(const float *map, const PoolGeom &g, int oa, int ob, float &best)
{
	int a0 = oa * g.stride - g.padding, b0 = ob * g.stride - g.padding;
	int arg = -1;
	best = -FLT_MAX;
	for (int da = 0; da < g.ksize; da++) {
		int a = a0 + da;
		if (a < 0 || a >= g.inA) continue;
		for (int db = 0; db < g.ksize; db++) {
			int b = b0 + db;
			if (b < 0 || b >= g.inB) continue;
			float t = map[a * g.inB + b];
			if (t > best) {
				best = t;
				arg = a * g.inB + b;
			}
		}
	}
	return arg;
}

// one thread per pooled cell
template <int MODE> // 0 max value, 1 average, 2 argmax index
__global__ void __launch_bounds__(256) pool_forward_kernel(const float *in, PoolGeom g, long maps, float *out, int *index)
{
	long total = maps * g.outA * g.outB;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		uint32_t q, ob, oa, map;
		g.divOutB.divmod((uint32_t)i, q, ob);
		g.divOutA.divmod(q, map, oa);
		const float *src = in + (size_t)map * g.inA * g.inB;
		if constexpr (MODE == 1) {
			int a0 = (int)oa * g.stride - g.padding, b0 = (int)ob * g.stride - g.padding;
			float s = 0.f;
			for (int da = 0; da < g.ksize; da++) {
				int a = a0 + da;
				if (a < 0 || a >= g.inA) continue;
				for (int db = 0; db < g.ksize; db++) {
					int b = b0 + db;
					if (b < 0 || b >= g.inB) continue;
					s += src[a * g.inB + b];
				}
			}
			out[i] = s / (float)(g.ksize * g.ksize);
		} else {
			float best;
			int arg = window_argmax(src, g, (int)oa, (int)ob, best);
			if constexpr (MODE == 0) out[i] = best;
			else index[i] = (arg < 0) ? INT_MAX : arg;
		}
	}
}

// out[pooled cell] = values[argmax of z over the cell's window]: what a max pool passes on of a
// second tensor that rides along (the directional derivative of its input)
__global__ void __launch_bounds__(256) pool_routed_kernel(const float *values, const float *z, PoolGeom g, long maps, float *out)
{
	long total = maps * g.outA * g.outB;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		uint32_t q, ob, oa, map;
		g.divOutB.divmod((uint32_t)i, q, ob);
		g.divOutA.divmod(q, map, oa);
		float best;
		int arg = window_argmax(z + (size_t)map * g.inA * g.inB, g, (int)oa, (int)ob, best);
		out[i] = (arg < 0) ? 0.f : values[(size_t)map * g.inA * g.inB + arg];
	}
}

// Gradient reaching input cell (a, b) of one map: sum over the windows that
// contain the cell.  No atomics: every input cell is owned by one thread.
template <int POOL> // 0 max, 1 average
__device__ __forceinline__ float pool_gather(const float *dmap, const float *zmap, const PoolGeom &g, int a, int b)
{
	// windows oa with oa*stride - padding <= a <= oa*stride - padding + ksize - 1
	int oaHi = (a + g.padding) / g.stride;
	int obHi = (b + g.padding) / g.stride;
	int oaLo = (a + g.padding - g.ksize + g.stride) / g.stride; // ceil((a+p-k+1)/s) for a+p-k+1 >= 1-s
	int obLo = (b + g.padding - g.ksize + g.stride) / g.stride;
	if (a + g.padding - g.ksize + 1 <= 0) oaLo = 0;
	if (b + g.padding - g.ksize + 1 <= 0) obLo = 0;
	if (oaHi >= g.outA) oaHi = g.outA - 1;
	if (obHi >= g.outB) obHi = g.outB - 1;
	float acc = 0.f;
	const int self = a * g.inB + b;
	for (int oa = oaLo; oa <= oaHi; oa++) {
		for (int ob = obLo; ob <= obHi; ob++) {
			if constexpr (POOL == 0) {
				float best;
				if (window_argmax(zmap, g, oa, ob, best) == self) acc += dmap[oa * g.outB + ob];
			} else {
				acc += dmap[oa * g.outB + ob] * (1.f / (float)(g.ksize * g.ksize));
			}
		}
	}
	return acc;
}


// One thread per input cell.  POOL: 0 max, 1 average, 2 none.  FUSE_ACT: also
// write dxAct = gradient * f'(.).
template <int POOL, bool FUSE_ACT>
__global__ void __launch_bounds__(256)
pool_backward_kernel(const float *delta, const float *z_in, const float *z_act, PoolGeom g, long maps, int actFun,
                     float *dxPool, float *dxAct)
{
	long perMap = (long)g.inA * g.inB;
	long total = maps * perMap;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		float gval;
		if constexpr (POOL == 2) {
			gval = delta[i];
		} else {
			uint32_t q, b, a, map;
			g.divInB.divmod((uint32_t)i, q, b);
			g.divInA.divmod(q, map, a);
			gval = pool_gather<POOL>(delta + (size_t)map * g.outA * g.outB, z_act + (size_t)map * perMap, g, (int)a, (int)b);
		}
		if (dxPool) dxPool[i] = gval;
		if constexpr (FUSE_ACT) {
			float zo = z_act ? z_act[i] : 0.f;
			float zi = z_in ? z_in[i] : 0.f;
			dxAct[i] = gval * act_derivative(actFun, zi, zo);
		}
	}
}

// 16-byte store; stream: nothing reads the value again soon and the tensor is larger than the caches
// can usefully hold, so it is written past them (measured on a 67 MB tensor: the pass 44 -> 36.5 us; on
// a 34 MB one the plain store is the faster)
__device__ __forceinline__ void store4(float *p, float4 v, bool stream)
{
	if (stream) {
		typedef float v4f __attribute__((ext_vector_type(4)));
		v4f t = { v.x, v.y, v.z, v.w };
		__builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
	} else {
		*reinterpret_cast<float4 *>(p) = v;
	}
}

// No pooling, 16-byte accesses: dxPool = delta (a snapshot, may be null), dxAct = delta * f'(.).
__global__ void __launch_bounds__(256)
nopool_act_backward_vec_kernel(const float4 *delta, const float4 *z_in, const float4 *z_act, long groups, int actFun, float4 *dxPool,
                               float4 *dxAct)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += stride) {
		const float4 d = delta[i];
		const float4 zo = z_act ? z_act[i] : make_float4(0.f, 0.f, 0.f, 0.f);
		const float4 zi = z_in ? z_in[i] : make_float4(0.f, 0.f, 0.f, 0.f);
		if (dxPool) dxPool[i] = d;
		float4 r;
		r.x = d.x * act_derivative(actFun, zi.x, zo.x);
		r.y = d.y * act_derivative(actFun, zi.y, zo.y);
		r.z = d.z * act_derivative(actFun, zi.z, zo.z);
		r.w = d.w * act_derivative(actFun, zi.w, zo.w);
		dxAct[i] = r;
	}
}

// Overlapping max-pool windows (e.g. 3x3 / stride 2): one workgroup per map keeps the map and the
// arg-max of every window in LDS, so a window is scanned once instead of once per cell it contains
// (up to four times for 3/2), and each cell then looks up the windows it belongs to.  Same scan and
// the same order of additions as pool_backward_kernel<0>: identical results.  Maps of up to
// kPoolMapCells cells and kPoolMapWindows windows.
constexpr int kPoolMapCells = 4096, kPoolMapWindows = 1280;
template <bool FUSE_ACT>
__global__ void __launch_bounds__(256)
maxpool_map_backward_kernel(const float *delta, const float *z_in, const float *z_act, PoolGeom g, int actFun, float *dxPool,
                            float *dxAct)
{
	__shared__ float zmap[kPoolMapCells];
	__shared__ int arg[kPoolMapWindows];
	const int cells = g.inA * g.inB, windows = g.outA * g.outB;
	const size_t mapOff = (size_t)blockIdx.x * cells;
	const float *dmap = delta + (size_t)blockIdx.x * windows;
	for (int i = threadIdx.x; i < cells; i += blockDim.x) zmap[i] = z_act[mapOff + i];
	__syncthreads();
	for (int w = threadIdx.x; w < windows; w += blockDim.x) {
		uint32_t oa, ob;
		g.divOutB.divmod((uint32_t)w, oa, ob);
		float best;
		arg[w] = window_argmax(zmap, g, (int)oa, (int)ob, best);
	}
	__syncthreads();
	for (int i = threadIdx.x; i < cells; i += blockDim.x) {
		uint32_t a, b;
		g.divInB.divmod((uint32_t)i, a, b);
		int oaHi = ((int)a + g.padding) / g.stride, obHi = ((int)b + g.padding) / g.stride;
		int oaLo = ((int)a + g.padding - g.ksize + g.stride) / g.stride, obLo = ((int)b + g.padding - g.ksize + g.stride) / g.stride;
		if ((int)a + g.padding - g.ksize + 1 <= 0) oaLo = 0;
		if ((int)b + g.padding - g.ksize + 1 <= 0) obLo = 0;
		if (oaHi >= g.outA) oaHi = g.outA - 1;
		if (obHi >= g.outB) obHi = g.outB - 1;
		float acc = 0.f;
		for (int oa = oaLo; oa <= oaHi; oa++)
			for (int ob = obLo; ob <= obHi; ob++)
				if (arg[oa * g.outB + ob] == i) acc += dmap[oa * g.outB + ob];
		if (dxPool) dxPool[mapOff + i] = acc;
		if constexpr (FUSE_ACT) {
			const float zi = z_in ? z_in[mapOff + i] : 0.f;
			dxAct[mapOff + i] = acc * act_derivative(actFun, zi, zmap[i]);
		}
	}
}

// The same for windows of compile-time extent and stride (3 / 2: AlexNet-style pools), moved with 16-byte
// accesses: a "group" is `mapsPerGroup` consecutive maps, i.e. one contiguous range of the tensor, walked in
// 16-byte groups aligned in global memory (the range may start anywhere: its first and last 16 bytes are
// handled cell by cell).  One group per workgroup: maps and
// pooled gradient to LDS (every load of a thread in flight at once), one scan per window, then every cell looks
// up the (at most ceil(KS/ST)^2) windows that contain it, in the same order as pool_backward_kernel<0>, so the
// results are identical.
struct PoolGroup {
	int nCells, nWin, lead, nVec;
	size_t vbase, dbase;
};
constexpr int kPoolVecPerThread = (kPoolMapCells + 8) / 4 / 256 + 1; // 5
constexpr int kPoolWinPerThread = kPoolMapWindows / 256;             // 5

__device__ __forceinline__ PoolGroup pool_group(long group, int mapsPerGroup, long maps, int cells, int windows)
{
	PoolGroup q;
	const long firstMap = group * mapsPerGroup;
	long n = maps - firstMap;
	if (n > mapsPerGroup) n = mapsPerGroup;
	if (n < 0) n = 0;
	q.nCells = (int)n * cells;
	q.nWin = (int)n * windows;
	const size_t g0 = (size_t)firstMap * cells;
	q.lead = (int)(g0 & 3);
	q.nVec = q.nCells ? (q.lead + q.nCells + 3) >> 2 : 0;
	q.vbase = g0 - q.lead; // multiple of four floats
	q.dbase = (size_t)firstMap * windows;
	return q;
}

__device__ __forceinline__ void pool_group_load(const PoolGroup &q, const float *z_act, const float *delta, int tid,
                                                float4 (&t)[kPoolVecPerThread], float (&d)[kPoolWinPerThread])
{
#pragma unroll
	for (int k = 0; k < kPoolVecPerThread; k++) {
		const int v = tid + 256 * k;
		const int e0 = 4 * v - q.lead;
		t[k] = make_float4(0.f, 0.f, 0.f, 0.f);
		if (v < q.nVec) {
			const float *src = z_act + q.vbase + 4 * (size_t)v;
			if (e0 >= 0 && e0 + 3 < q.nCells) {
				t[k] = *reinterpret_cast<const float4 *>(src);
			} else {
				if (e0 >= 0 && e0 < q.nCells) t[k].x = src[0];
				if (e0 + 1 >= 0 && e0 + 1 < q.nCells) t[k].y = src[1];
				if (e0 + 2 >= 0 && e0 + 2 < q.nCells) t[k].z = src[2];
				if (e0 + 3 >= 0 && e0 + 3 < q.nCells) t[k].w = src[3];
			}
		}
	}
#pragma unroll
	for (int k = 0; k < kPoolWinPerThread; k++) {
		const int w = tid + 256 * k;
		d[k] = (w < q.nWin) ? delta[q.dbase + w] : 0.f;
	}
}

template <bool FUSE_ACT, int KS, int ST>
__global__ void __launch_bounds__(256)
maxpool_maps_backward_kernel(const float *delta, const float *z_in, const float *z_act, PoolGeom g, int mapsPerGroup,
                             long maps, FastDiv divCells, FastDiv divWindows, int actFun, float *dxPool, float *dxAct, bool streamPool)
{
	// LDS sized by the launch for one group: [maps | pooled gradient | window arg-max]
	extern __shared__ __align__(16) unsigned char pool_lds[];
	float *zs = reinterpret_cast<float *>(pool_lds);
	float *dl = zs + ((mapsPerGroup * g.inA * g.inB + 8 + 3) & ~3);
	int *arg = reinterpret_cast<int *>(dl + mapsPerGroup * g.outA * g.outB);
	const int cells = g.inA * g.inB, windows = g.outA * g.outB;
	const int tid = threadIdx.x;
	constexpr int NC = (KS + ST - 1) / ST;

	{
		const PoolGroup cur = pool_group((long)blockIdx.x, mapsPerGroup, maps, cells, windows);
		// ---- global -> registers (every load of the thread in flight at once) -> LDS.  One group per workgroup:
		// a workgroup that walks several groups, with or without the next group's loads held in registers across
		// the work on the current one, was measured and is slower (86 resp. 110 registers instead of 56: the
		// kernel is bound by latency, i.e. by how many workgroups a compute unit holds).
		{
			float4 t[kPoolVecPerThread];
			float d[kPoolWinPerThread];
			pool_group_load(cur, z_act, delta, tid, t, d);
#pragma unroll
			for (int k = 0; k < kPoolVecPerThread; k++) {
				const int v = tid + 256 * k;
				if (v < cur.nVec) *reinterpret_cast<float4 *>(zs + 4 * v) = t[k];
			}
#pragma unroll
			for (int k = 0; k < kPoolWinPerThread; k++) {
				const int w = tid + 256 * k;
				if (w < cur.nWin) dl[w] = d[k];
			}
		}
		__syncthreads();

		// ---- one scan per window: first maximum in memory order (strict >), offset inside its map
		for (int w = tid; w < cur.nWin; w += 256) {
			uint32_t m, r, oa, ob;
			divWindows.divmod((uint32_t)w, m, r);
			g.divOutB.divmod(r, oa, ob);
			const float *zmap = zs + cur.lead + (int)m * cells;
			const int a0 = (int)oa * ST - g.padding, b0 = (int)ob * ST - g.padding;
			float best = -FLT_MAX;
			int at = -1;
#pragma unroll
			for (int da = 0; da < KS; da++) {
				const int a = a0 + da;
				if (a < 0 || a >= g.inA) continue;
#pragma unroll
				for (int db = 0; db < KS; db++) {
					const int b = b0 + db;
					if (b < 0 || b >= g.inB) continue;
					const float zv = zmap[a * g.inB + b];
					if (zv > best) {
						best = zv;
						at = a * g.inB + b;
					}
				}
			}
			arg[w] = at;
		}
		__syncthreads();

		// ---- every cell gathers from the windows that contain it: at most NC = ceil(KS / ST) along each axis, the
		// last of them (a + padding) / ST; all candidates are read at once and added in ascending window order
		for (int v = tid; v < cur.nVec; v += 256) {
			const int e0 = 4 * v - cur.lead;
			float acc[4], zo[4];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int i = e0 + e;
				acc[e] = 0.f;
				zo[e] = zs[4 * v + e];
				const bool live = i >= 0 && i < cur.nCells;
				uint32_t m, r, a, b;
				divCells.divmod((uint32_t)(live ? i : 0), m, r);
				g.divInB.divmod(r, a, b);
				const int ta = (int)a + g.padding, tb = (int)b + g.padding;
				const int oaHi = ta / ST, obHi = tb / ST;
				const int wbase = (int)m * windows;
				int hit[NC][NC];
				float dv[NC][NC];
#pragma unroll
				for (int da = NC - 1; da >= 0; da--) {
					const int oa = oaHi - da;
					const bool okA = live && oa >= 0 && oa < g.outA && ta - oa * ST < KS;
#pragma unroll
					for (int db = NC - 1; db >= 0; db--) {
						const int ob = obHi - db;
						const bool ok = okA && ob >= 0 && ob < g.outB && tb - ob * ST < KS;
						const int w = ok ? wbase + oa * g.outB + ob : 0;
						hit[da][db] = ok ? arg[w] : -2;
						dv[da][db] = dl[w];
					}
				}
#pragma unroll
				for (int da = NC - 1; da >= 0; da--)
#pragma unroll
					for (int db = NC - 1; db >= 0; db--)
						if (hit[da][db] == (int)r) acc[e] += dv[da][db];
			}
			const size_t at = cur.vbase + 4 * (size_t)v;
			const bool whole = e0 >= 0 && e0 + 3 < cur.nCells;
			if (dxPool) {
				if (whole) {
					store4(dxPool + at, make_float4(acc[0], acc[1], acc[2], acc[3]), streamPool);
				} else {
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (e0 + e >= 0 && e0 + e < cur.nCells) dxPool[at + e] = acc[e];
				}
			}
			if constexpr (FUSE_ACT) {
				float zi[4] = { 0.f, 0.f, 0.f, 0.f };
				if (z_in) {
					if (whole) {
						const float4 zq = *reinterpret_cast<const float4 *>(z_in + at);
						zi[0] = zq.x, zi[1] = zq.y, zi[2] = zq.z, zi[3] = zq.w;
					} else {
#pragma unroll
						for (int e = 0; e < 4; e++)
							if (e0 + e >= 0 && e0 + e < cur.nCells) zi[e] = z_in[at + e];
					}
				}
				float r4[4];
#pragma unroll
				for (int e = 0; e < 4; e++) r4[e] = acc[e] * act_derivative(actFun, zi[e], zo[e]);
				if (whole) {
					*reinterpret_cast<float4 *>(dxAct + at) = make_float4(r4[0], r4[1], r4[2], r4[3]);
				} else {
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (e0 + e >= 0 && e0 + e < cur.nCells) dxAct[at + e] = r4[e];
				}
			}
		}
	}
}

// LDS bytes of maxpool_maps_backward_kernel for groups of `per` maps
static size_t maps_group_lds(int cells, int windows, int per)
{
	return sizeof(float) * (size_t)((per * cells + 8 + 3) & ~3) + 2 * sizeof(float) * (size_t)per * windows;
}

// How many consecutive maps one workgroup of maxpool_maps_backward_kernel takes: as many as fit its LDS arrays,
// but no more than leaves about six workgroups per compute unit.
static int maps_per_group(int cells, int windows, long maps)
{
	long fit = kPoolMapCells / cells;
	if (kPoolMapWindows / windows < fit) fit = kPoolMapWindows / windows;
	long spread = maps / 1536;
	if (spread < 1) spread = 1;
	if (fit > spread) fit = spread;
	return (int)(fit < 1 ? 1 : fit);
}


// pool_routed_kernel for 2x2 / stride 2 / no padding windows on maps with B % 4 == 0 and A even: one thread per pair of
// pooled cells adjacent along B, i.e. a 2 x 4 patch of z and of the values, moved with 16-byte accesses.
__global__ void __launch_bounds__(256) pool_routed2_kernel(const float *values, const float *z, int inA, int inB, long maps, float *out)
{
	const int outB2 = inB / 4, outA = inA / 2, outB = inB / 2;
	const long perMap = (long)outA * outB2, total = maps * perMap;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		const long map = i / perMap;
		const int rem = (int)(i - map * perMap);
		const int oa = rem / outB2, pb = rem - oa * outB2;
		const size_t in = (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
		const float4 z0 = *reinterpret_cast<const float4 *>(z + in), z1 = *reinterpret_cast<const float4 *>(z + in + inB);
		const float4 v0 = *reinterpret_cast<const float4 *>(values + in), v1 = *reinterpret_cast<const float4 *>(values + in + inB);
		const int a = scan2x2(z0.x, z0.y, z1.x, z1.y), b = scan2x2(z0.z, z0.w, z1.z, z1.w);
		float2 r;
		r.x = a == 0 ? v0.x : (a == 1 ? v0.y : (a == 2 ? v1.x : (a == 3 ? v1.y : 0.f)));
		r.y = b == 0 ? v0.z : (b == 1 ? v0.w : (b == 2 ? v1.z : (b == 3 ? v1.w : 0.f)));
		*reinterpret_cast<float2 *>(out + (size_t)map * outA * outB + (size_t)oa * outB + 2 * pb) = r;
	}
}

// Non-overlapping 2x2 / stride 2 / no padding max pool, even extents: one
// thread per pair of pooled cells adjacent along B, i.e. a 2 x 4 input patch
// moved with 16-byte accesses.  Fused with the activation derivative.
template <bool FUSE_ACT>
__global__ void __launch_bounds__(256)
maxpool2_backward_kernel(const float *delta, const float *z_in, const float *z_act, int inA, int inB, long maps,
                         int actFun, float *dxPool, float *dxAct)
{
	const int outB2 = inB / 4; // pairs of pooled cells per pooled row
	const int outA = inA / 2;
	long total = maps * outA * outB2;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		long map = i / ((long)outA * outB2);
		int rem = (int)(i - map * outA * outB2);
		int oa = rem / outB2, pb = rem - oa * outB2;
		size_t inOff = (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
		size_t dOff = (size_t)map * outA * (inB / 2) + (size_t)oa * (inB / 2) + 2 * pb;
		float4 r0 = *reinterpret_cast<const float4 *>(z_act + inOff);
		float4 r1 = *reinterpret_cast<const float4 *>(z_act + inOff + inB);
		float2 d = *reinterpret_cast<const float2 *>(delta + dOff);
		// memory-order scan of each 2x2 window: (a0,b0), (a0,b1), (a1,b0), (a1,b1)
		float4 g0 = make_float4(0.f, 0.f, 0.f, 0.f), g1 = g0;
		int arg = scan2x2(r0.x, r0.y, r1.x, r1.y);
		if (arg == 0) g0.x = d.x;
		else if (arg == 1) g0.y = d.x;
		else if (arg == 2) g1.x = d.x;
		else if (arg == 3) g1.y = d.x;
		arg = scan2x2(r0.z, r0.w, r1.z, r1.w);
		if (arg == 0) g0.z = d.y;
		else if (arg == 1) g0.w = d.y;
		else if (arg == 2) g1.z = d.y;
		else if (arg == 3) g1.w = d.y;
		if (dxPool) {
			*reinterpret_cast<float4 *>(dxPool + inOff) = g0;
			*reinterpret_cast<float4 *>(dxPool + inOff + inB) = g1;
		}
		if constexpr (FUSE_ACT) {
			float4 i0 = r0, i1 = r1;
			if (z_in) {
				i0 = *reinterpret_cast<const float4 *>(z_in + inOff);
				i1 = *reinterpret_cast<const float4 *>(z_in + inOff + inB);
			}
			g0.x *= act_derivative(actFun, i0.x, r0.x);
			g0.y *= act_derivative(actFun, i0.y, r0.y);
			g0.z *= act_derivative(actFun, i0.z, r0.z);
			g0.w *= act_derivative(actFun, i0.w, r0.w);
			g1.x *= act_derivative(actFun, i1.x, r1.x);
			g1.y *= act_derivative(actFun, i1.y, r1.y);
			g1.z *= act_derivative(actFun, i1.z, r1.z);
			g1.w *= act_derivative(actFun, i1.w, r1.w);
			*reinterpret_cast<float4 *>(dxAct + inOff) = g0;
			*reinterpret_cast<float4 *>(dxAct + inOff + inB) = g1;
		}
	}
}

static int check_pool_shape(const char *fn, int channels, int samples, int inA, int inB, int ksize, int stride,
                            int padding, int outA, int outB)
{
	FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0 && ksize > 0 && stride > 0 && padding >= 0,
	              "%s: non-positive shape (C=%d N=%d A=%d B=%d k=%d s=%d p=%d)", fn, channels, samples, inA, inB,
	              ksize, stride, padding);
	FITRE_REQUIRE(outA == (inA + 2 * padding - ksize) / stride + 1 && outB == (inB + 2 * padding - ksize) / stride + 1 &&
	                  outA > 0 && outB > 0,
	              "%s: pooled extent %dx%d does not match input %dx%d, k=%d s=%d p=%d", fn, outA, outB, inA, inB, ksize,
	              stride, padding);
	FITRE_REQUIRE(padding < ksize, "%s: padding %d >= window %d leaves empty windows", fn, padding, ksize);
	FITRE_REQUIRE((double)channels * samples * inA * inB < 2147483647.0, "%s: tensor exceeds 2^31 elements", fn);
	return FITRE_OK;
}

// =====================================================================
// per-channel reductions and batch normalisation
// =====================================================================

constexpr int kRedBlock = 256;

// number of segments each channel is cut into
static int segments_for(int channels, long perChannel)
{
	long perBlockMin = 4096; // at least 16 elements per thread
	long s = (perChannel + perBlockMin - 1) / perBlockMin;
	long want = (2048 + channels - 1) / channels; // aim at >= 2048 workgroups
	if (s > want) s = want;
	if (s > 256) s = 256;
	if (s < 1) s = 1;
	return (int)s;
}

// Segment [lo, hi) of a channel handled by block (blockIdx.x of gridDim.x), in units of 4 elements
// so that 16-byte accesses stay aligned.
__device__ __forceinline__ void segment_range(long perChannel, long &lo, long &hi)
{
	long quads = (perChannel + 3) / 4;
	long per = (quads + gridDim.x - 1) / gridDim.x;
	lo = (long)blockIdx.x * per * 4;
	hi = lo + per * 4;
	if (hi > perChannel) hi = perChannel;
	if (lo > perChannel) lo = perChannel;
}

// sums per (channel, segment): MODE 0: sum x; 1: sum x, sum x*y; 2: sum x, sum x^2;
// 3: sum x, sum x*y, sum y (slots of four doubles instead of two)
template <int MODE, bool VEC>
__global__ void __launch_bounds__(kRedBlock)
channel_partial_kernel(const float *x, const float *y, long perChannel, double *partial)
{
	__shared__ double lds[kRedBlock / kWave];
	constexpr bool PAIR = (MODE == 1 || MODE == 3);
	const int c = blockIdx.y;
	const float *px = x + (size_t)c * perChannel;
	const float *py = PAIR ? y + (size_t)c * perChannel : nullptr;
	long lo, hi;
	segment_range(perChannel, lo, hi);
	double s0 = 0.0, s1 = 0.0, s2 = 0.0;
	if constexpr (VEC) {
		for (long i = lo + 4 * (long)threadIdx.x; i + 3 < hi; i += 4 * kRedBlock) {
			float4 a = *reinterpret_cast<const float4 *>(px + i);
			float t0 = (a.x + a.y) + (a.z + a.w);
			s0 += (double)t0;
			if constexpr (PAIR) {
				float4 b = *reinterpret_cast<const float4 *>(py + i);
				s1 += (double)(a.x * b.x) + (double)(a.y * b.y) + (double)(a.z * b.z) + (double)(a.w * b.w);
				if constexpr (MODE == 3) s2 += (double)((b.x + b.y) + (b.z + b.w));
			}
			if constexpr (MODE == 2)
				s1 += (double)a.x * a.x + (double)a.y * a.y + (double)a.z * a.z + (double)a.w * a.w;
		}
		long tail = lo + ((hi - lo) / 4) * 4;
		for (long i = tail + threadIdx.x; i < hi; i += kRedBlock) {
			float a = px[i];
			s0 += (double)a;
			if constexpr (PAIR) s1 += (double)(a * py[i]);
			if constexpr (MODE == 3) s2 += (double)py[i];
			if constexpr (MODE == 2) s1 += (double)a * a;
		}
	} else {
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			float a = px[i];
			s0 += (double)a;
			if constexpr (PAIR) s1 += (double)(a * py[i]);
			if constexpr (MODE == 3) s2 += (double)py[i];
			if constexpr (MODE == 2) s1 += (double)a * a;
		}
	}
	double t0 = block_sum<kRedBlock>(s0, lds);
	double t1 = 0.0, t2 = 0.0;
	if constexpr (MODE != 0) t1 = block_sum<kRedBlock>(s1, lds);
	if constexpr (MODE == 3) t2 = block_sum<kRedBlock>(s2, lds);
	if (threadIdx.x == 0) {
		constexpr int SLOT = (MODE == 3) ? 4 : 2;
		size_t slot = ((size_t)c * gridDim.x + blockIdx.x) * SLOT;
		partial[slot] = t0;
		partial[slot + 1] = t1;
		if constexpr (MODE == 3) partial[slot + 2] = t2;
	}
}

// out[c] = sum over segments of partial[c][s][which]
__global__ void channel_finish_kernel(const double *partial, int segments, int which, int channels, float *out)
{
	int c = blockIdx.x * blockDim.x + threadIdx.x;
	if (c >= channels) return;
	double acc = 0.0;
	for (int s = 0; s < segments; s++) acc += partial[((size_t)c * segments + s) * 2 + which];
	out[c] = (float)acc;
}

// batch-norm forward, statistics: mean, biased variance, running statistics
__global__ void bn_stats_kernel(const double *partial, int segments, int channels, long perChannel, float momentum,
                                float *mean, float *variance, float *runMean, float *runVar)
{
	int c = blockIdx.x * blockDim.x + threadIdx.x;
	if (c >= channels) return;
	double s = 0.0, ss = 0.0;
	for (int k = 0; k < segments; k++) {
		s += partial[((size_t)c * segments + k) * 2];
		ss += partial[((size_t)c * segments + k) * 2 + 1];
	}
	double m = s / (double)perChannel;
	double v = ss / (double)perChannel - m * m;
	if (v < 0.0) v = 0.0;
	mean[c] = (float)m;
	variance[c] = (float)v;
	runMean[c] = momentum * runMean[c] + (1.f - momentum) * (float)m;
	runVar[c] = momentum * runVar[c] + (1.f - momentum) * (float)v;
}

template <bool VEC>
__global__ void __launch_bounds__(kRedBlock)
bn_normalize_kernel(const float *x, const float *mean, const float *variance, float epsilon, long perChannel, float *zhat)
{
	const int c = blockIdx.y;
	const float mu = mean[c];
	const float inv = 1.f / sqrtf(variance[c] + epsilon);
	const float *px = x + (size_t)c * perChannel;
	float *po = zhat + (size_t)c * perChannel;
	long lo, hi;
	segment_range(perChannel, lo, hi);
	if constexpr (VEC) {
		for (long i = lo + 4 * (long)threadIdx.x; i + 3 < hi; i += 4 * kRedBlock) {
			float4 a = *reinterpret_cast<const float4 *>(px + i);
			a.x = (a.x - mu) * inv;
			a.y = (a.y - mu) * inv;
			a.z = (a.z - mu) * inv;
			a.w = (a.w - mu) * inv;
			*reinterpret_cast<float4 *>(po + i) = a;
		}
		long tail = lo + ((hi - lo) / 4) * 4;
		for (long i = tail + threadIdx.x; i < hi; i += kRedBlock) po[i] = (px[i] - mu) * inv;
	} else {
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) po[i] = (px[i] - mu) * inv;
	}
}

// the activation functions, as fitre_hip_activation_forward evaluates them
__device__ __forceinline__ float act_forward_value(int actFun, float x)
{
	switch (actFun) {
	case CNN_ACT_RELU: return x < 0.f ? 0.f : x;
	case CNN_ACT_SOFTPLUS: return x < 20.f ? logf(1.f + expf(x)) : x;
	case CNN_ACT_ELU: return x < 0.f ? (expf(x) - 1.f) : x;
	case CNN_ACT_SWISH: return x / (1.f + expf(-x));
	case ACT_LOGISTIC: return 1.f / (1.f + expf(-x));
	case ACT_TANH: return tanhf(x);
	default: return x;
	}
}
__device__ __forceinline__ float4 act_forward4(int actFun, float4 v)
{
	return make_float4(act_forward_value(actFun, v.x), act_forward_value(actFun, v.y), act_forward_value(actFun, v.z),
	                   act_forward_value(actFun, v.w));
}
// strict-> scan of a 2 x 2 window in memory order, as the pooling kernels scan it
__device__ __forceinline__ float max2x2(float v0, float v1, float v2, float v3)
{
	float best = -FLT_MAX;
	if (v0 > best) best = v0;
	if (v1 > best) best = v1;
	if (v2 > best) best = v2;
	if (v3 > best) best = v3;
	return best;
}

// Normalisation, activation and 2x2 / stride 2 max pooling of a layer in one pass over its convolution output: x is
// read once and zhat, the activation output and the pooled output are written (the three separate passes read four
// tensors for the same three results).  One (channel, segment) per workgroup.  `partial`: the per-segment sums of x and
// x^2 of channel_partial_kernel<2> (segmentsIn per channel) -- every workgroup of a channel adds them up in the same
// order, the first one also stores the statistics; null: statMean / statVar hold the statistics to use.  zhat null: no
// normalisation (x goes into the activation as it is).  POOL 0: the unit of work is a 2 x 4 patch (B % 4 == 0, A even);
// POOL 2: no pooling, the unit is a 16-byte group.
template <int POOL>
__global__ void __launch_bounds__(kRedBlock)
bn_act_pool_forward_kernel(const float *x, const double *partial, int segmentsIn, float momentum, float *mean, float *variance,
                           float *runMean, float *runVar, const float *statMean, const float *statVar, float epsilon, int samples,
                           int inA, int inB, int actFun, float *zhat, float *actOut, float *poolOut)
{
	const int c = blockIdx.y;
	const long perChannel = (long)samples * inA * inB;
	float mu = 0.f, inv = 1.f;
	if (zhat) {
		float var;
		if (partial) {
			double s = 0.0, ss = 0.0;
			for (int k = 0; k < segmentsIn; k++) {
				s += partial[((size_t)c * segmentsIn + k) * 2];
				ss += partial[((size_t)c * segmentsIn + k) * 2 + 1];
			}
			const double m = s / (double)perChannel;
			double v = ss / (double)perChannel - m * m;
			if (v < 0.0) v = 0.0;
			mu = (float)m;
			var = (float)v;
			if (blockIdx.x == 0 && threadIdx.x == 0) {
				mean[c] = mu;
				variance[c] = var;
				runMean[c] = momentum * runMean[c] + (1.f - momentum) * mu;
				runVar[c] = momentum * runVar[c] + (1.f - momentum) * var;
			}
		} else {
			mu = statMean[c];
			var = statVar[c];
		}
		inv = 1.f / sqrtf(var + epsilon);
	}
	const size_t base = (size_t)c * perChannel;
	if constexpr (POOL == 2) {
		const long groups = perChannel / 4;
		const long per = (groups + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < groups) ? lo + per : groups;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			float4 a = *reinterpret_cast<const float4 *>(x + base + 4 * i);
			if (zhat) {
				a.x = (a.x - mu) * inv, a.y = (a.y - mu) * inv, a.z = (a.z - mu) * inv, a.w = (a.w - mu) * inv;
				*reinterpret_cast<float4 *>(zhat + base + 4 * i) = a;
			}
			*reinterpret_cast<float4 *>(actOut + base + 4 * i) = act_forward4(actFun, a);
		}
	} else {
		const int outB2 = inB / 4, outA = inA / 2, outB = inB / 2;
		const int perMap = outA * outB2;
		const long patches = (long)samples * perMap;
		const long per = (patches + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < patches) ? lo + per : patches;
		const size_t pBase = (size_t)c * samples * outA * outB;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB2, pb = rem - oa * outB2;
			const size_t in = base + (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
			float4 a0 = *reinterpret_cast<const float4 *>(x + in);
			float4 a1 = *reinterpret_cast<const float4 *>(x + in + inB);
			if (zhat) {
				a0.x = (a0.x - mu) * inv, a0.y = (a0.y - mu) * inv, a0.z = (a0.z - mu) * inv, a0.w = (a0.w - mu) * inv;
				a1.x = (a1.x - mu) * inv, a1.y = (a1.y - mu) * inv, a1.z = (a1.z - mu) * inv, a1.w = (a1.w - mu) * inv;
				*reinterpret_cast<float4 *>(zhat + in) = a0;
				*reinterpret_cast<float4 *>(zhat + in + inB) = a1;
			}
			const float4 r0 = act_forward4(actFun, a0), r1 = act_forward4(actFun, a1);
			*reinterpret_cast<float4 *>(actOut + in) = r0;
			*reinterpret_cast<float4 *>(actOut + in + inB) = r1;
			*reinterpret_cast<float2 *>(poolOut + pBase + (size_t)map * outA * outB + (size_t)oa * outB + 2 * pb) =
			    make_float2(max2x2(r0.x, r0.y, r1.x, r1.y), max2x2(r0.z, r0.w, r1.z, r1.w));
		}
	}
}

// dx_i = (m*delta_i - sum(delta) - zhat_i * sum(delta*zhat)) / (m * sqrt(var + eps)), and its channel sum
// (the bias gradient) in closed form: -sum(delta*zhat) * sum(zhat) / (m * sqrt(var + eps)).
__device__ __forceinline__ float bn_backward_value(float m, float d, float z, float sum1, float sum2, float scale)
{
	return (m * d - sum1 - sum2 * z) * scale;
}

// batch-norm backward, elementwise part, from the per-segment sums of channel_partial_kernel<3>
template <bool VEC>
__global__ void __launch_bounds__(kRedBlock)
bn_backward_apply_kernel(const float *delta, const float *zhat, const float *variance, const double *partial,
                         int segmentsIn, float epsilon, long perChannel, float *out, float *biasGrad)
{
	FITRE_RAISE_WAVE_PRIORITY();
	__shared__ double lds[3 * kRedBlock / kWave];
	const int c = blockIdx.y;
	const float *pd = delta + (size_t)c * perChannel;
	const float *pz = zhat + (size_t)c * perChannel;
	float *po = out + (size_t)c * perChannel;
	long lo, hi;
	segment_range(perChannel, lo, hi);
	// the first group's loads are in flight while the segment sums are combined
	long i = lo + 4 * (long)threadIdx.x;
	float4 d = make_float4(0.f, 0.f, 0.f, 0.f), z = d;
	if constexpr (VEC) {
		if (i + 3 < hi) {
			d = *reinterpret_cast<const float4 *>(pd + i);
			z = *reinterpret_cast<const float4 *>(pz + i);
		}
	}
	double a1 = 0.0, a2 = 0.0, a3 = 0.0;
	for (int k = threadIdx.x; k < segmentsIn; k += kRedBlock) {
		const double *slot = partial + ((size_t)c * segmentsIn + k) * 4;
		a1 += slot[0], a2 += slot[1], a3 += slot[2];
	}
	block_sum3<kRedBlock>(a1, a2, a3, lds);
	const double d1 = a1, d2 = a2, d3 = a3;
	const float m = (float)perChannel;
	const float sum1 = (float)d1, sum2 = (float)d2;
	const float scale = 1.f / (m * sqrtf(epsilon + variance[c]));
	if (biasGrad && blockIdx.x == 0 && threadIdx.x == 0) biasGrad[c] = (float)(-d2 * d3 * (double)scale);
	if constexpr (VEC) {
		while (i + 3 < hi) {
			const long next = i + 4 * kRedBlock;
			float4 dn = d, zn = z;
			if (next + 3 < hi) {
				dn = *reinterpret_cast<const float4 *>(pd + next);
				zn = *reinterpret_cast<const float4 *>(pz + next);
			}
			float4 r;
			r.x = bn_backward_value(m, d.x, z.x, sum1, sum2, scale);
			r.y = bn_backward_value(m, d.y, z.y, sum1, sum2, scale);
			r.z = bn_backward_value(m, d.z, z.z, sum1, sum2, scale);
			r.w = bn_backward_value(m, d.w, z.w, sum1, sum2, scale);
			*reinterpret_cast<float4 *>(po + i) = r;
			d = dn, z = zn, i = next;
		}
		long tail = lo + ((hi - lo) / 4) * 4;
		for (long t = tail + threadIdx.x; t < hi; t += kRedBlock) po[t] = bn_backward_value(m, pd[t], pz[t], sum1, sum2, scale);
	} else {
		for (long t = lo + threadIdx.x; t < hi; t += kRedBlock) po[t] = bn_backward_value(m, pd[t], pz[t], sum1, sum2, scale);
	}
}

// The same for short channels: one workgroup per channel sums, then applies (the second read of
// delta and zhat comes from the cache), one launch instead of two.
constexpr long kBnSmallChannel = 4096;
template <bool VEC>
__global__ void __launch_bounds__(kRedBlock)
bn_backward_small_kernel(const float *delta, const float *zhat, const float *variance, float epsilon, long perChannel,
                         float *out, float *biasGrad)
{
	FITRE_RAISE_WAVE_PRIORITY();
	__shared__ double lds[kRedBlock / kWave];
	const int c = blockIdx.x;
	const float *pd = delta + (size_t)c * perChannel;
	const float *pz = zhat + (size_t)c * perChannel;
	float *po = out + (size_t)c * perChannel;
	double s1 = 0.0, s2 = 0.0, s3 = 0.0;
	if constexpr (VEC) {
		for (long i = 4 * (long)threadIdx.x; i < perChannel; i += 4 * kRedBlock) {
			float4 d = *reinterpret_cast<const float4 *>(pd + i);
			float4 z = *reinterpret_cast<const float4 *>(pz + i);
			s1 += (double)((d.x + d.y) + (d.z + d.w));
			s2 += (double)(d.x * z.x) + (double)(d.y * z.y) + (double)(d.z * z.z) + (double)(d.w * z.w);
			s3 += (double)((z.x + z.y) + (z.z + z.w));
		}
	} else {
		for (long i = threadIdx.x; i < perChannel; i += kRedBlock) {
			float d = pd[i], z = pz[i];
			s1 += (double)d, s2 += (double)(d * z), s3 += (double)z;
		}
	}
	const double d1 = block_sum<kRedBlock>(s1, lds);
	const double d2 = block_sum<kRedBlock>(s2, lds);
	const double d3 = block_sum<kRedBlock>(s3, lds);
	const float m = (float)perChannel;
	const float sum1 = (float)d1, sum2 = (float)d2;
	const float scale = 1.f / (m * sqrtf(epsilon + variance[c]));
	if (biasGrad && threadIdx.x == 0) biasGrad[c] = (float)(-d2 * d3 * (double)scale);
	if constexpr (VEC) {
		for (long i = 4 * (long)threadIdx.x; i < perChannel; i += 4 * kRedBlock) {
			float4 d = *reinterpret_cast<const float4 *>(pd + i);
			float4 z = *reinterpret_cast<const float4 *>(pz + i);
			float4 r;
			r.x = bn_backward_value(m, d.x, z.x, sum1, sum2, scale);
			r.y = bn_backward_value(m, d.y, z.y, sum1, sum2, scale);
			r.z = bn_backward_value(m, d.z, z.z, sum1, sum2, scale);
			r.w = bn_backward_value(m, d.w, z.w, sum1, sum2, scale);
			*reinterpret_cast<float4 *>(po + i) = r;
		}
	} else {
		for (long i = threadIdx.x; i < perChannel; i += kRedBlock) po[i] = bn_backward_value(m, pd[i], pz[i], sum1, sum2, scale);
	}
}

// ---------------------------------------------------------------------
// pool + activation + batch-norm backward in two launches (one for short channels)
// ---------------------------------------------------------------------
// The batch-norm backward sums are sums over the gradient this pass writes, so it leaves them behind
// and the batch-norm step is the elementwise pass alone: 12 bytes per element instead of 20.

// the four cells of a 16-byte group: gradient after the activation, and the sums' terms
__device__ __forceinline__ float4 act_backward4(int actFun, float4 g, float4 zi, float4 zo)
{
	g.x *= act_derivative(actFun, zi.x, zo.x);
	g.y *= act_derivative(actFun, zi.y, zo.y);
	g.z *= act_derivative(actFun, zi.z, zo.z);
	g.w *= act_derivative(actFun, zi.w, zo.w);
	return g;
}
__device__ __forceinline__ float4 relu4(float4 v)
{
	return make_float4(v.x > 0.f ? v.x : 0.f, v.y > 0.f ? v.y : 0.f, v.z > 0.f ? v.z : 0.f, v.w > 0.f ? v.w : 0.f);
}
__device__ __forceinline__ void bn_sums4(float4 g, float4 z, double &s1, double &s2, double &s3)
{
	// four terms in float, the running sums in double
	s1 += (double)((g.x + g.y) + (g.z + g.w));
	s2 += (double)((g.x * z.x + g.y * z.y) + (g.z * z.z + g.w * z.w));
	s3 += (double)((z.x + z.y) + (z.z + z.w));
}
// routes the two pooled gradients d of a 2 x 4 patch (rows r0, r1 of the pool input) to the window maxima
__device__ __forceinline__ void route2x4(float4 r0, float4 r1, float2 d, float4 &g0, float4 &g1)
{
	g0 = make_float4(0.f, 0.f, 0.f, 0.f);
	g1 = g0;
	int arg = scan2x2(r0.x, r0.y, r1.x, r1.y);
	if (arg == 0) g0.x = d.x;
	else if (arg == 1) g0.y = d.x;
	else if (arg == 2) g1.x = d.x;
	else if (arg == 3) g1.y = d.x;
	arg = scan2x2(r0.z, r0.w, r1.z, r1.w);
	if (arg == 0) g0.z = d.y;
	else if (arg == 1) g0.w = d.y;
	else if (arg == 2) g1.z = d.y;
	else if (arg == 3) g1.w = d.y;
}

// B == 2: a window is the 16-byte group (a, 0), (a, 1), (a + 1, 0), (a + 1, 1)
__device__ __forceinline__ float4 route2x2(float4 r, float d)
{
	float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
	const int arg = scan2x2(r.x, r.y, r.z, r.w);
	if (arg == 0) g.x = d;
	else if (arg == 1) g.y = d;
	else if (arg == 2) g.z = d;
	else if (arg == 3) g.w = d;
	return g;
}

// delta given as `splits` slabs `stride` floats apart: their sum in slab order, accumulated in double
// (what the split-K reduction kernel would have written)
// (four slabs are read before the first of them is added: a loop that adds each slab as it arrives pays one memory
// latency per slab)
template <class T>
__device__ __forceinline__ void add_in_double(double (&a)[sizeof(T) / sizeof(float)], const T &t)
{
	const float *f = reinterpret_cast<const float *>(&t);
#pragma unroll
	for (int v = 0; v < (int)(sizeof(T) / sizeof(float)); v++) a[v] += (double)f[v];
}
template <class T>
__device__ __forceinline__ T load_sum_groups(const float *p, int splits, long stride)
{
	constexpr int V = sizeof(T) / sizeof(float);
	if (splits == 1) return *reinterpret_cast<const T *>(p);
	double a[V];
#pragma unroll
	for (int v = 0; v < V; v++) a[v] = 0.0;
	int s = 0;
	for (; s + 4 <= splits; s += 4) {
		T t[4];
#pragma unroll
		for (int u = 0; u < 4; u++) t[u] = *reinterpret_cast<const T *>(p + (size_t)(s + u) * stride);
#pragma unroll
		for (int u = 0; u < 4; u++) add_in_double<T>(a, t[u]);
	}
	if (s + 2 <= splits) {
		T t[2];
#pragma unroll
		for (int u = 0; u < 2; u++) t[u] = *reinterpret_cast<const T *>(p + (size_t)(s + u) * stride);
#pragma unroll
		for (int u = 0; u < 2; u++) add_in_double<T>(a, t[u]);
		s += 2;
	}
	if (s < splits) add_in_double<T>(a, *reinterpret_cast<const T *>(p + (size_t)s * stride));
	T r;
	float *f = reinterpret_cast<float *>(&r);
#pragma unroll
	for (int v = 0; v < V; v++) f[v] = (float)a[v];
	return r;
}
__device__ __forceinline__ float4 load_sum4(const float *p, int splits, long stride) { return load_sum_groups<float4>(p, splits, stride); }
__device__ __forceinline__ float2 load_sum2(const float *p, int splits, long stride) { return load_sum_groups<float2>(p, splits, stride); }
__device__ __forceinline__ float load_sum1(const float *p, int splits, long stride) { return load_sum_groups<float>(p, splits, stride); }
// slab 0 += the other slabs (same order and precision)
__global__ void __launch_bounds__(256) sum_slabs_kernel(float *base, int splits, long stride, long n)
{
	const long step = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) base[i] = load_sum1(base + i, splits, stride);
}

// One (channel, segment) per workgroup.  POOL 0: 2x2 / stride 2 max pool (B % 4 == 0, A even), the
// unit of work is a 2 x 4 patch; POOL 1: the same for any even B, the unit is one 2 x 2 window moved as two 8-byte
// rows; POOL 2: no pooling, the unit is a 16-byte group; POOL 3: 2x2 / stride 2
// max pool of maps with B == 2, where pooled cell q of a channel is its 16-byte group q.  z_act == nullptr:
// the activation is ReLU and its output is max(zhat, 0).  partial: slots of four doubles
// (sum g, sum g*zhat, sum zhat) per (channel, segment).
template <int POOL>
__global__ void __launch_bounds__(kRedBlock)
pool_act_sums_kernel(const float *delta, int dSplits, long dStride, const float *zhat, const float *z_act, int inA, int inB,
                     int samples, int actFun, float *dxPool, bool streamPool, float *dxAct, double *partial)
{
	FITRE_RAISE_WAVE_PRIORITY();
	__shared__ double lds[3 * kRedBlock / kWave];
	const int c = blockIdx.y;
	const long perChannel = (long)samples * inA * inB;
	const size_t base = (size_t)c * perChannel;
	double s1 = 0.0, s2 = 0.0, s3 = 0.0;
	if constexpr (POOL == 2 || POOL == 3) {
		long lo, hi;
		segment_range(perChannel, lo, hi);
		for (long i = lo + 4 * (long)threadIdx.x; i + 3 < hi; i += 4 * kRedBlock) {
			const float4 zi = *reinterpret_cast<const float4 *>(zhat + base + i);
			const float4 zo = z_act ? *reinterpret_cast<const float4 *>(z_act + base + i) : relu4(zi);
			float4 g;
			if constexpr (POOL == 2) g = load_sum4(delta + base + i, dSplits, dStride);
			else g = route2x2(zo, load_sum1(delta + (base + i) / 4, dSplits, dStride));
			if (dxPool) store4(dxPool + base + i, g, streamPool);
			g = act_backward4(actFun, g, zi, zo);
			*reinterpret_cast<float4 *>(dxAct + base + i) = g;
			bn_sums4(g, zi, s1, s2, s3);
		}
	} else if constexpr (POOL == 1) {
		const int outB = inB / 2, outA = inA / 2;
		const int perMap = outA * outB;
		const long patches = (long)samples * perMap;
		const long per = (patches + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < patches) ? lo + per : patches;
		const size_t dBase = (size_t)c * samples * perMap;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB, pb = rem - oa * outB;
			const size_t inOff = base + (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 2 * pb;
			const float2 a0 = *reinterpret_cast<const float2 *>(zhat + inOff);
			const float2 a1 = *reinterpret_cast<const float2 *>(zhat + inOff + inB);
			const float4 zi = make_float4(a0.x, a0.y, a1.x, a1.y);
			float4 zo;
			if (z_act) {
				const float2 q0 = *reinterpret_cast<const float2 *>(z_act + inOff);
				const float2 q1 = *reinterpret_cast<const float2 *>(z_act + inOff + inB);
				zo = make_float4(q0.x, q0.y, q1.x, q1.y);
			} else {
				zo = relu4(zi);
			}
			float4 g = route2x2(zo, load_sum1(delta + dBase + i, dSplits, dStride));
			if (dxPool) {
				*reinterpret_cast<float2 *>(dxPool + inOff) = make_float2(g.x, g.y);
				*reinterpret_cast<float2 *>(dxPool + inOff + inB) = make_float2(g.z, g.w);
			}
			g = act_backward4(actFun, g, zi, zo);
			*reinterpret_cast<float2 *>(dxAct + inOff) = make_float2(g.x, g.y);
			*reinterpret_cast<float2 *>(dxAct + inOff + inB) = make_float2(g.z, g.w);
			bn_sums4(g, zi, s1, s2, s3);
		}
	} else {
		const int outB2 = inB / 4, outA = inA / 2;
		const int perMap = outA * outB2;
		const long patches = (long)samples * perMap;
		const long per = (patches + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < patches) ? lo + per : patches;
		const size_t dBase = (size_t)c * samples * outA * (inB / 2);
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB2, pb = rem - oa * outB2;
			const size_t inOff = base + (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
			const size_t dOff = dBase + (size_t)map * outA * (inB / 2) + (size_t)oa * (inB / 2) + 2 * pb;
			const float4 i0 = *reinterpret_cast<const float4 *>(zhat + inOff);
			const float4 i1 = *reinterpret_cast<const float4 *>(zhat + inOff + inB);
			const float4 r0 = z_act ? *reinterpret_cast<const float4 *>(z_act + inOff) : relu4(i0);
			const float4 r1 = z_act ? *reinterpret_cast<const float4 *>(z_act + inOff + inB) : relu4(i1);
			const float2 d = load_sum2(delta + dOff, dSplits, dStride);
			float4 g0, g1;
			route2x4(r0, r1, d, g0, g1);
			if (dxPool) {
				store4(dxPool + inOff, g0, streamPool);
				store4(dxPool + inOff + inB, g1, streamPool);
			}
			g0 = act_backward4(actFun, g0, i0, r0);
			g1 = act_backward4(actFun, g1, i1, r1);
			*reinterpret_cast<float4 *>(dxAct + inOff) = g0;
			*reinterpret_cast<float4 *>(dxAct + inOff + inB) = g1;
			bn_sums4(g0, i0, s1, s2, s3);
			bn_sums4(g1, i1, s1, s2, s3);
		}
	}
	block_sum3<kRedBlock>(s1, s2, s3, lds);
	if (threadIdx.x == 0) {
		double *slot = partial + ((size_t)c * gridDim.x + blockIdx.x) * 4;
		slot[0] = s1, slot[1] = s2, slot[2] = s3;
	}
}

// Short channels (at most kBnSmallChannel cells): one workgroup per channel keeps the gradient and zhat
// in registers between the sums and the batch-norm formula; one launch for the three steps.
template <int POOL>
__global__ void __launch_bounds__(kRedBlock)
pool_act_bn_small_kernel(const float *delta, int dSplits, long dStride, const float *zhat, const float *z_act,
                         const float *variance, int inA, int inB, int samples, int actFun, float epsilon, float *dxPool,
                         float *dxAct, float *dxBn, float *biasGrad)
{
	FITRE_RAISE_WAVE_PRIORITY();
	__shared__ double lds[3 * kRedBlock / kWave];
	constexpr int G = (int)(kBnSmallChannel / (4 * kRedBlock)); // 16-byte groups per thread
	static_assert(G >= 2 && G % 2 == 0, "a 2 x 4 patch is two groups");
	const int c = blockIdx.x;
	const long perChannel = (long)samples * inA * inB;
	const size_t base = (size_t)c * perChannel;
	float4 g[G], z[G];
	long off[G]; // offset of the group inside the channel, -1: none
	double s1 = 0.0, s2 = 0.0, s3 = 0.0;
	if constexpr (POOL == 2 || POOL == 3) {
#pragma unroll
		for (int k = 0; k < G; k++) {
			const long i = 4 * ((long)threadIdx.x + (long)k * kRedBlock);
			off[k] = (i + 3 < perChannel) ? i : -1;
			if (off[k] < 0) continue;
			z[k] = *reinterpret_cast<const float4 *>(zhat + base + i);
			const float4 zo = z_act ? *reinterpret_cast<const float4 *>(z_act + base + i) : relu4(z[k]);
			if constexpr (POOL == 2) g[k] = load_sum4(delta + base + i, dSplits, dStride);
			else g[k] = route2x2(zo, load_sum1(delta + (base + i) / 4, dSplits, dStride));
			if (dxPool) *reinterpret_cast<float4 *>(dxPool + base + i) = g[k];
			g[k] = act_backward4(actFun, g[k], z[k], zo);
			*reinterpret_cast<float4 *>(dxAct + base + i) = g[k];
			bn_sums4(g[k], z[k], s1, s2, s3);
		}
	} else {
		const int outB2 = inB / 4, outA = inA / 2;
		const int perMap = outA * outB2;
		const long patches = (long)samples * perMap;
		const size_t dBase = (size_t)c * samples * outA * (inB / 2);
#pragma unroll
		for (int k = 0; k < G / 2; k++) {
			const long i = (long)threadIdx.x + (long)k * kRedBlock;
			off[2 * k] = off[2 * k + 1] = -1;
			if (i >= patches) continue;
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB2, pb = rem - oa * outB2;
			const long in = map * inA * inB + (long)(2 * oa) * inB + 4 * pb;
			const size_t dOff = dBase + (size_t)map * outA * (inB / 2) + (size_t)oa * (inB / 2) + 2 * pb;
			off[2 * k] = in;
			off[2 * k + 1] = in + inB;
			z[2 * k] = *reinterpret_cast<const float4 *>(zhat + base + in);
			z[2 * k + 1] = *reinterpret_cast<const float4 *>(zhat + base + in + inB);
			const float4 r0 = z_act ? *reinterpret_cast<const float4 *>(z_act + base + in) : relu4(z[2 * k]);
			const float4 r1 = z_act ? *reinterpret_cast<const float4 *>(z_act + base + in + inB) : relu4(z[2 * k + 1]);
			const float2 d = load_sum2(delta + dOff, dSplits, dStride);
			route2x4(r0, r1, d, g[2 * k], g[2 * k + 1]);
			if (dxPool) {
				*reinterpret_cast<float4 *>(dxPool + base + in) = g[2 * k];
				*reinterpret_cast<float4 *>(dxPool + base + in + inB) = g[2 * k + 1];
			}
			g[2 * k] = act_backward4(actFun, g[2 * k], z[2 * k], r0);
			g[2 * k + 1] = act_backward4(actFun, g[2 * k + 1], z[2 * k + 1], r1);
			*reinterpret_cast<float4 *>(dxAct + base + in) = g[2 * k];
			*reinterpret_cast<float4 *>(dxAct + base + in + inB) = g[2 * k + 1];
			bn_sums4(g[2 * k], z[2 * k], s1, s2, s3);
			bn_sums4(g[2 * k + 1], z[2 * k + 1], s1, s2, s3);
		}
	}
	block_sum3<kRedBlock>(s1, s2, s3, lds);
	const double d1 = s1, d2 = s2, d3 = s3;
	const float m = (float)perChannel;
	const float sum1 = (float)d1, sum2 = (float)d2;
	const float scale = 1.f / (m * sqrtf(epsilon + variance[c]));
	if (biasGrad && threadIdx.x == 0) biasGrad[c] = (float)(-d2 * d3 * (double)scale);
#pragma unroll
	for (int k = 0; k < G; k++) {
		if (off[k] < 0) continue;
		float4 r;
		r.x = bn_backward_value(m, g[k].x, z[k].x, sum1, sum2, scale);
		r.y = bn_backward_value(m, g[k].y, z[k].y, sum1, sum2, scale);
		r.z = bn_backward_value(m, g[k].z, z[k].z, sum1, sum2, scale);
		r.w = bn_backward_value(m, g[k].w, z[k].w, sum1, sum2, scale);
		*reinterpret_cast<float4 *>(dxBn + base + off[k]) = r;
	}
}

// The directional derivative of a layer's batch norm, activation and 2x2 / stride 2 max pooling in one pass (the R
// operator's forward sweep): R{bn out} is the batch-norm backward formula applied to R{x} (sums of channel_partial_kernel<3>
// over (R{x}, zhat)), R{act out} = R{bn out} * f'(.), and the pooled value is the one at the arg-max of the activation
// output.  z_act null (ReLU only): the activation output is max(zhat, 0), bit for bit what the forward pass stored.
// POOL 0: units of 2 x 4 patches; POOL 2: no pooling, 16-byte groups.
template <int POOL>
__global__ void __launch_bounds__(kRedBlock)
bn_act_pool_rop_forward_kernel(const float *rx, const float *zhat, const float *z_act, const float *variance, const double *partial,
                               int segmentsIn, float epsilon, int samples, int inA, int inB, int actFun, float *rbn, float *ract,
                               float *rpool)
{
	__shared__ double lds[3 * kRedBlock / kWave];
	const int c = blockIdx.y;
	const long perChannel = (long)samples * inA * inB;
	double a1 = 0.0, a2 = 0.0, a3 = 0.0;
	for (int k = threadIdx.x; k < segmentsIn; k += kRedBlock) {
		const double *slot = partial + ((size_t)c * segmentsIn + k) * 4;
		a1 += slot[0], a2 += slot[1], a3 += slot[2];
	}
	block_sum3<kRedBlock>(a1, a2, a3, lds);
	const float m = (float)perChannel;
	const float sum1 = (float)a1, sum2 = (float)a2;
	const float scale = 1.f / (m * sqrtf(epsilon + variance[c]));
	const size_t base = (size_t)c * perChannel;
	auto step = [&](size_t at, float4 &zo) { // R{bn out} and R{act out} of one group; zo: its activation output
		const float4 d = *reinterpret_cast<const float4 *>(rx + at), z = *reinterpret_cast<const float4 *>(zhat + at);
		zo = z_act ? *reinterpret_cast<const float4 *>(z_act + at) : relu4(z);
		float4 r;
		r.x = bn_backward_value(m, d.x, z.x, sum1, sum2, scale);
		r.y = bn_backward_value(m, d.y, z.y, sum1, sum2, scale);
		r.z = bn_backward_value(m, d.z, z.z, sum1, sum2, scale);
		r.w = bn_backward_value(m, d.w, z.w, sum1, sum2, scale);
		*reinterpret_cast<float4 *>(rbn + at) = r;
		// a zero derivative gives +0 whatever the sign of R{bn out}, as the activation's own backward kernel does for ReLU
		const float fx = act_derivative(actFun, z.x, zo.x), fy = act_derivative(actFun, z.y, zo.y);
		const float fz = act_derivative(actFun, z.z, zo.z), fw = act_derivative(actFun, z.w, zo.w);
		r.x = fx == 0.f ? 0.f : r.x * fx, r.y = fy == 0.f ? 0.f : r.y * fy;
		r.z = fz == 0.f ? 0.f : r.z * fz, r.w = fw == 0.f ? 0.f : r.w * fw;
		*reinterpret_cast<float4 *>(ract + at) = r;
		return r;
	};
	if constexpr (POOL == 2) {
		const long groups = perChannel / 4;
		const long per = (groups + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < groups) ? lo + per : groups;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			float4 zo;
			step(base + 4 * i, zo);
		}
	} else {
		const int outB2 = inB / 4, outA = inA / 2, outB = inB / 2;
		const int perMap = outA * outB2;
		const long patches = (long)samples * perMap;
		const long per = (patches + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < patches) ? lo + per : patches;
		const size_t pBase = (size_t)c * samples * outA * outB;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB2, pb = rem - oa * outB2;
			const size_t in = base + (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
			float4 z0, z1;
			const float4 r0 = step(in, z0), r1 = step(in + inB, z1);
			const int a = scan2x2(z0.x, z0.y, z1.x, z1.y), b = scan2x2(z0.z, z0.w, z1.z, z1.w);
			float2 r;
			r.x = a == 0 ? r0.x : (a == 1 ? r0.y : (a == 2 ? r1.x : (a == 3 ? r1.y : 0.f)));
			r.y = b == 0 ? r0.z : (b == 1 ? r0.w : (b == 2 ? r1.z : (b == 3 ? r1.w : 0.f)));
			*reinterpret_cast<float2 *>(rpool + pBase + (size_t)map * outA * outB + (size_t)oa * outB + 2 * pb) = r;
		}
	}
}

// Directional derivative of the batch-norm backward formula.  Per channel, with s = sqrt(var + eps)
// and <.> the mean over the channel:
//   out = ( rdx - <rdx> - rzhat <dx zhat> - zhat ( <rdx zhat> + <dx rzhat> ) ) / s  -  dc <zhat rx> / s
// Pass 1: five sums per (channel, segment), slots of eight doubles.
template <bool VEC>
__global__ void __launch_bounds__(kRedBlock)
bn_rop_partial_kernel(const float *rdx, const float *dx, const float *zhat, const float *rzhat, const float *rx, long perChannel,
                      double *partial)
{
	__shared__ double lds[kRedBlock / kWave];
	const size_t base = (size_t)blockIdx.y * perChannel;
	long lo, hi;
	segment_range(perChannel, lo, hi);
	double s[5] = { 0.0, 0.0, 0.0, 0.0, 0.0 };
	if constexpr (VEC) { // 16-byte groups (perChannel % 4 == 0, aligned tensors: segments are whole groups)
		for (long i = lo + 4 * (long)threadIdx.x; i + 3 < hi; i += 4 * kRedBlock) {
			const float4 a = *reinterpret_cast<const float4 *>(rdx + base + i), d = *reinterpret_cast<const float4 *>(dx + base + i);
			const float4 z = *reinterpret_cast<const float4 *>(zhat + base + i), rz = *reinterpret_cast<const float4 *>(rzhat + base + i);
			const float4 x = *reinterpret_cast<const float4 *>(rx + base + i);
			s[0] += (double)((a.x + a.y) + (a.z + a.w));
			s[1] += (double)(d.x * z.x) + (double)(d.y * z.y) + (double)(d.z * z.z) + (double)(d.w * z.w);
			s[2] += (double)(a.x * z.x) + (double)(a.y * z.y) + (double)(a.z * z.z) + (double)(a.w * z.w);
			s[3] += (double)(d.x * rz.x) + (double)(d.y * rz.y) + (double)(d.z * rz.z) + (double)(d.w * rz.w);
			s[4] += (double)(z.x * x.x) + (double)(z.y * x.y) + (double)(z.z * x.z) + (double)(z.w * x.w);
		}
	} else {
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const float a = rdx[base + i], d = dx[base + i], z = zhat[base + i], rz = rzhat[base + i], x = rx[base + i];
			s[0] += (double)a;
			s[1] += (double)(d * z);
			s[2] += (double)(a * z);
			s[3] += (double)(d * rz);
			s[4] += (double)(z * x);
		}
	}
	double t[5];
#pragma unroll
	for (int k = 0; k < 5; k++) t[k] = block_sum<kRedBlock>(s[k], lds);
	if (threadIdx.x == 0) {
		double *slot = partial + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8;
#pragma unroll
		for (int k = 0; k < 5; k++) slot[k] = t[k];
	}
}
template <bool VEC>
__global__ void __launch_bounds__(kRedBlock)
bn_rop_apply_kernel(const float *rdx, const float *zhat, const float *rzhat, const float *dc, const float *variance,
                    const double *partial, int segments, float epsilon, long perChannel, float *out)
{
	const int c = blockIdx.y;
	double t[5] = { 0.0, 0.0, 0.0, 0.0, 0.0 };
	for (int k = 0; k < segments; k++) {
		const double *slot = partial + ((size_t)c * segments + k) * 8;
#pragma unroll
		for (int j = 0; j < 5; j++) t[j] += slot[j];
	}
	const double m = (double)perChannel;
	const float inv = 1.f / sqrtf(variance[c] + epsilon);
	const float a = (float)(t[0] / m), b = (float)(t[1] / m), cd = (float)((t[2] + t[3]) / m), e = (float)(t[4] / m);
	const size_t base = (size_t)c * perChannel;
	long lo, hi;
	segment_range(perChannel, lo, hi);
	if constexpr (VEC) {
		for (long i = lo + 4 * (long)threadIdx.x; i + 3 < hi; i += 4 * kRedBlock) {
			const float4 r = *reinterpret_cast<const float4 *>(rdx + base + i), rz = *reinterpret_cast<const float4 *>(rzhat + base + i);
			const float4 z = *reinterpret_cast<const float4 *>(zhat + base + i), d = *reinterpret_cast<const float4 *>(dc + base + i);
			float4 o;
			o.x = (r.x - a - rz.x * b - z.x * cd) * inv - d.x * e * inv;
			o.y = (r.y - a - rz.y * b - z.y * cd) * inv - d.y * e * inv;
			o.z = (r.z - a - rz.z * b - z.z * cd) * inv - d.z * e * inv;
			o.w = (r.w - a - rz.w * b - z.w * cd) * inv - d.w * e * inv;
			*reinterpret_cast<float4 *>(out + base + i) = o;
		}
	} else {
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock)
			out[base + i] = (rdx[base + i] - a - rzhat[base + i] * b - zhat[base + i] * cd) * inv - dc[base + i] * e * inv;
	}
}

// The backward sweep's first three R-steps of a layer with batch norm in one pass: the pooled R{delta} is routed to the
// arg-max cells (2x2 / stride 2 windows, POOL 0; POOL 2: no pooling), R{delta f'(x)} = R{delta} f'(x) + delta f''(x) R{x}
// is written to rdOut, and the five sums of bn_rop_partial_kernel over (rdOut, dxAct, zhat, rzhat, rx) are left per
// (channel, segment) -- what bn_rop_apply_kernel needs.  SECOND false: f'' is zero (ReLU, linear) and `delta` is not
// read.  z_act null (ReLU only): the activation output is max(zhat, 0).  rzhat is R{x} of the activation: R{bn out}.
template <int POOL, bool SECOND>
__global__ void __launch_bounds__(kRedBlock)
pool_act_bn_rop_sums_kernel(const float *rdeltaPooled, const float *delta, const float *zhat, const float *z_act, const float *rzhat,
                            const float *dxAct, const float *rx, int inA, int inB, int samples, int actFun, float *rdOut, double *partial)
{
	__shared__ double lds[kRedBlock / kWave];
	const int c = blockIdx.y;
	const long perChannel = (long)samples * inA * inB;
	const size_t base = (size_t)c * perChannel;
	double s[5] = { 0.0, 0.0, 0.0, 0.0, 0.0 };
	auto step = [&](size_t at, float4 g, float4 z, float4 zo) { // g: R{delta} at the activation output of this group
		const float4 rz = *reinterpret_cast<const float4 *>(rzhat + at), da = *reinterpret_cast<const float4 *>(dxAct + at);
		const float4 x = *reinterpret_cast<const float4 *>(rx + at);
		float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
		if constexpr (SECOND) d = *reinterpret_cast<const float4 *>(delta + at);
		float4 r;
		float f1, f2;
		act_derivatives(actFun, z.x, zo.x, f1, f2);
		r.x = SECOND ? g.x * f1 + d.x * f2 * rz.x : g.x * f1;
		act_derivatives(actFun, z.y, zo.y, f1, f2);
		r.y = SECOND ? g.y * f1 + d.y * f2 * rz.y : g.y * f1;
		act_derivatives(actFun, z.z, zo.z, f1, f2);
		r.z = SECOND ? g.z * f1 + d.z * f2 * rz.z : g.z * f1;
		act_derivatives(actFun, z.w, zo.w, f1, f2);
		r.w = SECOND ? g.w * f1 + d.w * f2 * rz.w : g.w * f1;
		*reinterpret_cast<float4 *>(rdOut + at) = r;
		s[0] += (double)((r.x + r.y) + (r.z + r.w));
		s[1] += (double)(da.x * z.x) + (double)(da.y * z.y) + (double)(da.z * z.z) + (double)(da.w * z.w);
		s[2] += (double)(r.x * z.x) + (double)(r.y * z.y) + (double)(r.z * z.z) + (double)(r.w * z.w);
		s[3] += (double)(da.x * rz.x) + (double)(da.y * rz.y) + (double)(da.z * rz.z) + (double)(da.w * rz.w);
		s[4] += (double)(z.x * x.x) + (double)(z.y * x.y) + (double)(z.z * x.z) + (double)(z.w * x.w);
	};
	if constexpr (POOL == 2) {
		const long groups = perChannel / 4;
		const long per = (groups + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < groups) ? lo + per : groups;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const size_t at = base + 4 * i;
			const float4 z = *reinterpret_cast<const float4 *>(zhat + at);
			const float4 zo = z_act ? *reinterpret_cast<const float4 *>(z_act + at) : relu4(z);
			step(at, *reinterpret_cast<const float4 *>(rdeltaPooled + at), z, zo);
		}
	} else {
		const int outB2 = inB / 4, outA = inA / 2, outB = inB / 2;
		const int perMap = outA * outB2;
		const long patches = (long)samples * perMap;
		const long per = (patches + gridDim.x - 1) / gridDim.x;
		const long lo = (long)blockIdx.x * per;
		const long hi = (lo + per < patches) ? lo + per : patches;
		const size_t pBase = (size_t)c * samples * outA * outB;
		for (long i = lo + threadIdx.x; i < hi; i += kRedBlock) {
			const long map = i / perMap;
			const int rem = (int)(i - map * perMap);
			const int oa = rem / outB2, pb = rem - oa * outB2;
			const size_t in = base + (size_t)map * inA * inB + (size_t)(2 * oa) * inB + 4 * pb;
			const float4 z0 = *reinterpret_cast<const float4 *>(zhat + in), z1 = *reinterpret_cast<const float4 *>(zhat + in + inB);
			const float4 o0 = z_act ? *reinterpret_cast<const float4 *>(z_act + in) : relu4(z0);
			const float4 o1 = z_act ? *reinterpret_cast<const float4 *>(z_act + in + inB) : relu4(z1);
			const float2 d = *reinterpret_cast<const float2 *>(rdeltaPooled + pBase + (size_t)map * outA * outB + (size_t)oa * outB + 2 * pb);
			float4 g0, g1;
			route2x4(o0, o1, d, g0, g1);
			step(in, g0, z0, o0);
			step(in + inB, g1, z1, o1);
		}
	}
	double t[5];
#pragma unroll
	for (int k = 0; k < 5; k++) t[k] = block_sum<kRedBlock>(s[k], lds);
	if (threadIdx.x == 0) {
		double *slot = partial + ((size_t)c * gridDim.x + blockIdx.x) * 8;
#pragma unroll
		for (int k = 0; k < 5; k++) slot[k] = t[k];
	}
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// =====================================================================
// softmax cross entropy
// =====================================================================

// one wave per row; classes strided over the lanes
__global__ void __launch_bounds__(256)
softmax_ce_kernel(const float *logits, const float *target, int rows, int classes, float *probs, float *errors, float *nll)
{
	const int lane = threadIdx.x % kWave;
	const int row = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
	if (row >= rows) return;
	const float *in = logits + (size_t)row * classes;
	float mx = -FLT_MAX;
	for (int c = lane; c < classes; c += kWave) mx = fmaxf(mx, in[c]);
	mx = wave_max(mx);
	float s = 0.f;
	for (int c = lane; c < classes; c += kWave) s += expf(in[c] - mx);
	s = wave_sum(s);
	const float inv = 1.f / s;
	const int label = (int)target[row]; // 1-based
	const float invRows = 1.f / (float)rows;
	for (int c = lane; c < classes; c += kWave) {
		float p = expf(in[c] - mx) * inv + 1e-10f;
		probs[(size_t)row * classes + c] = p;
		if (errors) errors[(size_t)row * classes + c] = (((c + 1) == label) ? p - 1.f : p) * invRows;
		if ((c + 1) == label) nll[row] = -logf(p);
	}
	if (lane == 0 && (label < 1 || label > classes)) nll[row] = 0.f;
}

// classes[r] = 1-based index of the first class whose cumulative probability reaches uniforms[r];
// classes + 1 if rounding keeps the total below it
__global__ void __launch_bounds__(256) multinomial_classes_kernel(const float *probs, const float *uniforms, int samples, int classes,
                                                                   float *out)
{
	const int r = blockIdx.x * blockDim.x + threadIdx.x;
	if (r >= samples) return;
	const float u = uniforms[r];
	float c = 0.f;
	int pick = classes + 1;
	for (int i = 0; i < classes; i++) {
		c += probs[(size_t)r * classes + i];
		if (c >= u) {
			pick = i + 1;
			break;
		}
	}
	out[r] = (float)pick;
}

// hits[r] = 1 when the first class with the largest probability (> 0) is the 1-based target, else 0
__global__ void __launch_bounds__(256) accuracy_hits_kernel(const float *probs, const float *target, int rows, int classes, float *hits)
{
	const int r = blockIdx.x * blockDim.x + threadIdx.x;
	if (r >= rows) return;
	float best = 0.f;
	int arg = 0;
	for (int c = 0; c < classes; c++) {
		const float p = probs[(size_t)r * classes + c];
		if (best < p) {
			best = p;
			arg = c;
		}
	}
	hits[r] = ((float)(arg + 1) == target[r]) ? 1.f : 0.f;
}

// rError[r][i] = p_i (rz_i - sum_j p_j rz_j) * scale
__global__ void __launch_bounds__(256) cross_entropy_rop_error_kernel(const float *rz, const float *probs, int rows, int classes,
                                                                       float scale, float *rError)
{
	const int r = blockIdx.x * blockDim.x + threadIdx.x;
	if (r >= rows) return;
	const float *p = probs + (size_t)r * classes, *z = rz + (size_t)r * classes;
	float s = 0.f;
	for (int j = 0; j < classes; j++) s += p[j] * z[j];
	for (int i = 0; i < classes; i++) rError[(size_t)r * classes + i] = p[i] * (z[i] - s) * scale;
}

__global__ void cross_entropy_error_kernel(const float *probs, const float *target, int rows, int classes, float *errors)
{
	long total = (long)rows * classes;
	long stride = (long)gridDim.x * blockDim.x;
	const float invRows = 1.f / (float)rows;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		int r = (int)(i / classes), c = (int)(i - (long)r * classes);
		float p = probs[i];
		errors[i] = (((float)(c + 1) == target[r]) ? p - 1.f : p) * invRows;
	}
}

__global__ void __launch_bounds__(256) mean_kernel(const float *x, int n, float *out)
{
	__shared__ double lds[4];
	double acc = 0.0;
	for (int i = threadIdx.x; i < n; i += 256) acc += (double)x[i];
	double t = block_sum<256>(acc, lds);
	if (threadIdx.x == 0) out[0] = (float)(t / (double)n);
}

static float *g_nll = nullptr;
static int g_nll_rows = 0;
static float *g_loss_host = nullptr;

void layers_release()
{
	if (g_nll) (void)hipFree(g_nll);
	if (g_loss_host) (void)hipHostFree(g_loss_host);
	g_nll = nullptr, g_loss_host = nullptr, g_nll_rows = 0;
}

// =====================================================================
// layout changes
// =====================================================================

// [right][left][chunk] -> [left][right][chunk]
__global__ void reshape_kernel(const float *in, int right, int left, int chunk, float *out)
{
	long total = (long)right * left * chunk;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		long t = i % chunk;
		long q = i / chunk;
		long l = q % left, r = q / left;
		out[(l * right + r) * chunk + t] = in[i];
	}
}

// TO_FC: in [C][N][a*B+b] -> out [N][C][b*A+a];  otherwise the inverse.
template <bool TO_FC>
__global__ void boundary_permute_kernel(const float *in, int C, int N, int A, int B, float *out)
{
	long total = (long)C * N * A * B;
	long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		// i enumerates the output
		long inner = i % ((long)A * B);
		long outer = i / ((long)A * B);
		if constexpr (TO_FC) {
			long c = outer % C, n = outer / C;
			long a = inner % A, b = inner / A;
			out[i] = in[((c * N + n) * A + a) * B + b];
		} else {
			long n = outer % N, c = outer / N;
			long b = inner % B, a = inner / B;
			out[i] = in[((n * C + c) * B + b) * A + a];
		}
	}
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// The per-(channel, segment) sums of the batch-norm backward step live in a file-scope device
// array instead of a caller's workspace.  Every GPU holds its own copy of the array at its own
// address; the address is looked up once per device, with that device current, by
// layers_device_setup() (called from fitre_hip_init) and host code only ever uses that pointer.
static __device__ __align__(256) unsigned char scratch[FITRE_HIP_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices] = {};

int layers_device_setup(int device)
{
	if (device < 0 || device >= kMaxDevices)
		return fail(FITRE_E_ARGUMENT, "device index %d beyond the %d this layer keeps a scratch address for", device, kMaxDevices);
	if (g_scratch_ptr[device]) return FITRE_OK;
	void *ptr = nullptr;
	FITRE_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
	if (!ptr) return fail(FITRE_E_DEVICE, "hipGetSymbolAddress returned a null address for the static scratch array");
	g_scratch_ptr[device] = ptr;
	return FITRE_OK;
}

} // namespace fitre

using namespace fitre;

extern "C" {

int fitre_hip_pool_forward(int poolType, const float *in, int channels, int samples, int inA, int inB, int ksize,
                           int stride, int padding, int outA, int outB, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && out, "fitre_hip_pool_forward: null pointer");
	int rc = check_pool_shape("fitre_hip_pool_forward", channels, samples, inA, inB, ksize, stride, padding, outA, outB);
	if (rc) return rc;
	PoolGeom g = make_geom(inA, inB, ksize, stride, padding, outA, outB);
	long maps = (long)channels * samples;
	long total = maps * outA * outB;
	LaunchScope scope(FITRE_KC_POOL_FWD, 4.0 * (double)(maps * inA * inB + total));
	if (poolType == MAX_POOL)
		pool_forward_kernel<0><<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(in, g, maps, out, nullptr);
	else if (poolType == AVG_POOL)
		pool_forward_kernel<1><<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(in, g, maps, out, nullptr);
	else
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_pool_forward: unknown pool type %d", poolType);
	return check_launch("pool_forward_kernel");
}

int fitre_hip_max_pool_argmax(const float *z_in, int channels, int samples, int inA, int inB, int ksize, int stride,
                              int padding, int outA, int outB, int *index)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(z_in && index, "fitre_hip_max_pool_argmax: null pointer");
	int rc = check_pool_shape("fitre_hip_max_pool_argmax", channels, samples, inA, inB, ksize, stride, padding, outA, outB);
	if (rc) return rc;
	PoolGeom g = make_geom(inA, inB, ksize, stride, padding, outA, outB);
	long maps = (long)channels * samples;
	long total = maps * outA * outB;
	LaunchScope scope(FITRE_KC_POOL_FWD, 4.0 * (double)(maps * inA * inB + total));
	pool_forward_kernel<2><<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(z_in, g, maps, nullptr, index);
	return check_launch("pool_forward_kernel<argmax>");
}

int fitre_hip_pool_act_backward(int poolType, int actFun, const float *delta, const float *z_in, const float *z_act,
                                int channels, int samples, int inA, int inB, int ksize, int stride, int padding,
                                int outA, int outB, float *dxPool, float *dxAct)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && dxAct, "fitre_hip_pool_act_backward: null pointer");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_pool_act_backward: unknown activation code %d", actFun);
	FITRE_REQUIRE(!act_needs_zin(actFun) || z_in, "fitre_hip_pool_act_backward: activation %d needs z_in", actFun);
	FITRE_REQUIRE(!(act_needs_zout(actFun) || poolType == MAX_POOL) || z_act,
	              "fitre_hip_pool_act_backward: z_act is required");
	long maps = (long)channels * samples;
	long total = maps * inA * inB;
	if (poolType == NO_POOL) {
		FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0, "fitre_hip_pool_act_backward: non-positive shape");
		FITRE_REQUIRE((double)total < 2147483647.0, "fitre_hip_pool_act_backward: tensor exceeds 2^31 elements");
	} else {
		int rc = check_pool_shape("fitre_hip_pool_act_backward", channels, samples, inA, inB, ksize, stride, padding, outA, outB);
		if (rc) return rc;
	}
	PoolGeom g = make_geom(inA, inB, ksize > 0 ? ksize : 1, stride > 0 ? stride : 1, padding, outA > 0 ? outA : 1, outB > 0 ? outB : 1);
	double bytes = 4.0 * (double)total * (1 + (dxPool ? 1 : 0) + (act_needs_zin(actFun) ? 1 : 0) + 1) +
	               4.0 * (double)maps * (poolType == NO_POOL ? inA * inB : outA * outB);
	LaunchScope scope(FITRE_KC_POOL_ACT_BWD, bytes);
	unsigned blocks = blocks_for(total, 512, 16384);
	if (poolType == MAX_POOL) {
		bool fast = ksize == 2 && stride == 2 && padding == 0 && (inB % 4 == 0) && (inA % 2 == 0) && aligned16(z_act) &&
		            aligned16(dxAct) && (!dxPool || aligned16(dxPool)) && (!z_in || aligned16(z_in)) &&
		            (((uintptr_t)delta & 7) == 0);
		const bool perMap = !fast && inA * inB <= kPoolMapCells && outA * outB <= kPoolMapWindows && inA * inB >= 64 &&
		                    maps <= 0x7fffffffL;
		const bool grouped = perMap && ksize == 3 && stride == 2 && aligned16(z_act) && aligned16(dxAct) &&
		                     (!dxPool || aligned16(dxPool)) && (!z_in || aligned16(z_in));
		if (fast)
			maxpool2_backward_kernel<true><<<blocks_for(total / 8, 256, 16384), 256, 0, stream()>>>(
			    delta, act_needs_zin(actFun) ? z_in : nullptr, z_act, inA, inB, maps, actFun, dxPool, dxAct);
		else if (grouped) {
			const int per = maps_per_group(inA * inB, outA * outB, maps);
			const long groups = (maps + per - 1) / per;
			maxpool_maps_backward_kernel<true, 3, 2><<<(unsigned)groups, 256, maps_group_lds(inA * inB, outA * outB, per), stream()>>>(
			    delta, act_needs_zin(actFun) ? z_in : nullptr, z_act, g, per, maps, FastDiv((uint32_t)(inA * inB)),
			    FastDiv((uint32_t)(outA * outB)), actFun, dxPool, dxAct, 4.0 * (double)total >= 48.0 * 1024 * 1024);
		} else if (perMap)
			maxpool_map_backward_kernel<true><<<(unsigned)maps, 256, 0, stream()>>>(delta, act_needs_zin(actFun) ? z_in : nullptr, z_act, g,
			                                                                      actFun, dxPool, dxAct);
		else
			pool_backward_kernel<0, true><<<blocks, 256, 0, stream()>>>(delta, z_in, z_act, g, maps, actFun, dxPool, dxAct);
	} else if (poolType == AVG_POOL) {
		pool_backward_kernel<1, true><<<blocks, 256, 0, stream()>>>(delta, z_in, z_act, g, maps, actFun, dxPool, dxAct);
	} else if (poolType == NO_POOL) {
		if (total % 4 == 0 && aligned16(delta) && aligned16(dxAct) && (!dxPool || aligned16(dxPool)) && (!z_in || aligned16(z_in)) &&
		    (!z_act || aligned16(z_act)))
			nopool_act_backward_vec_kernel<<<blocks_for(total / 4, 256, 16384), 256, 0, stream()>>>(
			    reinterpret_cast<const float4 *>(delta), reinterpret_cast<const float4 *>(act_needs_zin(actFun) ? z_in : nullptr),
			    reinterpret_cast<const float4 *>(z_act), total / 4, actFun, reinterpret_cast<float4 *>(dxPool),
			    reinterpret_cast<float4 *>(dxAct));
		else
			pool_backward_kernel<2, true><<<blocks, 256, 0, stream()>>>(delta, z_in, z_act, g, maps, actFun, dxPool, dxAct);
	} else {
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_pool_act_backward: unknown pool type %d", poolType);
	}
	return check_launch("pool_act_backward");
}

int fitre_hip_pool_backward(int poolType, const float *delta, const float *z_in, int channels, int samples, int inA,
                            int inB, int ksize, int stride, int padding, int outA, int outB, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && out, "fitre_hip_pool_backward: null pointer");
	FITRE_REQUIRE(poolType != MAX_POOL || z_in, "fitre_hip_pool_backward: max pooling needs the pool input");
	int rc = check_pool_shape("fitre_hip_pool_backward", channels, samples, inA, inB, ksize, stride, padding, outA, outB);
	if (rc) return rc;
	PoolGeom g = make_geom(inA, inB, ksize, stride, padding, outA, outB);
	long maps = (long)channels * samples;
	long total = maps * inA * inB;
	LaunchScope scope(FITRE_KC_POOL_BWD, 4.0 * (double)(total * (poolType == MAX_POOL ? 2 : 1) + maps * outA * outB));
	unsigned blocks = blocks_for(total, 512, 16384);
	if (poolType == MAX_POOL) {
		bool fast = ksize == 2 && stride == 2 && padding == 0 && (inB % 4 == 0) && (inA % 2 == 0) && aligned16(z_in) &&
		            aligned16(out) && (((uintptr_t)delta & 7) == 0);
		const bool perMap = !fast && inA * inB <= kPoolMapCells && outA * outB <= kPoolMapWindows && inA * inB >= 64 &&
		                    maps <= 0x7fffffffL;
		if (fast)
			maxpool2_backward_kernel<false><<<blocks_for(total / 8, 256, 16384), 256, 0, stream()>>>(
			    delta, nullptr, z_in, inA, inB, maps, CNN_ACT_NONE, out, nullptr);
		else if (perMap && ksize == 3 && stride == 2 && aligned16(z_in) && aligned16(out)) {
			const int per = maps_per_group(inA * inB, outA * outB, maps);
			const long groups = (maps + per - 1) / per;
			maxpool_maps_backward_kernel<false, 3, 2><<<(unsigned)groups, 256, maps_group_lds(inA * inB, outA * outB, per), stream()>>>(
			    delta, nullptr, z_in, g, per, maps, FastDiv((uint32_t)(inA * inB)), FastDiv((uint32_t)(outA * outB)), CNN_ACT_NONE, out,
			    nullptr, false);
		} else if (perMap)
			maxpool_map_backward_kernel<false><<<(unsigned)maps, 256, 0, stream()>>>(delta, nullptr, z_in, g, CNN_ACT_NONE, out, nullptr);
		else
			pool_backward_kernel<0, false><<<blocks, 256, 0, stream()>>>(delta, nullptr, z_in, g, maps, CNN_ACT_NONE, out, nullptr);
	} else if (poolType == AVG_POOL) {
		pool_backward_kernel<1, false><<<blocks, 256, 0, stream()>>>(delta, nullptr, nullptr, g, maps, CNN_ACT_NONE, out, nullptr);
	} else {
		return fail(FITRE_E_UNSUPPORTED, "fitre_hip_pool_backward: unknown pool type %d", poolType);
	}
	return check_launch("pool_backward_kernel");
}

size_t fitre_hip_batch_norm_workspace(int channels, long perChannel)
{
	if (channels <= 0 || perChannel <= 0) return 0;
	return (size_t)channels * segments_for(channels, perChannel) * 8 * sizeof(double) + 64; // slots of up to eight sums
}

size_t fitre_hip_channel_sum_workspace(int channels, long perChannel)
{
	return fitre_hip_batch_norm_workspace(channels, perChannel);
}

static int check_channels(const char *fn, int channels, long perChannel, void *ws, size_t wsBytes)
{
	FITRE_REQUIRE(channels > 0 && perChannel > 0, "%s: non-positive shape (channels=%d, perChannel=%ld)", fn, channels, perChannel);
	FITRE_REQUIRE(channels <= 65535, "%s: %d channels exceed the grid limit", fn, channels);
	FITRE_REQUIRE(ws != nullptr && (((uintptr_t)ws) & 7) == 0, "%s: workspace is null or not 8-byte aligned", fn);
	if (wsBytes < fitre_hip_batch_norm_workspace(channels, perChannel))
		return fail(FITRE_E_WORKSPACE, "%s: workspace of %zu bytes is smaller than the %zu required", fn, wsBytes,
		            fitre_hip_batch_norm_workspace(channels, perChannel));
	return FITRE_OK;
}

int fitre_hip_channel_sum(const float *x, int channels, long perChannel, float *out, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(x && out, "fitre_hip_channel_sum: null pointer");
	int rc = check_channels("fitre_hip_channel_sum", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	int S = segments_for(channels, perChannel);
	double *partial = (double *)ws;
	LaunchScope scope(FITRE_KC_BIAS_GRAD, 4.0 * (double)channels * (double)perChannel);
	dim3 grid(S, channels);
	bool vec = aligned16(x) && (perChannel % 4 == 0);
	if (vec)
		channel_partial_kernel<0, true><<<grid, kRedBlock, 0, stream()>>>(x, nullptr, perChannel, partial);
	else
		channel_partial_kernel<0, false><<<grid, kRedBlock, 0, stream()>>>(x, nullptr, perChannel, partial);
	channel_finish_kernel<<<blocks_for(channels, 64), 64, 0, stream()>>>(partial, S, 0, channels, out);
	return check_launch("channel_sum");
}

int fitre_hip_batch_norm_forward(const float *in, int channels, long perChannel, float *zhat, float *mean, float *variance,
                                 float *runningMean, float *runningVariance, float epsilon, float momentum, int train,
                                 void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && zhat && mean && variance && runningMean && runningVariance, "fitre_hip_batch_norm_forward: null pointer");
	int rc = check_channels("fitre_hip_batch_norm_forward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	int S = segments_for(channels, perChannel);
	double *partial = (double *)ws;
	LaunchScope scope(FITRE_KC_BN_FWD, 4.0 * (double)channels * (double)perChannel * (train ? 3 : 2));
	dim3 grid(S, channels);
	bool vec = aligned16(in) && aligned16(zhat) && (perChannel % 4 == 0);
	if (train) {
		if (vec)
			channel_partial_kernel<2, true><<<grid, kRedBlock, 0, stream()>>>(in, nullptr, perChannel, partial);
		else
			channel_partial_kernel<2, false><<<grid, kRedBlock, 0, stream()>>>(in, nullptr, perChannel, partial);
		bn_stats_kernel<<<blocks_for(channels, 64), 64, 0, stream()>>>(partial, S, channels, perChannel, momentum, mean,
		                                                            variance, runningMean, runningVariance);
	}
	const float *mu = train ? mean : runningMean;
	const float *var = train ? variance : runningVariance;
	if (vec)
		bn_normalize_kernel<true><<<grid, kRedBlock, 0, stream()>>>(in, mu, var, epsilon, perChannel, zhat);
	else
		bn_normalize_kernel<false><<<grid, kRedBlock, 0, stream()>>>(in, mu, var, epsilon, perChannel, zhat);
	return check_launch("batch_norm_forward");
}

int fitre_hip_bn_act_pool_forward(const float *in, int channels, int samples, int inA, int inB, float *zhat, float *mean,
                                  float *variance, float *runningMean, float *runningVariance, float epsilon, float momentum,
                                  int train, int actFun, float *actOut, int poolType, int ksize, int stride, int padding, int outA,
                                  int outB, float *poolOut, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && actOut, "fitre_hip_bn_act_pool_forward: null pointer");
	FITRE_REQUIRE(!zhat || (mean && variance && runningMean && runningVariance), "fitre_hip_bn_act_pool_forward: null statistics");
	FITRE_REQUIRE(poolType == NO_POOL || poolOut, "fitre_hip_bn_act_pool_forward: null pooled output");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_bn_act_pool_forward: unknown activation code %d", actFun);
	FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0, "fitre_hip_bn_act_pool_forward: non-positive shape");
	const long perChannel = (long)samples * inA * inB, count = perChannel * channels;
	int rc;
	if (zhat) {
		rc = check_channels("fitre_hip_bn_act_pool_forward", channels, perChannel, ws, wsBytes);
		if (rc) return rc;
	}
	const bool pool2 = poolType == MAX_POOL && ksize == 2 && stride == 2 && padding == 0 && inB % 4 == 0 && inA % 2 == 0 &&
	                   outA == inA / 2 && outB == inB / 2 && (((uintptr_t)poolOut) & 7) == 0;
	const bool fused = (poolType == NO_POOL || pool2) && perChannel % 4 == 0 && channels <= 65535 && aligned16(in) && aligned16(actOut) &&
	                   (!zhat || aligned16(zhat));
	if (!fused) {
		const float *actIn = in;
		if (zhat) {
			rc = fitre_hip_batch_norm_forward(in, channels, perChannel, zhat, mean, variance, runningMean, runningVariance, epsilon, momentum,
			                                  train, ws, wsBytes);
			if (rc) return rc;
			actIn = zhat;
		}
		rc = fitre_hip_activation_forward(actFun, actIn, actOut, count);
		if (rc || poolType == NO_POOL) return rc;
		return fitre_hip_pool_forward(poolType, actOut, channels, samples, inA, inB, ksize, stride, padding, outA, outB, poolOut);
	}
	const int S = segments_for(channels, perChannel);
	double *partial = nullptr;
	const dim3 grid(S, channels);
	if (zhat && train) {
		partial = (double *)ws;
		LaunchScope scope(FITRE_KC_BN_FWD, 4.0 * (double)count);
		channel_partial_kernel<2, true><<<grid, kRedBlock, 0, stream()>>>(in, nullptr, perChannel, partial);
	}
	const double moved = 4.0 * (double)count * (zhat ? 3 : 2) + (poolType == NO_POOL ? 0.0 : (double)count);
	LaunchScope scope(zhat ? FITRE_KC_BN_FWD : FITRE_KC_ACT_FWD, moved);
	if (poolType == NO_POOL)
		bn_act_pool_forward_kernel<2><<<grid, kRedBlock, 0, stream()>>>(in, partial, S, momentum, mean, variance, runningMean, runningVariance,
		                                                                runningMean, runningVariance, epsilon, samples, inA, inB, actFun,
		                                                                zhat, actOut, poolOut);
	else
		bn_act_pool_forward_kernel<0><<<grid, kRedBlock, 0, stream()>>>(in, partial, S, momentum, mean, variance, runningMean, runningVariance,
		                                                                runningMean, runningVariance, epsilon, samples, inA, inB, actFun,
		                                                                zhat, actOut, poolOut);
	return check_launch("bn_act_pool_forward_kernel");
}

// The launches of the stand-alone batch-norm backward step; `partial` holds the per-(channel, segment) sums.
static int bn_backward_launch(const float *delta, const float *zhat, const float *variance, int channels, long perChannel,
                              float epsilon, float *out, float *biasGrad, double *partial)
{
	int S = segments_for(channels, perChannel);
	LaunchScope scope(FITRE_KC_BN_BWD, 12.0 * (double)channels * (double)perChannel + 8.0 * channels);
	dim3 grid(S, channels);
	bool vec = aligned16(delta) && aligned16(zhat) && aligned16(out) && (perChannel % 4 == 0);
	if (perChannel <= kBnSmallChannel && channels >= 128) {
		if (vec)
			bn_backward_small_kernel<true><<<channels, kRedBlock, 0, stream()>>>(delta, zhat, variance, epsilon, perChannel, out, biasGrad);
		else
			bn_backward_small_kernel<false><<<channels, kRedBlock, 0, stream()>>>(delta, zhat, variance, epsilon, perChannel, out, biasGrad);
	} else if (vec) {
		channel_partial_kernel<3, true><<<grid, kRedBlock, 0, stream()>>>(delta, zhat, perChannel, partial);
		bn_backward_apply_kernel<true><<<grid, kRedBlock, 0, stream()>>>(delta, zhat, variance, partial, S, epsilon, perChannel,
		                                                                 out, biasGrad);
	} else {
		channel_partial_kernel<3, false><<<grid, kRedBlock, 0, stream()>>>(delta, zhat, perChannel, partial);
		bn_backward_apply_kernel<false><<<grid, kRedBlock, 0, stream()>>>(delta, zhat, variance, partial, S, epsilon, perChannel,
		                                                                  out, biasGrad);
	}
	return check_launch("batch_norm_backward");
}

int fitre_hip_batch_norm_backward(const float *delta, const float *zhat, const float *variance, int channels,
                                  long perChannel, float epsilon, float *out, float *biasGrad, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && zhat && variance && out, "fitre_hip_batch_norm_backward: null pointer");
	int rc = check_channels("fitre_hip_batch_norm_backward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	return bn_backward_launch(delta, zhat, variance, channels, perChannel, epsilon, out, biasGrad, (double *)ws);
}

int fitre_hip_batch_norm_backward_static(const float *delta, const float *zhat, const float *variance, int channels,
                                         long perChannel, float epsilon, float *out, float *biasGrad)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(delta && zhat && variance && out, "fitre_hip_batch_norm_backward_static: null pointer");
	FITRE_REQUIRE(channels > 0 && perChannel > 0, "fitre_hip_batch_norm_backward_static: non-positive shape (channels=%d, perChannel=%ld)",
	              channels, perChannel);
	FITRE_REQUIRE(channels <= 65535, "fitre_hip_batch_norm_backward_static: %d channels exceed the grid limit", channels);
	const size_t need = fitre_hip_batch_norm_workspace(channels, perChannel);
	if (need > (size_t)FITRE_HIP_STATIC_SCRATCH_BYTES)
		return fail(FITRE_E_WORKSPACE,
		            "fitre_hip_batch_norm_backward_static: %d channels of %ld elements need %zu bytes of partial sums, the static "
		            "scratch array holds %d; use fitre_hip_batch_norm_backward with a workspace",
		            channels, perChannel, need, FITRE_HIP_STATIC_SCRATCH_BYTES);
	const int device = current_device();
	void *ptr = (device >= 0 && device < kMaxDevices) ? g_scratch_ptr[device] : nullptr;
	if (!ptr) return fail(FITRE_E_DEVICE, "fitre_hip_batch_norm_backward_static: no scratch address for device %d", device);
	// every (channel, segment) slot the apply pass reads is written by the partial-sum pass of the
	// same call, so nothing of an earlier call's contents has to be cleared
	return bn_backward_launch(delta, zhat, variance, channels, perChannel, epsilon, out, biasGrad, (double *)ptr);
}

int fitre_hip_pool_act_bn_backward(int poolType, int actFun, float *delta, int deltaSplits, long deltaStride, const float *zhat,
                                   const float *z_act, const float *variance, int channels, int samples, int inA, int inB,
                                   int ksize, int stride, int padding, int outA, int outB, float epsilon, float *dxPool,
                                   float *dxAct, float *dxBn, float *biasGrad, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(deltaSplits >= 1 && (deltaSplits == 1 || deltaStride > 0),
	              "fitre_hip_pool_act_bn_backward: bad split view (%d slabs, stride %ld)", deltaSplits, deltaStride);
	FITRE_REQUIRE(delta && zhat && variance && dxAct && dxBn, "fitre_hip_pool_act_bn_backward: null pointer");
	FITRE_REQUIRE(z_act || actFun == CNN_ACT_RELU,
	              "fitre_hip_pool_act_bn_backward: z_act may be left out for ReLU only (activation %d)", actFun);
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_pool_act_bn_backward: unknown activation code %d", actFun);
	FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0, "fitre_hip_pool_act_bn_backward: non-positive shape");
	const long perChannel = (long)samples * inA * inB;
	int rc = check_channels("fitre_hip_pool_act_bn_backward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	FITRE_REQUIRE((double)channels * (double)perChannel < 2147483647.0, "fitre_hip_pool_act_bn_backward: tensor exceeds 2^31 elements");
	const bool aligned = aligned16(zhat) && aligned16(dxAct) && aligned16(dxBn) && (!z_act || aligned16(z_act)) &&
	                     (!dxPool || aligned16(dxPool));
	bool fused = false;
	if (poolType == NO_POOL)
		fused = aligned && aligned16(delta) && perChannel % 4 == 0 && (deltaSplits == 1 || deltaStride % 4 == 0);
	else if (poolType == MAX_POOL)
		fused = aligned && ksize == 2 && stride == 2 && padding == 0 && inB % 2 == 0 && inA % 2 == 0 && perChannel % 4 == 0 &&
		        outA == inA / 2 && outB == inB / 2 && (((uintptr_t)delta & 7) == 0) && (deltaSplits == 1 || deltaStride % 2 == 0);
	const int variant = (poolType == NO_POOL) ? 2 : (inB == 2 ? 3 : (inB % 4 == 0 ? 0 : 1));
	if (!fused) {
		// other windows / layouts: the separate passes (slabs summed, z_act rebuilt for the ReLU shortcut)
		if (deltaSplits > 1) {
			const long nd = (poolType == NO_POOL) ? (long)channels * perChannel : (long)channels * samples * outA * outB;
			sum_slabs_kernel<<<blocks_for(nd, 256, 8192), 256, 0, stream()>>>(delta, deltaSplits, deltaStride, nd);
			rc = check_launch("sum_slabs_kernel");
			if (rc) return rc;
		}
		const float *zo = z_act;
		if (!zo) {
			rc = fitre_hip_activation_forward(actFun, zhat, dxBn, (long)channels * perChannel);
			if (rc) return rc;
			zo = dxBn; // free until the batch-norm step writes it
		}
		rc = fitre_hip_pool_act_backward(poolType, actFun, delta, zhat, zo, channels, samples, inA, inB, ksize, stride, padding,
		                                 outA, outB, dxPool, dxAct);
		if (rc) return rc;
		return fitre_hip_batch_norm_backward(dxAct, zhat, variance, channels, perChannel, epsilon, dxBn, biasGrad, ws, wsBytes);
	}
	const double total = (double)channels * (double)perChannel;
	const double poolBytes = 4.0 * total * (2 + (dxPool ? 1 : 0) + (z_act ? 1 : 0)) +
	                         4.0 * deltaSplits * (poolType == NO_POOL ? total : total / 4);
	if (perChannel <= kBnSmallChannel && channels >= 128 && variant != 1) {
		LaunchScope scope(FITRE_KC_POOL_ACT_BWD, poolBytes + 4.0 * total);
		if (variant == 2)
			pool_act_bn_small_kernel<2><<<channels, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, variance, inA, inB, samples, actFun,
			                                                                 epsilon, dxPool, dxAct, dxBn, biasGrad);
		else if (variant == 3)
			pool_act_bn_small_kernel<3><<<channels, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, variance, inA, inB, samples, actFun,
			                                                                 epsilon, dxPool, dxAct, dxBn, biasGrad);
		else
			pool_act_bn_small_kernel<0><<<channels, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, variance, inA, inB, samples, actFun,
			                                                                 epsilon, dxPool, dxAct, dxBn, biasGrad);
		return check_launch("pool_act_bn_small_kernel");
	}
	const int S = segments_for(channels, perChannel);
	double *partial = (double *)ws;
	dim3 grid(S, channels);
	const bool streamPool = 4.0 * total >= 48.0 * 1024 * 1024; // the pool gradient is a snapshot nothing reads in this pass
	{
		LaunchScope scope(FITRE_KC_POOL_ACT_BWD, poolBytes);
		if (variant == 1)
			pool_act_sums_kernel<1><<<grid, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, inA, inB, samples, actFun, dxPool, streamPool, dxAct, partial);
		else if (variant == 2)
			pool_act_sums_kernel<2><<<grid, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, inA, inB, samples, actFun, dxPool, streamPool, dxAct, partial);
		else if (variant == 3)
			pool_act_sums_kernel<3><<<grid, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, inA, inB, samples, actFun, dxPool, streamPool, dxAct, partial);
		else
			pool_act_sums_kernel<0><<<grid, kRedBlock, 0, stream()>>>(delta, deltaSplits, deltaStride, zhat, z_act, inA, inB, samples, actFun, dxPool, streamPool, dxAct, partial);
		rc = check_launch("pool_act_sums_kernel");
		if (rc) return rc;
	}
	LaunchScope scope(FITRE_KC_BN_BWD, 12.0 * total + 8.0 * channels);
	bn_backward_apply_kernel<true><<<grid, kRedBlock, 0, stream()>>>(dxAct, zhat, variance, partial, S, epsilon, perChannel, dxBn,
	                                                                 biasGrad);
	return check_launch("bn_backward_apply_kernel");
}

int fitre_hip_softmax_cross_entropy(const float *logits, const float *target, int rows, int classes, float *probs,
                                    float *errors, float *lossHost)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(logits && target && probs && lossHost, "fitre_hip_softmax_cross_entropy: null pointer");
	FITRE_REQUIRE(rows > 0 && classes > 0, "fitre_hip_softmax_cross_entropy: non-positive shape (%d x %d)", rows, classes);
	if (rows > g_nll_rows) {
		FITRE_HIP_TRY(hipDeviceSynchronize()); // the buffer is shared by every lane
		if (g_nll) FITRE_HIP_TRY(hipFree(g_nll));
		g_nll = nullptr;
		g_nll_rows = 0;
		int cap = rows < 4096 ? 4096 : rows;
		FITRE_HIP_TRY(hipMalloc((void **)&g_nll, sizeof(float) * ((size_t)cap + 16)));
		g_nll_rows = cap;
	}
	if (!g_loss_host) FITRE_HIP_TRY(hipHostMalloc((void **)&g_loss_host, 64, hipHostMallocDefault));
	{
		LaunchScope scope(FITRE_KC_SOFTMAX, 4.0 * rows * classes * 2);
		softmax_ce_kernel<<<blocks_for(rows, 4), 256, 0, stream()>>>(logits, target, rows, classes, probs, errors, g_nll);
		mean_kernel<<<1, 256, 0, stream()>>>(g_nll, rows, g_nll + g_nll_rows);
		int rc = check_launch("softmax_ce_kernel");
		if (rc) return rc;
	}
	FITRE_HIP_TRY(hipMemcpyAsync(g_loss_host, g_nll + g_nll_rows, sizeof(float), hipMemcpyDeviceToHost, stream()));
	FITRE_HIP_TRY(hipStreamSynchronize(stream()));
	*lossHost = *g_loss_host;
	return FITRE_OK;
}

int fitre_hip_cross_entropy_rop_error(const float *rz, const float *probs, int rows, int classes, float *rError)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(rz && probs && rError, "fitre_hip_cross_entropy_rop_error: null pointer");
	FITRE_REQUIRE(rows > 0 && classes > 0, "fitre_hip_cross_entropy_rop_error: non-positive shape %d x %d", rows, classes);
	LaunchScope scope(FITRE_KC_SOFTMAX, 12.0 * (double)rows * classes);
	cross_entropy_rop_error_kernel<<<blocks_for(rows, 256), 256, 0, stream()>>>(rz, probs, rows, classes, 1.f / (float)rows, rError);
	return check_launch("cross_entropy_rop_error_kernel");
}

int fitre_hip_column_softmax_rop(const float *probs, const float *rx, int rows, int cols, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(probs && rx && out, "fitre_hip_column_softmax_rop: null pointer");
	FITRE_REQUIRE(rows > 0 && cols > 0, "fitre_hip_column_softmax_rop: non-positive shape %d x %d", rows, cols);
	LaunchScope scope(FITRE_KC_SOFTMAX, 12.0 * (double)rows * cols);
	cross_entropy_rop_error_kernel<<<blocks_for(cols, 256), 256, 0, stream()>>>(rx, probs, cols, rows, 1.f, out);
	return check_launch("cross_entropy_rop_error_kernel");
}

int fitre_hip_batch_norm_rop_backward(const float *rdelta_x, const float *delta_x, const float *zhat, const float *rzhat,
                                      const float *rx, const float *delta_c, const float *variance, int channels,
                                      long perChannel, float epsilon, float *out, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(rdelta_x && delta_x && zhat && rzhat && rx && delta_c && variance && out,
	              "fitre_hip_batch_norm_rop_backward: null pointer");
	int rc = check_channels("fitre_hip_batch_norm_rop_backward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	const int S = segments_for(channels, perChannel);
	if (wsBytes < (size_t)channels * S * 8 * sizeof(double))
		return fail(FITRE_E_WORKSPACE, "fitre_hip_batch_norm_rop_backward: workspace of %zu bytes is smaller than the %zu required",
		            wsBytes, (size_t)channels * S * 8 * sizeof(double));
	double *partial = (double *)ws;
	LaunchScope scope(FITRE_KC_BN_BWD, 28.0 * (double)channels * (double)perChannel);
	dim3 grid(S, channels);
	const bool vec = perChannel % 4 == 0 && aligned16(rdelta_x) && aligned16(delta_x) && aligned16(zhat) && aligned16(rzhat) && aligned16(rx) &&
	                 aligned16(delta_c) && aligned16(out);
	if (vec) {
		bn_rop_partial_kernel<true><<<grid, kRedBlock, 0, stream()>>>(rdelta_x, delta_x, zhat, rzhat, rx, perChannel, partial);
		bn_rop_apply_kernel<true><<<grid, kRedBlock, 0, stream()>>>(rdelta_x, zhat, rzhat, delta_c, variance, partial, S, epsilon, perChannel, out);
	} else {
		bn_rop_partial_kernel<false><<<grid, kRedBlock, 0, stream()>>>(rdelta_x, delta_x, zhat, rzhat, rx, perChannel, partial);
		bn_rop_apply_kernel<false><<<grid, kRedBlock, 0, stream()>>>(rdelta_x, zhat, rzhat, delta_c, variance, partial, S, epsilon, perChannel, out);
	}
	return check_launch("batch_norm_rop_backward");
}

int fitre_hip_pool_act_bn_rop_backward(int poolType, int actFun, const float *rdelta, const float *delta, const float *zhat,
                                       const float *z_act, const float *rzhat, const float *delta_x, const float *rx,
                                       const float *delta_c, const float *variance, int channels, int samples, int inA, int inB,
                                       int ksize, int stride, int padding, int outA, int outB, float epsilon, float *rdeltaAct,
                                       float *rdeltaX, float *out, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(rdelta && delta && zhat && rzhat && delta_x && rx && delta_c && variance && rdeltaX && out,
	              "fitre_hip_pool_act_bn_rop_backward: null pointer");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_pool_act_bn_rop_backward: unknown activation code %d", actFun);
	FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0, "fitre_hip_pool_act_bn_rop_backward: non-positive shape");
	const long perChannel = (long)samples * inA * inB, count = perChannel * channels;
	int rc = check_channels("fitre_hip_pool_act_bn_rop_backward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	const int S = segments_for(channels, perChannel);
	if (wsBytes < (size_t)channels * S * 8 * sizeof(double))
		return fail(FITRE_E_WORKSPACE, "fitre_hip_pool_act_bn_rop_backward: workspace of %zu bytes is smaller than the %zu required", wsBytes,
		            (size_t)channels * S * 8 * sizeof(double));
	const bool pool2 = poolType == MAX_POOL && ksize == 2 && stride == 2 && padding == 0 && inB % 4 == 0 && inA % 2 == 0 &&
	                   outA == inA / 2 && outB == inB / 2 && (((uintptr_t)rdelta) & 7) == 0;
	const bool second = !(actFun == CNN_ACT_RELU || actFun == ACT_LINEAR || actFun == CNN_ACT_NONE);
	const bool fused = (pool2 || (poolType == NO_POOL && aligned16(rdelta))) && perChannel % 4 == 0 && aligned16(zhat) && aligned16(rzhat) &&
	                   aligned16(delta_x) && aligned16(rx) && aligned16(delta_c) && aligned16(rdeltaX) && aligned16(out) &&
	                   (!z_act || aligned16(z_act)) && (!second || aligned16(delta)) && (z_act || actFun == CNN_ACT_RELU);
	if (!fused) {
		FITRE_REQUIRE(z_act, "fitre_hip_pool_act_bn_rop_backward: this shape runs the separate passes, which need z_act");
		const float *atAct = rdelta;
		if (poolType != NO_POOL) {
			FITRE_REQUIRE(rdeltaAct, "fitre_hip_pool_act_bn_rop_backward: the separate passes need a buffer for the routed R{delta}");
			rc = fitre_hip_pool_backward(poolType, rdelta, z_act, channels, samples, inA, inB, ksize, stride, padding, outA, outB, rdeltaAct);
			if (rc) return rc;
			atAct = rdeltaAct;
		}
		rc = fitre_hip_activation_rop_backward(actFun, atAct, delta, zhat, z_act, rzhat, rdeltaX, count);
		if (rc) return rc;
		return fitre_hip_batch_norm_rop_backward(rdeltaX, delta_x, zhat, rzhat, rx, delta_c, variance, channels, perChannel, epsilon, out, ws,
		                                         wsBytes);
	}
	double *partial = (double *)ws;
	const dim3 grid(S, channels);
	LaunchScope scope(FITRE_KC_BN_BWD, 4.0 * (double)count * (11.0 + (second ? 1.0 : 0.0) + (z_act ? 1.0 : 0.0)));
	if (poolType == NO_POOL) {
		if (second)
			pool_act_bn_rop_sums_kernel<2, true><<<grid, kRedBlock, 0, stream()>>>(rdelta, delta, zhat, z_act, rzhat, delta_x, rx, inA, inB, samples,
			                                                                       actFun, rdeltaX, partial);
		else
			pool_act_bn_rop_sums_kernel<2, false><<<grid, kRedBlock, 0, stream()>>>(rdelta, delta, zhat, z_act, rzhat, delta_x, rx, inA, inB, samples,
			                                                                        actFun, rdeltaX, partial);
	} else {
		if (second)
			pool_act_bn_rop_sums_kernel<0, true><<<grid, kRedBlock, 0, stream()>>>(rdelta, delta, zhat, z_act, rzhat, delta_x, rx, inA, inB, samples,
			                                                                       actFun, rdeltaX, partial);
		else
			pool_act_bn_rop_sums_kernel<0, false><<<grid, kRedBlock, 0, stream()>>>(rdelta, delta, zhat, z_act, rzhat, delta_x, rx, inA, inB, samples,
			                                                                        actFun, rdeltaX, partial);
	}
	bn_rop_apply_kernel<true><<<grid, kRedBlock, 0, stream()>>>(rdeltaX, zhat, rzhat, delta_c, variance, partial, S, epsilon, perChannel, out);
	return check_launch("pool_act_bn_rop_backward");
}

int fitre_hip_pool_forward_routed(int poolType, const float *values, const float *z_act, int channels, int samples, int inA,
                                  int inB, int ksize, int stride, int padding, int outA, int outB, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(values && out, "fitre_hip_pool_forward_routed: null pointer");
	if (poolType == AVG_POOL) return fitre_hip_pool_forward(AVG_POOL, values, channels, samples, inA, inB, ksize, stride, padding, outA, outB, out);
	if (poolType != MAX_POOL) return fail(FITRE_E_UNSUPPORTED, "fitre_hip_pool_forward_routed: unknown pool type %d", poolType);
	FITRE_REQUIRE(z_act, "fitre_hip_pool_forward_routed: z_act is required for max pooling");
	int rc = check_pool_shape("fitre_hip_pool_forward_routed", channels, samples, inA, inB, ksize, stride, padding, outA, outB);
	if (rc) return rc;
	PoolGeom g = make_geom(inA, inB, ksize, stride, padding, outA, outB);
	const long maps = (long)channels * samples;
	LaunchScope scope(FITRE_KC_POOL_FWD, 4.0 * (double)maps * (2.0 * inA * inB + (double)outA * outB));
	if (ksize == 2 && stride == 2 && padding == 0 && inB % 4 == 0 && inA % 2 == 0 && outA == inA / 2 && outB == inB / 2 && aligned16(values) &&
	    aligned16(z_act) && (((uintptr_t)out) & 7) == 0) {
		pool_routed2_kernel<<<blocks_for(maps * outA * (inB / 4), 256, 16384), 256, 0, stream()>>>(values, z_act, inA, inB, maps, out);
		return check_launch("pool_routed2_kernel");
	}
	pool_routed_kernel<<<blocks_for(maps * outA * outB, 256, 16384), 256, 0, stream()>>>(values, z_act, g, maps, out);
	return check_launch("pool_routed_kernel");
}

int fitre_hip_bn_act_pool_rop_forward(const float *rx, const float *zhat, const float *z_act, const float *variance, int channels,
                                      int samples, int inA, int inB, float epsilon, int actFun, float *rbn, float *ract, int poolType,
                                      int ksize, int stride, int padding, int outA, int outB, float *rpool, void *ws, size_t wsBytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(rx && zhat && variance && rbn && ract, "fitre_hip_bn_act_pool_rop_forward: null pointer");
	FITRE_REQUIRE(poolType == NO_POOL || rpool, "fitre_hip_bn_act_pool_rop_forward: null pooled output");
	FITRE_REQUIRE(act_known(actFun), "fitre_hip_bn_act_pool_rop_forward: unknown activation code %d", actFun);
	FITRE_REQUIRE(z_act || actFun == CNN_ACT_RELU, "fitre_hip_bn_act_pool_rop_forward: z_act is required (only ReLU's output can be derived)");
	FITRE_REQUIRE(channels > 0 && samples > 0 && inA > 0 && inB > 0, "fitre_hip_bn_act_pool_rop_forward: non-positive shape");
	const long perChannel = (long)samples * inA * inB, count = perChannel * channels;
	int rc = check_channels("fitre_hip_bn_act_pool_rop_forward", channels, perChannel, ws, wsBytes);
	if (rc) return rc;
	const bool pool2 = poolType == MAX_POOL && ksize == 2 && stride == 2 && padding == 0 && inB % 4 == 0 && inA % 2 == 0 &&
	                   outA == inA / 2 && outB == inB / 2 && (((uintptr_t)rpool) & 7) == 0;
	const bool fused = (poolType == NO_POOL || pool2) && perChannel % 4 == 0 && aligned16(rx) && aligned16(zhat) && aligned16(rbn) &&
	                   aligned16(ract) && (!z_act || aligned16(z_act));
	if (!fused) {
		FITRE_REQUIRE(z_act, "fitre_hip_bn_act_pool_rop_forward: this shape runs the separate passes, which need z_act");
		rc = fitre_hip_batch_norm_backward(rx, zhat, variance, channels, perChannel, epsilon, rbn, nullptr, ws, wsBytes);
		if (rc) return rc;
		rc = fitre_hip_activation_backward(actFun, rbn, zhat, z_act, ract, count);
		if (rc || poolType == NO_POOL) return rc;
		return fitre_hip_pool_forward_routed(poolType, ract, z_act, channels, samples, inA, inB, ksize, stride, padding, outA, outB, rpool);
	}
	const int S = segments_for(channels, perChannel);
	double *partial = (double *)ws;
	const dim3 grid(S, channels);
	LaunchScope scope(FITRE_KC_BN_BWD, 4.0 * (double)count * (2 + 2 + 2 + (z_act ? 1 : 0)) + (poolType == NO_POOL ? 0.0 : (double)count));
	channel_partial_kernel<3, true><<<grid, kRedBlock, 0, stream()>>>(rx, zhat, perChannel, partial);
	if (poolType == NO_POOL)
		bn_act_pool_rop_forward_kernel<2><<<grid, kRedBlock, 0, stream()>>>(rx, zhat, z_act, variance, partial, S, epsilon, samples, inA, inB,
		                                                                    actFun, rbn, ract, rpool);
	else
		bn_act_pool_rop_forward_kernel<0><<<grid, kRedBlock, 0, stream()>>>(rx, zhat, z_act, variance, partial, S, epsilon, samples, inA, inB,
		                                                                    actFun, rbn, ract, rpool);
	return check_launch("bn_act_pool_rop_forward_kernel");
}

int fitre_hip_multinomial_classes(const float *probs, const float *uniforms, int samples, int classes, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(probs && uniforms && out, "fitre_hip_multinomial_classes: null pointer");
	FITRE_REQUIRE(samples > 0 && classes > 0, "fitre_hip_multinomial_classes: non-positive shape %d x %d", samples, classes);
	LaunchScope scope(FITRE_KC_SOFTMAX, 4.0 * (double)samples * (classes + 2));
	multinomial_classes_kernel<<<blocks_for(samples, 256), 256, 0, stream()>>>(probs, uniforms, samples, classes, out);
	return check_launch("multinomial_classes_kernel");
}

int fitre_hip_accuracy_hits(const float *probs, const float *target, int rows, int classes, float *hits)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(probs && target && hits, "fitre_hip_accuracy_hits: null pointer");
	FITRE_REQUIRE(rows > 0 && classes > 0, "fitre_hip_accuracy_hits: non-positive shape %d x %d", rows, classes);
	LaunchScope scope(FITRE_KC_SOFTMAX, 4.0 * (double)rows * (classes + 2));
	accuracy_hits_kernel<<<blocks_for(rows, 256), 256, 0, stream()>>>(probs, target, rows, classes, hits);
	return check_launch("accuracy_hits_kernel");
}

int fitre_hip_cross_entropy_error(const float *probs, const float *target, int rows, int classes, float *errors)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(probs && target && errors, "fitre_hip_cross_entropy_error: null pointer");
	FITRE_REQUIRE(rows > 0 && classes > 0, "fitre_hip_cross_entropy_error: non-positive shape (%d x %d)", rows, classes);
	LaunchScope scope(FITRE_KC_SOFTMAX, 8.0 * rows * classes);
	cross_entropy_error_kernel<<<blocks_for((long)rows * classes, 256, 4096), 256, 0, stream()>>>(probs, target, rows, classes, errors);
	return check_launch("cross_entropy_error_kernel");
}

int fitre_hip_reshape(const float *in, int right, int left, int chunk, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && out && in != out, "fitre_hip_reshape: null or aliased pointers");
	FITRE_REQUIRE(right > 0 && left > 0 && chunk > 0, "fitre_hip_reshape: non-positive shape");
	long total = (long)right * left * chunk;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * total);
	reshape_kernel<<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(in, right, left, chunk, out);
	return check_launch("reshape_kernel");
}

int fitre_hip_conv_to_fc(const float *in, int channels, int samples, int extA, int extB, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && out && in != out, "fitre_hip_conv_to_fc: null or aliased pointers");
	FITRE_REQUIRE(channels > 0 && samples > 0 && extA > 0 && extB > 0, "fitre_hip_conv_to_fc: non-positive shape");
	long total = (long)channels * samples * extA * extB;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * total);
	boundary_permute_kernel<true><<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(in, channels, samples, extA, extB, out);
	return check_launch("boundary_permute_kernel");
}

int fitre_hip_fc_to_conv(const float *in, int channels, int samples, int extA, int extB, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && out && in != out, "fitre_hip_fc_to_conv: null or aliased pointers");
	FITRE_REQUIRE(channels > 0 && samples > 0 && extA > 0 && extB > 0, "fitre_hip_fc_to_conv: non-positive shape");
	long total = (long)channels * samples * extA * extB;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * total);
	boundary_permute_kernel<false><<<blocks_for(total, 512, 8192), 256, 0, stream()>>>(in, channels, samples, extA, extB, out);
	return check_launch("boundary_permute_kernel");
}

} // extern "C"
