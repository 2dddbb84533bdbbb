// Weight gradient of a wide fully connected layer at a small batch: dW(out x in) = delta(out x n) * zin(in x n)',
// db = delta * 1, n <= 64 (functions/cnn_backward.cu:189-197, :216-224; AlexNet's 9216-4096-4096-1000 tail at batch 64).
//
// The reduction is the batch, so the whole of it fits registers: a result element costs n multiply-adds and four bytes
// of HBM, and the product is bound by writing dW (151 MB for 9216 x 4096) as much as by the matrix pipes.  A workgroup
// therefore keeps its 128 rows of delta as MFMA fragments for its whole life and walks along the inputs: per 128 x
// 128 tile it reads the 128 x n block of zin straight into fragments (both operands are contiguous along the index that a
// fragment's 32 lanes span, so no LDS staging is needed); a finished tile is put into LDS and leaves from there as whole
// 512-byte rows BETWEEN the matrix steps of the next tile, so that the writes to HBM run at an even rate beside the
// matrix work instead of in bursts.  Two workgroups share a compute unit.  No reduction
// split, no second launch.
#pragma once
#include "gemm_engine.h"

namespace fitre {

constexpr int kSkinnyBatch = 64; // largest batch; it must be even
constexpr int kSkinnySteps = kSkinnyBatch / 2;

struct SkinnyDwParams {
	const float *delta; // out x n, column-major
	const float *zin;   // in x n, column-major
	float *dW;          // out x in, column-major
	float *db;          // out, or null
	int out, in, n;
	int inBlocks, inBlocksPerGroup;
};

constexpr int kSkinnyLd = 128 + 4; // row stride of the tile in LDS: 16-byte aligned rows, conflict-free both ways

// 2 x 32 fragments of a 64-row strip of a column-major (rows x n) matrix: element (row0 + 32 b + lane % 32, 2 step + lane / 32)
__device__ __forceinline__ void skinny_load(float (&f)[2][kSkinnySteps], __amdgpu_buffer_rsrc_t rs, int rows, int row0, int steps,
                                            int l32, int khalf)
{
#pragma unroll
	for (int b = 0; b < 2; b++) {
		const int row = row0 + 32 * b + l32;
		// a row outside the matrix: an offset beyond any buffer this kernel takes, which adding a step's share cannot wrap
		const uint32_t voff = row < rows ? 4u * (uint32_t)(khalf * rows + row) : 0x80000000u;
#pragma unroll
		for (int s = 0; s < kSkinnySteps; s++) {
			f[b][s] = 0.f;
			if (s < steps) // uniform
				f[b][s] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, (int)(voff + 8u * (uint32_t)(s * rows)), 0, 0));
		}
	}
}

// VEC: out % 4 == 0 and dW is 16-byte aligned, so a tile leaves through LDS as whole 512-byte rows (16 bytes per lane)
template <bool VEC>
__global__ void __launch_bounds__(256, 2) fc_dw_skinny_kernel(const SkinnyDwParams p)
{
	FITRE_RAISE_MATRIX_WAVE_PRIORITY();
	extern __shared__ float tileLds[]; // VEC: 128 rows (inputs) of kSkinnyLd
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, khalf = lane >> 5;
	const int wo = wave & 1, wi = wave >> 1; // the wave's 64 x 64 quarter of the tile
	const int steps = p.n >> 1;
	const __amdgpu_buffer_rsrc_t dRs = make_rsrc(p.delta, 4u * (uint32_t)p.out * (uint32_t)p.n);
	const __amdgpu_buffer_rsrc_t zRs = make_rsrc(p.zin, 4u * (uint32_t)p.in * (uint32_t)p.n);
	const int ob0 = (int)blockIdx.x * 128, o0 = ob0 + wo * 64;
	float dfr[2][kSkinnySteps];
	skinny_load(dfr, dRs, p.out, o0, steps, l32, khalf);
	const int ibBeg = (int)blockIdx.y * p.inBlocksPerGroup;
	const int ibEnd = (ibBeg + p.inBlocksPerGroup < p.inBlocks) ? ibBeg + p.inBlocksPerGroup : p.inBlocks;

	if (p.db != nullptr && blockIdx.y == 0 && wi == 0) {
		// row sums of delta from the fragments: a lane holds every second sample of two rows
#pragma unroll
		for (int b = 0; b < 2; b++) {
			float s = 0.f;
#pragma unroll
			for (int k = 0; k < kSkinnySteps; k++) s += dfr[b][k];
			s += __shfl_xor(s, 32);
			const int o = o0 + 32 * b + l32;
			if (khalf == 0 && o < p.out) p.db[o] = s;
		}
	}

	// a row piece of the tile in LDS (the previous tile of this workgroup) to memory: 16 bytes per lane
	auto store_piece = [&](int t, int ibPrev) {
		typedef float f4 __attribute__((ext_vector_type(4)));
		const int idx = tid + 256 * t, row = idx >> 5, c4 = (idx & 31) * 4;
		const f4 val = *reinterpret_cast<const f4 *>(tileLds + row * kSkinnyLd + c4);
		if (ibPrev * 128 + row < p.in && ob0 + c4 < p.out)
			__builtin_nontemporal_store(val, reinterpret_cast<f4 *>(p.dW + (size_t)(ibPrev * 128 + row) * p.out + ob0 + c4));
	};

	float zf[2][kSkinnySteps];
	if (ibBeg < ibEnd) skinny_load(zf, zRs, p.in, ibBeg * 128 + wi * 64, steps, l32, khalf);
	for (int ib = ibBeg; ib < ibEnd; ib++) {
		const int i0 = ib * 128 + wi * 64;
		const bool drain = VEC && ib != ibBeg; // the previous tile sits in LDS: it leaves between this tile's matrix steps
		v16f acc[2][2];
#pragma unroll
		for (int bi = 0; bi < 2; bi++)
#pragma unroll
			for (int bo = 0; bo < 2; bo++)
#pragma unroll
				for (int v = 0; v < 16; v++) acc[bi][bo][v] = 0.f;
#pragma unroll
		for (int s = 0; s < kSkinnySteps; s++) {
			if (s < steps) {
#pragma unroll
				for (int bi = 0; bi < 2; bi++)
#pragma unroll
					for (int bo = 0; bo < 2; bo++)
						acc[bi][bo] = __builtin_amdgcn_mfma_f32_32x32x2f32(zf[bi][s], dfr[bo][s], acc[bi][bo], 0, 0, 0);
			}
			if (VEC && (s & 1) && drain) store_piece(s >> 1, ib - 1); // sixteen pieces over thirty-two steps
		}
		// the next block of zin is requested into the fragments the matrix pipes have just finished with
		if (ib + 1 < ibEnd) skinny_load(zf, zRs, p.in, (ib + 1) * 128 + wi * 64, steps, l32, khalf);
		// register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 (an input), column l % 32 (an output unit)
		if (VEC) {
			if (drain) __syncthreads(); // the previous tile has left LDS
#pragma unroll
			for (int bi = 0; bi < 2; bi++)
#pragma unroll
				for (int bo = 0; bo < 2; bo++)
#pragma unroll
					for (int v = 0; v < 16; v++)
						tileLds[(wi * 64 + 32 * bi + 8 * (v / 4) + 4 * khalf + (v % 4)) * kSkinnyLd + wo * 64 + 32 * bo + l32] = acc[bi][bo][v];
			__syncthreads();
		} else {
#pragma unroll
			for (int bi = 0; bi < 2; bi++) {
#pragma unroll
				for (int bo = 0; bo < 2; bo++) {
					const int o = o0 + 32 * bo + l32;
#pragma unroll
					for (int v = 0; v < 16; v++) {
						const int i = i0 + 32 * bi + 8 * (v / 4) + 4 * khalf + (v % 4);
						if (o < p.out && i < p.in) __builtin_nontemporal_store(acc[bi][bo][v], p.dW + (size_t)i * p.out + o);
					}
				}
			}
		}
	}
	if (VEC && ibBeg < ibEnd) {
#pragma unroll
		for (int t = 0; t < 16; t++) store_piece(t, ibEnd - 1);
	}
}

static inline bool skinny_dw_fits(int in, int out, int n)
{
	return n >= 2 && n <= kSkinnyBatch && (n & 1) == 0 && in >= 512 && out >= 512 && (double)in * n * 4.0 < 2.0e9 &&
	       (double)out * n * 4.0 < 2.0e9 && (double)in * out >= 2.0e6;
}

static inline int launch_skinny_dw(int in, int out, int n, const float *delta, const float *zin, float *dW, float *db, int cus)
{
	SkinnyDwParams p{};
	p.delta = delta, p.zin = zin, p.dW = dW, p.db = db;
	p.out = out, p.in = in, p.n = n;
	const int outBlocks = (out + 127) / 128;
	p.inBlocks = (in + 127) / 128;
	int groups = 2 * cus / outBlocks; // two workgroups per compute unit
	groups = groups < 1 ? 1 : (groups > p.inBlocks ? p.inBlocks : groups);
	p.inBlocksPerGroup = (p.inBlocks + groups - 1) / groups;
	groups = (p.inBlocks + p.inBlocksPerGroup - 1) / p.inBlocksPerGroup;
	const bool vec = (out & 3) == 0 && (((uintptr_t)dW) & 15) == 0;
	const dim3 grid((unsigned)outBlocks, (unsigned)groups);
	LaunchScope scope(FITRE_KC_FC_GEMM, 2.0 * (double)in * out * n, 9);
	if (vec) {
		constexpr size_t ldsBytes = sizeof(float) * 128 * kSkinnyLd;
		static bool attributeSet = false;
		if (!attributeSet) {
			FITRE_HIP_TRY(hipFuncSetAttribute((const void *)fc_dw_skinny_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
			attributeSet = true;
		}
		fc_dw_skinny_kernel<true><<<grid, 256, ldsBytes, stream()>>>(p);
	} else {
		fc_dw_skinny_kernel<false><<<grid, 256, 0, stream()>>>(p);
	}
	return check_launch("fc_dw_skinny_kernel");
}

} // namespace fitre
