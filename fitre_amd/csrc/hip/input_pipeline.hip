// Mini-batch selection and augmentation on the device.
// Replaces device/extract_columns.cu and augmentation/dev_crop.cu, dev_flip.cu, dev_normalize.cu of the
// reference, which run one pass over the batch per step (layout change, crop, flip, normalise); here one
// gather kernel produces the layer-0 input from the selected columns in a single pass: every output cell
// computes where it comes from.
#include "common.h"

namespace fitre {

constexpr int kMaxImageChannels = 8;

struct GatherParams {
	int samples, channels, width, height; // A = width (columns), B = height (rows, fastest)
	int sampleMajor;                      // source is [N][C][cells] (else [C][N][cells])
	int padding;                          // crop: shifts in [-padding, padding]; < 0: no crop
	float fill;                           // value of cells the shift moves in from outside
	int normalise;
	float scale;                          // pixel scale (255)
	float mean[kMaxImageChannels], stdv[kMaxImageChannels];
};

// uniform in (0, 1] -> shift in [-padding, padding]   (ker_convert, augmentation/dev_crop.cu:52-58)
__device__ __forceinline__ int crop_shift(float u, int padding)
{
	return (int)((double)u * 100.) % (2 * padding + 1) - padding;
}

// out[c][n][col][row].  cropUniforms: row shifts of the samples, then their column shifts (or null);
// flipUniforms: an image with a value below one half is mirrored along the column axis (or null).
__global__ void __launch_bounds__(256)
image_gather_kernel(const float *src, GatherParams p, const float *cropUniforms, const float *flipUniforms, float *out)
{
	const int cells = p.width * p.height;
	const long total = (long)p.channels * p.samples * cells;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		const int cell = (int)(i % cells);
		const long map = i / cells;
		const int n = (int)(map % p.samples), c = (int)(map / p.samples);
		int row = cell % p.height, col = cell / p.height;
		if (flipUniforms && flipUniforms[n] < 0.5f) col = p.width - 1 - col;
		bool inside = true;
		if (cropUniforms) {
			row += crop_shift(cropUniforms[n], p.padding);
			col += crop_shift(cropUniforms[p.samples + n], p.padding);
			inside = row >= 0 && col >= 0 && row < p.height && col < p.width;
		}
		float v = p.fill;
		if (inside) {
			const size_t image = p.sampleMajor ? ((size_t)n * p.channels + c) : ((size_t)c * p.samples + n);
			v = src[image * cells + (size_t)col * p.height + row];
		}
		if (p.normalise) {
			v /= p.scale;
			v = (v - p.mean[c]) / p.stdv[c];
		}
		out[i] = v;
	}
}

// crop with shifts that are already integers (randomCrop's second kernel on its own)
__global__ void __launch_bounds__(256)
image_shift_kernel(const float *src, int samples, int channels, int width, int height, const int *shiftRow, const int *shiftCol,
                   float fill, float *out)
{
	const int cells = width * height;
	const long total = (long)channels * samples * cells;
	const long stride = (long)gridDim.x * blockDim.x;
	for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		const int cell = (int)(i % cells);
		const long map = i / cells;
		const int n = (int)(map % samples);
		const int row = cell % height + shiftRow[n], col = cell / height + shiftCol[n];
		float v = fill;
		if (row >= 0 && col >= 0 && row < height && col < width) v = src[map * cells + (size_t)col * height + row];
		out[i] = v;
	}
}

__global__ void __launch_bounds__(256) crop_shift_kernel(const float *uniforms, int count, int padding, int *shifts)
{
	int i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < count) shifts[i] = crop_shift(uniforms[i], padding);
}

// tgt column j = src column indices[j]; columns of `rows` values
template <typename T>
__global__ void __launch_bounds__(256) extract_columns_kernel(T *tgt, const T *src, const int *indices, int rows, long numElements)
{
	const long stride = (long)gridDim.x * blockDim.x;
	for (long j = (long)blockIdx.x * blockDim.x + threadIdx.x; j < numElements; j += stride) {
		const long colId = j / rows;
		const int rowId = (int)(j - colId * rows);
		tgt[j] = src[(size_t)indices[colId] * rows + rowId];
	}
}

static int fill_params(const char *fn, GatherParams &p, int samples, int channels, int height, int width, const float *mean,
                       const float *stdv, float scale)
{
	FITRE_REQUIRE(samples > 0 && channels > 0 && height > 0 && width > 0, "%s: non-positive shape (N=%d C=%d H=%d W=%d)", fn, samples,
	              channels, height, width);
	FITRE_REQUIRE((double)samples * channels * height * width < 2147483647.0, "%s: batch exceeds 2^31 elements", fn);
	p.samples = samples, p.channels = channels, p.width = width, p.height = height;
	p.normalise = (mean && stdv) ? 1 : 0;
	p.scale = scale;
	if (p.normalise) {
		FITRE_REQUIRE(channels <= kMaxImageChannels, "%s: normalisation of %d channels (at most %d)", fn, channels, kMaxImageChannels);
		FITRE_REQUIRE(scale != 0.f, "%s: pixel scale is zero", fn);
		for (int c = 0; c < channels; c++) {
			FITRE_REQUIRE(stdv[c] != 0.f, "%s: standard deviation of channel %d is zero", fn, c);
			p.mean[c] = mean[c], p.stdv[c] = stdv[c];
		}
	}
	return FITRE_OK;
}

} // namespace fitre

using namespace fitre;

extern "C" {

int fitre_hip_extract_columns(float *tgt, const float *src, const int *indices, int rows, int columns)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(tgt && src && indices, "fitre_hip_extract_columns: null pointer");
	FITRE_REQUIRE(rows > 0 && columns >= 0, "fitre_hip_extract_columns: bad shape (%d rows, %d columns)", rows, columns);
	if (columns == 0) return FITRE_OK;
	const long n = (long)rows * columns;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * (double)n);
	extract_columns_kernel<float><<<blocks_for(n, 256, 8192), 256, 0, stream()>>>(tgt, src, indices, rows, n);
	return check_launch("extract_columns_kernel");
}

int fitre_hip_augment_batch(const float *sampled, int sampleMajor, int samples, int channels, int height, int width,
                            const float *cropUniforms, int padding, float fill, const float *flipUniforms, const float *mean,
                            const float *stdv, float scale, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(sampled && out, "fitre_hip_augment_batch: null pointer");
	FITRE_REQUIRE(sampled != out || (!sampleMajor && !cropUniforms && !flipUniforms),
	              "fitre_hip_augment_batch: only the normalisation alone can run in place");
	FITRE_REQUIRE(!cropUniforms || padding >= 0, "fitre_hip_augment_batch: negative crop padding %d", padding);
	GatherParams p;
	int rc = fill_params("fitre_hip_augment_batch", p, samples, channels, height, width, mean, stdv, scale);
	if (rc) return rc;
	p.sampleMajor = sampleMajor ? 1 : 0;
	p.padding = padding;
	p.fill = fill;
	const long n = (long)samples * channels * height * width;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * (double)n);
	image_gather_kernel<<<blocks_for(n, 256, 8192), 256, 0, stream()>>>(sampled, p, cropUniforms, flipUniforms, out);
	return check_launch("image_gather_kernel");
}

int fitre_hip_crop_shifts(const float *uniforms, int count, int padding, int *shifts)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(uniforms && shifts, "fitre_hip_crop_shifts: null pointer");
	FITRE_REQUIRE(count > 0 && padding >= 0, "fitre_hip_crop_shifts: bad arguments (count %d, padding %d)", count, padding);
	crop_shift_kernel<<<blocks_for(count, 256), 256, 0, stream()>>>(uniforms, count, padding, shifts);
	return check_launch("crop_shift_kernel");
}

int fitre_hip_shift_images(const float *in, int samples, int channels, int height, int width, const int *shiftRow,
                           const int *shiftCol, float fill, float *out)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(in && out && shiftRow && shiftCol, "fitre_hip_shift_images: null pointer");
	FITRE_REQUIRE(in != out, "fitre_hip_shift_images: the batch cannot be rewritten in place");
	GatherParams p;
	int rc = fill_params("fitre_hip_shift_images", p, samples, channels, height, width, nullptr, nullptr, 1.f);
	if (rc) return rc;
	const long n = (long)samples * channels * height * width;
	LaunchScope scope(FITRE_KC_PERMUTE, 8.0 * (double)n);
	image_shift_kernel<<<blocks_for(n, 256, 8192), 256, 0, stream()>>>(in, samples, channels, width, height, shiftRow, shiftCol, fill, out);
	return check_launch("image_shift_kernel");
}

} // extern "C"
