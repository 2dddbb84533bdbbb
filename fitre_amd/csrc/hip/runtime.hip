// Environment, memory and timing entry points of the device layer.
// Replaces device/cuda_environment.c, device/cuda_utils.c and device/query.c
// of the reference (handles become four streams -- "lanes" -- owned by this file:
// everything is queued on the selected lane, lane 0 unless a caller overlaps
// independent work on the others).
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "common.h"

namespace fitre {

static thread_local char g_error[512] = "";
constexpr int kLanes = kMaxLanes;
static hipStream_t g_lanes[kLanes] = {};
static hipStream_t g_stream = nullptr; // the selected lane
static int g_lane = 0;
static bool g_lanes_on = true;
// Compute units a kernel launched on each lane can occupy.  Lane 1 can be created with a
// compute-unit mask that leaves a share of every XCD free (FITRE_LANE1_CUS), so that work on
// lane 0 always finds idle compute units while a chip-filling kernel runs on lane 1; the
// planners size their grids for the lane's share.  Off unless asked for: on the gradient path
// it measured within noise of two unmasked lanes.
static int g_lane_cus[kLanes] = { 256, 256, 256, 256 };
static int g_dw_eighths = 8; // share of the compute units the 3 x 3 weight gradients are planned for
constexpr int kJoinEvents = 64;
static hipEvent_t g_join[kJoinEvents];
static int g_join_next = 0;
static bool g_ready = false;
static int g_device = -1;

// accounting state
struct ClassTotals {
	long launches;
	double ms;
	double work;
};
static bool g_profile = false;
static ClassTotals g_totals[FITRE_KC_COUNT][FITRE_TILE_VARIANTS];
struct Pending {
	hipEvent_t start, stop;
	int cls, tile;
	double work;
};
// every accounted launch in issue order, for per-launch figures (bounded: the oldest are kept)
struct LaunchRecord {
	int cls, tile;
	double work, ms;
};
constexpr size_t kMaxLaunchRecords = 1 << 16;
static std::vector<LaunchRecord> g_records;
static std::vector<Pending> g_pending;
static std::vector<hipEvent_t> g_event_pool;

void set_error(const char *fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
}

int fail(int code, const char *fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
	return code;
}

hipStream_t stream() { return g_stream; }
int lane() { return g_lane; }
int lane_compute_units() { return g_lane_cus[g_lane]; }
int lane_compute_units_min()
{
	int m = g_lane_cus[0];
	for (int i = 1; i < kLanes; i++) m = g_lane_cus[i] < m ? g_lane_cus[i] : m;
	return m;
}
int device_compute_units() { return g_lane_cus[0]; }
int share_of_units(int cus, int eighths)
{
	const int share = (cus * eighths / 8) & ~7;
	return share >= 8 ? share : cus;
}
int weight_grad_units() { return g_dw_eighths < 8 ? share_of_units(g_lane_cus[g_lane], g_dw_eighths) : g_lane_cus[g_lane]; }
bool ready() { return g_ready; }
int current_device() { return g_ready ? g_device : -1; }

int check_launch(const char *what)
{
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) return fail(FITRE_E_DEVICE, "launch of %s failed: %s", what, hipGetErrorString(e));
	return FITRE_OK;
}

static hipEvent_t take_event()
{
	if (!g_event_pool.empty()) {
		hipEvent_t e = g_event_pool.back();
		g_event_pool.pop_back();
		return e;
	}
	hipEvent_t e = nullptr;
	if (hipEventCreate(&e) != hipSuccess) return nullptr;
	return e;
}

static void drain_pending()
{
	for (Pending &p : g_pending) {
		float ms = 0.f;
		if (hipEventSynchronize(p.stop) == hipSuccess && hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
			g_totals[p.cls][p.tile].ms += ms;
			if (g_records.size() < kMaxLaunchRecords) g_records.push_back({ p.cls, p.tile, p.work, (double)ms });
		}
		g_event_pool.push_back(p.start);
		g_event_pool.push_back(p.stop);
	}
	g_pending.clear();
}

LaunchScope::LaunchScope(int kernelClass, double work, int tile) : slot(-1)
{
	if (!g_profile || kernelClass < 0 || kernelClass >= FITRE_KC_COUNT || tile < 0 || tile >= FITRE_TILE_VARIANTS) return;
	Pending p;
	p.start = take_event();
	p.stop = take_event();
	p.cls = kernelClass;
	p.tile = tile;
	p.work = work;
	if (!p.start || !p.stop) return;
	g_totals[kernelClass][tile].launches += 1;
	g_totals[kernelClass][tile].work += work;
	(void)hipEventRecord(p.start, g_stream);
	g_pending.push_back(p);
	slot = (int)g_pending.size() - 1;
}

LaunchScope::~LaunchScope()
{
	if (slot < 0) return;
	(void)hipEventRecord(g_pending[slot].stop, g_stream);
	if (g_pending.size() >= 2048) drain_pending();
}

// Plain device-to-device copy as a kernel: cheaper to queue than a runtime copy for the small
// tensors of a pass.
__global__ void copy_bytes_kernel(unsigned char *dst, const unsigned char *src, size_t n, int wide)
{
	const size_t stride = (size_t)gridDim.x * blockDim.x;
	const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	size_t done = 0;
	if (wide) {
		const size_t words = n / 16;
		const uint4 *s16 = reinterpret_cast<const uint4 *>(src);
		uint4 *d16 = reinterpret_cast<uint4 *>(dst);
		for (size_t i = first; i < words; i += stride) d16[i] = s16[i];
		done = words * 16;
	}
	for (size_t i = done + first; i < n; i += stride) dst[i] = src[i];
}

// Byte fill as a kernel: a memset node recorded into a captured graph is not
// reliable on this platform, a kernel node is.
__global__ void fill_bytes_kernel(unsigned char *p, unsigned char v, size_t n)
{
	size_t words = n / 16;
	uint4 *p16 = reinterpret_cast<uint4 *>(p);
	unsigned w = v * 0x01010101u;
	size_t stride = (size_t)gridDim.x * blockDim.x;
	for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride)
		p16[i] = make_uint4(w, w, w, w);
	for (size_t i = words * 16 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = v;
}

} // namespace fitre

using namespace fitre;

extern "C" {

int fitre_hip_init(int device)
{
	int count = 0;
	FITRE_HIP_TRY(hipGetDeviceCount(&count));
	if (device < 0 || device >= count)
		return fail(FITRE_E_ARGUMENT, "fitre_hip_init: device %d out of range (%d visible)", device, count);
	FITRE_HIP_TRY(hipSetDevice(device));
	if (g_ready && g_device == device) return FITRE_OK;
	if (g_ready) fitre_hip_shutdown();
	if (int rc = layers_device_setup(device)) return rc;
	int cus = 0;
	FITRE_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
	if (cus <= 0 || cus > 1024) return fail(FITRE_E_DEVICE, "fitre_hip_init: device reports %d compute units", cus);
	for (int i = 0; i < kLanes; i++) {
		FITRE_HIP_TRY(hipStreamCreate(&g_lanes[i])); // default priority
		g_lane_cus[i] = cus;
	}
	for (int i = 0; i < kJoinEvents; i++) FITRE_HIP_TRY(hipEventCreateWithFlags(&g_join[i], hipEventDisableTiming));
	g_join_next = 0;
	g_stream = g_lanes[0];
	g_lane = 0;
	g_device = device;
	g_ready = true;
	memset(g_totals, 0, sizeof(g_totals));
	return FITRE_OK;
}

int fitre_hip_shutdown(void)
{
	if (!g_ready) return FITRE_OK;
	for (int i = 0; i < kLanes; i++) (void)hipStreamSynchronize(g_lanes[i]);
	drain_pending();
	layers_release();
	elementwise_release();
	conv_gemm_release();
	for (hipEvent_t e : g_event_pool) (void)hipEventDestroy(e);
	g_event_pool.clear();
	for (int i = 0; i < kJoinEvents; i++) (void)hipEventDestroy(g_join[i]);
	for (int i = 0; i < kLanes; i++) {
		(void)hipStreamDestroy(g_lanes[i]);
		g_lanes[i] = nullptr;
	}
	g_stream = nullptr;
	g_ready = false;
	g_profile = false;
	return FITRE_OK;
}

int fitre_hip_sync(void)
{
	FITRE_NEED_INIT();
	for (int i = 0; i < kLanes; i++) FITRE_HIP_TRY(hipStreamSynchronize(g_lanes[i]));
	return FITRE_OK;
}

int fitre_hip_lane_select(int laneIndex)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(laneIndex >= 0 && laneIndex < kLanes, "fitre_hip_lane_select: lane %d out of range", laneIndex);
	// with per-launch accounting on, everything runs on lane 0 so that durations are not shared
	g_lane = (g_profile || !g_lanes_on) ? 0 : laneIndex;
	g_stream = g_lanes[g_lane];
	return FITRE_OK;
}

int fitre_hip_lanes_enable(int on)
{
	FITRE_NEED_INIT();
	for (int i = 0; i < kLanes; i++) FITRE_HIP_TRY(hipStreamSynchronize(g_lanes[i]));
	g_lanes_on = (on != 0);
	g_lane = 0;
	g_stream = g_lanes[0];
	return FITRE_OK;
}

int fitre_hip_weight_grad_share(int eighths)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(eighths >= 4 && eighths <= 8, "fitre_hip_weight_grad_share: %d eighths (4 to 8)", eighths);
	g_dw_eighths = eighths;
	return FITRE_OK;
}

int fitre_hip_lane_wait(int waiter, int signaller)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(waiter >= 0 && waiter < kLanes && signaller >= 0 && signaller < kLanes,
	              "fitre_hip_lane_wait: lane out of range (%d waits for %d)", waiter, signaller);
	if (waiter == signaller) return FITRE_OK;
	if (g_profile || !g_lanes_on) return FITRE_OK; // everything is queued on lane 0: already in order
	hipEvent_t e = g_join[g_join_next];
	g_join_next = (g_join_next + 1) % kJoinEvents;
	FITRE_HIP_TRY(hipEventRecord(e, g_lanes[signaller]));
	FITRE_HIP_TRY(hipStreamWaitEvent(g_lanes[waiter], e, 0));
	return FITRE_OK;
}

const char *fitre_hip_last_error(void) { return g_error; }

void *fitre_hip_stream(void) { return (void *)g_stream; }

int fitre_hip_device_info(int *computeUnits, int *waveSize, int *maxThreadsPerBlock, size_t *totalBytes,
                          size_t *freeBytes, char *name, int nameLen)
{
	FITRE_NEED_INIT();
	hipDeviceProp_t prop;
	FITRE_HIP_TRY(hipGetDeviceProperties(&prop, g_device));
	if (computeUnits) *computeUnits = prop.multiProcessorCount;
	if (waveSize) *waveSize = prop.warpSize;
	if (maxThreadsPerBlock) *maxThreadsPerBlock = prop.maxThreadsPerBlock;
	size_t fr = 0, tot = 0;
	FITRE_HIP_TRY(hipMemGetInfo(&fr, &tot));
	if (totalBytes) *totalBytes = tot;
	if (freeBytes) *freeBytes = fr;
	if (name && nameLen > 0) {
		snprintf(name, (size_t)nameLen, "%s (%s)", prop.name, prop.gcnArchName);
	}
	return FITRE_OK;
}

int fitre_hip_malloc(void **ptr, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(ptr != nullptr, "fitre_hip_malloc: null result pointer");
	FITRE_REQUIRE(bytes > 0, "fitre_hip_malloc: zero bytes requested");
	FITRE_HIP_TRY(hipMalloc(ptr, bytes));
	return FITRE_OK;
}

int fitre_hip_free(void *ptr)
{
	FITRE_NEED_INIT();
	if (!ptr) return FITRE_OK;
	for (int i = 0; i < kLanes; i++) FITRE_HIP_TRY(hipStreamSynchronize(g_lanes[i]));
	FITRE_HIP_TRY(hipFree(ptr));
	return FITRE_OK;
}

int fitre_hip_malloc_host(void **ptr, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(ptr != nullptr, "fitre_hip_malloc_host: null result pointer");
	FITRE_REQUIRE(bytes > 0, "fitre_hip_malloc_host: zero bytes requested");
	FITRE_HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
	return FITRE_OK;
}

int fitre_hip_free_host(void *ptr)
{
	FITRE_NEED_INIT();
	if (!ptr) return FITRE_OK;
	for (int i = 0; i < kLanes; i++) FITRE_HIP_TRY(hipStreamSynchronize(g_lanes[i]));
	FITRE_HIP_TRY(hipHostFree(ptr));
	return FITRE_OK;
}

int fitre_hip_memset(void *ptr, int value, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(ptr != nullptr, "fitre_hip_memset: null pointer");
	if (bytes == 0) return FITRE_OK;
	unsigned char *p = (unsigned char *)ptr;
	// head up to 16-byte alignment, then the aligned body
	size_t head = (16 - ((uintptr_t)p & 15)) & 15;
	if (head > bytes) head = bytes;
	if (head) {
		fill_bytes_kernel<<<1, 64, 0, g_stream>>>(p, (unsigned char)value, head);
		p += head;
		bytes -= head;
	}
	if (bytes) {
		unsigned blocks = blocks_for((long)(bytes / 16 + 1), 256, 4096);
		fill_bytes_kernel<<<blocks, 256, 0, g_stream>>>(p, (unsigned char)value, bytes);
	}
	return check_launch("fill_bytes_kernel");
}

int fitre_hip_copy_h2d(void *dev, const void *host, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(dev && host, "fitre_hip_copy_h2d: null pointer");
	if (bytes == 0) return FITRE_OK;
	FITRE_HIP_TRY(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, g_stream));
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	return FITRE_OK;
}

int fitre_hip_copy_d2h(void *host, const void *dev, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(dev && host, "fitre_hip_copy_d2h: null pointer");
	if (bytes == 0) return FITRE_OK;
	FITRE_HIP_TRY(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, g_stream));
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	return FITRE_OK;
}

int fitre_hip_copy_d2d(void *dst, const void *src, size_t bytes)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(dst && src, "fitre_hip_copy_d2d: null pointer");
	if (bytes == 0 || dst == src) return FITRE_OK;
	if (bytes <= ((size_t)4 << 20)) {
		const int wide = (((uintptr_t)dst | (uintptr_t)src) & 15) == 0;
		unsigned blocks = blocks_for((long)(bytes / 16 + 1), 256, 4096);
		copy_bytes_kernel<<<blocks, 256, 0, g_stream>>>((unsigned char *)dst, (const unsigned char *)src, bytes, wide);
		return check_launch("copy_bytes_kernel");
	}
	FITRE_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
	return FITRE_OK;
}

int fitre_hip_event_create(void **event)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(event != nullptr, "fitre_hip_event_create: null result pointer");
	hipEvent_t e;
	FITRE_HIP_TRY(hipEventCreate(&e));
	*event = (void *)e;
	return FITRE_OK;
}

int fitre_hip_event_destroy(void *event)
{
	FITRE_NEED_INIT();
	if (!event) return FITRE_OK;
	FITRE_HIP_TRY(hipEventDestroy((hipEvent_t)event));
	return FITRE_OK;
}

int fitre_hip_event_record(void *event)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(event != nullptr, "fitre_hip_event_record: null event");
	FITRE_HIP_TRY(hipEventRecord((hipEvent_t)event, g_stream));
	return FITRE_OK;
}

int fitre_hip_event_elapsed_ms(void *start, void *stop, float *ms)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(start && stop && ms, "fitre_hip_event_elapsed_ms: null argument");
	FITRE_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
	FITRE_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
	return FITRE_OK;
}

int fitre_hip_profile_enable(int on)
{
	FITRE_NEED_INIT();
	for (int i = 0; i < kLanes; i++) FITRE_HIP_TRY(hipStreamSynchronize(g_lanes[i]));
	drain_pending();
	if (on) {
		memset(g_totals, 0, sizeof(g_totals));
		g_records.clear();
	}
	g_profile = (on != 0);
	if (g_profile) {
		g_lane = 0;
		g_stream = g_lanes[0];
	}
	return FITRE_OK;
}

int fitre_hip_profile_read(int kernelClass, long *launches, double *milliseconds, double *work)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(kernelClass >= 0 && kernelClass < FITRE_KC_COUNT, "fitre_hip_profile_read: class %d unknown", kernelClass);
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	drain_pending();
	long n = 0;
	double ms = 0.0, wk = 0.0;
	for (int t = 0; t < FITRE_TILE_VARIANTS; t++) {
		n += g_totals[kernelClass][t].launches;
		ms += g_totals[kernelClass][t].ms;
		wk += g_totals[kernelClass][t].work;
	}
	if (launches) *launches = n;
	if (milliseconds) *milliseconds = ms;
	if (work) *work = wk;
	return FITRE_OK;
}

int fitre_hip_profile_read_tile(int kernelClass, int tile, long *launches, double *milliseconds, double *work)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(kernelClass >= 0 && kernelClass < FITRE_KC_COUNT && tile >= 0 && tile < FITRE_TILE_VARIANTS,
	              "fitre_hip_profile_read_tile: class %d / tile %d unknown", kernelClass, tile);
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	drain_pending();
	if (launches) *launches = g_totals[kernelClass][tile].launches;
	if (milliseconds) *milliseconds = g_totals[kernelClass][tile].ms;
	if (work) *work = g_totals[kernelClass][tile].work;
	return FITRE_OK;
}

int fitre_hip_profile_launch_count(long *count)
{
	FITRE_NEED_INIT();
	FITRE_REQUIRE(count != nullptr, "fitre_hip_profile_launch_count: null result pointer");
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	drain_pending();
	*count = (long)g_records.size();
	return FITRE_OK;
}

int fitre_hip_profile_read_launch(long index, int *kernelClass, int *tile, double *milliseconds, double *work)
{
	FITRE_NEED_INIT();
	FITRE_HIP_TRY(hipStreamSynchronize(g_stream));
	drain_pending();
	FITRE_REQUIRE(index >= 0 && (size_t)index < g_records.size(), "fitre_hip_profile_read_launch: index %ld of %zu records", index,
	              g_records.size());
	const LaunchRecord &r = g_records[(size_t)index];
	if (kernelClass) *kernelClass = r.cls;
	if (tile) *tile = r.tile;
	if (milliseconds) *milliseconds = r.ms;
	if (work) *work = r.work;
	return FITRE_OK;
}

} // extern "C"
