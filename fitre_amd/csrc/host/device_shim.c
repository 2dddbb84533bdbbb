/*
 * The reference's device-shim names (device/cuda_utils.c, device/cuda_environment.c,
 * device/query.c) implemented on the C-ABI device layer.  Failure behaviour is
 * the reference's: a message on stderr, then exit with the caller's code.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "fitre_hip.h"
#include "fitre_shim.h"

int BLOCK_SIZE = 1024;
int WARP_SIZE = 64;
int DEVICE_NUM_BLOCKS = 0;
int __THREADS_PER_SAMPLE__ = 1;

static void die(const char *what, int err_code)
{
	fprintf(stderr, "%s failed (res %d): %s\n", what, err_code, fitre_hip_last_error());
	exit(err_code);
}

void getDeviceParameters(void)
{
	int cus = 0, wave = 0, maxThreads = 0;
	size_t total = 0, freeb = 0;
	char name[128];
	if (fitre_hip_init(0)) die("fitre_hip_init", -1);
	if (fitre_hip_device_info(&cus, &wave, &maxThreads, &total, &freeb, name, sizeof(name)))
		die("fitre_hip_device_info", -1);
	BLOCK_SIZE = maxThreads;
	WARP_SIZE = wave;
	/* 2048 resident threads per compute unit, six waves of workgroups */
	DEVICE_NUM_BLOCKS = (cus * 2048 * 6) / (maxThreads > 0 ? maxThreads : 1);
	fprintf(stderr, "device: %s, compute units: %d, wavefront: %d, max threads per workgroup: %d\n", name, cus,
	        wave, maxThreads);
	fprintf(stderr, "ideal workgroup count: %d, sizeof(real): %zu\n", DEVICE_NUM_BLOCKS, sizeof(real));
}

void fitre_env_init(SCRATCH_AREA *scratch, int gpu, size_t hostBytes)
{
	if (fitre_hip_init(gpu)) die("fitre_hip_init", -1);
	if (hostBytes == 0) hostBytes = FITRE_DEFAULT_HOST_WORKSPACE;
	memset(scratch, 0, sizeof(*scratch));
	scratch->hostWorkspace = (real *)malloc(hostBytes);
	if (!scratch->hostWorkspace) {
		fprintf(stderr, "host workspace of %zu bytes could not be allocated\n", hostBytes);
		exit(ERROR_MEM_ALLOC);
	}
	scratch->nextHostPtr = scratch->hostWorkspace;
}

void cuda_env_init(SCRATCH_AREA *scratch, int gpu) { fitre_env_init(scratch, gpu, 0); }

void fitre_allocate_workspace(SCRATCH_AREA *scratch, size_t deviceBytes)
{
	cuda_malloc((void **)&scratch->devWorkspace, deviceBytes, 0, ERR_MEM_ALLOC);
	cuda_malloc_host((void **)&scratch->pageLckWorkspace, PAGE_LOCKED_WORKSPACE_SIZE, 0, ERR_MEM_ALLOC);
	scratch->nextDevPtr = scratch->devWorkspace;
	scratch->nextPageLckPtr = scratch->pageLckWorkspace;
}

void cuda_allocate_workspace(SCRATCH_AREA *scratch, int device)
{
	(void)device;
	size_t total = 0, freeb = 0;
	if (fitre_hip_device_info(NULL, NULL, NULL, &total, &freeb, NULL, 0)) die("fitre_hip_device_info", ERR_MEM_ALLOC);
	size_t reserve = (size_t)500 * 1024 * 1024;
	if (freeb <= reserve) {
		fprintf(stderr, "only %zu bytes of device memory are free\n", freeb);
		exit(ERR_MEM_ALLOC);
	}
	size_t bytes = freeb - reserve;
	fprintf(stderr, "device workspace size: %zu (MB)\n", bytes / (1024 * 1024));
	fitre_allocate_workspace(scratch, bytes);
}

void cuda_env_cleanup(SCRATCH_AREA *scratch)
{
	free(scratch->hostWorkspace);
	cuda_free((void *)scratch->devWorkspace, ERR_MEM_FREE);
	cuda_free_host((void *)scratch->pageLckWorkspace, ERR_MEM_FREE);
	memset(scratch, 0, sizeof(*scratch));
}

void cuda_malloc(void **ptr, size_t size, int zero, int err_code)
{
	if (fitre_hip_malloc(ptr, size)) die("device allocation", err_code);
	if (zero && (fitre_hip_memset(*ptr, 0, size) || fitre_hip_sync())) die("device memset", err_code);
}

void cuda_malloc_host(void **ptr, size_t size, int zero, int err_code)
{
	if (fitre_hip_malloc_host(ptr, size)) die("pinned allocation", err_code);
	if (zero) memset(*ptr, 0, size);
}

void cuda_free(void *ptr, int err_code)
{
	if (!ptr) return;
	if (fitre_hip_free(ptr)) fprintf(stderr, "device free failed (res %d): %s\n", err_code, fitre_hip_last_error());
}

void cuda_free_host(void *ptr, int err_code)
{
	if (!ptr) return;
	if (fitre_hip_free_host(ptr)) fprintf(stderr, "pinned free failed (res %d): %s\n", err_code, fitre_hip_last_error());
}

void cuda_memset(void *ptr, int value, size_t size, int err_code)
{
	if (fitre_hip_memset(ptr, value, size) || fitre_hip_sync()) die("device memset", err_code);
}

void copy_host_device(void *host, void *dev, size_t size, enum cudaMemcpyKind dir, int err_code)
{
	int rc;
	if (dir == cudaMemcpyHostToDevice)
		rc = fitre_hip_copy_h2d(dev, host, size);
	else if (dir == cudaMemcpyDeviceToHost)
		rc = fitre_hip_copy_d2h(host, dev, size);
	else {
		fprintf(stderr, "copy_host_device: unknown direction %d\n", (int)dir);
		exit(err_code);
	}
	if (rc) die("host/device copy", err_code);
}

void copy_device(void *dst, void *src, size_t size, int err_code)
{
	if (fitre_hip_copy_d2d(dst, src, size) || fitre_hip_sync()) die("device copy", err_code);
}

void print_device_mem_usage(void)
{
	size_t total = 0, freeb = 0;
	if (fitre_hip_device_info(NULL, NULL, NULL, &total, &freeb, NULL, 0)) die("fitre_hip_device_info", -1);
	fprintf(stderr, "device memory: used %zu MB, free %zu MB, total %zu MB\n", (total - freeb) >> 20, freeb >> 20,
	        total >> 20);
}

void getRandomVector(int n, real *hostPtr, real *devPtr, RAND_GENERATOR r)
{
	int rc = (r == RAND_NORMAL) ? fitre_hip_random_normal(devPtr, n) : fitre_hip_random_uniform(devPtr, n);
	if (rc) die("getRandomVector", -1);
	if (hostPtr != NULL && fitre_hip_copy_d2h(hostPtr, devPtr, sizeof(real) * (size_t)n)) die("getRandomVector: copy", -1);
	if (hostPtr == NULL && fitre_hip_sync()) die("getRandomVector: sync", -1);
}

void writeVector(real *mat, int rows, char *file, int hostData, real *dscratch)
{
	FILE *f = fopen(file, "w");
	real *t = dscratch;
	if (f == NULL) {
		fprintf(stderr, "Error opening the path .... !\n");
		exit(-1);
	}
	if (hostData == 1)
		t = mat;
	else if (fitre_hip_copy_d2h(t, mat, sizeof(real) * (size_t)rows))
		die("writeVector: copy", -1);
	for (int i = 0; i < rows; i++) fprintf(f, "%6.10f\n", t[i]);
	fclose(f);
}

int readVector(real *vec, int rows, char *file, int offset, real *dscratch)
{
	(void)dscratch;
	FILE *handle = fopen(file, "r");
	char line[1024];
	int index = 0;
	if (handle == NULL) {
		fprintf(stderr, "Error opening the path... \n");
		exit(-1);
	}
	while (index < rows && fgets(line, sizeof(line), handle) != NULL) {
		if (line[0] == 0 || line[0] == '\n') break;
		vec[index++] = (real)atof(line) + (real)offset;
	}
	fclose(handle);
	return index;
}
