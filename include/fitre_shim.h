/*
 * fitre_shim.h -- the reference's device-shim names on top of fitre_hip.h, so
 * that its solver and driver sources build against this library unchanged.
 *
 * Same names, argument order and failure behaviour (message on stderr, then
 * exit with the given error code) as device/cuda_utils.h:15-26,
 * device/cuda_environment.h:6-9, device/query.h and the globals of
 * drivers/main_driver.c:52-60.  The four vendor-library handles of
 * device/handles.h have no counterpart: the device layer owns its stream.
 */
#ifndef FITRE_SHIM_H
#define FITRE_SHIM_H

#include "fitre_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* direction argument of copy_host_device, with the values the reference's
 * call sites spell out */
enum cudaMemcpyKind { cudaMemcpyHostToDevice = 1, cudaMemcpyDeviceToHost = 2 };

extern int BLOCK_SIZE;              /* max threads per workgroup (1024) */
extern int WARP_SIZE;               /* wavefront size (64) */
extern int DEVICE_NUM_BLOCKS;       /* workgroups that fill the device six times over */
extern int __THREADS_PER_SAMPLE__;

void getDeviceParameters(void);

/* hostBytes of host arena (the reference fixes 12 GiB); 0 selects the default */
void fitre_env_init(SCRATCH_AREA *scratch, int gpu, size_t hostBytes);
void cuda_env_init(SCRATCH_AREA *scratch, int gpu);
/* device arena = free memory - 500 MiB, plus the 1 MiB pinned arena */
void cuda_allocate_workspace(SCRATCH_AREA *scratch, int device);
/* device arena of a chosen size (no counterpart in the reference) */
void fitre_allocate_workspace(SCRATCH_AREA *scratch, size_t deviceBytes);
void cuda_env_cleanup(SCRATCH_AREA *scratch);

void cuda_malloc(void **ptr, size_t size, int zero, int err_code);
void cuda_malloc_host(void **ptr, size_t size, int zero, int err_code);
void cuda_free(void *ptr, int err_code);
void cuda_free_host(void *ptr, int err_code);
void cuda_memset(void *ptr, int value, size_t size, int err_code);
void copy_host_device(void *host, void *dev, size_t size, enum cudaMemcpyKind dir, int err_code);
void copy_device(void *dst, void *src, size_t size, int err_code);
void print_device_mem_usage(void);

/* utilities/print_utils.c:136-186: one value per line, "%6.10f".  writeVector: hostData == 1 writes the
 * host vector mat; otherwise mat is a device vector and dscratch a host buffer of at least rows reals.
 * readVector: reads up to rows values into the HOST vector vec, adds offset to each, returns the count
 * (the format of the <net>_<init>.params files, e.g. pytorch/kfac/lenet_xavier.txt). */
void writeVector(real *mat, int rows, char *file, int hostData, real *dscratch);
int readVector(real *vec, int rows, char *file, int offset, real *dscratch);

/* device/gen_random.h:6-13: n standard-normal or uniform (0, 1] reals into devPtr, copied to hostPtr
 * when it is not NULL.  The stream is seeded with fitre_hip_random_seed(). */
typedef enum random_generator { RAND_NORMAL = 1, RAND_UNIFORM } RAND_GENERATOR;
void getRandomVector(int n, real *hostPtr, real *devPtr, RAND_GENERATOR r);

#ifdef __cplusplus
}
#endif
#endif
