/*
 * fitre_blas_compat.h -- the vendor BLAS names the reference's solvers call, as macros over the level-1 and GEMM entry
 * points of fitre_hip.h, so that solver sources such as solvers/cg_steihaug.c:87-177 or
 * solvers/kfac_trust_region.cu:364-366 compile against this library unchanged.
 *
 * The handle argument is accepted and ignored (the device layer owns its streams); increments must be 1, as they are
 * at every call site of the reference.  Results of dot / nrm2 / asum are written to host memory and are complete on
 * return, which is what the solvers' reads of their pinned scalars expect.  `real` is float, so the D-names map to
 * the float entry points.
 */
#ifndef FITRE_BLAS_COMPAT_H
#define FITRE_BLAS_COMPAT_H

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include "fitre_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* device/handles.h:13-18: the globals the solvers pass around; opaque here */
#ifndef FITRE_VENDOR_HANDLES_DEFINED
#define FITRE_VENDOR_HANDLES_DEFINED
typedef void *cublasHandle_t;
typedef void *cudaStream_t;
typedef void *cusolverDnHandle_t;
#endif
typedef void *cusparseHandle_t;
typedef void *curandGenerator_t;
extern cublasHandle_t cublasHandle;
extern cusparseHandle_t cusparseHandle;
extern cusolverDnHandle_t cusolverHandle;
extern curandGenerator_t curandGeneratorHandle;

typedef enum { CUBLAS_OP_N = 0, CUBLAS_OP_T = 1 } cublasOperation_t;

/* device/cuda_utils.h:28-31 (cublasCheckError / cudaCheckError / ...): message on stderr and exit, as there */
static inline void fitre_check_status(int rc, const char *file, int line)
{
	if (rc != FITRE_OK) {
		fprintf(stderr, "%s:%d: device call failed with code %d: %s\n", file, line, rc, fitre_hip_last_error());
		exit(-1);
	}
}
#define cublasCheckError(x) fitre_check_status((x), __FILE__, __LINE__)
#define cudaCheckError() fitre_check_status(fitre_hip_sync(), __FILE__, __LINE__)
#define cudaDeviceSynchronize() fitre_hip_sync()
#define cudaThreadSynchronize() fitre_hip_sync()

#define cublasDaxpy(h, n, alpha, x, incx, y, incy) fitre_hip_axpy((n), *(alpha), (x), (y))
#define cublasDscal(h, n, alpha, x, incx) fitre_hip_scal((n), *(alpha), (x))
#define cublasDcopy(h, n, x, incx, y, incy) fitre_hip_copy((n), (x), (y))
#define cublasDdot(h, n, x, incx, y, incy, result) fitre_hip_dot((n), (x), (y), (result))
#define cublasDnrm2(h, n, x, incx, result) fitre_hip_nrm2((n), (x), (result))
#define cublasDasum(h, n, x, incx, result) fitre_hip_asum((n), (x), (result))
#define cublasDgeam(h, ta, tb, m, n, alpha, A, lda, beta, B, ldb, C, ldc)                                               \
	fitre_hip_geam((ta) != CUBLAS_OP_N, (tb) != CUBLAS_OP_N, (m), (n), *(alpha), (A), (lda), *(beta), (B), (ldb), (C), (ldc))
/* The products need a workspace, which cuBLAS hides: the caller sets fitre_blas_workspace / fitre_blas_workspace_bytes
 * (device memory, 256-byte aligned, fitre_hip_gemm_workspace(M, N, K) bytes for the largest product) once. */
extern void *fitre_blas_workspace;
extern size_t fitre_blas_workspace_bytes;
#define cublasDgemm(h, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)                                            \
	fitre_hip_gemm((ta) != CUBLAS_OP_N, (tb) != CUBLAS_OP_N, (m), (n), (k), *(alpha), (A), (lda), (B), (ldb), *(beta), (C),    \
	               (ldc), NULL, fitre_blas_workspace, fitre_blas_workspace_bytes)

#ifdef __cplusplus
}
#endif
#endif
