/* A caller written the way the reference's solvers are: the reference's include paths and its vendor-BLAS spelling
 * (the pattern of solvers/kfac_trust_region.cu:352-366 -- gradient, then axpy / dot / nrm2 on the result), resolved by
 * include/compat and include/fitre_blas_compat.h.  Compiled and linked by tests/test_compat_headers.py. */
#include <core/datadefs.h>
#include <core/structdefs.h>
#include <core/errors.h>
#include <nn/nn_decl.h>
#include <device/device_defines.h>
#include <device/cuda_utils.h>
#include <device/handles.h>
#include <functions/cnn_gradient.h>
#include <functions/cnn_forward.h>
#include <functions/cnn_backward.h>
#include <solvers/kfac_structs.h>
#include <solvers/kfac_inverses.h>
#include <solvers/kfac_natural_gradient.h>

cublasHandle_t cublasHandle;
cusparseHandle_t cusparseHandle;
cusolverDnHandle_t cusolverHandle;
curandGenerator_t curandGeneratorHandle;
void *fitre_blas_workspace;
size_t fitre_blas_workspace_bytes;

real gradient_step(CNN_MODEL *model, DEVICE_DATASET *data, SCRATCH_AREA *scratch, real *z, real *dx, real *probs, real *errors,
                   real *gradient, real *weights, real stepSize)
{
	real alpha = -stepSize, norm = 0, dot = 0;
	real loss = computeCNNGradient(model, data, scratch, z, dx, probs, errors, gradient, 0, model->batchSize, 0);
	cublasCheckError(cublasDnrm2(cublasHandle, model->pSize, gradient, 1, &norm));
	cublasCheckError(cublasDdot(cublasHandle, model->pSize, gradient, 1, weights, 1, &dot));
	cublasCheckError(cublasDaxpy(cublasHandle, model->pSize, &alpha, gradient, 1, weights, 1));
	cublasCheckError(cublasDscal(cublasHandle, model->pSize, &alpha, gradient, 1));
	cuda_memset(errors, 0, sizeof(real) * 16, ERROR_MEMSET);
	return loss + norm + dot;
}

int main(void)
{
	return sizeof(KFAC_CURVATURE_INFO) > 0 && BLOCK_SIZE >= 0 ? 0 : 1; /* never touches a device */
}
