"""Loads the two in-tree shared libraries and declares their C-ABI to ctypes.

There is no fallback: if a library is missing or a symbol is not exported the
import fails with the reason.  Build with ``python -m fitre_amd.build``.
"""
import ctypes as C
import os

from .structs import (CNN_MODEL, CONV_LAYER, DEVICE_DATASET, KFAC_CURVATURE_INFO, NN_MODEL, POOL_LAYER, SCRATCH_AREA,
                      fitre_conv_shape, fitre_matrix)

_PKG = os.path.dirname(os.path.abspath(__file__))
HIP_LIB_PATH = os.path.join(_PKG, "libfitre_hip.so")
CNN_LIB_PATH = os.path.join(_PKG, "libfitre_cnn.so")

vp, i32, f32, lng, sz = C.c_void_p, C.c_int, C.c_float, C.c_long, C.c_size_t
pvp, pi32, pf32 = C.POINTER(C.c_void_p), C.POINTER(C.c_int), C.POINTER(C.c_float)
pshape = C.POINTER(fitre_conv_shape)
pmodel, pdata, pscratch = C.POINTER(CNN_MODEL), C.POINTER(DEVICE_DATASET), C.POINTER(SCRATCH_AREA)
pkfac = C.POINTER(KFAC_CURVATURE_INFO)
pnn = C.POINTER(NN_MODEL)
f64, pmat = C.c_double, C.POINTER(fitre_matrix)

# name -> (restype, argtypes); mirrors include/fitre_hip.h
HIP_API = {
    "fitre_hip_init": (i32, [i32]),
    "fitre_hip_shutdown": (i32, []),
    "fitre_hip_sync": (i32, []),
    "fitre_hip_last_error": (C.c_char_p, []),
    "fitre_hip_device_info": (i32, [pi32, pi32, pi32, C.POINTER(sz), C.POINTER(sz), C.c_char_p, i32]),
    "fitre_hip_stream": (vp, []),
    "fitre_hip_malloc": (i32, [pvp, sz]),
    "fitre_hip_free": (i32, [vp]),
    "fitre_hip_malloc_host": (i32, [pvp, sz]),
    "fitre_hip_free_host": (i32, [vp]),
    "fitre_hip_memset": (i32, [vp, i32, sz]),
    "fitre_hip_copy_h2d": (i32, [vp, vp, sz]),
    "fitre_hip_copy_d2h": (i32, [vp, vp, sz]),
    "fitre_hip_copy_d2d": (i32, [vp, vp, sz]),
    "fitre_hip_event_create": (i32, [pvp]),
    "fitre_hip_event_destroy": (i32, [vp]),
    "fitre_hip_event_record": (i32, [vp]),
    "fitre_hip_event_elapsed_ms": (i32, [vp, vp, pf32]),
    "fitre_hip_profile_enable": (i32, [i32]),
    "fitre_hip_profile_read": (i32, [i32, C.POINTER(lng), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "fitre_hip_profile_read_tile": (i32, [i32, i32, C.POINTER(lng), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "fitre_hip_profile_launch_count": (i32, [C.POINTER(lng)]),
    "fitre_hip_profile_read_launch": (i32, [lng, pi32, pi32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "fitre_hip_axpy": (i32, [i32, f32, vp, vp]),
    "fitre_hip_scal": (i32, [i32, f32, vp]),
    "fitre_hip_copy": (i32, [i32, vp, vp]),
    "fitre_hip_copy_2d": (i32, [vp, lng, vp, lng, i32, i32]),
    "fitre_hip_geam": (i32, [i32, i32, i32, i32, f32, vp, i32, f32, vp, i32, vp, i32]),
    "fitre_hip_dot": (i32, [i32, vp, vp, pf32]),
    "fitre_hip_nrm2": (i32, [i32, vp, pf32]),
    "fitre_hip_asum": (i32, [i32, vp, pf32]),
    "fitre_hip_norm_inf": (i32, [i32, vp, pf32]),
    "fitre_hip_sum": (i32, [i32, vp, pf32]),
    "fitre_hip_fill": (i32, [vp, lng, f32]),
    "fitre_hip_hadamard": (i32, [vp, vp, lng]),
    "fitre_hip_hadamard2": (i32, [vp, vp, vp, vp, lng, vp]),
    "fitre_hip_elem_inv_scale": (i32, [vp, vp, f32, lng, vp]),
    "fitre_hip_elem_sqr": (i32, [vp, lng, vp]),
    "fitre_hip_elem_sqr_decay": (i32, [vp, vp, f32, lng, vp]),
    "fitre_hip_mat_mat_scale": (i32, [vp, vp, lng, vp]),
    "fitre_hip_mat_row_vec_scale": (i32, [vp, i32, i32, vp, vp]),
    "fitre_hip_add_column": (i32, [vp, i32, i32, vp]),
    "fitre_hip_add_channel_bias": (i32, [vp, i32, lng, vp]),
    "fitre_hip_activation_forward": (i32, [i32, vp, vp, lng]),
    "fitre_hip_activation_backward": (i32, [i32, vp, vp, vp, vp, lng]),
    "fitre_hip_pool_forward": (i32, [i32, vp] + [i32] * 9 + [vp]),
    "fitre_hip_pool_backward": (i32, [i32, vp, vp] + [i32] * 9 + [vp]),
    "fitre_hip_max_pool_argmax": (i32, [vp] + [i32] * 9 + [vp]),
    "fitre_hip_pool_act_backward": (i32, [i32, i32, vp, vp, vp] + [i32] * 9 + [vp, vp]),
    "fitre_hip_pool_act_bn_backward": (i32, [i32, i32, vp, i32, lng, vp, vp, vp] + [i32] * 9 + [f32, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_pair_supported": (i32, [pshape, i32]),
    "fitre_hip_conv_pair_workspace": (sz, [pshape, i32]),
    "fitre_hip_conv_forward_pair": (i32, [pshape, vp, vp, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_input_grad_pair": (i32, [pshape, vp, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_weight_grad_pair": (i32, [pshape, vp, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_input_grad_split": (i32, [pshape, vp, vp, vp, vp, sz, vp]),
    "fitre_hip_conv_input_grad_prepared_bytes": (sz, [pshape]),
    "fitre_hip_conv_input_grad_prepare": (i32, [pshape, vp, vp, sz]),
    "fitre_hip_conv_input_grad_split_prepared": (i32, [pshape, vp, vp, vp, vp, vp, sz, vp]),
    "fitre_hip_extract_columns": (i32, [vp, vp, vp, i32, i32]),
    "fitre_hip_augment_batch": (i32, [vp, i32, i32, i32, i32, i32, vp, i32, f32, vp, vp, vp, f32, vp]),
    "fitre_hip_crop_shifts": (i32, [vp, i32, i32, vp]),
    "fitre_hip_shift_images": (i32, [vp, i32, i32, i32, i32, vp, vp, f32, vp]),
    "fitre_hip_batch_norm_workspace": (sz, [i32, lng]),
    "fitre_hip_batch_norm_forward": (i32, [vp, i32, lng, vp, vp, vp, vp, vp, f32, f32, i32, vp, sz]),
    "fitre_hip_bn_act_pool_forward": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, vp, vp, f32, f32, i32, i32, vp, i32, i32, i32, i32, i32,
                                            i32, vp, vp, sz]),
    "fitre_hip_batch_norm_backward": (i32, [vp, vp, vp, i32, lng, f32, vp, vp, vp, sz]),
    "fitre_hip_batch_norm_backward_static": (i32, [vp, vp, vp, i32, lng, f32, vp, vp]),
    "fitre_hip_channel_sum_workspace": (sz, [i32, lng]),
    "fitre_hip_channel_sum": (i32, [vp, i32, lng, vp, vp, sz]),
    "fitre_hip_row_sum": (i32, [vp, i32, i32, vp]),
    "fitre_hip_softmax_cross_entropy": (i32, [vp, vp, i32, i32, vp, vp, pf32]),
    "fitre_hip_cross_entropy_error": (i32, [vp, vp, i32, i32, vp]),
    "fitre_hip_accuracy_hits": (i32, [vp, vp, i32, i32, vp]),
    "fitre_hip_multinomial_classes": (i32, [vp, vp, i32, i32, vp]),
    "fitre_hip_column_softmax": (i32, [vp, i32, i32]),
    "fitre_hip_output_terms": (i32, [i32, vp, vp, lng, f32, vp]),
    "fitre_hip_random_seed": (i32, [C.c_ulonglong]),
    "fitre_hip_random_uniform": (i32, [vp, lng]),
    "fitre_hip_random_normal": (i32, [vp, lng]),
    "fitre_hip_reshape": (i32, [vp, i32, i32, i32, vp]),
    "fitre_hip_conv_to_fc": (i32, [vp, i32, i32, i32, i32, vp]),
    "fitre_hip_fc_to_conv": (i32, [vp, i32, i32, i32, i32, vp]),
    "fitre_hip_conv_forward_workspace": (sz, [pshape]),
    "fitre_hip_conv_forward": (i32, [pshape, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_weight_grad_workspace": (sz, [pshape]),
    "fitre_hip_conv_weight_grad_runs_beside": (i32, [pshape]),
    "fitre_hip_conv_weight_grad": (i32, [pshape, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_weight_bias_grad_workspace": (sz, [pshape]),
    "fitre_hip_conv_weight_bias_grad": (i32, [pshape, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_thin_reduce_bytes": (sz, [pshape]),
    "fitre_hip_thin_reduce_defer": (i32, [i32]),
    "fitre_hip_thin_reduce_flush": (i32, []),
    "fitre_hip_conv_input_grad_workspace": (sz, [pshape]),
    "fitre_hip_conv_input_grad": (i32, [pshape, vp, vp, vp, vp, sz]),
    "fitre_hip_conv_input_grad_folds_pool": (i32, [pshape]),
    "fitre_hip_conv_input_grad_pool_act": (i32, [pshape, vp, vp, vp, i32, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_gemm_workspace": (sz, [i32, i32, i32]),
    "fitre_hip_gemm": (i32, [i32, i32, i32, i32, i32, f32, vp, i32, vp, i32, f32, vp, i32, vp, vp, sz]),
    "fitre_hip_linear_is_small": (i32, [i32, i32, i32]),
    "fitre_hip_linear_weight_grad_workspace": (sz, [i32, i32, i32]),
    "fitre_hip_linear_input_grad": (i32, [i32, i32, i32, vp, vp, i32, vp, vp, i32, i32, vp, vp, vp, sz, vp]),
    "fitre_hip_linear_weight_grad": (i32, [i32, i32, i32, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_fc_tail_fits": (i32, [i32, vp, i32]),
    "fitre_hip_fc_tail_workspace": (sz, [i32, vp, i32]),
    "fitre_hip_fc_tail_backward": (i32, [i32, vp, i32, vp, i32, i32, vp, vp, sz]),
    "fitre_hip_fc_tail_backward_pool_act": (i32, [i32, vp, i32, vp, i32, i32, vp, i32, vp, vp, vp, vp, vp, sz]),
    "fitre_hip_lane_select": (i32, [i32]),
    "fitre_hip_lane_wait": (i32, [i32, i32]),
    "fitre_hip_weight_grad_share": (i32, [i32]),
    "fitre_hip_lanes_enable": (i32, [i32]),
    "fitre_hip_activation_rop_backward": (i32, [i32, vp, vp, vp, vp, vp, vp, lng]),
    "fitre_hip_pool_forward_routed": (i32, [i32, vp, vp] + [i32] * 9 + [vp]),
    "fitre_hip_bn_act_pool_rop_forward": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, f32, i32, vp, vp, i32, i32, i32, i32, i32, i32, vp, vp,
                                                sz]),
    "fitre_hip_pool_act_bn_rop_backward": (i32, [i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, i32,
                                                 f32, vp, vp, vp, vp, sz]),
    "fitre_hip_batch_norm_rop_backward": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, lng, f32, vp, vp, sz]),
    "fitre_hip_cross_entropy_rop_error": (i32, [vp, vp, i32, i32, vp]),
    "fitre_hip_fc_rop_backward": (i32, [i32, vp, vp, vp, vp, vp, lng]),
    "fitre_hip_column_softmax_rop": (i32, [vp, vp, i32, i32, vp]),
    "fitre_hip_spd_inverse_workspace": (sz, [i32]),
    "fitre_hip_spd_inverse": (i32, [vp, i32, f32, vp, vp, sz, pi32]),
    "fitre_hip_spd_inverse_queued": (i32, [vp, i32, f32, vp, vp, sz, vp]),
    "fitre_hip_spd_inverse_batched_queued": (i32, [i32, vp, lng, i32, f32, vp, lng, vp, sz, lng, vp]),
    "fitre_hip_kfac_conv_input_factor_workspace": (sz, [vp, i32]),
    "fitre_hip_kfac_conv_input_factor": (i32, [vp, vp, i32, vp, vp, sz]),
    "fitre_hip_kfac_gram_workspace": (sz, [i32, C.c_long]),
    "fitre_hip_kfac_conv_output_factor": (i32, [vp, vp, vp, vp, sz]),
    "fitre_hip_kfac_fc_input_factor": (i32, [vp, i32, i32, i32, vp, vp, sz]),
    "fitre_hip_kfac_fc_output_factor": (i32, [vp, i32, i32, vp, vp, sz]),
    "fitre_hip_gemm_f64_workspace": (sz, [lng, lng, lng, i32]),
    "fitre_hip_gemm_f64": (i32, [lng, lng, lng, f64, pmat, pmat, f64, pmat, f64, i32, vp, sz]),
    "fitre_hip_gemm_f64_add": (i32, [lng, lng, lng, f64, pmat, pmat, f64, pmat, pmat, vp, sz]),
    "fitre_hip_kfac_conv_input_rows": (i32, [vp, vp, i32, vp]),
    "fitre_hip_kfac_fc_input_rows": (i32, [vp, i32, i32, i32, vp]),
    "fitre_hip_gather_headers": (i32, [vp, i32, vp]),
    "fitre_hip_write_header": (i32, [vp, vp, i32]),
    "fitre_hip_spd_inverse_f64_workspace": (sz, [i32]),
    "fitre_hip_spd_inverse_f64_queued": (i32, [vp, i32, vp, i32, vp, sz, vp]),
    "fitre_hip_widen_shift": (i32, [vp, i32, f64, vp]),
    "fitre_hip_pair_to_f64": (i32, [vp, lng, i32, vp, lng]),
    "fitre_hip_kfac_conv_input_factor_f64_workspace": (sz, [vp, i32]),
    "fitre_hip_kfac_conv_input_factor_f64": (i32, [vp, vp, i32, f64, vp, vp, sz]),
    "fitre_hip_kfac_conv_output_factor_f64": (i32, [vp, vp, f64, vp, vp, sz]),
    "fitre_hip_kfac_fc_input_factor_f64": (i32, [vp, i32, i32, i32, f64, vp, vp, sz]),
    "fitre_hip_kfac_fc_output_factor_f64": (i32, [vp, i32, i32, f64, vp, vp, sz]),
}

pconv, ppool = C.POINTER(CONV_LAYER), C.POINTER(POOL_LAYER)
# mirrors include/fitre_cnn.h and include/fitre_shim.h
CNN_API = {
    "getDimensions": (None, [i32, i32, i32, i32, i32, pi32, pi32]),
    "computeParamSize": (None, [pmodel]),
    "computeWeightOffsets": (None, [pmodel]),
    "computeWeightBiasOffsets": (None, [pmodel]),
    "computeZOffsets": (None, [pmodel, i32, i32, i32]),
    "makeLayer": (None, [pconv, ppool, i32, i32, i32, i32, i32, pi32, pi32, i32, i32]),
    "readVGG11": (None, [pmodel, i32, i32, i32, i32, i32, i32, i32, i32]),
    "readLenetCNN": (None, [pmodel, i32, i32, i32, i32, i32, i32]),
    "readAlexNetCNN": (None, [pmodel, i32, i32, i32, i32, i32, i32]),
    "readVGG13": (None, [pmodel, i32, i32, i32, i32, i32, i32, i32, i32]),
    "readVGG16": (None, [pmodel, i32, i32, i32, i32, i32, i32, i32, i32]),
    "readVGG19": (None, [pmodel, i32, i32, i32, i32, i32, i32, i32, i32]),
    "fitre_make_conv_layer": (None, [pconv, ppool] + [i32] * 13 + [pi32, pi32]),
    "fitre_finalize_model": (None, [pmodel, i32, i32, i32]),
    "fitre_build_lenet": (None, [pmodel] + [i32] * 9),
    "fitre_build_vgg11": (None, [pmodel] + [i32] * 8),
    "fitre_build_alexnet": (None, [pmodel] + [i32] * 8),
    "cnnForwardMemRequired": (lng, [pmodel]),
    "cnnForward": (f32, [pmodel, pdata, pscratch, vp, vp, vp, i32, i32, i32]),
    "cnnBackwardMemRequired": (lng, [pmodel]),
    "cnnBackward": (None, [pmodel, pdata, vp, vp, vp, vp, vp, vp, i32, i32, vp]),
    "fitreBackwardUnsupportedLayer": (i32, [pmodel]),
    "fitreSetBackwardLanes": (None, [i32]),
    "fitreBackwardUsesLanes": (i32, [pmodel, i32]),
    "evaluateCNNModel": (f32, [pmodel, pdata, pscratch, vp, vp, vp, i32, i32]),
    "computeCNNGradient": (f32, [pmodel, pdata, pscratch, vp, vp, vp, vp, vp, i32, i32, f32]),
    "computeAccuracy": (f32, [vp, vp, i32, i32, vp, pf32]),
    "computeCrossEntropyError": (None, [vp, i32, i32, vp, vp]),
    "getMultinomialDistSample": (None, [vp, i32, i32, vp, vp]),
    "computeDistributionErrors": (None, [vp, vp, vp, i32, i32, vp, vp]),
    "getRandomVector": (None, [i32, vp, vp, i32]),
    "writeVector": (None, [vp, i32, C.c_char_p, i32, vp]),
    "readVector": (i32, [vp, i32, C.c_char_p, i32, vp]),
    # include/fitre_input.h
    "selectColumnMatrix": (None, [pdata, i32, vp, i32]),
    "selectHostMatrix": (None, [vp, vp, vp, i32, vp, i32, vp]),
    "randomCrop": (None, [vp, i32, i32, i32, i32, i32, vp, vp, vp, f32, vp]),
    "flipData": (None, [vp, vp, i32, i32, i32, i32, vp, vp, vp]),
    "normalizeCIFAR10": (None, [vp, i32, i32, i32, i32, vp, vp, i32]),
    "augmentData": (None, [pmodel, pdata, i32, i32, vp, vp, i32, i32]),
    "computeTestGeneralizationErrors": (None, [pmodel, pdata, pscratch, vp, vp, vp, pf32, pf32]),
    "computeTrainGeneralizationErrors": (None, [pmodel, pdata, vp, pscratch, vp, vp, vp, pf32, pf32]),
    # include/fitre_kfac.h
    "computeKFACStorageIndices": (None, [pmodel, pkfac]),
    "kfacFactorsMemRequired": (lng, [pmodel, i32]),
    "computeOmegaZFactors": (None, [pkfac, pmodel, pdata, i32, vp, vp, vp, pi32, pi32, vp]),
    "computeLambdaDeltaFactors": (None, [pkfac, pmodel, i32, vp, vp, vp, pi32, pi32, vp]),
    "kfacInverseMemRequired": (lng, [pmodel, i32]),
    "computeMatrixInverse": (None, [vp, vp, i32, vp, f32, f32]),
    "matrixInverseMemRequired": (lng, [i32]),
    "computeOmegaZ": (None, [pkfac, pmodel, pdata, i32, vp, vp, vp, pi32, pi32, vp, vp, vp, vp, vp]),
    "computeLambdaDelta": (None, [pkfac, pmodel, i32, vp, vp, vp, pi32, pi32, vp, vp, vp, vp, vp]),
    "computeOmegaZAndLambdaDelta": (None, [pkfac, pmodel, pdata, i32, vp, vp, vp, vp, pi32, pi32, vp]),
    "kfacNaturalGradientMemRequired": (lng, [pmodel]),
    "computeNaturalGradient": (None, [pmodel, pkfac, vp, vp]),
    # include/fitre_solver.h
    "genRandomVector": (None, [pi32, i32, i32]),
    "allocSampledDataset": (None, [pdata, i32]),
    "initBatchNormData": (None, [pmodel, vp, pi32]),
    "updateRunningStats": (None, [vp, vp, i32, f32]),
    "computeSpeedUpOmegaZ": (None, [pkfac, pmodel, pdata, i32, vp, pi32, vp, vp, pi32, i32]),
    "computeSpeedUpLambdaDelta": (None, [pkfac, pmodel, i32, vp, vp, pi32, pi32, i32]),
    "kfacTrustRegionMemRequired": (lng, [pmodel, pdata, pkfac]),
    "kfacTrustRegionHostMemRequired": (lng, [pdata]),
    "kfacTrustRegionReports": (i32, [vp, i32]),
    "subsampledTrustRegionKFAC": (None, [pmodel, pdata, vp, pkfac, vp, pscratch, i32, i32]),
    # include/fitre_dataset.h
    "convertToColumnMajor": (None, [vp, i32, i32, vp]),
    "convertCIFARToColumnMajor": (None, [vp, vp, i32, i32, i32, i32]),
    "imageNormalization": (None, [vp, i32, i32, i32, i32, f32, i32]),
    "readDelimitedMatrix": (None, [C.c_char_p, C.POINTER(C.POINTER(C.c_float)), pi32, pi32]),
    "readCIFARDataset": (None, [C.c_char_p, C.c_char_p, i32, C.c_char_p, vp, vp, i32, i32, i32, i32, i32]),
    "initialize_device_data": (None, [vp, pdata]),
    "initialize_device_image": (None, [vp, pdata]),
    "cleanup_dataset": (None, [vp, pdata]),
    "fitreSetDatasetFolder": (None, [i32, C.c_char_p]),
    "fitreSetWeightsFolder": (None, [C.c_char_p]),
    "getCIFAR10": (i32, [pmodel, vp, pdata, pscratch]),
    "getCIFAR100": (i32, [pmodel, vp, pdata, pscratch]),
    "getTinyImageNet": (i32, [pmodel, vp, pdata, pscratch]),
    "cnnInitializations": (None, [pmodel, pdata]),
    "initKFACTrustRegionParams": (None, [vp, i32]),
    "initKFACInfo": (None, [pkfac]),
    "kfacParamsFileName": (i32, [pmodel, i32, i32, C.c_char_p, i32]),
    "testKFACTrustRegion": (None, [pmodel, pdata, vp, pscratch, f32, f32, i32, i32, i32, i32, i32, i32, f32, i32]),
    # include/fitre_hv.h
    "cnnHvMemRequired": (lng, [pmodel]),
    "cnnHv": (None, [pmodel, pdata, vp, vp, vp, vp, vp, vp, i32, i32, vp, vp, f32]),
    "computeQuadraticModel": (f32, [pmodel, pdata, vp, vp, vp, vp, vp, vp, f32, i32, i32, f32, vp, vp, pf32]),
    # include/fitre_fc.h
    "fitre_build_nn": (None, [pnn, pi32, pi32, i32, i32, i32]),
    "initSampledZOffsets": (None, [pnn, i32]),
    "initRZOffsets": (None, [pnn, i32]),
    "initSampledROffsets": (None, [pnn, i32]),
    "nnForwardMemRequired": (lng, [pnn, i32]),
    "nnGradientMemRequired": (lng, [pnn, i32]),
    "applyLayerActivation": (None, [i32, vp, i32, i32, vp, i32, vp, i32, i32, vp, vp, vp]),
    "nnForwardPass": (None, [pnn, pdata, vp, vp, vp, pf32, pf32, vp, vp, i32, i32]),
    "evaluateModel": (None, [pnn, pdata, pscratch, vp, pf32, pf32, i32, i32]),
    "computeGradient": (None, [pnn, pdata, pscratch, vp, vp, vp, vp, pf32, pf32, i32]),
    "nnHessianVecMemRequired": (lng, [pnn, pdata, i32]),
    "hessianVec": (None, [pnn, pdata, vp, vp, vp, vp, pscratch, i32]),
    "gaussNewtonHessianVec": (None, [pnn, pdata, vp, vp, vp, vp, pscratch, i32]),
    "getDeviceParameters": (None, []),
    "fitre_env_init": (None, [pscratch, i32, sz]),
    "cuda_env_init": (None, [pscratch, i32]),
    "cuda_allocate_workspace": (None, [pscratch, i32]),
    "fitre_allocate_workspace": (None, [pscratch, sz]),
    "cuda_env_cleanup": (None, [pscratch]),
    "cuda_malloc": (None, [pvp, sz, i32, i32]),
    "cuda_malloc_host": (None, [pvp, sz, i32, i32]),
    "cuda_free": (None, [vp, i32]),
    "cuda_free_host": (None, [vp, i32]),
    "cuda_memset": (None, [vp, i32, sz, i32]),
    "copy_host_device": (None, [vp, vp, sz, i32, i32]),
    "copy_device": (None, [vp, vp, sz, i32]),
    "print_device_mem_usage": (None, []),
}


def _load(path, api):
    if not os.path.exists(path):
        raise ImportError("%s is missing: build it with `python -m fitre_amd.build`" % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (restype, argtypes) in api.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise ImportError("%s does not export %s" % (path, name))
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


hip = _load(HIP_LIB_PATH, HIP_API)
cnn = _load(CNN_LIB_PATH, CNN_API)


class FitreError(RuntimeError):
    pass


def check(rc, what=""):
    """Raises FitreError with the device layer's message when rc is not 0."""
    if rc != 0:
        raise FitreError("%s failed with code %d: %s" % (what or "device call", rc, hip.fitre_hip_last_error().decode()))
