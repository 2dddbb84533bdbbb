"""ctypes mirrors of the records in include/fitre_types.h and include/fitre_nn.h.

Field names and order are those of the reference's nn/nn_decl.h:64-155 and
core/structdefs.h:25-83; `real` is float.
"""
import ctypes as C

MAX_LAYERS = 20
real = C.c_float
real_p = C.POINTER(real)

# enumerators (nn/nn_decl.h:13-62, 97-101)
PERFORM_NO_BATCH_NORM, PERFORM_BATCH_NORM, PERFORM_BATCH_NORM_TRAINABLE = 0, 10, 20
MODEL_TRAIN, MODEL_TRAIN_ACCURACY, MODEL_TEST_ACCURACY = 10, 20, 30
ACT_NONE, ACT_LOGISTIC, ACT_TANH, ACT_LINEAR, ACT_SOFTMAX = 0, 1, 2, 3, 4
CNN_ACT_NONE, CNN_ACT_SOFTPLUS, CNN_ACT_ELU, CNN_ACT_RELU, CNN_ACT_SWISH = 10, 11, 12, 13, 14
MAX_POOL, AVG_POOL, NO_POOL = 0, 1, 2
CIFAR10, CIFAR100, IMAGENET = 10, 20, 30
INT_MAX = 2 ** 31 - 1


class CONV_LAYER(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "inChannels", "outChannels", "width", "height", "outWidth", "outHeight", "kSize", "stride",
        "padding", "activationOffset", "poolOffset", "batchNormOffset", "outputOffset", "batchNorm",
        "meansOffset", "variancesOffset", "runningMeansOffset", "runningVariancesOffset", "convVolumn",
        "activationVolumn", "poolVolumn", "batchNormVolumn")]


class POOL_LAYER(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "height", "width", "outHeight", "outWidth", "type", "pSize", "padding", "stride")]


class FC_LAYER(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("in_", "out", "actFun", "batchNorm", "offset")]


class CNN_MODEL(C.Structure):
    _fields_ = [
        ("convLayer", CONV_LAYER * MAX_LAYERS),
        ("actFuns", C.c_int * MAX_LAYERS),
        ("poolLayer", POOL_LAYER * MAX_LAYERS),
        ("cLayers", C.c_int),
        ("lLayers", C.c_int),
        ("fcLayer", FC_LAYER * MAX_LAYERS),
        ("bias", C.c_int),
        ("pSize", C.c_int),
        ("zSize", C.c_int),
        ("batchSize", C.c_int),
        ("maxDeltaSize", C.c_int),
        ("name", C.c_int),
        ("enableBatchNorm", C.c_int),
        ("wOffsets", C.c_int * MAX_LAYERS),
        ("bOffsets", C.c_int * MAX_LAYERS),
        ("zOffsets", C.c_int * MAX_LAYERS),
        ("zztSize", C.c_int),
        ("zztOffsets", C.c_int * MAX_LAYERS),
        ("rZOffsets", C.c_int * MAX_LAYERS),
    ]


class NN_MODEL(C.Structure):
    """include/fitre_nn.h (nn/nn_decl.h:157-183 of the reference)."""
    _fields_ = ([("layerSizes", C.c_int * MAX_LAYERS), ("actFuns", C.c_int * MAX_LAYERS)] +
                [(n, C.c_int) for n in ("numLayers", "type", "pSize", "zSize", "sampledZSize", "sampledRSize", "rFullSize")] +
                [(n, C.c_int * MAX_LAYERS) for n in ("wOffsets", "bOffsets", "zOffsets", "sZOffsets", "rZOffsets",
                                                     "sRZOffsets")])


MODEL_TYPE_MSE, MODEL_TYPE_CLASSIFICATION = 0, 1
TEST_DATA, TRAIN_DATA = 0, 1
FULL_DATASET, SAMPLED_DATASET = 0, 1


class SCRATCH_AREA(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "hostWorkspace", "devWorkspace", "pageLckWorkspace", "nextDevPtr", "nextHostPtr", "nextPageLckPtr")]


class HOST_DATASET(C.Structure):
    """include/fitre_types.h (core/structdefs.h of the reference): the data set in host memory."""
    _fields_ = ([(n, C.POINTER(C.c_float)) for n in ("trainSetX", "trainSetY", "testSetX", "testSetY")] +
                [(n, C.c_int) for n in ("trainSizeX", "trainSizeY", "testSizeX", "testSizeY", "features", "height", "width",
                                        "numClasses", "datasetType")])


class SparseDataset(C.Structure):
    _fields_ = [("rowPtr", C.c_void_p), ("colPtr", C.c_void_p), ("rowCsrPtr", C.c_void_p),
                ("valPtr", C.c_void_p), ("nnz", C.c_int), ("sortedVals", C.c_void_p), ("P", C.c_void_p),
                ("descr", C.c_void_p)]


class DEVICE_DATASET(C.Structure):
    _fields_ = [
        ("trainSetX", C.c_void_p), ("trainSetY", C.c_void_p), ("testSetX", C.c_void_p),
        ("testSetY", C.c_void_p), ("weights", C.c_void_p), ("numClasses", C.c_int),
        ("datasetType", C.c_int), ("features", C.c_int), ("height", C.c_int), ("width", C.c_int),
        ("testSizeX", C.c_int), ("testSizeY", C.c_int), ("trainSizeX", C.c_int), ("trainSizeY", C.c_int),
        ("sampleSize", C.c_int), ("sampledTrainX", C.c_void_p), ("sampledTrainY", C.c_void_p),
        ("currentBatch", C.c_void_p), ("spSamplingMatrix", SparseDataset),
    ]


class KFAC_CURVATURE_INFO(C.Structure):
    """include/fitre_kfac.h (solvers/kfac_structs.h:13-52 of the reference)."""
    _fields_ = ([(n, C.c_void_p) for n in ("OmegaZZT", "LambdaGGT", "OmegaZInv", "LambdaGInv", "vec", "nGradient",
                                           "gradient")] +
                [("OmegaZOffsets", C.c_int * MAX_LAYERS), ("LambdaGOffsets", C.c_int * MAX_LAYERS)] +
                [(n, C.c_float) for n in ("stats_decay", "momentum", "regLambda", "dampGamma")] +
                [("checkGrad", C.c_int), ("dampedInputSize", C.c_int)] +
                [(n, C.c_void_p) for n in ("dampedInput", "dampedZ", "dampedLambda")] +
                [("inverseFreq", C.c_int)])


class TRUST_REGION_PARAMS(C.Structure):
    """include/fitre_solver.h (solvers/params.h:12-35 of the reference)."""
    _fields_ = ([(n, C.c_float) for n in ("delta", "minDelta", "maxDelta", "eta1", "eta2", "gamma1", "gamma2")] +
                [("maxProps", C.c_ulong), ("maxMatVecs", C.c_int), ("maxEpochs", C.c_int), ("maxIters", C.c_int),
                 ("hessianType", C.c_int), ("alpha", C.c_float), ("curIteration", C.c_int), ("hs", C.c_float),
                 ("lambda_", C.c_float)])


class KFAC_TR_EPOCH_REPORT(C.Structure):
    """include/fitre_solver.h: what one pass over the training set left behind."""
    _fields_ = ([("iteration", C.c_int), ("miniBatches", C.c_int), ("rejectedSteps", C.c_int)] +
                [(n, C.c_float) for n in ("trainLikelihood", "trainAccuracy", "testLikelihood", "testAccuracy",
                                          "weightNorm", "delta", "seconds")])


class fitre_split_view(C.Structure):
    """include/fitre_hip.h: unsummed split partials of an input gradient."""
    _fields_ = [("base", C.c_void_p), ("splits", C.c_int), ("stride", C.c_long)]


class fitre_conv_shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "samples", "inChannels", "outChannels", "inA", "inB", "outA", "outB", "ksize", "stride", "padding")]


FITRE_MAT_F32, FITRE_MAT_F64, FITRE_MAT_SYM_PAIR = 0, 1, 2
FITRE_GEMM_SYMMETRIC, FITRE_GEMM_A_LOWER, FITRE_GEMM_A_UPPER, FITRE_GEMM_B_LOWER, FITRE_GEMM_B_UPPER = 1, 2, 4, 8, 16


class fitre_matrix(C.Structure):
    """Operand of the float64 products (include/fitre_hip.h)."""
    _fields_ = [("data", C.c_void_p), ("rowStride", C.c_long), ("colStride", C.c_long), ("kind", C.c_int),
                ("onesRow", C.c_long), ("onesCol", C.c_long), ("onesValue", C.c_double)]


class fitre_fc_tail_layer(C.Structure):
    """One layer of fitre_hip_fc_tail_backward (include/fitre_hip.h)."""
    _fields_ = [("in_", C.c_int), ("out", C.c_int), ("act", C.c_int), ("W", C.c_void_p), ("zPre", C.c_void_p),
                ("zPost", C.c_void_p), ("zin", C.c_void_p), ("slot", C.c_void_p), ("dW", C.c_void_p), ("db", C.c_void_p)]
