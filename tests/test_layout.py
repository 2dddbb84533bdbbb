"""Flat parameter / activation-store layout (nn/utils.c:12-172, nn/read_vgg.c:25-120) and ABI surface."""
import ctypes as C
import json
import os
import re

import numpy as np

from fitre_amd import lib as L
from fitre_amd.structs import (CNN_ACT_RELU, CNN_ACT_SWISH, CNN_MODEL, INT_MAX, MAX_POOL, NO_POOL)
from helpers import build_alexnet, build_custom, build_lenet, build_vgg11

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_lenet_offsets_match_reference_log():
    want = json.load(open(os.path.join(HERE, "golden", "lenet_offsets.json")))["offsets"]
    m = build_lenet(128, bn=False, bias=1)
    got = []
    for l in range(m.cLayers + m.lLayers):
        got += [m.wOffsets[l], m.bOffsets[l]]
    got.append(m.pSize)
    assert got == want


def test_param_sizes_of_the_benchmark_configs():
    # 3x3 convs 3-64-128-256-256-512-512-512-512 + FC 512->10, with biases
    convs = [(3, 64), (64, 128), (128, 256), (256, 256), (256, 512), (512, 512), (512, 512), (512, 512)]
    want = sum(9 * a * b + b for a, b in convs) + 512 * 10 + 10
    m = build_vgg11(256)
    assert m.pSize == want == 9225610
    assert m.zSize == 124403456
    assert build_alexnet(64).pSize == 62378344
    # AlexNet extents 224 -> 55 -> 27 -> 27 -> 13 -> 13/13/13 -> 6
    a = build_alexnet(64)
    assert [a.convLayer[i].outHeight for i in range(5)] == [55, 27, 13, 13, 13]
    assert [a.poolLayer[i].outHeight for i in range(5)] == [27, 13, 13, 13, 6]
    assert a.fcLayer[0].in_ == 9216


def test_no_bias_offsets():
    m = build_lenet(4, bias=0)
    assert m.pSize == 450 + 2400 + 48000 + 10080 + 840
    assert [m.wOffsets[i] for i in range(6)] == [0, 450, 2850, 50850, 60930, 61770]
    assert all(m.bOffsets[i] == INT_MAX for i in range(5))


def test_slab_offsets_with_and_without_batch_norm():
    B = 4
    # one pooled and one unpooled 3x3 layer on 8x8, 2 -> 3 -> 5 channels
    for bn in (False, True):
        m = build_custom(B, 8, 8, 2, [dict(cout=3, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=bn),
                                      dict(cout=5, k=3, pad=1, pool=None, bn=bn)], [(7, 10)])
        c0, c1 = m.convLayer[0], m.convLayer[1]
        V0, P0, V1 = 8 * 8 * 3 * B, 4 * 4 * 3 * B, 4 * 4 * 5 * B
        if not bn:
            assert (c0.activationOffset, c0.poolOffset, c0.outputOffset) == (V0, 2 * V0, 2 * V0)
            assert c0.batchNormOffset == INT_MAX and c0.meansOffset == INT_MAX
            assert (c1.activationOffset, c1.poolOffset, c1.outputOffset) == (V1, INT_MAX, V1)
            slab0, slab1 = 2 * V0 + P0, 2 * V1
        else:
            assert c0.batchNormOffset == V0 and c0.meansOffset == V0 and c0.variancesOffset == V0 + 3
            assert c0.runningMeansOffset == V0 + 6 and c0.runningVariancesOffset == V0 + 9
            assert c0.activationOffset == 2 * V0 + 12 and c0.poolOffset == 3 * V0 + 12
            assert c1.activationOffset == 2 * V1 + 20 and c1.outputOffset == c1.activationOffset
            slab0, slab1 = 3 * V0 + 12 + P0, 3 * V1 + 20
        assert [m.zOffsets[i] for i in range(5)] == [0, 0, slab0, slab0 + slab1, slab0 + slab1 + 2 * 7 * B]
        assert m.zSize == slab0 + slab1 + 2 * 7 * B
        assert m.maxDeltaSize == max(slab0, slab1)
        assert m.fcLayer[0].in_ == 5 * 4 * 4 and m.fcLayer[0].offset == 7 * B


def test_readVGG11_is_the_swish_network():
    m = CNN_MODEL()
    L.cnn.readVGG11(C.byref(m), 8, 32, 32, 10, 3, 0, 0, 10)
    assert m.cLayers == 8 and m.lLayers == 1 and all(m.actFuns[i] == CNN_ACT_SWISH for i in range(8))
    assert [m.poolLayer[i].type for i in range(8)] == [MAX_POOL, MAX_POOL, NO_POOL, MAX_POOL, NO_POOL, MAX_POOL, NO_POOL, MAX_POOL]
    assert m.fcLayer[0].in_ == 512


def test_get_dimensions():
    h, w = C.c_int(), C.c_int()
    L.cnn.getDimensions(224, 224, 2, 4, 11, C.byref(h), C.byref(w))
    assert (h.value, w.value) == (55, 55)
    L.cnn.getDimensions(27, 13, 0, 2, 3, C.byref(h), C.byref(w))
    assert (h.value, w.value) == (13, 6)


def _declared(header, pattern):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(pattern, text)))


def test_libraries_export_every_declared_symbol():
    hip_names = _declared("fitre_hip.h", r"\b(fitre_hip_\w+)\s*\(")
    assert len(hip_names) > 50
    for n in hip_names:
        assert hasattr(L.hip, n), n
        assert n in L.HIP_API, "ctypes table lacks %s" % n
    cnn_names = (_declared("fitre_cnn.h", r"\b([A-Za-z_]\w*)\s*\(") + _declared("fitre_shim.h", r"\b([A-Za-z_]\w*)\s*\(") +
                 _declared("fitre_kfac.h", r"\b([A-Za-z_]\w*)\s*\(") + _declared("fitre_fc.h", r"\b([A-Za-z_]\w*)\s*\(") +
                 _declared("fitre_hv.h", r"\b([A-Za-z_]\w*)\s*\(") + _declared("fitre_input.h", r"\b([A-Za-z_]\w*)\s*\(") + _declared("fitre_solver.h", r"\b([A-Za-z_]\w*)\s*\(") +
                 _declared("fitre_dataset.h", r"\b([A-Za-z_]\w*)\s*\("))
    cnn_names = [n for n in cnn_names if n not in ("defined",)]
    assert "cnnBackward" in cnn_names and "computeCNNGradient" in cnn_names and "copy_host_device" in cnn_names
    assert "computeOmegaZFactors" in cnn_names and "computeKFACStorageIndices" in cnn_names
    assert "cnnHv" in cnn_names and "computeQuadraticModel" in cnn_names
    assert "augmentData" in cnn_names and "selectColumnMatrix" in cnn_names and "computeTestGeneralizationErrors" in cnn_names
    assert "computeOmegaZAndLambdaDelta" in cnn_names
    assert "subsampledTrustRegionKFAC" in cnn_names and "genRandomVector" in cnn_names
    assert "readCIFARDataset" in cnn_names and "testKFACTrustRegion" in cnn_names and "selectHostMatrix" in cnn_names
    assert "computeGradient" in cnn_names and "nnForwardPass" in cnn_names and "computeNaturalGradient" in cnn_names
    for n in cnn_names:
        assert hasattr(L.cnn, n), n
    for g in ("BLOCK_SIZE", "WARP_SIZE", "DEVICE_NUM_BLOCKS"):
        assert C.c_int.in_dll(L.cnn, g) is not None


def test_struct_sizes_match_the_c_side():
    # a C-side check would need a compiler run; the builders fill every field through C, so a
    # mismatch in field order shows as garbage here
    m = build_vgg11(2)
    assert m.batchSize == 2 and m.bias == 1 and m.cLayers == 8
    assert m.convLayer[7].outChannels == 512 and m.poolLayer[7].outHeight == 1
    assert C.sizeof(CNN_MODEL) == 20 * 22 * 4 + 20 * 4 + 20 * 8 * 4 + 8 + 20 * 5 * 4 + 7 * 4 + 3 * 80 + 4 + 2 * 80


def test_kfac_storage_indices_follow_the_reference_formula():
    # solvers/kfac_utils.cu:17-45: input-side slots (K+1)^2 whatever the bias setting, output-side Cout^2
    from fitre_amd.structs import KFAC_CURVATURE_INFO
    for m in (build_vgg11(4), build_lenet(4, bias=0)):
        info = KFAC_CURVATURE_INFO()
        L.cnn.computeKFACStorageIndices(C.byref(m), C.byref(info))
        o = l = 0
        for i in range(m.cLayers):
            c = m.convLayer[i]
            assert (info.OmegaZOffsets[i], info.LambdaGOffsets[i]) == (o, l)
            o += (c.inChannels * c.kSize ** 2 + 1) ** 2
            l += c.outChannels ** 2
        for i in range(m.lLayers):
            f = m.fcLayer[i]
            assert (info.OmegaZOffsets[m.cLayers + i], info.LambdaGOffsets[m.cLayers + i]) == (o, l)
            o += (f.in_ + 1) ** 2
            l += f.out ** 2
        assert (info.OmegaZOffsets[m.cLayers + m.lLayers], info.LambdaGOffsets[m.cLayers + m.lLayers]) == (o, l)
        assert L.cnn.kfacFactorsMemRequired(C.byref(m), 4) > 0


def test_workspace_requirements_are_positive_and_modest():
    m = build_vgg11(256)
    fwd, bwd = L.cnn.cnnForwardMemRequired(C.byref(m)), L.cnn.cnnBackwardMemRequired(C.byref(m))
    assert 0 < fwd * 4 < 512e6 and 0 < bwd * 4 < 512e6


def test_vector_text_io_round_trip(tmp_path):
    """readVector / writeVector (utilities/print_utils.c:136-186): the first lines of the reference's LeNet weight
    file parse to the values numpy reads, and a written vector reads back to the printed precision."""
    here = os.path.dirname(os.path.abspath(__file__))
    path = os.path.join(here, "golden", "lenet_xavier_head.txt")
    want = np.loadtxt(path)
    vec = np.zeros(100, dtype=np.float32)
    got = L.cnn.readVector(vec.ctypes.data_as(C.c_void_p), 100, path.encode(), 0, None)
    assert got == want.size == 64
    np.testing.assert_array_equal(vec[:64], want.astype(np.float32))
    # fewer rows than lines, and the additive offset (used for 1-based labels)
    got = L.cnn.readVector(vec.ctypes.data_as(C.c_void_p), 10, path.encode(), 1, None)
    assert got == 10
    np.testing.assert_allclose(vec[:10], want[:10] + 1, atol=1e-6)
    out = str(tmp_path / "v.txt").encode()
    src = np.array([0.5, -1.25, 3.0000000001, 1e-11], dtype=np.float32)
    L.cnn.writeVector(src.ctypes.data_as(C.c_void_p), 4, out, 1, None)
    assert open(out).read().splitlines() == ["0.5000000000", "-1.2500000000", "3.0000000000", "0.0000000000"]
    back = np.zeros(4, dtype=np.float32)
    assert L.cnn.readVector(back.ctypes.data_as(C.c_void_p), 4, out, 0, None) == 4
    np.testing.assert_allclose(back, src, atol=1e-10)


def test_vgg_family_parameter_counts():
    """readVGG11/13/16/19 (nn/read_vgg.c): the convolution stacks are the standard ones, whose parameter counts are
    known (9 220 480, 9 404 992, 14 714 688 and 20 024 384 with biases), plus the 512 -> 10 linear layer."""
    from fitre_amd.structs import CNN_MODEL
    known = {"readVGG11": (8, 9220480, 2), "readVGG13": (10, 9404992, 3), "readVGG16": (13, 14714688, 4),
             "readVGG19": (16, 20024384, 5)}
    for reader, (convs, conv_params, name) in known.items():
        m = CNN_MODEL()
        getattr(L.cnn, reader)(C.byref(m), 32, 32, 32, 10, 3, 1, 1, 10)
        assert (m.cLayers, m.lLayers, m.name, m.bias, m.enableBatchNorm) == (convs, 1, name, 1, 1)
        assert m.pSize == conv_params + 512 * 10 + 10
        assert all(m.actFuns[i] == 14 for i in range(convs))                      # swish
        assert sum(1 for i in range(convs) if m.poolLayer[i].type != 2) == 5      # five max pools: 32 -> 1
        assert m.poolLayer[convs - 1].outHeight == 1 and m.fcLayer[0].in_ == 512
        m64 = CNN_MODEL()
        getattr(L.cnn, reader)(C.byref(m64), 8, 64, 64, 200, 3, 0, 0, 30)
        assert m64.fcLayer[0].in_ == 2048 and m64.bias == 0                       # 64 x 64 images: 512 * 4 features


def test_small_reference_networks():
    """readLenetCNN (nn/read_nn.c:500-700) and readAlexNetCNN (nn/read_alexnet.c:14-215): layer shapes as written there."""
    from fitre_amd.structs import CNN_MODEL
    m = CNN_MODEL()
    L.cnn.readLenetCNN(C.byref(m), 3, 32, 32, 64, 1, 0)
    assert (m.cLayers, m.lLayers, m.name, m.pSize) == (2, 3, 0, 62006)
    assert [m.poolLayer[i].type for i in range(2)] == [1, 1] and [m.actFuns[i] for i in range(2)] == [14, 14]   # average pool, swish
    assert (m.fcLayer[0].in_, m.fcLayer[0].out, m.fcLayer[1].out, m.fcLayer[2].out) == (400, 120, 84, 10)
    assert (m.fcLayer[0].actFun, m.fcLayer[1].actFun, m.fcLayer[2].actFun) == (14, 14, 10)          # swish, swish, none
    a = CNN_MODEL()
    L.cnn.readAlexNetCNN(C.byref(a), 32, 32, 32, 10, 1, 1)
    assert (a.cLayers, a.lLayers, a.name) == (2, 3, 1)
    assert [(a.convLayer[i].kSize, a.convLayer[i].padding, a.convLayer[i].outChannels) for i in range(2)] == [(5, 2, 64)] * 2
    assert [(a.poolLayer[i].pSize, a.poolLayer[i].stride, a.poolLayer[i].padding, a.poolLayer[i].type) for i in range(2)] == [(3, 2, 1, 0)] * 2
    assert (a.poolLayer[0].outHeight, a.poolLayer[1].outHeight, a.fcLayer[0].in_) == (16, 8, 64 * 8 * 8)
    assert a.pSize == 4864 + 102464 + 1573248 + 73920 + 1930


def test_strided_convolution_above_the_first_layer_is_rejected_before_any_launch():
    """Back-propagation is implemented for stride-1 convolutions; a model with a strided layer above the first is
    reported by fitreBackwardUnsupportedLayer, and cnnBackward exits with a message before it touches the device (run
    in a child process: the reference's error convention is exit(-1))."""
    import subprocess
    import sys
    ok = build_custom(2, 16, 16, 3, [dict(cout=4, k=5, stride=2, pad=2), dict(cout=4, k=3, pad=1)], [(3, 0)])
    assert L.cnn.fitreBackwardUnsupportedLayer(C.byref(ok)) == 0           # a strided FIRST layer is fine (AlexNet)
    bad = build_custom(2, 16, 16, 3, [dict(cout=4, k=3, pad=1), dict(cout=4, k=3, stride=2, pad=1)], [(3, 0)])
    assert L.cnn.fitreBackwardUnsupportedLayer(C.byref(bad)) == 2
    code = (
        "import ctypes as C, sys\n"
        "sys.path.insert(0, %r)\n"
        "from fitre_amd import lib as L\n"
        "from fitre_amd.harness import build_custom\n"
        "from fitre_amd.structs import DEVICE_DATASET\n"
        "m = build_custom(2, 16, 16, 3, [dict(cout=4, k=3, pad=1), dict(cout=4, k=3, stride=2, pad=1)], [(3, 0)])\n"
        "L.cnn.cnnBackward(C.byref(m), C.byref(DEVICE_DATASET()), None, None, None, None, None, None, 0, 2, None)\n"
        "print('returned')\n" % ROOT)
    proc = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0 and "returned" not in proc.stdout
    assert "stride 2" in proc.stderr and "layer 2" in proc.stderr
