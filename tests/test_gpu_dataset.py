"""From record files to a trained network: the data-set readers' device copies (utilities/dataset.c:606-706), the
driver that reads a start point and runs the solver (drivers/kfac_trust_region_driver.cu:201-498), and the solver on a
training set kept in host memory (selectHostMatrix, utilities/dataset_utils.c:10-25; solvers/kfac_trust_region.cu:322-337;
functions/cnn_accuracy.cu:136-143).  The files are written here: separable synthetic images, one template per class."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import CNN_MODEL, DEVICE_DATASET, HOST_DATASET, KFAC_CURVATURE_INFO, KFAC_TR_EPOCH_REPORT, SCRATCH_AREA, \
    TRUST_REGION_PARAMS
from helpers import build_lenet, he_weights

pytestmark = pytest.mark.gpu
hip, cnn = L.hip, L.cnn
libc = C.CDLL(None)
CIFAR10, IMAGENET = 10, 30


def write_records(path, rng, templates, per_class, classes_used):
    """Shuffled records `label byte + pixels` around the class templates; returns how many."""
    rows = []
    for c in classes_used:
        px = np.clip(templates[c] + 25.0 * rng.standard_normal((per_class, templates.shape[1])), 0, 255).astype(np.uint8)
        rows.append(np.concatenate([np.full((per_class, 1), c, np.uint8), px], axis=1))
    rows = np.concatenate(rows)
    rows = rows[rng.permutation(rows.shape[0])]
    path.write_bytes(rows.tobytes())
    return rows.shape[0]


def as_array(ptr, n):
    return np.ctypeslib.as_array(ptr, shape=(n,)).copy()


def make_scratch(dev, model, data, epochs_host_reals):
    info = KFAC_CURVATURE_INFO()
    info.inverseFreq = 1
    need = cnn.kfacTrustRegionMemRequired(C.byref(model), C.byref(data), C.byref(info))
    arena = dev.zeros(need)
    host_reals = max(cnn.kfacTrustRegionHostMemRequired(C.byref(data)), epochs_host_reals) + 1024
    host_arena = (C.c_float * host_reals)()
    pinned = (C.c_float * 8)()
    scratch = SCRATCH_AREA()
    scratch.devWorkspace = scratch.nextDevPtr = arena.value
    scratch.hostWorkspace = scratch.nextHostPtr = C.addressof(host_arena)
    scratch.pageLckWorkspace = scratch.nextPageLckPtr = C.addressof(pinned)
    return scratch, arena, (host_arena, pinned)


def reports_of(epochs):
    reports = (KFAC_TR_EPOCH_REPORT * epochs)()
    assert cnn.kfacTrustRegionReports(reports, epochs) == epochs
    return list(reports)


def cifar10_folder(tmp_path, rng):
    folder = tmp_path / "cifar10"
    folder.mkdir()
    templates = rng.integers(40, 216, size=(10, 3072)).astype(np.float32)
    train = sum(write_records(folder / ("data_batch_%d.bin" % i), rng, templates, 9, range(10)) for i in range(1, 6))
    test = write_records(folder / "test_batch.bin", rng, templates, 13, range(10))
    return folder, train, test


def test_files_to_device_and_back(dev, tmp_path):
    rng = np.random.default_rng(1)
    folder, train, test = cifar10_folder(tmp_path, rng)
    cnn.fitreSetDatasetFolder(1, (str(folder) + "/").encode())
    model = build_lenet(64, bn=True)
    host, data = HOST_DATASET(), DEVICE_DATASET()
    assert cnn.getCIFAR10(C.byref(model), C.byref(host), C.byref(data), None) == 0
    cnn.fitreSetDatasetFolder(1, None)
    assert (host.trainSizeX, host.testSizeX, host.features, host.numClasses) == (train, test, 3072, 10) == (450, 130, 3072, 10)
    assert (data.trainSizeX, data.testSizeX, data.features, data.numClasses, data.height, data.width) == (450, 130, 3072, 10, 32, 32)
    assert data.datasetType == CIFAR10 and host.datasetType == CIFAR10
    for dptr, hptr, n in ((data.trainSetX, host.trainSetX, 450 * 3072), (data.trainSetY, host.trainSetY, 450),
                          (data.testSetX, host.testSetX, 130 * 3072), (data.testSetY, host.testSetY, 130)):
        np.testing.assert_array_equal(dev.download(C.c_void_p(dptr), n), as_array(hptr, n))
    labels = as_array(host.trainSetY, 450)
    assert labels.min() == 1 and labels.max() == 10
    cnn.cleanup_dataset(C.byref(host), C.byref(data))
    assert not host.trainSetX and data.trainSetX is None and data.testSetY is None


def test_driver_trains_from_files(dev, tmp_path):
    """Files -> getCIFAR10 -> parameter file -> testKFACTrustRegion; the same start point and settings given to
    subsampledTrustRegionKFAC directly end at the same weights, bit for bit."""
    rng = np.random.default_rng(2)
    folder, _, _ = cifar10_folder(tmp_path, rng)
    weights_dir = tmp_path / "weights"
    (weights_dir / "cifar10").mkdir(parents=True)
    cnn.fitreSetDatasetFolder(1, (str(folder) + "/").encode())
    cnn.fitreSetWeightsFolder((str(weights_dir) + "/").encode())
    model = build_lenet(64, bn=True)
    host, data = HOST_DATASET(), DEVICE_DATASET()
    cnn.getCIFAR10(C.byref(model), C.byref(host), C.byref(data), None)
    cnn.cnnInitializations(C.byref(model), C.byref(data))
    assert data.weights is not None

    start = he_weights(model, rng).astype(np.float32)
    name = C.create_string_buffer(1024)
    assert cnn.kfacParamsFileName(C.byref(model), 1, 0, name, 1024) == 0
    assert name.value.decode() == str(weights_dir) + "/cifar10/lenet_default_bias.params"
    cnn.writeVector(start.ctypes.data_as(C.c_void_p), model.pSize, name.value, 1, None)

    epochs = 3
    scratch, arena, keep = make_scratch(dev, model, data, model.pSize)
    libc.srand(7)
    L.check(hip.fitre_hip_random_seed(7))
    cnn.testKFACTrustRegion(C.byref(model), C.byref(data), C.byref(host), C.byref(scratch), 0.1, 4.0, 0, 0, 0, 1, epochs, 1, 0.0, 0)
    reports = reports_of(epochs)
    trained = dev.download(C.c_void_p(data.weights), model.pSize)
    assert np.isfinite(trained).all()
    # the arenas' pointers are back where they were, so the struct serves the second run below as it is
    assert (scratch.nextDevPtr, scratch.nextHostPtr, scratch.nextPageLckPtr) == (
        scratch.devWorkspace, scratch.hostWorkspace, scratch.pageLckWorkspace)
    assert all(r.miniBatches == 7 for r in reports)
    assert reports[-1].trainAccuracy > 70.0 and reports[-1].testAccuracy > 70.0, [(r.trainAccuracy, r.testAccuracy) for r in reports]
    assert reports[-1].delta <= 4.0
    cnn.cuda_free(data.sampledTrainX, -1)
    cnn.cuda_free(data.sampledTrainY, -1)

    # the same run without the driver: its defaults, the file's values as the start point
    read_back = np.empty(model.pSize, np.float32)
    assert cnn.readVector(read_back.ctypes.data_as(C.c_void_p), model.pSize, name.value, 0, None) == model.pSize
    np.testing.assert_allclose(read_back, start, rtol=0, atol=1e-9)
    L.check(hip.fitre_hip_copy_h2d(C.c_void_p(data.weights), read_back.ctypes.data_as(C.c_void_p), read_back.nbytes))
    tr, info = TRUST_REGION_PARAMS(), KFAC_CURVATURE_INFO()
    cnn.initKFACTrustRegionParams(C.byref(tr), 450)
    cnn.initKFACInfo(C.byref(info))
    info.dampGamma, info.checkGrad, info.inverseFreq, info.regLambda = 0.1, 0, 1, 0.0
    tr.maxDelta, tr.maxIters = 4.0, epochs
    libc.srand(7)
    L.check(hip.fitre_hip_random_seed(7))
    cnn.subsampledTrustRegionKFAC(C.byref(model), C.byref(data), C.byref(host), C.byref(info), C.byref(tr), C.byref(scratch), 0, 0)
    np.testing.assert_array_equal(dev.download(C.c_void_p(data.weights), model.pSize), trained)

    cnn.cuda_free(data.sampledTrainX, -1)
    cnn.cuda_free(data.sampledTrainY, -1)
    cnn.cuda_free(data.weights, -1)
    cnn.cleanup_dataset(C.byref(host), C.byref(data))
    dev.free(arena)
    cnn.fitreSetDatasetFolder(1, None)
    cnn.fitreSetWeightsFolder(None)


def tiny_folder(tmp_path, rng):
    folder = tmp_path / "tiny"
    folder.mkdir()
    classes_used = [3, 17, 42, 64, 99, 120, 150, 163, 180, 199]
    templates = rng.integers(40, 216, size=(200, 3 * 64 * 64)).astype(np.float32)
    train = sum(write_records(folder / ("train_%d.bin" % i), rng, templates, 1, classes_used) for i in range(1, 20))
    test = sum(write_records(folder / ("test_%d.bin" % i), rng, templates, 2, classes_used) for i in (1, 2))
    return folder, train, test


def test_selection_from_host_memory_matches_selection_on_the_device(dev, tmp_path):
    rng = np.random.default_rng(3)
    folder, train, test = tiny_folder(tmp_path, rng)
    cnn.fitreSetDatasetFolder(3, (str(folder) + "/").encode())
    model = CNN_MODEL()
    cnn.fitre_build_lenet(C.byref(model), 32, 64, 64, 3, 200, 1, 1, 1, 1)
    host, data = HOST_DATASET(), DEVICE_DATASET()
    cnn.getTinyImageNet(C.byref(model), C.byref(host), C.byref(data), None)
    cnn.fitreSetDatasetFolder(3, None)
    assert (train, test) == (190, 40) == (host.trainSizeX, host.testSizeX)
    assert data.trainSetX is None and data.trainSetY is None and data.testSetX is not None
    assert data.datasetType == IMAGENET and data.features == 12288 and data.numClasses == 200

    feats, n = 12288, 32
    order = rng.permutation(190).astype(np.int32)
    outX, outY = dev.zeros(n * feats), dev.zeros(n)
    labels = np.zeros(n, np.float32)
    cnn.selectHostMatrix(C.byref(host), outX, outY, n, order.ctypes.data_as(C.c_void_p), 40, labels.ctypes.data_as(C.c_void_p))
    allX, allY = as_array(host.trainSetX, 190 * feats).reshape(190, feats), as_array(host.trainSetY, 190)
    np.testing.assert_array_equal(dev.download(outX, n * feats).reshape(n, feats), allX[order[40:72]])
    np.testing.assert_array_equal(dev.download(outY, n), allY[order[40:72]])
    np.testing.assert_array_equal(labels, allY[order[40:72]])

    # the device-side selection on an uploaded copy of the same set
    data.trainSetX, data.trainSetY = dev.upload(allX.reshape(-1)).value, dev.upload(allY).value
    data.sampledTrainX, data.sampledTrainY = dev.zeros(2 * n * feats).value, dev.zeros(n).value
    d_order = dev.upload(order, dtype=np.int32)
    cnn.selectColumnMatrix(C.byref(data), n, d_order, 40)
    np.testing.assert_array_equal(dev.download(C.c_void_p(data.sampledTrainX), n * feats), dev.download(outX, n * feats))
    np.testing.assert_array_equal(dev.download(C.c_void_p(data.sampledTrainY), n), dev.download(outY, n))
    for q in (data.sampledTrainX, data.sampledTrainY, data.trainSetX, data.trainSetY):
        dev.free(C.c_void_p(q))
    data.trainSetX = data.trainSetY = None
    dev.free(outX), dev.free(outY), dev.free(d_order)
    cnn.cleanup_dataset(C.byref(host), C.byref(data))


def test_solver_on_a_training_set_kept_in_host_memory(dev, tmp_path):
    """64 x 64 images, 200 classes (ten of them present), the training set on the host only: mini-batches and the
    whole-set evaluation read it through the host struct."""
    rng = np.random.default_rng(4)
    folder, _, _ = tiny_folder(tmp_path, rng)
    weights_dir = tmp_path / "weights"
    (weights_dir / "imagenet").mkdir(parents=True)
    cnn.fitreSetDatasetFolder(3, (str(folder) + "/").encode())
    cnn.fitreSetWeightsFolder((str(weights_dir) + "/").encode())
    model = CNN_MODEL()
    cnn.fitre_build_lenet(C.byref(model), 32, 64, 64, 3, 200, 1, 1, 1, 1)
    host, data = HOST_DATASET(), DEVICE_DATASET()
    cnn.getTinyImageNet(C.byref(model), C.byref(host), C.byref(data), None)
    cnn.cnnInitializations(C.byref(model), C.byref(data))
    start = he_weights(model, rng).astype(np.float32)
    name = C.create_string_buffer(1024)
    assert cnn.kfacParamsFileName(C.byref(model), 3, 1, name, 1024) == 0 and name.value.endswith(b"imagenet/lenet_kaiming_bias.params")
    cnn.writeVector(start.ctypes.data_as(C.c_void_p), model.pSize, name.value, 1, None)

    epochs = 4
    scratch, arena, keep = make_scratch(dev, model, data, model.pSize)
    libc.srand(5)
    L.check(hip.fitre_hip_random_seed(5))
    cnn.testKFACTrustRegion(C.byref(model), C.byref(data), C.byref(host), C.byref(scratch), 0.1, 4.0, 0, 0, 0, 1, epochs, 3, 0.0, 1)
    reports = reports_of(epochs)
    trained = dev.download(C.c_void_p(data.weights), model.pSize)
    assert np.isfinite(trained).all()
    assert all(r.miniBatches == 5 for r in reports)            # 190 images, batch 32: the last 30 are left out
    losses = [r.trainLikelihood for r in reports]
    assert np.isfinite(losses).all() and losses[-1] < losses[0], losses
    assert reports[-1].trainAccuracy > 50.0 and reports[-1].testAccuracy > 50.0, [(r.trainAccuracy, r.testAccuracy) for r in reports]
    cnn.cuda_free(data.sampledTrainX, -1)
    cnn.cuda_free(data.sampledTrainY, -1)
    cnn.cuda_free(data.weights, -1)
    cnn.cleanup_dataset(C.byref(host), C.byref(data))
    dev.free(arena)
    cnn.fitreSetDatasetFolder(3, None)
    cnn.fitreSetWeightsFolder(None)
