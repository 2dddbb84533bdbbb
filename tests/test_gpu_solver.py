"""The sub-sampled KFAC trust-region solver's host loop (solvers/kfac_trust_region.cu:92-660) run end to end
through subsampledTrustRegionKFAC on a small separable synthetic set, plus its helpers against numpy:
updateRunningStats (solvers/kfac_inverses.cu:106-124) and the packed running averages of
computeSpeedUpOmegaZ / computeSpeedUpLambdaDelta (:386-446, :699-755)."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import DEVICE_DATASET, KFAC_CURVATURE_INFO, KFAC_TR_EPOCH_REPORT, SCRATCH_AREA, TRUST_REGION_PARAMS
from helpers import at, build_lenet, he_weights

pytestmark = pytest.mark.gpu
hip = L.hip
CIFAR10 = 10
libc = C.CDLL(None)


def synthetic_sets(rng, classes, per_class, test_per_class, features):
    """Pixel images (0..255) around one random template per class; columns of a features x images matrix."""
    templates = rng.integers(40, 216, size=(classes, features)).astype(np.float32)

    def draw(count):
        X = np.concatenate([np.clip(templates[c] + 25.0 * rng.standard_normal((count, features)), 0, 255)
                            for c in range(classes)]).astype(np.float32)
        Y = np.repeat(np.arange(1, classes + 1), count).astype(np.float32)
        order = rng.permutation(X.shape[0])
        return X[order], Y[order]
    return draw(per_class), draw(test_per_class)


def run_solver(dev, inverse_freq, epochs, seed, check_grad=0, momentum=0.0, reg_lambda=0.0, vgg=False):
    rng = np.random.default_rng(seed)
    classes, feats = 10, 3 * 32 * 32
    if vgg:   # the benchmark's network at its batch size: 1 300 training images, 5 mini-batches per pass
        from helpers import build_vgg11
        batch = 256
        model = build_vgg11(batch, bn=True)
        (X, Y), (TX, TY) = synthetic_sets(rng, classes, 130, 30, feats)
    else:
        batch = 64
        model = build_lenet(batch, bn=True)
        (X, Y), (TX, TY) = synthetic_sets(rng, classes, 45, 13, feats)     # 450 training images: 7 mini-batches per pass
    w = dev.upload(he_weights(model, rng).astype(np.float32))
    trainX, trainY, testX, testY = dev.upload(X.reshape(-1)), dev.upload(Y), dev.upload(TX.reshape(-1)), dev.upload(TY)

    data = DEVICE_DATASET()
    data.trainSetX, data.trainSetY, data.testSetX, data.testSetY = trainX.value, trainY.value, testX.value, testY.value
    data.trainSizeX = data.trainSizeY = X.shape[0]
    data.testSizeX = data.testSizeY = TX.shape[0]
    data.weights, data.numClasses, data.datasetType = w.value, classes, CIFAR10
    data.features, data.height, data.width = feats, 32, 32

    info = KFAC_CURVATURE_INFO()
    info.regLambda, info.dampGamma, info.momentum, info.stats_decay = reg_lambda, (0.05 if vgg else 0.1), momentum, 0.9
    info.checkGrad, info.inverseFreq = check_grad, inverse_freq
    tr = TRUST_REGION_PARAMS()
    tr.delta, tr.minDelta, tr.maxDelta, tr.maxIters = 0.5, 1e-3, 4.0, epochs

    need = L.cnn.kfacTrustRegionMemRequired(C.byref(model), C.byref(data), C.byref(info))
    arena = dev.zeros(need)
    host_reals = L.cnn.kfacTrustRegionHostMemRequired(C.byref(data)) + 1024
    host_arena = (C.c_float * host_reals)()
    pinned = (C.c_float * 8)()
    scratch = SCRATCH_AREA()
    scratch.devWorkspace = scratch.nextDevPtr = arena.value
    scratch.hostWorkspace = scratch.nextHostPtr = C.addressof(host_arena)
    scratch.pageLckWorkspace = scratch.nextPageLckPtr = C.addressof(pinned)

    libc.srand(seed)
    L.check(hip.fitre_hip_random_seed(seed))
    L.cnn.subsampledTrustRegionKFAC(C.byref(model), C.byref(data), None, C.byref(info), C.byref(tr), C.byref(scratch), 0, 0)
    reports = (KFAC_TR_EPOCH_REPORT * epochs)()
    assert L.cnn.kfacTrustRegionReports(reports, epochs) == epochs
    weights = dev.download(w, model.pSize)
    L.cnn.cuda_free(data.sampledTrainX, -1)
    L.cnn.cuda_free(data.sampledTrainY, -1)
    for q in (w, trainX, trainY, testX, testY, arena):
        dev.free(q)
    return list(reports), weights, tr.delta


@pytest.mark.parametrize("inverse_freq,epochs", [(1, 3), (3, 5)])
def test_solver_trains_a_separable_set(dev, inverse_freq, epochs):
    # measured: every mini-batch's own factors: accuracy 90+ % after three passes; factors from running averages,
    # inverted every third mini-batch: 33 / 55 / 73 % after passes one to three (the whole-set figures are
    # taken with the batch-norm layers' running statistics, which lag behind the weights)
    reports, weights, delta = run_solver(dev, inverse_freq, epochs, seed=7)
    assert np.isfinite(weights).all()
    assert [r.iteration for r in reports] == list(range(epochs))
    assert all(r.miniBatches == 7 for r in reports)         # 450 images, batch 64: the last 2 images are left out
    assert 1e-3 <= delta <= 4.0 and abs(reports[-1].delta - delta) < 1e-6
    losses = [r.trainLikelihood for r in reports]
    assert np.isfinite(losses).all() and losses[-1] < 1.0, losses   # ten classes, random weights: log(10) = 2.3
    assert losses[-1] < losses[0] or losses[0] < 0.2, losses
    assert reports[-1].trainAccuracy > 70.0 and reports[-1].testAccuracy > 70.0, [(r.trainAccuracy, r.testAccuracy) for r in reports]
    assert sum(r.rejectedSteps for r in reports) <= 7, [r.rejectedSteps for r in reports]
    assert all(r.weightNorm > 0 and r.seconds > 0 for r in reports)


def test_solver_with_gradient_check_momentum_and_weight_decay(dev):
    """The branch that compares the natural-gradient step with the plain gradient step (checkGrad), a momentum
    term on the step and L2 regularisation in gradient and curvature: the loop still trains."""
    reports, weights, delta = run_solver(dev, 1, 3, seed=5, check_grad=1, momentum=0.2, reg_lambda=1e-4)
    assert np.isfinite(weights).all()
    losses = [r.trainLikelihood for r in reports]
    assert np.isfinite(losses).all() and losses[-1] < 1.5 and losses[-1] < losses[0], losses
    assert reports[-1].trainAccuracy > 60.0, [r.trainAccuracy for r in reports]


def test_solver_on_the_benchmark_network(dev):
    """VGG-11 with batch norm at batch 256 (factors up to order 4609, batched inverses, 2.5 GB of arena): two passes
    over a separable synthetic set.  Measured: 24 ms per mini-batch; whole-set accuracy (taken with the batch-norm
    layers' running statistics, which lag behind the weights) 10 % after the first pass of five mini-batches, 77 % after
    the second."""
    reports, weights, delta = run_solver(dev, 1, 3, seed=3, vgg=True)
    assert np.isfinite(weights).all()
    assert all(r.miniBatches == 5 for r in reports)
    losses = [r.trainLikelihood for r in reports]
    assert np.isfinite(losses).all() and losses[-1] < losses[0] and losses[-1] < 1.0, losses
    assert reports[-1].trainAccuracy > 70.0 and reports[-1].testAccuracy > 70.0, [(r.trainAccuracy, r.testAccuracy) for r in reports]


def test_solver_is_reproducible(dev):
    a = run_solver(dev, 1, 1, seed=11)
    b = run_solver(dev, 1, 1, seed=11)
    np.testing.assert_array_equal(a[1], b[1])       # same seeds, same shuffles and draws, deterministic kernels
    assert a[0][0].trainLikelihood == b[0][0].trainLikelihood


def test_update_running_stats(dev):
    rng = np.random.default_rng(3)
    n = 10007
    src, upd = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    ps, pu = dev.upload(src), dev.upload(upd)
    L.cnn.updateRunningStats(ps, pu, n, 0.9)
    np.testing.assert_allclose(dev.download(ps, n), 0.9 * src + 0.1 * upd, rtol=0, atol=2e-6)
    L.cnn.updateRunningStats(ps, pu, n, 0.0)
    np.testing.assert_array_equal(dev.download(ps, n), upd)
    dev.free(ps), dev.free(pu)


def test_running_averages_are_packed_at_zzt_offsets(dev):
    rng = np.random.default_rng(5)
    batch = 8
    model = build_lenet(batch, bn=True)
    feats = 3 * 32 * 32
    info = KFAC_CURVATURE_INFO()
    info.stats_decay = 0.81                       # decay sqrt(0.81) = 0.9
    z0, z1 = (rng.standard_normal(model.zSize).astype(np.float32) for _ in range(2))
    x0, x1 = (rng.standard_normal(batch * feats).astype(np.float32) for _ in range(2))
    pz, px = dev.upload(z0), dev.upload(x0)
    d_in, d_z, d_l = dev.zeros(batch * feats), dev.zeros(model.zztSize), dev.zeros(model.zztSize)
    data = DEVICE_DATASET()
    data.currentBatch, data.features = px.value, feats

    def packed(z, omega):
        out = np.zeros(model.zztSize, np.float32)
        for i in range(model.cLayers):
            c, p = model.convLayer[i], model.poolLayer[i]
            if omega:
                cells = c.outHeight * c.outWidth if p.type == 2 else p.outHeight * p.outWidth   # NO_POOL = 2
                src = model.zOffsets[i + 1] + c.outputOffset
            else:
                cells = c.outHeight * c.outWidth
                src = model.zOffsets[i + 1] + (c.batchNormOffset if c.batchNorm else c.activationOffset)
            n = cells * c.outChannels * batch
            out[model.zztOffsets[i + 1]:model.zztOffsets[i + 1] + n] = z[src:src + n]
        for l in range(model.lLayers):
            k = l + 1 + model.cLayers
            n = model.fcLayer[l].out * batch
            out[model.zztOffsets[k]:model.zztOffsets[k] + n] = z[model.zOffsets[k]:model.zOffsets[k] + n]
        return out

    for omega in (True, False):
        target = d_z if omega else d_l

        def call(count):
            if omega:
                L.cnn.computeSpeedUpOmegaZ(C.byref(info), C.byref(model), C.byref(data), batch, pz, model.zOffsets, d_in, d_z,
                                           model.zztOffsets, count)
            else:
                L.cnn.computeSpeedUpLambdaDelta(C.byref(info), C.byref(model), batch, pz, d_l, model.zOffsets, model.zztOffsets, count)
        L.check(hip.fitre_hip_copy_h2d(pz, z0.ctypes.data_as(C.c_void_p), z0.nbytes))
        L.check(hip.fitre_hip_copy_h2d(px, x0.ctypes.data_as(C.c_void_p), x0.nbytes))
        call(0)
        first = dev.download(target, model.zztSize)
        want0 = packed(z0, omega)
        touched = want0 != 0
        np.testing.assert_array_equal(first[touched], want0[touched])
        if omega:
            np.testing.assert_array_equal(dev.download(d_in, x0.size), x0)
        L.check(hip.fitre_hip_copy_h2d(pz, z1.ctypes.data_as(C.c_void_p), z1.nbytes))
        L.check(hip.fitre_hip_copy_h2d(px, x1.ctypes.data_as(C.c_void_p), x1.nbytes))
        call(5)
        second = dev.download(target, model.zztSize)
        want1 = 0.9 * want0 + 0.1 * packed(z1, omega)
        np.testing.assert_allclose(second[touched], want1[touched], rtol=0, atol=3e-6)
        if omega:
            np.testing.assert_allclose(dev.download(d_in, x0.size), 0.9 * x0 + 0.1 * x1, rtol=0, atol=3e-6)
    for q in (pz, px, d_in, d_z, d_l):
        dev.free(q)
