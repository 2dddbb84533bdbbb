"""One KFAC trust-region mini-batch after another, through the library's reference-named entry points in
the order the reference's solver calls them (solvers/kfac_trust_region.cu:299-613): batch selection and
augmentation, forward, backward, the sampled-target backward for the Fisher factors, both factor/inverse
passes, the natural gradient, the quadratic model along it (a Hessian-vector product), the step, the new
loss, rho and the radius update.  The loop itself is the caller's (here: this test); what is checked is
that the pieces compose on the device the way the solver needs them to: the predicted reduction is
negative, rho is close to one for a small radius, and training a small network on a separable synthetic
set brings the loss down."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import KFAC_CURVATURE_INFO
from helpers import GpuModel, at, build_lenet, he_weights

pytestmark = pytest.mark.gpu
hip = L.hip
CIFAR10 = 10


def synthetic_set(rng, classes, per_class, features):
    """Pixel images (0..255) around one random template per class: separable, so a few steps learn it."""
    templates = rng.integers(40, 216, size=(classes, features)).astype(np.float32)
    X = np.concatenate([np.clip(templates[c] + 25.0 * rng.standard_normal((per_class, features)), 0, 255)
                        for c in range(classes)]).astype(np.float32)
    Y = np.repeat(np.arange(1, classes + 1), per_class).astype(np.float32)
    return X, Y   # X: one image per row = one column of the features x images matrix


def test_kfac_trust_region_minibatches(dev):
    rng = np.random.default_rng(2024)
    batch, classes = 64, 10
    model = build_lenet(batch, bn=True)
    feats = 3 * 32 * 32
    X, Y = synthetic_set(rng, classes, 64, feats)
    train = X.shape[0]
    w0 = he_weights(model, rng).astype(np.float32)
    gm = GpuModel(dev, model, w0, np.zeros(batch * feats, np.float32), np.ones(batch, np.float32), batch)
    data, P = gm.data, model.pSize

    trainX, trainY = dev.upload(X.reshape(-1)), dev.upload(Y)
    sampledX, sampledY = dev.zeros(2 * batch * feats), dev.zeros(batch)
    data.trainSetX, data.trainSetY = trainX.value, trainY.value
    data.sampledTrainX, data.sampledTrainY = sampledX.value, sampledY.value
    data.trainSizeX, data.features = train, feats

    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    layers = model.cLayers + model.lLayers
    oinv, linv = dev.zeros(info.OmegaZOffsets[layers]), dev.zeros(info.LambdaGOffsets[layers])
    ngrad, dist_grad, dist_dx = dev.zeros(P), dev.zeros(P), dev.zeros(model.zSize)
    dist_target, dist_err = dev.zeros(batch), dev.zeros(max(model.maxDeltaSize, classes * batch))
    info.regLambda, info.dampGamma, info.momentum = 0.0, 0.1, 0.0
    info.OmegaZInv, info.LambdaGInv = oinv.value, linv.value
    info.gradient, info.nGradient = gm.grad.value, ngrad.value
    need = max(L.cnn.kfacInverseMemRequired(C.byref(model), batch), L.cnn.kfacNaturalGradientMemRequired(C.byref(model)),
               L.cnn.cnnHvMemRequired(C.byref(model)) + P, L.cnn.cnnBackwardMemRequired(C.byref(model)) + 2 * model.maxDeltaSize,
               4 * batch)
    ws = dev.zeros(need + 1024)
    pinned = (C.c_float * 4)()
    ok = L.check

    delta, max_delta, min_delta = 0.5, 4.0, 1e-3
    ok(hip.fitre_hip_random_seed(99))
    losses, rhos, accs = [], [], []
    for epoch in range(2):
        order = dev.upload(rng.permutation(train).astype(np.int32), np.int32)
        for offset in range(0, train - batch + 1, batch):
            L.cnn.selectColumnMatrix(C.byref(data), batch, order, offset)
            L.cnn.augmentData(C.byref(model), C.byref(data), offset, batch, ws, None, 1, CIFAR10)
            loss = gm.forward()                        # z, probs, loss errors
            gm.backward()                              # gradient, dx
            # sampled targets -> second backward: the deltas of the Fisher factors
            L.cnn.computeDistributionErrors(gm.probs, dist_target, dist_err, batch, classes, ws, None)
            L.cnn.cnnBackward(C.byref(model), C.byref(data), at(ws, 2 * model.maxDeltaSize), gm.z, dist_grad, dist_dx, dist_err,
                              ws, offset, batch, None)
            L.cnn.computeOmegaZ(C.byref(info), C.byref(model), C.byref(data), batch, None, gm.z, oinv, model.zOffsets,
                                model.zztOffsets, ws, None, None, None, None)
            L.cnn.computeLambdaDelta(C.byref(info), C.byref(model), batch, dist_dx, None, linv, model.zOffsets, model.zztOffsets,
                                     ws, None, None, None, None)
            L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws, None)
            # quadratic model along the natural gradient; scales ngrad to the step
            m_err = L.cnn.computeQuadraticModel(C.byref(model), C.byref(data), gm.z, gm.probs, gm.errors, gm.dx, gm.grad, ngrad,
                                                delta, offset, batch, 0.0, ws, None, pinned)
            assert np.isfinite(m_err) and m_err < 0, (epoch, offset, m_err)
            ok(hip.fitre_hip_axpy(P, -1.0, ngrad, gm.w))
            new_loss = L.cnn.evaluateCNNModel(C.byref(model), C.byref(data), C.byref(gm.scratch), gm.z, gm.probs, gm.errors,
                                              offset, batch)
            acc = L.cnn.computeAccuracy(gm.probs, sampledY, batch, classes, ws, pinned)
            rho = (new_loss - loss) / (m_err - 1e-16)
            assert np.isfinite(new_loss) and np.isfinite(rho)
            if rho > 0.75:
                delta = min(max_delta, 2 * delta)
            if rho < 0.25:
                delta = max(min_delta, 0.5 * delta)
            if rho < 1e-4 or new_loss > 10 * loss:
                ok(hip.fitre_hip_axpy(P, 1.0, ngrad, gm.w))   # revert
                new_loss = loss
            losses.append((loss, new_loss))
            rhos.append(rho)
            accs.append(acc)
        dev.free(order)

    # loss on each fresh batch before its step (measured run: 3.25 -> 0.55, accuracy 12 % -> 100 %, rho 0.64..0.99)
    first, last = losses[0][0], np.mean([l for l, _ in losses[-3:]])
    assert first > 1.5                      # ten classes, random weights: above log(10)
    assert last < 0.35 * first, losses
    assert all(after < before for before, after in losses), losses   # every accepted step lowers its batch's loss
    assert np.mean(accs[-3:]) > np.mean(accs[:3]) + 20.0, accs
    # the quadratic model is a usable predictor: most steps are accepted with rho of order one
    good = [r for r in rhos if 0.1 < r < 3.0]
    assert len(good) >= len(rhos) // 2, rhos
    assert np.isfinite(dev.download(gm.w, P)).all()
    for q in (trainX, trainY, sampledX, sampledY, oinv, linv, ngrad, dist_grad, dist_dx, dist_target, dist_err, ws):
        dev.free(q)
    gm.release()
