"""Mini-batch selection and augmentation on the device against the CPU oracle
(device/extract_columns.cu, augmentation/dev_crop.cu, dev_flip.cu, dev_normalize.cu, solvers/kfac_da.cu).
Data movement is compared bit for bit; the normalisation within float32 rounding."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import DEVICE_DATASET
from helpers import at, build_lenet, rel_err

pytestmark = pytest.mark.gpu
hip = L.hip

CIFAR10, CIFAR100, IMAGENET = 10, 20, 30
STATS = {CIFAR10: ([0.4914, 0.4822, 0.4465], [0.2470, 0.2435, 0.2616]),
         CIFAR100: ([0.5071, 0.4865, 0.4409], [0.2673, 0.2564, 0.2762]),
         IMAGENET: ([0.4799, 0.4478, 0.3972], [0.2769, 0.2690, 0.2820])}


def ok(rc):
    L.check(rc)


def f32p(values):
    a = np.ascontiguousarray(values, dtype=np.float32)
    return a, a.ctypes.data_as(C.c_void_p)


def test_extract_columns(dev, oracle64):
    rng = np.random.default_rng(1)
    rows, cols = 3072, 50
    src = rng.integers(0, 256, size=rows * cols).astype(np.float32)
    idx = rng.permutation(cols)[:17].astype(np.int32)
    ps, pi = dev.upload(src), dev.upload(idx, np.int32)
    out = dev.zeros(rows * idx.size)
    ok(hip.fitre_hip_extract_columns(out, ps, pi, rows, idx.size))
    np.testing.assert_array_equal(dev.download(out, rows * idx.size), oracle64.extract_columns(src, idx, rows).astype(np.float32))
    ok(hip.fitre_hip_extract_columns(out, ps, pi, rows, 0))   # empty selection: nothing to do
    assert hip.fitre_hip_extract_columns(out, ps, pi, 0, 4) == 2


@pytest.mark.parametrize("C_,N,W,H", [(3, 9, 32, 32), (3, 4, 5, 7), (1, 130, 8, 8), (8, 3, 6, 4)])
def test_crop_flip_steps(dev, oracle64, C_, N, W, H):
    rng = np.random.default_rng(N * W + H)
    x = rng.integers(0, 256, size=C_ * N * W * H).astype(np.float32)
    u = rng.random(2 * N).astype(np.float32)
    px, pu = dev.upload(x), dev.upload(u)
    shifts = dev.zeros(2 * N, np.int32)
    ok(hip.fitre_hip_crop_shifts(pu, 2 * N, 4, shifts))
    want_s = oracle64.crop_shifts(u, N, 4)
    np.testing.assert_array_equal(dev.download(shifts, 2 * N, np.int32), want_s)
    out = dev.zeros(x.size)
    ok(hip.fitre_hip_shift_images(px, N, C_, H, W, shifts, at(shifts, N), -3.0, out))
    want = oracle64.random_crop(x, N, H, W, C_, want_s[:N], want_s[N:], default=-3.0)
    np.testing.assert_array_equal(dev.download(out, x.size), want.astype(np.float32))
    # the same crop from the uniforms, through the one-pass entry point
    ok(hip.fitre_hip_augment_batch(px, 0, N, C_, H, W, pu, 4, -3.0, None, None, None, 1.0, out))
    np.testing.assert_array_equal(dev.download(out, x.size), want.astype(np.float32))
    # flip alone
    pr = rng.random(N).astype(np.float32)
    pr[0] = 0.5   # the boundary: not flipped
    ok(hip.fitre_hip_augment_batch(px, 0, N, C_, H, W, None, 0, 0.0, dev.upload(pr), None, None, 1.0, out))
    np.testing.assert_array_equal(dev.download(out, x.size), oracle64.random_flip(x, N, C_, H, W, pr).astype(np.float32))


@pytest.mark.parametrize("N,W,H,enable", [(16, 32, 32, 1), (5, 8, 6, 1), (7, 32, 32, 0), (256, 32, 32, 1)])
def test_augment_batch_one_pass(dev, oracle64, N, W, H, enable):
    rng = np.random.default_rng(N + W)
    C_ = 3
    sampled = rng.integers(0, 256, size=N * C_ * W * H).astype(np.float32)
    cu, fu = rng.random(2 * N).astype(np.float32), rng.random(N).astype(np.float32)
    mean, std = STATS[CIFAR100]
    (ma, mp), (sa, sp) = f32p(mean), f32p(std)
    out = dev.zeros(sampled.size)
    ok(hip.fitre_hip_augment_batch(dev.upload(sampled), 1, N, C_, H, W, dev.upload(cu) if enable else None, 4, 0.0,
                                   dev.upload(fu) if enable else None, mp, sp, 255.0, out))
    want = oracle64.augment_data(sampled, N, C_, H, W, enable, cu, fu, ma, sa)
    got = dev.download(out, sampled.size)
    assert rel_err(got, want) < 1e-6
    # filled cells are normalised zeros: the same value everywhere they occur
    if enable:
        fill = ((0.0 / 255 - ma) / sa).astype(np.float32)
        shifts = oracle64.crop_shifts(cu, N, 4)
        assert np.any(shifts != 0)
        img = got.reshape(C_, N, W, H)
        n = int(np.argmax(np.abs(shifts[:N]) + np.abs(shifts[N:])))
        moved_in = oracle64.random_flip(oracle64.random_crop(np.ones(sampled.size), N, H, W, C_, shifts[:N], shifts[N:]),
                                        N, C_, H, W, fu).reshape(C_, N, W, H)[:, n] == 0
        for c in range(C_):
            np.testing.assert_allclose(img[c, n][moved_in[c]], fill[c], rtol=1e-6)


def test_augment_batch_argument_errors(dev):
    p = dev.zeros(3 * 4 * 16)
    (ma, mp), (sa, sp) = f32p([0.5] * 3), f32p([0.25, 0.0, 0.25])
    assert hip.fitre_hip_augment_batch(p, 1, 4, 3, 4, 4, None, 0, 0.0, None, None, None, 1.0, p) == 2   # in place with a layout change
    assert hip.fitre_hip_augment_batch(p, 0, 4, 3, 4, 4, None, 0, 0.0, None, mp, sp, 255.0, p) == 2     # zero deviation
    assert b"standard deviation" in hip.fitre_hip_last_error()
    assert hip.fitre_hip_augment_batch(p, 0, 0, 3, 4, 4, None, 0, 0.0, None, None, None, 1.0, dev.zeros(16)) == 2


@pytest.mark.parametrize("enable,dataset", [(1, CIFAR10), (0, CIFAR100), (1, IMAGENET)])
def test_select_and_augment_with_the_reference_names(dev, oracle64, enable, dataset):
    """selectColumnMatrix + augmentData as the KFAC solver calls them (solvers/kfac_trust_region.cu:325-337)."""
    rng = np.random.default_rng(dataset)
    model = build_lenet(8)            # 3 x 32 x 32 input
    N, C_, W, H = 8, 3, 32, 32
    feats, train = C_ * W * H, 40
    X = rng.integers(0, 256, size=feats * train).astype(np.float32)
    Y = rng.integers(1, 11, size=train).astype(np.float32)
    order = rng.permutation(train).astype(np.int32)
    offset = 5
    data = DEVICE_DATASET()
    px, py, pidx = dev.upload(X), dev.upload(Y), dev.upload(order, np.int32)
    sampled = dev.zeros(2 * N * feats)
    labels = dev.zeros(N)
    data.trainSetX, data.trainSetY = px, py
    data.sampledTrainX, data.sampledTrainY = sampled, labels
    data.features, data.trainSizeX = feats, train
    L.cnn.selectColumnMatrix(C.byref(data), N, pidx, offset)
    picked = order[offset:offset + N]
    np.testing.assert_array_equal(dev.download(sampled, N * feats), oracle64.extract_columns(X, picked, feats).astype(np.float32))
    np.testing.assert_array_equal(dev.download(labels, N), Y[picked])

    scratch = dev.zeros(4 * N)
    seed = 77
    ok(hip.fitre_hip_random_seed(seed))
    L.cnn.augmentData(C.byref(model), C.byref(data), offset, N, scratch, None, enable, dataset)
    assert data.currentBatch == sampled.value + 4 * N * feats
    got = dev.download(at(sampled, N * feats), N * feats)
    # the uniforms the call drew: samples (never read), 2*samples (crop), samples (flip)
    stream = oracle64.uniform_stream(seed, 0, 4 * N)
    cu, fu = stream[N:3 * N], stream[3 * N:4 * N]
    mean, std = STATS[dataset]
    want = oracle64.augment_data(X.reshape(train, feats)[picked].reshape(-1), N, C_, H, W, enable, cu, fu,
                                 np.float32(mean), np.float32(std))
    assert rel_err(got, want) < 1e-6
    if enable:
        plain = oracle64.augment_data(X.reshape(train, feats)[picked].reshape(-1), N, C_, H, W, 0, cu, fu, np.float32(mean), np.float32(std))
        assert rel_err(got, plain) > 1e-3   # the augmentation did move pixels


def test_generalization_error_sweeps(dev, oracle64):
    """computeTestGeneralizationErrors / computeTrainGeneralizationErrors (functions/cnn_accuracy.cu:61-174): whole-set
    loss and accuracy in batches, against the oracle's forward pass on the oracle's normalised batches.  20 images in
    batches of 8: the test sweep ends with a batch of 4, the training sweep stops before it (as the reference does)
    and still divides by 20."""
    from helpers import GpuModel, he_weights
    rng = np.random.default_rng(31)
    batch, size, classes = 8, 20, 10
    model = build_lenet(batch)
    feats = 3 * 32 * 32
    X = rng.integers(0, 256, size=(size, feats)).astype(np.float32)
    Y = rng.integers(1, classes + 1, size=size).astype(np.float32)
    w = he_weights(model, rng).astype(np.float32) * np.float32(0.3)
    gm = GpuModel(dev, model, w, np.zeros(batch * feats, np.float32), np.ones(batch, np.float32), batch)
    data = gm.data
    setX, setY = dev.upload(X.reshape(-1)), dev.upload(Y)
    sampledX, sampledY = dev.zeros(2 * batch * feats), dev.zeros(batch)
    data.trainSetX, data.trainSetY, data.testSetX, data.testSetY = setX.value, setY.value, setX.value, setY.value
    data.trainSizeX, data.testSizeX, data.features, data.datasetType = size, size, feats, CIFAR10
    data.sampledTrainX, data.sampledTrainY = sampledX.value, sampledY.value
    pinned = (C.c_float * 4)()
    gm.scratch.nextPageLckPtr = C.cast(pinned, C.c_void_p).value
    mean, std = STATS[CIFAR10]

    def reference(limit_full_batches):
        nll, hits, idx = 0.0, 0, 0
        while idx < size:
            n = min(batch, size - idx)
            if limit_full_batches and n < batch:
                break
            xb = oracle64.augment_data(X[idx:idx + n].reshape(-1), n, 3, 32, 32, 0, np.zeros(2 * n), np.zeros(n),
                                       np.float32(mean), np.float32(std))
            loss, _, probs, _ = oracle64.forward(model, w, xb, Y[idx:idx + n], classes, n, mode=30)
            nll += loss * n
            hits += int((np.argmax(probs.reshape(n, classes), axis=1) + 1 == Y[idx:idx + n]).sum())
            idx += n
        return nll / size, 100.0 * hits / size

    like, acc = C.c_float(), C.c_float()
    L.cnn.computeTestGeneralizationErrors(C.byref(model), C.byref(data), C.byref(gm.scratch), gm.z, gm.probs, gm.errors,
                                          C.byref(like), C.byref(acc))
    want_l, want_a = reference(False)
    assert abs(like.value - want_l) < 1e-4 * abs(want_l) and abs(acc.value - want_a) < 1e-4
    L.cnn.computeTrainGeneralizationErrors(C.byref(model), C.byref(data), None, C.byref(gm.scratch), gm.z, gm.probs, gm.errors,
                                           C.byref(like), C.byref(acc))
    want_l, want_a = reference(True)
    assert abs(like.value - want_l) < 1e-4 * abs(want_l) and abs(acc.value - want_a) < 1e-4
    for q in (setX, setY, sampledX, sampledY):
        dev.free(q)
    gm.release()
