"""cnnForward / cnnBackward / computeCNNGradient through the C boundary against the float64 oracle:
loss, probabilities, every z and dx slot and the flat gradient; then size-independent properties at
the full benchmark shapes."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import (CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SWISH, MAX_POOL, NO_POOL, PERFORM_NO_BATCH_NORM)
from helpers import GpuModel, batch_inputs, build_alexnet, build_custom, build_lenet, build_vgg11, he_weights, num_classes, rel_err
from test_oracle_model import MODELS, slot, smooth_models

pytestmark = pytest.mark.gpu
TOL = 1e-4


def compare_with_oracle(dev, oracle64, model, batch, seed, weight_decay=0.0, tol=TOL, end_to_end=False):
    """Forward: every z slot, probabilities, errors and the loss against the float64 forward.
    Backward: the flat gradient and every dx slot against the float64 cnnBackward restatement run on
    the SAME inputs cnnBackward received (the z the GPU produced, and its loss errors) -- ReLU masks
    and pooling selections are functions of z, so both sides then take identical decisions and the
    comparison measures arithmetic only.  end_to_end additionally compares with the all-float64
    pipeline (small models, where no pre-activation sits within rounding of a kink)."""
    rng = np.random.default_rng(seed)
    w = he_weights(model, rng, bias_scale=0.05)
    x, y = batch_inputs(model, batch, rng)
    w32, x32 = w.astype(np.float32), x.astype(np.float32)
    classes = num_classes(model)
    gm = GpuModel(dev, model, w32, x32, y, batch)
    loss = gm.gradient(weight_decay)
    z, dx, grad = gm.get("z"), gm.get("dx"), gm.get("grad")
    probs, errors = gm.get("probs"), gm.get("errors")
    gm.release()

    # ---- forward
    fl, fz, fprobs, ferrors = oracle64.forward(model, w32, x32, y, classes, batch)
    assert abs(loss - fl) < 1e-5 * max(1.0, abs(fl))
    assert rel_err(probs, fprobs) < tol and rel_err(errors, ferrors) < tol
    for l in range(model.cLayers):
        c, p = model.convLayer[l], model.poolLayer[l]
        names = ["conv", "act"] + (["bn"] if c.batchNorm != PERFORM_NO_BATCH_NORM else []) + (["pool"] if p.type != NO_POOL else [])
        for nme in names:
            assert rel_err(slot(z, model, l, nme), slot(fz, model, l, nme)) < tol, "z %s of layer %d" % (nme, l)
    for f in range(model.lLayers):
        base = model.zOffsets[model.cLayers + f + 1]
        cnt = model.fcLayer[f].out * batch
        assert rel_err(z[base:base + 2 * cnt], fz[base:base + 2 * cnt]) < tol, "z of FC layer %d" % f

    # ---- backward on identical inputs
    rgrad, rdx = oracle64.backward(model, w32, x32, z.astype(np.float64), errors.astype(np.float64), batch)
    rgrad = rgrad + weight_decay * w32.astype(np.float64)
    assert rel_err(grad, rgrad) < tol, "flat gradient"
    nl = model.cLayers + model.lLayers
    for l in range(nl):  # per-layer blocks: a small layer must not hide behind a large one
        a = model.wOffsets[l]
        b = model.bOffsets[l] if model.bias else (model.wOffsets[l + 1] if l + 1 < nl else model.pSize)
        assert rel_err(grad[a:b], rgrad[a:b]) < tol, "weight gradient of layer %d" % l
        if model.bias:
            e = model.wOffsets[l + 1] if l + 1 < nl else model.pSize
            if l < model.cLayers and model.convLayer[l].batchNorm != PERFORM_NO_BATCH_NORM:
                # behind batch norm the bias gradient is a sum that cancels to zero; what is left is rounding
                cl = model.convLayer[l]
                cancel = np.abs(slot(rdx, model, l, "bn")).reshape(cl.outChannels, -1).sum(1).max()
                assert np.abs(grad[b:e] - rgrad[b:e]).max() < 1e-5 * cancel, "bias gradient of layer %d" % l
            else:
                assert rel_err(grad[b:e], rgrad[b:e]) < tol, "bias gradient of layer %d" % l
    for l in range(model.cLayers):
        c = model.convLayer[l]
        for nme in ["conv", "act"] + (["bn"] if c.batchNorm != PERFORM_NO_BATCH_NORM else []):
            assert rel_err(slot(dx, model, l, nme), slot(rdx, model, l, nme)) < tol, "dx %s of layer %d" % (nme, l)
    for f in range(model.lLayers):
        base = model.zOffsets[model.cLayers + f + 1]
        cnt = model.fcLayer[f].out * batch
        assert rel_err(dx[base:base + cnt], rdx[base:base + cnt]) < tol, "dx of FC layer %d" % f

    if end_to_end:
        ref = oracle64.gradient(model, w32, x32, y, classes, batch, weight_decay)
        assert rel_err(grad, ref["gradient"]) < tol, "flat gradient, all-float64 pipeline"
    return grad, rgrad


@pytest.mark.parametrize("name,model,batch", MODELS, ids=[m[0] for m in MODELS])
def test_small_models_every_slot(dev, oracle64, name, model, batch):
    compare_with_oracle(dev, oracle64, model, batch, seed=sum(map(ord, name)), end_to_end=True)


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_smooth_models(dev, oracle64, idx):
    model, batch = list(smooth_models())[idx]
    compare_with_oracle(dev, oracle64, model, batch, seed=idx, weight_decay=0.01, end_to_end=True)


def test_lenet_batch128(dev, oracle64):
    compare_with_oracle(dev, oracle64, build_lenet(128, bn=False), 128, seed=11)


def test_lenet_bn_batch1024(dev, oracle64):
    compare_with_oracle(dev, oracle64, build_lenet(1024, bn=True), 1024, seed=12)


def test_lenet_batch1024_on_two_lanes(dev, oracle64):
    """Without batch norm and above the lane limit: the pooling steps folded into the launches above them, the weight
    gradients on the second lane and their reductions held back to one launch, against the oracle."""
    model = build_lenet(1024, bn=False)
    assert L.cnn.fitreBackwardUsesLanes(C.byref(model), 1024) == 1
    compare_with_oracle(dev, oracle64, model, 1024, seed=13)


def test_vgg11_bn_reduced_batch(dev, oracle64):
    # the benchmark network at its real layer shapes; batch trimmed so that the oracle takes seconds
    compare_with_oracle(dev, oracle64, build_vgg11(16, bn=True), 16, seed=13)


def test_vgg11_swish_reference_network(dev, oracle64):
    compare_with_oracle(dev, oracle64, build_vgg11(8, bn=True, act=CNN_ACT_SWISH, bias=0), 8, seed=14)


@pytest.mark.parametrize("reader,convs", [("readVGG13", 10), ("readVGG16", 13), ("readVGG19", 16)])
def test_deeper_vgg_members_as_the_reference_builds_them(dev, oracle64, reader, convs):
    """nn/read_vgg.c:345-750: swish after every convolution, batch norm, bias; forward, loss and gradient against the oracle."""
    import ctypes as C
    from fitre_amd import lib as L
    from fitre_amd.structs import CNN_MODEL
    model = CNN_MODEL()
    getattr(L.cnn, reader)(C.byref(model), 6, 32, 32, 10, 3, 1, 1, 10)
    assert model.cLayers == convs and model.lLayers == 1 and model.fcLayer[0].in_ == 512
    compare_with_oracle(dev, oracle64, model, 6, seed=30 + convs)


@pytest.mark.parametrize("which,bn", [("lenet", 0), ("lenet", 1), ("alexnet", 0), ("alexnet", 1)])
def test_small_reference_networks_as_the_reference_builds_them(dev, oracle64, which, bn):
    """readLenetCNN (swish, average pools) and readAlexNetCNN (5x5 / pad 2, 3 / 2 / 1 max pools), nn/read_nn.c:500-700,
    nn/read_alexnet.c:14-215."""
    import ctypes as C
    from fitre_amd import lib as L
    from fitre_amd.structs import CNN_MODEL
    model = CNN_MODEL()
    if which == "lenet":
        L.cnn.readLenetCNN(C.byref(model), 3, 32, 32, 12, 1, bn)
    else:
        L.cnn.readAlexNetCNN(C.byref(model), 12, 32, 32, 10, 1, bn)
    compare_with_oracle(dev, oracle64, model, 12, seed=40 + bn)


def test_alexnet_reduced(dev, oracle64):
    # AlexNet layer types at a reduced image (67 -> 16 -> 7 -> 3 -> 1): 11x11/s4/p2, 5x5/p2, 3x3, maxpool 3/2
    compare_with_oracle(dev, oracle64, build_alexnet(4, classes=50, size=67), 4, seed=15)


def test_smaller_batch_than_model(dev, oracle64):
    """The solvers call with curBatchSize <= model->batchSize (last mini-batch of an epoch)."""
    model = build_custom(8, 8, 8, 3, [dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=True)], [(5, CNN_ACT_NONE)])
    rng = np.random.default_rng(5)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, 5, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, 5)
    loss = gm.gradient()
    ref_model = build_custom(8, 8, 8, 3, [dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=True)], [(5, CNN_ACT_NONE)])
    ref = oracle64.gradient(ref_model, w, x.astype(np.float32), y, 5, 5)
    assert abs(loss - ref["loss"]) < 1e-5
    assert rel_err(gm.get("grad"), ref["gradient"]) < TOL
    gm.release()


def test_scratch_cursors_are_restored(dev):
    model = build_lenet(4)
    rng = np.random.default_rng(6)
    x, y = batch_inputs(model, 4, rng)
    gm = GpuModel(dev, model, he_weights(model, rng).astype(np.float32), x.astype(np.float32), y, 4)
    before = (gm.scratch.nextDevPtr, gm.scratch.nextHostPtr, gm.scratch.nextPageLckPtr)
    gm.gradient()
    assert (gm.scratch.nextDevPtr, gm.scratch.nextHostPtr, gm.scratch.nextPageLckPtr) == before
    gm.release()


# ------------------------------------------------------------------ full benchmark shapes: properties
@pytest.fixture(scope="module")
def vgg_full(dev):
    batch = 256
    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(2024)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
    yield gm, w
    gm.release()


def test_vgg11_full_size_properties(vgg_full, dev):
    gm, w = vgg_full
    model, batch = gm.model, gm.batch
    loss = gm.forward()
    assert np.isfinite(loss) and 1.0 < loss < 10.0
    probs = gm.get("probs").reshape(batch, 10)
    np.testing.assert_allclose(probs.sum(1), 1.0, atol=1e-5)
    err = gm.get("errors").reshape(batch, 10)
    np.testing.assert_allclose(err.sum(1), 0.0, atol=1e-7)
    gm.backward()
    g1 = gm.get("grad")
    assert np.isfinite(g1).all() and np.abs(g1).max() > 0
    # bitwise run-to-run determinism (no atomics anywhere on the path)
    gm.backward()
    np.testing.assert_array_equal(g1, gm.get("grad"))
    # batch-norm backward invariants per channel: sum(dx) = 0 = the bias gradient, sum(dx * zhat) ~ 0
    z, dx = gm.get("z"), gm.get("dx")
    for l in (0, 3, 7):
        c = model.convLayer[l]
        per = batch * c.outHeight * c.outWidth
        d = slot(dx, model, l, "bn").reshape(c.outChannels, per).astype(np.float64)
        zh = slot(z, model, l, "bn").reshape(c.outChannels, per).astype(np.float64)
        scale = np.abs(d).sum(1).max()
        assert np.abs(d.sum(1)).max() < 1e-5 * scale
        assert np.abs((d * zh).sum(1)).max() < 1e-3 * scale
        b = g1[model.bOffsets[l]:model.bOffsets[l] + c.outChannels]
        assert np.abs(b).max() < 1e-5 * scale
    # FC bias gradient = column sums of the loss errors; FC weight gradient = errors x features
    fcw = g1[model.wOffsets[8]:model.wOffsets[8] + 5120].reshape(512, 10).astype(np.float64)
    feat = z[model.zOffsets[8] + model.convLayer[7].outputOffset:][:512 * batch].reshape(batch, 512).astype(np.float64)
    want = feat.T @ err.astype(np.float64)
    assert rel_err(fcw, want) < TOL
    np.testing.assert_allclose(g1[model.bOffsets[8]:model.bOffsets[8] + 10], err.astype(np.float64).sum(0), atol=1e-6)


def test_vgg11_full_size_backward_is_linear_in_delta(vgg_full, dev):
    """cnnBackward is linear in the incoming errors: B(2*delta) = 2*B(delta) up to rounding,
    and exactly so for a power-of-two factor."""
    gm, w = vgg_full
    gm.forward()
    gm.backward()
    g1 = gm.get("grad")
    L.check(L.hip.fitre_hip_scal(10 * gm.batch, 2.0, gm.errors))
    gm.backward()
    g2 = gm.get("grad")
    np.testing.assert_array_equal(g2, 2 * g1)


def test_vgg11_full_size_one_lane_gives_the_same_bits(vgg_full, dev):
    """At this size cnnBackward spreads its launches over the lanes; with the lanes switched off everything is queued
    on one stream.  The kernels and the order of every sum are the same, so gradient and dx must be too, bit for bit."""
    gm, w = vgg_full
    gm.forward()
    gm.backward()
    grad, dx = gm.get("grad"), gm.get("dx")
    L.check(L.hip.fitre_hip_lanes_enable(0))
    try:
        L.check(L.hip.fitre_hip_memset(gm.grad, 0xFF, 4 * gm.model.pSize))
        gm.backward()
        np.testing.assert_array_equal(gm.get("grad").view(np.uint32), grad.view(np.uint32))
        np.testing.assert_array_equal(gm.get("dx").view(np.uint32), dx.view(np.uint32))
    finally:
        L.check(L.hip.fitre_hip_lanes_enable(1))


@pytest.mark.parametrize("name", ["lenet_bn_b1024", "lenet_b1024", "alexnet_b64", "vgg11_no_bn_b32"])
def test_forced_lanes_give_the_same_bits(dev, name):
    """Networks on either side of cnnBackward's lane limit and without the batch-norm steps the lanes were built around
    (LeNet + batch norm at batch 1024: just above it; AlexNet; a VGG-11 without batch norm at a small batch) and the
    override fitreSetBackwardLanes: one lane and the lanes give the same gradient and dx, bit for bit."""
    from helpers import GpuModel, batch_inputs, build_alexnet, build_lenet, build_vgg11, he_weights
    if name == "lenet_bn_b1024":
        batch, model = 1024, build_lenet(1024, bn=True)
    elif name == "lenet_b1024":  # without batch norm: folded pooling steps and held-back reductions, on two lanes
        batch, model = 1024, build_lenet(1024, bn=False)
    elif name == "alexnet_b64":
        batch, model = 64, build_alexnet(64)
    else:
        batch, model = 32, build_vgg11(32, bn=False)
    rng = np.random.default_rng(len(name))
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
    gm.forward()
    results = []
    try:
        for mode in (0, 1):
            L.cnn.fitreSetBackwardLanes(mode)
            assert L.cnn.fitreBackwardUsesLanes(C.byref(model), batch) == mode
            L.check(L.hip.fitre_hip_memset(gm.grad, 0xFF, 4 * model.pSize))
            gm.forward()
            gm.backward()
            results.append((gm.get("grad").view(np.uint32), gm.get("dx").view(np.uint32)))
    finally:
        L.cnn.fitreSetBackwardLanes(-1)
    gm.release()
    assert np.isfinite(results[0][0].view(np.float32)).all()
    np.testing.assert_array_equal(results[0][0], results[1][0])
    np.testing.assert_array_equal(results[0][1], results[1][1])


def test_vgg11_full_size_directional_derivative(vgg_full, dev):
    """g'd against a central difference of the loss along a random direction d (fp32 forward)."""
    gm, w = vgg_full
    gm.forward()
    gm.backward()
    g = gm.get("grad").astype(np.float64)
    rng = np.random.default_rng(99)
    d = rng.standard_normal(w.size)
    d *= 1.0 / np.linalg.norm(d)
    h = 2e-2
    losses = []
    for sgn in (+1, -1):
        L.check(L.hip.fitre_hip_copy_h2d(gm.w, (w + np.float32(sgn * h) * d.astype(np.float32)).ctypes.data_as(C.c_void_p), 4 * w.size))
        losses.append(gm.forward())
    L.check(L.hip.fitre_hip_copy_h2d(gm.w, w.ctypes.data_as(C.c_void_p), 4 * w.size))
    fd = (losses[0] - losses[1]) / (2 * h)
    assert abs(fd - np.dot(g, d)) < 0.05 * abs(np.dot(g, d)) + 1e-3


# ------------------------------------------------------------------ AlexNet at its full size: properties
@pytest.fixture(scope="module")
def alexnet_full(dev):
    """3 x 224 x 224, batch 64, 1000 classes: 11x11/s4, 5x5, 3x3 convolutions, max-pool 3/2, FC 9216-4096-4096-1000
    (62 M parameters).  Too large for the CPU oracle in a test; checked through what holds at any size."""
    batch = 64
    model = build_alexnet(batch)
    rng = np.random.default_rng(4242)
    w = he_weights(model, rng).astype(np.float32)
    # He-normal weights on N(0,1) pixels give logits in the hundreds; the loss then sits on the floor the
    # reference puts under the probabilities (p + 1e-10, functions/softmax_loss.cu) and stops following the
    # gradient.  A small last layer keeps the softmax in its smooth range.
    last = model.cLayers + model.lLayers - 1
    w[model.wOffsets[last]:model.bOffsets[last]] *= np.float32(0.02)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
    yield gm, w
    gm.release()


def test_alexnet_full_size_properties(alexnet_full, dev):
    gm, w = alexnet_full
    model, batch = gm.model, gm.batch
    assert model.cLayers == 5 and model.lLayers == 3 and model.fcLayer[0].in_ == 9216
    loss = gm.forward()
    assert np.isfinite(loss) and 5.0 < loss < 12.0        # log(1000) = 6.9 for uninformed predictions
    probs = gm.get("probs").reshape(batch, 1000)
    np.testing.assert_allclose(probs.sum(1), 1.0, atol=1e-5)
    err = gm.get("errors").reshape(batch, 1000)
    gm.backward()
    g1 = gm.get("grad")
    assert np.isfinite(g1).all()
    for l in range(8):                                      # every layer receives a gradient
        n = model.bOffsets[l] - model.wOffsets[l]
        assert np.abs(g1[model.wOffsets[l]:model.wOffsets[l] + n]).max() > 0, l
    gm.backward()
    np.testing.assert_array_equal(g1, gm.get("grad"))       # bitwise run-to-run determinism
    # last FC layer in closed form: bias gradient = column sums of the loss errors, weight gradient = errors x input
    z = gm.get("z")
    last = model.cLayers + model.lLayers - 1
    f = model.fcLayer[model.lLayers - 1]
    zin = z[model.zOffsets[last]:][:f.in_ * batch].reshape(batch, f.in_).astype(np.float64)
    want = zin.T @ err.astype(np.float64)
    got = g1[model.wOffsets[last]:model.wOffsets[last] + f.in_ * f.out].reshape(f.in_, f.out)
    assert rel_err(got, want) < TOL
    np.testing.assert_allclose(g1[model.bOffsets[last]:model.bOffsets[last] + f.out], err.astype(np.float64).sum(0), atol=1e-6)
    # linear in the incoming errors, exactly for a power of two
    L.check(L.hip.fitre_hip_scal(1000 * batch, 2.0, gm.errors))
    gm.backward()
    np.testing.assert_array_equal(gm.get("grad"), 2 * g1)


def test_alexnet_full_size_directional_derivative(alexnet_full, dev):
    """g'd against a central difference of the loss along a random direction d (fp32 forward)."""
    gm, w = alexnet_full
    gm.forward()
    gm.backward()
    g = gm.get("grad").astype(np.float64)
    rng = np.random.default_rng(98)
    d = rng.standard_normal(w.size).astype(np.float32)
    d *= np.float32(1.0 / np.linalg.norm(d.astype(np.float64)))
    h = 5e-2
    losses = []
    for sgn in (+1, -1):
        L.check(L.hip.fitre_hip_copy_h2d(gm.w, (w + np.float32(sgn * h) * d).ctypes.data_as(C.c_void_p), 4 * w.size))
        losses.append(gm.forward())
    L.check(L.hip.fitre_hip_copy_h2d(gm.w, w.ctypes.data_as(C.c_void_p), 4 * w.size))
    fd = (losses[0] - losses[1]) / (2 * h)
    gd = float(np.dot(g, d.astype(np.float64)))
    assert abs(fd - gd) < 0.05 * abs(gd) + 1e-3, (fd, gd)


def test_vgg11_full_size_against_the_oracle(dev, oracle64):
    """The benchmark network at the benchmark batch (256): every z and dx slot and the flat gradient against the
    float64 oracle (tens of seconds of host time on the GPU box's cores)."""
    compare_with_oracle(dev, oracle64, build_vgg11(256, bn=True), 256, seed=21)


def test_alexnet_full_size_against_the_oracle(dev, oracle64):
    """AlexNet at 3 x 224 x 224, batch 64, 1000 classes against the float64 oracle: 11x11 / stride 4 and 5x5
    convolutions, 3/2 max pooling, FC 9216-4096-4096-1000."""
    compare_with_oracle(dev, oracle64, build_alexnet(64), 64, seed=22)


def test_backward_pass_leaves_the_device_layer_settings_as_it_found_them(vgg_full, dev):
    """cnnBackward plans some weight gradients for a share of the chip and holds small layers' reductions back while it runs;
    after it returns the device layer is back at its defaults: a weight gradient called directly gives the bits it gives
    with the share set to the whole chip explicitly, and a small layer's call writes its result at once."""
    from helpers import conv_shape
    gm, w = vgg_full
    gm.forward()
    gm.backward()
    hip = L.hip
    rng = np.random.default_rng(5)
    # a 3 x 3 layer the share would apply to
    shape = conv_shape(32, 64, 128, 16, 16, 3, 1, 1)
    x = dev.upload(rng.standard_normal(64 * 32 * 256).astype(np.float32))
    d = dev.upload(rng.standard_normal(128 * 32 * 256).astype(np.float32))
    nb = hip.fitre_hip_conv_weight_grad_workspace(C.byref(shape))
    ws, dw = dev.alloc(nb), dev.zeros(128 * 64 * 9)
    L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), x, d, dw, ws, nb))
    after = dev.download(dw, 128 * 64 * 9).view(np.uint32)
    L.check(hip.fitre_hip_weight_grad_share(8))
    L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), x, d, dw, ws, nb))
    np.testing.assert_array_equal(dev.download(dw, 128 * 64 * 9).view(np.uint32), after)
    for q in (x, d, ws, dw):
        dev.free(q)
    # a LeNet-sized layer: the reduction is not held back
    lenet = build_lenet(16, bn=False)
    wl = he_weights(lenet, rng).astype(np.float32)
    xl, yl = batch_inputs(lenet, 16, rng)
    g2 = GpuModel(dev, lenet, wl, xl.astype(np.float32), yl, 16)
    g2.forward()
    g2.backward()
    g2.release()
    shape = conv_shape(8, 3, 6, 32, 32, 5, 1, 0)
    x = dev.upload(rng.standard_normal(3 * 8 * 1024).astype(np.float32))
    d = dev.upload(rng.standard_normal(6 * 8 * 28 * 28).astype(np.float32))
    nb = max(hip.fitre_hip_conv_weight_bias_grad_workspace(C.byref(shape)), 256)
    ws, dw, db = dev.alloc(nb), dev.upload(np.full(6 * 75, np.nan, np.float32)), dev.upload(np.full(6, np.nan, np.float32))
    L.check(hip.fitre_hip_conv_weight_bias_grad(C.byref(shape), x, d, dw, db, ws, nb))
    assert np.isfinite(dev.download(dw, 6 * 75)).all() and np.isfinite(dev.download(db, 6)).all()
    for q in (x, d, ws, dw, db):
        dev.free(q)
