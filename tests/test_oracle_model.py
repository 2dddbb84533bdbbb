"""Whole-model pins of the oracle: float64 autograd of the textbook layers (every z and dx slot, the
flat gradient) and the reference's own Taylor-remainder test (utilities/cnn_derivative_test.cu:124-223)."""
import numpy as np
import pytest

from oracle import torchref
from fitre_amd.structs import (ACT_LOGISTIC, ACT_TANH, AVG_POOL, CNN_ACT_ELU, CNN_ACT_NONE, CNN_ACT_RELU,
                               CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, MAX_POOL, NO_POOL, PERFORM_NO_BATCH_NORM)
from helpers import batch_inputs, build_custom, build_lenet, he_weights, num_classes, rel_err


def small_models():
    B = 4
    yield "lenet_like", build_custom(B, 12, 12, 3, [
        dict(cout=4, k=5, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU),
        dict(cout=6, k=3, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU)], [(9, CNN_ACT_RELU), (7, CNN_ACT_RELU), (5, CNN_ACT_NONE)]), B
    yield "lenet_bn", build_custom(B, 12, 12, 3, [
        dict(cout=4, k=5, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU, bn=True),
        dict(cout=6, k=3, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU, bn=True)], [(9, CNN_ACT_RELU), (5, CNN_ACT_NONE)]), B
    yield "vgg_like_bn", build_custom(B, 8, 8, 3, [
        dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU, bn=True),
        dict(cout=8, k=3, pad=1, pool=None, act=CNN_ACT_RELU, bn=True),
        dict(cout=8, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU, bn=True)], [(10, CNN_ACT_NONE)]), B
    yield "vgg_like_swish_nobias", build_custom(B, 8, 8, 3, [
        dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_SWISH),
        dict(cout=6, k=3, pad=1, pool=None, act=CNN_ACT_SWISH, bn=True)], [(10, CNN_ACT_NONE)], bias=0), B
    yield "alexnet_like", build_custom(2, 35, 35, 3, [
        dict(cout=4, k=11, stride=4, pad=2, pool=(MAX_POOL, 3, 2, 0), act=CNN_ACT_RELU),
        dict(cout=6, k=5, pad=2, pool=None, act=CNN_ACT_RELU),
        dict(cout=5, k=3, pad=1, pool=(MAX_POOL, 3, 2, 0), act=CNN_ACT_RELU)], [(12, CNN_ACT_RELU), (6, CNN_ACT_NONE)]), 2
    yield "avgpool_softplus_tanh", build_custom(3, 9, 9, 2, [
        dict(cout=3, k=3, pad=1, pool=(AVG_POOL, 3, 3, 0), act=CNN_ACT_SOFTPLUS),
        dict(cout=4, k=2, pool=(MAX_POOL, 3, 2, 1), act=CNN_ACT_ELU)], [(6, ACT_TANH), (5, ACT_LOGISTIC), (4, CNN_ACT_NONE)]), 3
    yield "rectangular", build_custom(2, 6, 10, 2, [
        dict(cout=3, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_RELU, bn=True)], [(4, CNN_ACT_NONE)]), 2


MODELS = list(small_models())


def floored_loss(logits, y):
    """mean(-log(softmax + 1e-10)): the reference adds 1e-10 to every probability
    (functions/softmax_loss.cu:55), which shows in the loss when a target probability is tiny."""
    import torch
    p = torch.softmax(torch.tensor(logits), 1).numpy() + 1e-10
    return float(np.mean(-np.log(p[np.arange(len(y)), np.asarray(y, dtype=int) - 1])))


def slot(arr, model, l, name):
    c, p = model.convLayer[l], model.poolLayer[l]
    base = model.zOffsets[l + 1]
    n = model.batchSize
    V = c.outHeight * c.outWidth * c.outChannels * n
    if name == "conv":
        return arr[base:base + V]
    if name == "bn":
        return arr[base + c.batchNormOffset:base + c.batchNormOffset + V]
    if name == "act":
        return arr[base + c.activationOffset:base + c.activationOffset + V]
    if name == "pool":
        P = p.outHeight * p.outWidth * c.outChannels * n
        return arr[base + c.poolOffset:base + c.poolOffset + P]
    raise KeyError(name)


@pytest.mark.parametrize("name,model,batch", MODELS, ids=[m[0] for m in MODELS])
def test_oracle_matches_autograd(oracle64, name, model, batch):
    rng = np.random.default_rng(sum(map(ord, name)))
    w = he_weights(model, rng, bias_scale=0.1)
    x, y = batch_inputs(model, batch, rng)
    got = oracle64.gradient(model, w, x, y, num_classes(model), batch)
    ref = torchref.run(model, w, x, y, batch)

    assert abs(got["loss"] - floored_loss(ref["logits"], y)) < 1e-9
    assert rel_err(got["gradient"], ref["gradient"]) < 1e-9
    last = model.cLayers - 1
    for l in range(model.cLayers):
        st = ref["stages"][l]
        c = model.convLayer[l]
        for key in st:
            if l == last and key == ("pool" if "pool" in st else "act"):
                continue  # rewritten in place into the FC layout, checked below
            np.testing.assert_allclose(slot(got["z"], model, l, key), torchref.from_nchw(st[key]), atol=1e-9,
                                       err_msg="z %s layer %d" % (key, l))
        # dx slots (functions/cnn_backward.cu:513, 605, 653): + 0 = dL/d(act out), + activationOffset =
        # dL/d(act in), + batchNormOffset = dL/d(conv out)
        np.testing.assert_allclose(slot(got["dx"], model, l, "conv"), torchref.from_nchw(st["act"].grad), atol=1e-10)
        pre = st["bn"] if c.batchNorm != PERFORM_NO_BATCH_NORM else st["conv"]
        np.testing.assert_allclose(slot(got["dx"], model, l, "act"), torchref.from_nchw(pre.grad), atol=1e-10)
        if c.batchNorm != PERFORM_NO_BATCH_NORM:
            np.testing.assert_allclose(slot(got["dx"], model, l, "bn"), torchref.from_nchw(st["conv"].grad), atol=1e-10)
    # FC input = torch's flatten of NCHW: [N][C*h*w]
    st = ref["stages"][last]
    feat = st["pool"] if "pool" in st else st["act"]
    key = "pool" if "pool" in st else "act"
    np.testing.assert_allclose(slot(got["z"], model, last, key), feat.detach().reshape(batch, -1).numpy().reshape(-1), atol=1e-9)
    # FC slabs: output then saved pre-activation; dx = dL/d(pre-activation)
    for f in range(model.lLayers):
        fc = model.fcLayer[f]
        base = model.zOffsets[model.cLayers + f + 1]
        cnt = fc.out * batch
        fs = ref["fc_stages"][f]
        np.testing.assert_allclose(got["z"][base:base + cnt], fs["out"].detach().numpy().reshape(-1), atol=1e-9)
        np.testing.assert_allclose(got["z"][base + fc.offset:base + fc.offset + cnt], fs["pre"].detach().numpy().reshape(-1), atol=1e-9)
        np.testing.assert_allclose(got["dx"][base:base + cnt], fs["pre"].grad.numpy().reshape(-1), atol=1e-10)
    # probabilities and loss errors, class fastest
    import torch
    p = torch.softmax(torch.tensor(ref["logits"]), 1).numpy().reshape(-1)
    np.testing.assert_allclose(got["probs"], p, atol=1e-9)


def test_weight_decay_term(oracle64):
    name, model, batch = MODELS[0]
    rng = np.random.default_rng(5)
    w = he_weights(model, rng)
    x, y = batch_inputs(model, batch, rng)
    g0 = oracle64.gradient(model, w, x, y, num_classes(model), batch, 0.0)["gradient"]
    g1 = oracle64.gradient(model, w, x, y, num_classes(model), batch, 0.25)["gradient"]
    np.testing.assert_allclose(g1 - g0, 0.25 * w, atol=1e-12)


def smooth_models():
    """No max pooling and no ReLU: the loss is smooth in the weights, so the remainder test is exact."""
    yield build_custom(4, 8, 8, 3, [
        dict(cout=4, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0), act=CNN_ACT_SWISH, bn=True),
        dict(cout=6, k=3, pad=1, pool=None, act=CNN_ACT_SWISH, bn=True),
        dict(cout=5, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0), act=CNN_ACT_SWISH, bn=True)], [(10, CNN_ACT_NONE)]), 4
    yield build_custom(3, 9, 9, 2, [
        dict(cout=3, k=3, pad=1, pool=(AVG_POOL, 3, 3, 0), act=CNN_ACT_SOFTPLUS),
        dict(cout=4, k=2, pool=None, act=CNN_ACT_SWISH)], [(6, ACT_TANH), (5, ACT_LOGISTIC), (4, CNN_ACT_NONE)]), 3
    yield build_custom(2, 19, 19, 2, [
        dict(cout=3, k=7, stride=3, pad=2, pool=(AVG_POOL, 2, 2, 0), act=CNN_ACT_SWISH)], [(5, CNN_ACT_SWISH), (3, CNN_ACT_NONE)], bias=0), 2


@pytest.mark.parametrize("model,batch", list(smooth_models()), ids=["bn_swish", "softplus_tanh_logistic", "strided_nobias"])
def test_taylor_remainder_decays_quadratically(oracle64, model, batch):
    """f(W0 + d) - f(W0) - g'd = O(|d|^2): halving d must quarter the remainder
    (utilities/cnn_derivative_test.cu:112-124, 197, 222-223: W0, Wr uniform * 0.1, Wr halved each step)."""
    rng = np.random.default_rng(23)
    W0 = rng.uniform(0, 1, model.pSize) * 0.1
    Wr = rng.uniform(0, 1, model.pSize) * 0.1
    x, y = batch_inputs(model, batch, rng)
    classes = num_classes(model)
    base = oracle64.gradient(model, W0, x, y, classes, batch)
    f0, g = base["loss"], base["gradient"]
    rem = []
    for i in range(10):
        d = Wr / 2 ** i
        fd = oracle64.forward(model, W0 + d, x, y, classes, batch)[0]
        rem.append(abs(fd - f0 - np.dot(g, d)))
    ratios = [rem[i] / rem[i + 1] for i in range(len(rem) - 1) if rem[i + 1] > 1e-12]
    assert len(ratios) >= 5, rem
    assert all(3.5 < r < 4.6 for r in ratios[2:]), ratios
    # a gradient with the last layer's block dropped must fail the same test
    bad = g.copy()
    bad[model.wOffsets[model.cLayers + model.lLayers - 1]:] = 0
    rem_bad = [abs(oracle64.forward(model, W0 + Wr / 2 ** i, x, y, classes, batch)[0] - f0 - np.dot(bad, Wr / 2 ** i))
               for i in (6, 7)]
    assert rem_bad[0] / rem_bad[1] < 3.0


def test_full_size_lenet_against_autograd(oracle64):
    """The LeNet configuration at its real layer shapes (batch trimmed to keep the CPU suite short)."""
    batch = 16
    model = build_lenet(batch, bn=True)
    rng = np.random.default_rng(31)
    w = he_weights(model, rng)
    x, y = batch_inputs(model, batch, rng)
    got = oracle64.gradient(model, w, x, y, 10, batch)
    ref = torchref.run(model, w, x, y, batch, want_intermediates=False)
    assert abs(got["loss"] - floored_loss(ref["logits"], y)) < 1e-9
    assert rel_err(got["gradient"], ref["gradient"]) < 1e-9
