"""Hessian-vector product (R-operator passes): the oracle against float64 double backward, symmetry and the
second-order Taylor remainder (CPU), and the HIP path against the oracle through the C boundary (GPU)."""
import ctypes as C

import numpy as np
import pytest

from oracle import torchref
from fitre_amd.structs import (ACT_TANH, AVG_POOL, CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, MAX_POOL)
from helpers import batch_inputs, build_custom, he_weights, rel_err


def models():
    yield "swish_maxpool_fc", build_custom(6, 8, 8, 2, [dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_SWISH),
                                                        dict(cout=5, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_SWISH)],
                                           [(7, CNN_ACT_SWISH), (4, CNN_ACT_NONE)]), 6
    yield "bn_softplus_avgpool", build_custom(5, 6, 6, 3, [dict(cout=4, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0), bn=True, act=CNN_ACT_SOFTPLUS),
                                                           dict(cout=3, k=3, pad=1, pool=None, bn=True, act=CNN_ACT_SWISH)],
                                              [(5, CNN_ACT_NONE)]), 5
    yield "bn_relu_maxpool", build_custom(7, 8, 8, 1, [dict(cout=3, k=5, pad=2, pool=(MAX_POOL, 2, 2, 0), bn=True, act=CNN_ACT_RELU),
                                                       dict(cout=4, k=3, pad=0, pool=None, bn=False, act=CNN_ACT_SWISH)],
                                          [(6, ACT_TANH), (3, CNN_ACT_NONE)]), 7
    yield "no_bias_unpooled_last", build_custom(4, 5, 5, 2, [dict(cout=3, k=3, pad=1, pool=None, act=CNN_ACT_SWISH)],
                                                [(3, CNN_ACT_NONE)], bias=0), 4


MODELS = {name: (m, b) for name, m, b in models()}


def setup(name, rng):
    model, batch = MODELS[name]
    w = he_weights(model, rng) * 1.5
    x, y = batch_inputs(model, batch, rng)
    v = rng.standard_normal(model.pSize)
    return model, batch, w, x, y, v


def classes_of(model):
    return model.fcLayer[model.lLayers - 1].out


@pytest.mark.parametrize("name", list(MODELS))
def test_oracle_hv_against_double_backward(oracle64, name):
    rng = np.random.default_rng(sum(map(ord, name)))
    model, batch, w, x, y, v = setup(name, rng)
    k = classes_of(model)
    ref = oracle64.gradient(model, w, x, y, k, batch)
    hv = oracle64.hessian_vector(model, w, x, ref["z"], ref["probs"], ref["errors"], ref["dx"], v, k, batch)
    want = torchref.hessian_vector(model, w, x, y, batch, v)
    assert rel_err(hv, want) < 1e-8, name


@pytest.mark.parametrize("name", ["swish_maxpool_fc", "bn_softplus_avgpool"])
def test_oracle_hv_symmetry_and_taylor(oracle64, name):
    rng = np.random.default_rng(7)
    model, batch, w, x, y, v = setup(name, rng)
    k = classes_of(model)
    u = rng.standard_normal(model.pSize)
    ref = oracle64.gradient(model, w, x, y, k, batch)
    args = (model, w, x, ref["z"], ref["probs"], ref["errors"], ref["dx"])
    hv, hu = oracle64.hessian_vector(*args, v, k, batch), oracle64.hessian_vector(*args, u, k, batch)
    assert abs(u @ hv - v @ hu) < 1e-9 * max(1.0, abs(u @ hv))
    if name == "bn_softplus_avgpool":   # smooth everywhere: the remainder of the quadratic model decays like t^3
        g, f0 = ref["gradient"], ref["loss"]
        d = v / np.linalg.norm(v)
        hd = oracle64.hessian_vector(*args, d, k, batch)
        rem = []
        for t in (1e-2, 5e-3, 2.5e-3):
            ft = oracle64.gradient(model, w + t * d, x, y, k, batch)["loss"]
            rem.append(abs(ft - f0 - t * (g @ d) - 0.5 * t * t * (d @ hd)))
        assert rem[0] / rem[1] > 6 and rem[1] / rem[2] > 6, rem   # 8 for an exact Hessian, 4 for a wrong one


# ------------------------------------------------------------------------------------------ GPU
from fitre_amd import lib as L  # noqa: E402

TOL = 1e-4


def gpu_hv(dev, gm, model, batch, v32):
    pv = dev.upload(v32)
    hv = dev.upload(np.full(model.pSize, np.nan, dtype=np.float32))
    ws = dev.alloc(4 * L.cnn.cnnHvMemRequired(C.byref(model)) + 512)
    L.cnn.cnnHv(C.byref(model), C.byref(gm.data), gm.z, gm.probs, gm.errors, gm.dx, pv, hv, 0, batch, ws, None, 0.0)
    out = dev.download(hv, model.pSize)
    for q in (pv, hv, ws):
        dev.free(q)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(MODELS))
def test_gpu_hv_against_oracle_on_the_same_inputs(dev, oracle64, name):
    """cnnHv against the oracle's R passes run on the z / probs / errors / dx the device produced (the ReLU masks
    and pooling selections are functions of z; see the gradient tests)."""
    from helpers import GpuModel
    rng = np.random.default_rng(sum(map(ord, name)) + 3)
    model, batch, w, x, y, v = setup(name, rng)
    w32, x32, v32 = w.astype(np.float32), x.astype(np.float32), v.astype(np.float32)
    gm = GpuModel(dev, model, w32, x32, y, batch)
    gm.gradient()
    got = gpu_hv(dev, gm, model, batch, v32)
    k = classes_of(model)
    want = oracle64.hessian_vector(model, w32, x32, gm.get("z"), gm.get("probs"), gm.get("errors"), gm.get("dx"), v32, k, batch)
    assert np.isfinite(got).all()
    assert rel_err(got, want) < TOL
    # and end to end against double backward (small smooth-enough models: a looser bound)
    assert rel_err(got, torchref.hessian_vector(model, w32, x32, y, batch, v32)) < 5e-4
    gm.release()


@pytest.mark.gpu
def test_gpu_quadratic_model_step(dev, oracle64):
    from helpers import GpuModel
    name = "swish_maxpool_fc"
    rng = np.random.default_rng(11)
    model, batch, w, x, y, v = setup(name, rng)
    w32, x32, v32 = w.astype(np.float32), x.astype(np.float32), v.astype(np.float32)
    gm = GpuModel(dev, model, w32, x32, y, batch)
    gm.gradient()
    g = gm.get("grad")
    hv = gpu_hv(dev, gm, model, batch, v32).astype(np.float64)
    decay = 1e-3
    hv_d = hv + decay * w32                      # the reference adds weightDecay * weights
    vhv, gv, nrm = hv_d @ v32, g.astype(np.float64) @ v32, np.linalg.norm(v32.astype(np.float64))
    for delta in (1e-3, 1e3):
        pv = dev.upload(v32)
        ws = dev.alloc(4 * (L.cnn.cnnHvMemRequired(C.byref(model)) + model.pSize) + 512)
        host = (C.c_float * 3)()
        m = L.cnn.computeQuadraticModel(C.byref(model), C.byref(gm.data), gm.z, gm.probs, gm.errors, gm.dx, gm.grad, pv,
                                        delta, 0, batch, decay, ws, None, host)
        if vhv < 0:
            step = delta / nrm
        else:
            step = min(gv / (vhv + 1e-6), delta / (nrm + 1e-16))
        want = 0.5 * vhv * step * step - gv * step
        assert abs(host[1] - vhv) < 1e-3 * max(1, abs(vhv)) and abs(host[0] - gv) < 1e-3 * max(1, abs(gv))
        assert abs(m - want) < 1e-3 * max(1e-6, abs(want))
        assert rel_err(dev.download(pv, model.pSize), step * v32) < 1e-3
        dev.free(pv)
        dev.free(ws)
    gm.release()


@pytest.mark.gpu
def test_gpu_hv_full_size_vgg_symmetry_and_finite_difference(dev):
    """A network of VGG-11's shape (eight 3x3 convolutions 64..512 with batch norm and swish, FC 512->10), batch 64,
    with average instead of max pooling so that the loss is smooth: u'Hv = v'Hu, and Hv against the central
    difference of the gradient along v (across a max-pool arg-max flip the gradient jumps, which a difference
    quotient sees and a Hessian does not)."""
    from helpers import GpuModel
    batch = 64
    widths, pooled = [64, 128, 256, 256, 512, 512, 512, 512], {0, 1, 3, 5, 7}
    convs = [dict(cout=c, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0) if i in pooled else None, bn=True, act=CNN_ACT_SWISH)
             for i, c in enumerate(widths)]
    model = build_custom(batch, 32, 32, 3, convs, [(10, CNN_ACT_NONE)])
    rng = np.random.default_rng(2024)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    x = x.astype(np.float32)
    u = rng.standard_normal(model.pSize).astype(np.float32)
    # a direction that perturbs every weight by a fraction of its own size, so that a float32 gradient
    # difference stays far above the rounding noise of the gradients
    v = (w * rng.standard_normal(model.pSize)).astype(np.float32)
    gm = GpuModel(dev, model, w, x, y, batch)
    gm.gradient()
    hv, hu = gpu_hv(dev, gm, model, batch, v), gpu_hv(dev, gm, model, batch, u)
    assert np.isfinite(hv).all() and np.isfinite(hu).all()
    a, b = float(u.astype(np.float64) @ hv), float(v.astype(np.float64) @ hu)
    assert abs(a - b) < 2e-3 * max(abs(a), abs(b)), (a, b)
    # central difference of the gradient, projected on a few random directions to average the float32 noise
    eps = 5e-3
    grads = []
    for sign in (1.0, -1.0):
        gm2 = GpuModel(dev, model, (w + sign * eps * v).astype(np.float32), x, y, batch)
        gm2.gradient()
        grads.append(gm2.get("grad").astype(np.float64))
        gm2.release()
    fd = (grads[0] - grads[1]) / (2 * eps)
    for r in (u, v):
        p, q = float(r.astype(np.float64) @ fd), float(r.astype(np.float64) @ hv)
        assert abs(p - q) < 5e-2 * max(abs(p), abs(q)), (p, q)
    gm.release()


@pytest.mark.gpu
def test_gpu_hv_full_size_vgg_against_oracle(dev, oracle64):
    """The benchmark's Hessian-vector configuration at its full size: VGG-11 (batch norm, ReLU, max pooling), batch
    256, a seeded N(0,1) direction; cnnHv against the oracle's R passes on the z / probs / errors / dx the device
    produced.  Per-layer blocks are compared separately so that a small layer cannot hide behind a large one."""
    from helpers import GpuModel, batch_inputs, build_vgg11, he_weights
    batch = 256
    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(0xF17E)
    w32 = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    x32 = x.astype(np.float32)
    v32 = rng.standard_normal(model.pSize).astype(np.float32)
    gm = GpuModel(dev, model, w32, x32, y, batch)
    gm.gradient()
    got = gpu_hv(dev, gm, model, batch, v32)
    want = oracle64.hessian_vector(model, w32, x32, gm.get("z"), gm.get("probs"), gm.get("errors"), gm.get("dx"), v32, 10, batch)
    gm.release()
    assert np.isfinite(got).all()
    assert rel_err(got, want) < TOL
    nl = model.cLayers + model.lLayers
    for l in range(nl):
        a, b = model.wOffsets[l], model.bOffsets[l]
        assert rel_err(got[a:b], want[a:b]) < TOL, "weights of layer %d" % l
