"""The fully connected model family (functions/eval_gradient.cu): oracle pins against torch autograd and
closed forms (CPU), and the HIP path against the oracle through the C boundary (GPU)."""
import ctypes as C

import numpy as np
import pytest
import torch

from fitre_amd import lib as L
from fitre_amd.structs import (ACT_LINEAR, ACT_LOGISTIC, ACT_SOFTMAX, ACT_TANH, DEVICE_DATASET, FULL_DATASET,
                               MODEL_TYPE_CLASSIFICATION, MODEL_TYPE_MSE, NN_MODEL, SAMPLED_DATASET, SCRATCH_AREA, TEST_DATA,
                               TRAIN_DATA)
from helpers import rel_err

TOL = 1e-4


def build_nn(sizes, acts, kind, points):
    m = NN_MODEL()
    L.cnn.fitre_build_nn(C.byref(m), (C.c_int * len(sizes))(*sizes), (C.c_int * len(acts))(*acts), len(acts), kind, points)
    L.cnn.initRZOffsets(C.byref(m), points)
    L.cnn.initSampledZOffsets(C.byref(m), points)
    L.cnn.initSampledROffsets(C.byref(m), points)
    return m


CASES = {
    "autoencoder_logistic": ([12, 7, 3, 7, 12], [ACT_LOGISTIC, ACT_LINEAR, ACT_TANH, ACT_LOGISTIC], MODEL_TYPE_MSE),
    "regression_linear": ([9, 6, 4], [ACT_TANH, ACT_LINEAR], MODEL_TYPE_MSE),
    "classifier_softmax": ([10, 8, 5], [ACT_LOGISTIC, ACT_SOFTMAX], MODEL_TYPE_CLASSIFICATION),
    "one_layer_logistic": ([6, 6], [ACT_LOGISTIC], MODEL_TYPE_MSE),
}


def make_data(name, n, rng):
    sizes, acts, kind = CASES[name]
    m = build_nn(sizes, acts, kind, n)
    w = rng.standard_normal(m.pSize) * 0.4
    x = rng.standard_normal((n, sizes[0]))          # column-major features x n: sample-major memory
    if acts[-1] == ACT_SOFTMAX:
        y = np.eye(sizes[-1])[rng.integers(0, sizes[-1], n)]
    elif acts[-1] == ACT_LOGISTIC:
        y = rng.random((n, sizes[-1]))
    else:
        y = rng.standard_normal((n, sizes[-1]))
    return m, w, x, y


def torch_loss(m, w, x, y):
    """The loss whose gradient the reference computes: mean over points of squared error (linear head),
    Bernoulli negative log-likelihood of the logits (logistic head) or cross entropy (softmax head)."""
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    h = torch.tensor(x, dtype=torch.float64)
    nl = m.numLayers
    logits = None
    for i in range(nl):
        out, inn = m.layerSizes[i + 1], m.layerSizes[i]
        W = wt[m.wOffsets[i]:m.wOffsets[i] + out * inn].reshape(inn, out).t()   # column-major out x in
        b = wt[m.bOffsets[i]:m.bOffsets[i] + out]
        a = h @ W.t() + b
        logits = a
        act = m.actFuns[i]
        h = {ACT_LOGISTIC: torch.sigmoid, ACT_TANH: torch.tanh, ACT_LINEAR: lambda t: t,
             ACT_SOFTMAX: lambda t: torch.softmax(t, dim=1)}[act](a)
    yt = torch.tensor(y, dtype=torch.float64)
    head = m.actFuns[nl - 1]
    n = x.shape[0]
    if head == ACT_LINEAR:
        loss = ((yt - h) ** 2).sum() / n
        shown = -loss                      # the reference reports -(1/n) * sum of squares for this head
    elif head == ACT_LOGISTIC:
        loss = -(yt * logits - torch.nn.functional.softplus(logits)).sum() / n
        shown = loss
    else:
        loss = -(yt * torch.log(h)).sum() / n
        shown = loss
    loss.backward()
    return float(shown.detach()), wt.grad.numpy(), h.detach().numpy()


@pytest.mark.parametrize("name", list(CASES))
def test_oracle_gradient_against_autograd(oracle64, name):
    rng = np.random.default_rng(sum(map(ord, name)))
    n = 11
    m, w, x, y = make_data(name, n, rng)
    ll, merr, grad, z, dx = oracle64.nn_gradient(m, w, x.reshape(-1), y.reshape(-1), n)
    shown, want, out = torch_loss(m, w, x, y)
    assert abs(ll - shown) < 1e-12 * max(1, abs(shown))
    np.testing.assert_allclose(grad, want, atol=1e-12 * max(1, np.abs(want).max()))
    zl = z[m.zOffsets[m.numLayers]:m.zOffsets[m.numLayers] + out.size].reshape(out.shape)
    np.testing.assert_allclose(zl, out, atol=1e-13)
    if CASES[name][2] == MODEL_TYPE_MSE:
        assert abs(merr - ((y - out) ** 2).sum() / n) < 1e-12
    else:
        assert merr == 0


def torch_net(m, wt, x, upto=None):
    """(last pre-activation, last output) of the first `upto` layers (all by default) at the flat parameters wt."""
    h = torch.tensor(x, dtype=torch.float64)
    a = None
    for i in range(m.numLayers if upto is None else upto):
        out, inn = m.layerSizes[i + 1], m.layerSizes[i]
        W = wt[m.wOffsets[i]:m.wOffsets[i] + out * inn].reshape(inn, out).t()
        a = h @ W.t() + wt[m.bOffsets[i]:m.bOffsets[i] + out]
        h = {ACT_LOGISTIC: torch.sigmoid, ACT_TANH: torch.tanh, ACT_LINEAR: lambda t: t,
             ACT_SOFTMAX: lambda t: torch.softmax(t, dim=1)}[m.actFuns[i]](a)
    return a, h


def torch_nll(m, wt, x, y):
    logits, h = torch_net(m, wt, x)
    yt = torch.tensor(y, dtype=torch.float64)
    if m.actFuns[m.numLayers - 1] == ACT_LOGISTIC:
        return -(yt * logits - torch.nn.functional.softplus(logits)).sum() / x.shape[0]
    return -(yt * torch.log(h)).sum() / x.shape[0]


HV_CASES = ["autoencoder_logistic", "classifier_softmax", "one_layer_logistic"]


@pytest.mark.parametrize("name", HV_CASES)
def test_oracle_hessian_vector_product_against_double_backward(oracle64, name):
    """hessianVec (functions/eval_hessian_vec.cu) is the Hessian of the loss whose gradient computeGradient
    returns, times the vector: pinned by differentiating autograd's gradient once more."""
    rng = np.random.default_rng(sum(map(ord, name)) + 1)
    n = 9
    m, w, x, y = make_data(name, n, rng)
    v = rng.standard_normal(m.pSize)
    _, _, grad, z, dx = oracle64.nn_gradient(m, w, x.reshape(-1), y.reshape(-1), n)
    got = oracle64.nn_hessian_vec(m, w, v, x.reshape(-1), n, z, dx)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    g, = torch.autograd.grad(torch_nll(m, wt, x, y), wt, create_graph=True)
    np.testing.assert_allclose(g.detach().numpy(), grad, atol=1e-12)
    want, = torch.autograd.grad(g @ torch.tensor(v), wt)
    np.testing.assert_allclose(got, want.numpy(), atol=1e-11 * max(1, np.abs(want.numpy()).max()))
    # symmetry of the Hessian: u' H v == v' H u
    u = rng.standard_normal(m.pSize)
    hu = oracle64.nn_hessian_vec(m, w, u, x.reshape(-1), n, z, dx)
    assert abs(u @ got - v @ hu) < 1e-10 * max(1, abs(u @ got))


@pytest.mark.parametrize("name", HV_CASES)
def test_oracle_gauss_newton_product(oracle64, name):
    """Without the top layer's VW' dx term the product is J' H_L J v (J: logits by parameters, H_L: the head's
    Hessian in the logits); with it (as eval_gauss_newton_hessian_vec.cu:262-275 has it) the difference is that
    term back-propagated through the layers below, -(1/n) vjp(z_{L-1}; VW_L' (y - out))."""
    rng = np.random.default_rng(sum(map(ord, name)) + 2)
    n = 8
    m, w, x, y = make_data(name, n, rng)
    v = rng.standard_normal(m.pSize)
    _, _, _, z, dx = oracle64.nn_gradient(m, w, x.reshape(-1), y.reshape(-1), n)
    plain = oracle64.nn_hessian_vec(m, w, v, x.reshape(-1), n, z, dx, gauss_newton=True, top_layer_term=False)
    as_reference = oracle64.nn_hessian_vec(m, w, v, x.reshape(-1), n, z, dx, gauss_newton=True, top_layer_term=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    logits_of = lambda p: torch_net(m, p, x)[0]
    logits, ju = torch.autograd.functional.jvp(logits_of, wt, torch.tensor(v))
    out = torch.sigmoid(logits) if m.actFuns[m.numLayers - 1] == ACT_LOGISTIC else torch.softmax(logits, dim=1)
    if m.actFuns[m.numLayers - 1] == ACT_LOGISTIC:
        hju = out * (1 - out) * ju
    else:
        hju = out * ju - out * (out * ju).sum(dim=1, keepdim=True)
    _, want = torch.autograd.functional.vjp(logits_of, wt, hju / n)
    np.testing.assert_allclose(plain, want.numpy(), atol=1e-11 * max(1, np.abs(want.numpy()).max()))
    # positive semi-definite
    assert v @ plain > -1e-12
    nl = m.numLayers
    if nl == 1:
        np.testing.assert_array_equal(as_reference, plain)
        return
    o, i = m.layerSizes[nl], m.layerSizes[nl - 1]
    VW = torch.tensor(v[m.wOffsets[nl - 1]:m.wOffsets[nl - 1] + o * i]).reshape(i, o).t()
    cot = (torch.tensor(y) - out) @ VW                               # n x in: (VW' dx)' per point
    _, extra = torch.autograd.functional.vjp(lambda p: torch_net(m, p, x, upto=nl - 1)[1], wt, cot)
    np.testing.assert_allclose(as_reference - plain, -extra.numpy() / n, atol=1e-11 * max(1, np.abs(extra.numpy()).max()))
    assert np.abs(as_reference - plain).max() > 1e-6                 # the term is there


@pytest.mark.parametrize("name", HV_CASES)
def test_oracle_second_order_taylor_remainder(oracle64, name):
    """utilities/derivative_test.cu:150-199 for this family: f(w + e v) - f(w) - e g'v - e^2/2 v'Hv shrinks like e^3."""
    rng = np.random.default_rng(sum(map(ord, name)) + 3)
    n = 10
    m, w, x, y = make_data(name, n, rng)
    v = rng.standard_normal(m.pSize)
    v /= np.linalg.norm(v)
    f0, _, g, z, dx = oracle64.nn_gradient(m, w, x.reshape(-1), y.reshape(-1), n)
    hv = oracle64.nn_hessian_vec(m, w, v, x.reshape(-1), n, z, dx)
    rem = []
    for e in (1e-1, 5e-2, 2.5e-2):
        f1 = oracle64.nn_forward(m, w + e * v, x.reshape(-1), y.reshape(-1), n, n)[0]
        rem.append(abs(f1 - f0 - e * (g @ v) - 0.5 * e * e * (v @ hv)))
    assert rem[0] > 1e-9                                # not trivially zero
    for a, b in zip(rem, rem[1:]):
        assert 6.0 < a / b < 10.5, rem                  # halving e divides the remainder by about 8


def test_oracle_hessian_vector_refuses_the_linear_head(oracle64):
    m, w, x, y = make_data("regression_linear", 5, np.random.default_rng(0))
    _, _, _, z, dx = oracle64.nn_gradient(m, w, x.reshape(-1), y.reshape(-1), 5)
    with pytest.raises(ValueError):
        oracle64.nn_hessian_vec(m, w, w, x.reshape(-1), 5, z, dx)


def test_oracle_offsets_follow_the_reference_arithmetic(oracle64):
    m = build_nn([5, 4, 3], [ACT_LOGISTIC, ACT_LINEAR], MODEL_TYPE_MSE, 10)
    assert (m.wOffsets[0], m.bOffsets[0], m.wOffsets[1], m.bOffsets[1], m.pSize) == (0, 20, 24, 36, 39)
    assert (m.zOffsets[0], m.zOffsets[1], m.zOffsets[2], m.zSize) == (0, 50, 90, 120)   # slots sized by the layer below
    assert (m.rZOffsets[0], m.rZOffsets[1], m.rZOffsets[2], m.rFullSize) == (0, 40, 70, 70)
    assert L.cnn.nnGradientMemRequired(C.byref(m), 10) > L.cnn.nnForwardMemRequired(C.byref(m), 10) > 0


# ------------------------------------------------------------------------------------------ GPU
def device_setup(dev, m, w, x, y, n, sampled=False):
    data = DEVICE_DATASET()
    px, py, pw = dev.upload(x.reshape(-1)), dev.upload(y.reshape(-1)), dev.upload(w)
    data.features = m.layerSizes[0]
    if sampled:
        data.sampledTrainX, data.sampleSize = px.value, n
    else:
        data.trainSetX, data.trainSetY, data.trainSizeX, data.trainSizeY = px.value, py.value, n, n
        data.testSetX, data.testSetY, data.testSizeX, data.testSizeY = px.value, py.value, n, n
    need = L.cnn.nnGradientMemRequired(C.byref(m), n) + m.zSize + m.rFullSize + 4096
    arena = dev.zeros(2 * need)
    scratch = SCRATCH_AREA()
    scratch.devWorkspace = scratch.nextDevPtr = arena.value
    return data, scratch, pw


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("n", [11, 300])
def test_gpu_gradient_against_oracle(dev, oracle64, name, n):
    rng = np.random.default_rng(sum(map(ord, name)) + n)
    m, w, x, y = make_data(name, n, rng)
    w32, x32, y32 = w.astype(np.float32), x.astype(np.float32), y.astype(np.float32)
    data, scratch, pw = device_setup(dev, m, w32, x32, y32, n)
    z, dx, grad = dev.zeros(m.zSize), dev.zeros(m.rFullSize), dev.upload(np.full(m.pSize, np.nan, np.float32))
    ll, merr = C.c_float(), C.c_float()
    L.cnn.computeGradient(C.byref(m), C.byref(data), C.byref(scratch), pw, z, dx, grad, C.byref(ll), C.byref(merr), FULL_DATASET)
    oll, omerr, ograd, oz, odx = oracle64.nn_gradient(m, w32, x32.reshape(-1), y32.reshape(-1), n)
    assert abs(ll.value - oll) < TOL * max(1, abs(oll))
    assert abs(merr.value - omerr) < TOL * max(1, abs(omerr))
    assert rel_err(dev.download(grad, m.pSize), ograd) < TOL
    gz = dev.download(z, m.zSize)
    for i in range(1, m.numLayers + 1):
        a, b = m.zOffsets[i], m.zOffsets[i] + m.layerSizes[i] * n
        assert rel_err(gz[a:b], oz[a:b]) < TOL, ("z", i)
    assert rel_err(dev.download(dx, m.rFullSize), odx) < TOL
    # the same through the scratch-carved buffers (z == NULL), and evaluateModel on train and test data
    grad2 = dev.zeros(m.pSize)
    L.cnn.computeGradient(C.byref(m), C.byref(data), C.byref(scratch), pw, None, None, grad2, C.byref(ll), C.byref(merr), FULL_DATASET)
    np.testing.assert_array_equal(dev.download(grad2, m.pSize), dev.download(grad, m.pSize))
    for kind in (TRAIN_DATA, TEST_DATA):
        l2, e2 = C.c_float(), C.c_float()
        L.cnn.evaluateModel(C.byref(m), C.byref(data), C.byref(scratch), pw, C.byref(l2), C.byref(e2), FULL_DATASET, kind)
        assert abs(l2.value - oll) < TOL * max(1, abs(oll)) and abs(e2.value - omerr) < TOL * max(1, abs(omerr))


@pytest.mark.gpu
def test_gpu_sampled_dataset_uses_the_input_as_target(dev, oracle64):
    name, n = "autoencoder_logistic", 64
    rng = np.random.default_rng(3)
    m, w, x, _ = make_data(name, n, rng)
    x = rng.random((n, m.layerSizes[0]))          # an auto-encoder of values in (0, 1)
    w32, x32 = w.astype(np.float32), x.astype(np.float32)
    data, scratch, pw = device_setup(dev, m, w32, x32, x32, n, sampled=True)
    grad = dev.zeros(m.pSize)
    z, dx = dev.zeros(m.sampledZSize), dev.zeros(m.sampledRSize)
    ll, merr = C.c_float(), C.c_float()
    L.cnn.computeGradient(C.byref(m), C.byref(data), C.byref(scratch), pw, z, dx, grad, C.byref(ll), C.byref(merr), SAMPLED_DATASET)
    oll, omerr, ograd, _, _ = oracle64.nn_gradient(m, w32, x32.reshape(-1), x32.reshape(-1), n)
    assert abs(ll.value - oll) < TOL * max(1, abs(oll))
    assert rel_err(dev.download(grad, m.pSize), ograd) < TOL


@pytest.mark.gpu
def test_gpu_apply_layer_activation_keeps_the_pre_activation_copy(dev, oracle64):
    rng = np.random.default_rng(8)
    rows, cols, n = 5, 7, 9
    W, b, zin = rng.standard_normal((cols, rows)), rng.standard_normal(rows), rng.standard_normal((n, cols))
    pW, pb, pz = dev.upload(W.reshape(-1)), dev.upload(b), dev.upload(zin.reshape(-1))
    out = dev.zeros(2 * rows * n)
    L.cnn.applyLayerActivation(ACT_SOFTMAX, pW, rows, cols, pb, rows, pz, cols, n, out, None, None)
    got = dev.download(out, 2 * rows * n)
    pre = zin @ W + b                                   # n x rows, sample-major == column-major rows x n
    want = np.exp(pre) / np.exp(pre).sum(1, keepdims=True)
    assert rel_err(got[:rows * n].reshape(n, rows), want) < 1e-5
    assert rel_err(got[rows * n:].reshape(n, rows), pre) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("name", HV_CASES)
@pytest.mark.parametrize("n", [11, 300])
def test_gpu_hessian_vector_products_against_oracle(dev, oracle64, name, n):
    """hessianVec and gaussNewtonHessianVec after computeGradient at the same point, result at the head of the arena."""
    rng = np.random.default_rng(sum(map(ord, name)) + 7 * n)
    m, w, x, y = make_data(name, n, rng)
    w32, x32, y32 = w.astype(np.float32), x.astype(np.float32), y.astype(np.float32)
    v32 = rng.standard_normal(m.pSize).astype(np.float32)
    data, scratch, pw = device_setup(dev, m, w32, x32, y32, n)
    z, dx, grad, pv = dev.zeros(m.zSize), dev.zeros(m.rFullSize), dev.zeros(m.pSize), dev.upload(v32)
    ll, merr = C.c_float(), C.c_float()
    L.cnn.computeGradient(C.byref(m), C.byref(data), C.byref(scratch), pw, z, dx, grad, C.byref(ll), C.byref(merr), FULL_DATASET)
    need = L.cnn.nnHessianVecMemRequired(C.byref(m), C.byref(data), FULL_DATASET)
    arena = dev.upload(np.full(need, np.nan, np.float32))          # nothing may rely on a cleared arena
    hv_scratch = SCRATCH_AREA()
    hv_scratch.devWorkspace = hv_scratch.nextDevPtr = arena.value
    _, _, _, oz, odx = oracle64.nn_gradient(m, w32, x32.reshape(-1), y32.reshape(-1), n)
    L.cnn.hessianVec(C.byref(m), C.byref(data), z, dx, pv, pw, C.byref(hv_scratch), FULL_DATASET)
    want = oracle64.nn_hessian_vec(m, w32, v32, x32.reshape(-1), n, oz, odx)
    assert rel_err(dev.download(arena, m.pSize), want) < TOL
    L.cnn.gaussNewtonHessianVec(C.byref(m), C.byref(data), z, dx, pv, pw, C.byref(hv_scratch), FULL_DATASET)
    want = oracle64.nn_hessian_vec(m, w32, v32, x32.reshape(-1), n, oz, odx, gauss_newton=True)
    assert rel_err(dev.download(arena, m.pSize), want) < TOL
    for q in (z, dx, grad, pv, arena):
        dev.free(q)


@pytest.mark.gpu
def test_gpu_hessian_vector_product_on_the_sampled_set(dev, oracle64):
    name, n = "autoencoder_logistic", 64
    rng = np.random.default_rng(13)
    m, w, _, _ = make_data(name, n, rng)
    x = rng.random((n, m.layerSizes[0]))
    w32, x32 = w.astype(np.float32), x.astype(np.float32)
    v32 = rng.standard_normal(m.pSize).astype(np.float32)
    data, scratch, pw = device_setup(dev, m, w32, x32, x32, n, sampled=True)
    z, dx, grad, pv = dev.zeros(m.sampledZSize), dev.zeros(m.sampledRSize), dev.zeros(m.pSize), dev.upload(v32)
    ll, merr = C.c_float(), C.c_float()
    L.cnn.computeGradient(C.byref(m), C.byref(data), C.byref(scratch), pw, z, dx, grad, C.byref(ll), C.byref(merr), SAMPLED_DATASET)
    need = L.cnn.nnHessianVecMemRequired(C.byref(m), C.byref(data), SAMPLED_DATASET)
    arena = dev.upload(np.full(need, np.nan, np.float32))
    hv_scratch = SCRATCH_AREA()
    hv_scratch.devWorkspace = hv_scratch.nextDevPtr = arena.value
    L.cnn.hessianVec(C.byref(m), C.byref(data), z, dx, pv, pw, C.byref(hv_scratch), SAMPLED_DATASET)
    _, _, _, oz, odx = oracle64.nn_gradient(m, w32, x32.reshape(-1), x32.reshape(-1), n)
    want = oracle64.nn_hessian_vec(m, w32, v32, x32.reshape(-1), n, oz, odx)
    assert rel_err(dev.download(arena, m.pSize), want) < TOL
    for q in (z, dx, grad, pv, arena):
        dev.free(q)


@pytest.mark.gpu
def test_gpu_rop_pieces_against_their_formulas(dev):
    rng = np.random.default_rng(21)
    n = 5000
    z = rng.random(n).astype(np.float32) * 1.8 - 0.9
    rdz, rx, dxv = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    pz, prdz, prx, pdx, out = dev.upload(z), dev.upload(rdz), dev.upload(rx), dev.upload(dxv), dev.zeros(n)
    z64, rdz64, rx64, dx64 = (a.astype(np.float64) for a in (z, rdz, rx, dxv))
    forms = {ACT_LOGISTIC: ((1 - z64) * z64, 1 - 2 * z64), ACT_TANH: ((1 + z64) * (1 - z64), -2 * z64),
             ACT_LINEAR: (np.ones(n), np.zeros(n))}
    for act, (f1, g) in forms.items():
        L.check(L.hip.fitre_hip_fc_rop_backward(act, pz, prdz, prx, pdx, out, n))
        np.testing.assert_allclose(dev.download(out, n), f1 * rdz64 + rx64 * g * dx64, rtol=0, atol=2e-6)
        L.check(L.hip.fitre_hip_fc_rop_backward(act, pz, prdz, None, None, out, n))
        np.testing.assert_allclose(dev.download(out, n), f1 * rdz64, rtol=0, atol=1e-6)
    assert L.hip.fitre_hip_fc_rop_backward(ACT_SOFTMAX, pz, prdz, prx, pdx, out, n) != 0      # not an element-wise activation
    rows, cols = 7, 300
    logits = rng.standard_normal((cols, rows))
    p = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    r = rng.standard_normal((cols, rows))
    pp, pr, po = dev.upload(p.reshape(-1)), dev.upload(r.reshape(-1)), dev.zeros(rows * cols)
    L.check(L.hip.fitre_hip_column_softmax_rop(pp, pr, rows, cols, po))
    want = p * r - p * (p * r).sum(axis=1, keepdims=True)
    np.testing.assert_allclose(dev.download(po, rows * cols).reshape(cols, rows), want, rtol=0, atol=1e-6)
    assert abs(dev.download(po, rows * cols).reshape(cols, rows).sum(axis=1)).max() < 1e-6    # the directions sum to zero
    for q in (pz, prdz, prx, pdx, out, pp, pr, po):
        dev.free(q)
