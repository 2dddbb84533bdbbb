"""The reference's derivative test (utilities/cnn_derivative_test.cu:48-235) run on the HIP path.

The reference draws W0 and Wr uniform in (0,1) scaled by 0.1 (:112-118), and for numPoints halvings of Wr
(:222-223) evaluates f(W0 + Wr) with evaluateCNNModel (:150-151), f(W0) and g with computeCNNGradient
(:158-159), H*Wr with cnnHv (:160-161), the two dot products g'Wr and Wr'H Wr (:167-178) and reports

    d2error = |f(W0+Wr) - (f(W0) + g'Wr)|                    / |f(W0+Wr)|     (:197)
    d3error = |f(W0+Wr) - (f(W0) + g'Wr + 0.5 Wr'H Wr)|      / |f(W0+Wr)|     (:198-199)

next to |Wr|^2 and |Wr|^3: the first must fall like |Wr|^2 (a factor 4 per halving), the second like |Wr|^3 (a
factor 8).  Here the same calls go through the C boundary on the GPU — evaluateCNNModel, computeCNNGradient,
cnnHv, fitre_hip_dot — on networks whose loss is smooth in the weights (swish, average pooling), and the test
asserts the two slopes.

What float32 resolves.  The loss is about 2.3 and is returned as a float: one unit in its last place is 2.4e-7,
and the forward pass itself carries a few of those.  The first-order remainder starts near 5e-2 and is still
1e-5 after six halvings: slopes of halvings 0..6 are usable (seven points).  The second-order remainder starts
near 5e-3 and reaches 1e-5 after three halvings: four points.  Beyond that the differences are rounding noise
(the float64 oracle, tests/test_oracle_model.py, shows slopes 2.00 and 2.9-3.0 for ten halvings).  A wrong
gradient gives a first-order slope of 1 and a wrong Hessian a second-order slope of 2; both are checked here
as negative controls.
"""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.harness import GpuModel, batch_inputs, build_custom
from fitre_amd.structs import AVG_POOL, CNN_ACT_NONE, CNN_ACT_SWISH

pytestmark = pytest.mark.gpu

FIRST_ORDER_POINTS = 7
SECOND_ORDER_POINTS = 4


def vgg_shaped(batch, widths, size=32):
    pooled = {0, 1, 3, 5, 7}
    convs = [dict(cout=c, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0) if i in pooled else None, bn=True, act=CNN_ACT_SWISH)
             for i, c in enumerate(widths)]
    return build_custom(batch, size, size, 3, convs, [(10, CNN_ACT_NONE)])


def fitted_slope(norms, errors):
    """Least-squares slope of log(error) against log(|Wr|)."""
    return float(np.polyfit(np.log(norms), np.log(errors), 1)[0])


def device_dot(n, a, b):
    out = C.c_float()
    L.check(L.hip.fitre_hip_dot(n, a, b, C.byref(out)))
    return float(out.value)


@pytest.mark.parametrize("name,batch,widths", [
    ("narrow", 16, [16, 32, 64, 64, 128, 128, 128, 128]),
    ("vgg11_widths", 32, [64, 128, 256, 256, 512, 512, 512, 512]),
])
def test_derivative_test_of_the_reference_on_the_device(dev, name, batch, widths):
    model = vgg_shaped(batch, widths)
    n = model.pSize
    rng = np.random.default_rng(2718 + batch)
    w0 = (rng.uniform(0, 1, n) * 0.1).astype(np.float32)
    wr = (rng.uniform(0, 1, n) * 0.1).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w0, x.astype(np.float32), y, batch)
    p_w0, p_wr, p_wc = dev.upload(w0), dev.upload(wr), dev.zeros(n)
    hv = dev.zeros(n)
    ws = dev.alloc(4 * L.cnn.cnnHvMemRequired(C.byref(model)) + 512)

    d2, d3, norms, d3_without_h = [], [], [], []
    for i in range(FIRST_ORDER_POINTS):
        # Wc = W0 + Wr; f(c)
        L.check(L.hip.fitre_hip_copy(n, p_w0, p_wc))
        L.check(L.hip.fitre_hip_axpy(n, 1.0, p_wr, p_wc))
        L.check(L.hip.fitre_hip_copy(n, p_wc, gm.w))
        f_c = L.cnn.evaluateCNNModel(C.byref(model), C.byref(gm.data), C.byref(gm.scratch), gm.z, gm.probs, gm.errors, 0, batch)
        # f(0), g, H * Wr at W0
        L.check(L.hip.fitre_hip_copy(n, p_w0, gm.w))
        f_0 = gm.gradient()
        L.cnn.cnnHv(C.byref(model), C.byref(gm.data), gm.z, gm.probs, gm.errors, gm.dx, p_wr, hv, 0, batch, ws, None, 0.0)
        first = device_dot(n, p_wr, gm.grad)
        second = device_dot(n, hv, p_wr)
        nrm = C.c_float()
        L.check(L.hip.fitre_hip_nrm2(n, p_wr, C.byref(nrm)))
        d2.append(abs(f_c - (f_0 + first)) / abs(f_c))
        d3.append(abs(f_c - (f_0 + first + 0.5 * second)) / abs(f_c))
        d3_without_h.append(abs(f_c - (f_0 + first + 0.25 * second)) / abs(f_c))     # negative control: half the curvature
        norms.append(float(nrm.value))
        L.check(L.hip.fitre_hip_scal(n, 0.5, p_wr))                                   # Wr = Wr / 2
    for q in (p_w0, p_wr, p_wc, hv, ws):
        dev.free(q)
    gm.release()

    norms = np.array(norms)
    np.testing.assert_allclose(norms[:-1] / norms[1:], 2.0, rtol=1e-6)
    # the slopes are those of the limit |Wr| -> 0: the largest steps still carry the next order of the expansion
    # (the first-order remainder of the first halvings is 0.5 Wr'H Wr plus a cubic term of opposite sign and a
    # third of its size), so each fit uses the smallest steps float32 resolves
    s1 = fitted_slope(norms[3:], d2[3:])
    lo = SECOND_ORDER_POINTS - 3
    s2 = fitted_slope(norms[lo:SECOND_ORDER_POINTS], d3[lo:SECOND_ORDER_POINTS])
    s2_bad = fitted_slope(norms[lo:SECOND_ORDER_POINTS], d3_without_h[lo:SECOND_ORDER_POINTS])
    print("%s: first-order remainders %s slope %.3f; second-order remainders %s slope %.3f (half the curvature: %.3f)"
          % (name, ["%.2e" % v for v in d2], s1, ["%.2e" % v for v in d3[:SECOND_ORDER_POINTS]], s2, s2_bad))
    assert 1.9 < s1 < 2.1, (s1, d2)
    assert 2.6 < s2 < 3.3, (s2, d3)
    assert s2_bad < 2.3, (s2_bad, d3_without_h)
    # every single halving of the first-order remainder: a factor that rises towards 4
    ratios = np.array(d2[:-1]) / np.array(d2[1:])
    assert np.all((3.0 < ratios) & (ratios < 4.6)), ratios
    assert np.all((3.6 < ratios[3:]) & (ratios[3:] < 4.4)), ratios
    # the remainders themselves: the quadratic model is the better one at every resolved point
    assert all(b < a for a, b in zip(d2[:SECOND_ORDER_POINTS], d3[:SECOND_ORDER_POINTS]))


def test_derivative_test_detects_a_wrong_gradient(dev):
    """The same sequence with the last layer's block of the gradient left out: the first-order remainder then falls
    like |Wr| (slope 1), which the slope assertion of the test above would reject."""
    batch = 16
    model = vgg_shaped(batch, [16, 32, 64, 64, 128, 128, 128, 128])
    n = model.pSize
    rng = np.random.default_rng(2718 + batch)
    w0 = (rng.uniform(0, 1, n) * 0.1).astype(np.float32)
    wr = (rng.uniform(0, 1, n) * 0.1).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w0, x.astype(np.float32), y, batch)
    f_0 = gm.gradient()
    g = gm.get("grad").astype(np.float64)
    g[model.wOffsets[model.cLayers + model.lLayers - 1]:] = 0
    d2, norms = [], []
    for i in range(FIRST_ORDER_POINTS):
        d = (wr / np.float32(2 ** i)).astype(np.float32)
        L.check(L.hip.fitre_hip_copy_h2d(gm.w, (w0 + d).ctypes.data_as(C.c_void_p), 4 * n))
        f_c = L.cnn.evaluateCNNModel(C.byref(model), C.byref(gm.data), C.byref(gm.scratch), gm.z, gm.probs, gm.errors, 0, batch)
        d2.append(abs(f_c - (f_0 + float(g @ d.astype(np.float64)))) / abs(f_c))
        norms.append(float(np.linalg.norm(d.astype(np.float64))))
    gm.release()
    assert fitted_slope(np.array(norms[2:]), d2[2:]) < 1.5, d2
