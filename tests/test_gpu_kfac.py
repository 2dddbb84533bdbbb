"""Kronecker factors of the KFAC approximation (symmetric fp32-MFMA products with mirrored tiles)
against the float64 oracle, through the C boundary."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from helpers import conv_shape, stored_inverse, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4
hip = L.hip

# N, Cin, Cout, A(width), B(height), k, stride, pad
FACTOR_CASES = [
    (2, 3, 6, 32, 32, 5, 1, 0),     # LeNet conv1: order 76, one 128-tile
    (4, 3, 64, 32, 32, 3, 1, 1),    # VGG conv1: order 28, long reduction (split)
    (2, 64, 128, 16, 16, 3, 1, 1),  # VGG conv2: order 577 = 4 tiles + 65 rows
    (3, 30, 8, 8, 8, 3, 1, 1),      # order 271: partial tile on the diagonal
    (8, 43, 8, 4, 4, 3, 1, 1),      # order 388, short reduction (no split)
    (2, 8, 12, 13, 13, 5, 1, 2),    # AlexNet conv2 geometry
    (2, 3, 8, 67, 67, 11, 4, 2),    # strided window
    (3, 5, 7, 9, 6, 3, 1, 1),       # rectangular
    (1, 1, 1, 5, 5, 3, 1, 0),       # degenerate
    (2, 7, 5, 7, 7, 1, 1, 0),       # 1x1 window: order 8
    # small maps, channels in whole tiles: rows by tap over cell-major positions, reduction cut to the cells both taps see
    (16, 128, 8, 4, 4, 3, 1, 1),    # order 1153
    (16, 128, 8, 2, 2, 3, 1, 1),    # 2 x 2 map: opposite taps share no cell (zero tiles)
    (32, 128, 8, 8, 8, 3, 1, 1),    # 8 x 8 map, split reduction
    (16, 256, 8, 4, 4, 3, 1, 1),    # order 2305
    (16, 128, 8, 4, 2, 3, 1, 1),    # rectangular map
    (16, 128, 4, 4, 4, 5, 1, 2),    # 5 x 5 window: order 3201
    (16, 128, 4, 6, 6, 3, 1, 0),    # no padding: every tap inside at every cell
    (8, 128, 8, 4, 4, 3, 1, 1),     # eight images: not whole reduction slices per cell, plain rows
]


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("case", FACTOR_CASES)
def test_conv_input_factor(dev, oracle64, case, bias):
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    n = Cin * k * k + (1 if bias else 0)
    rng = np.random.default_rng(sum(case) + 7)
    x = (rng.standard_normal(Cin * N * A * B) + 0.3).astype(np.float32)
    px = dev.upload(x)
    nb = hip.fitre_hip_kfac_conv_input_factor_workspace(C.byref(shape), int(bias))
    ws = dev.alloc(nb)
    out = dev.upload(np.full(n * n, np.nan, dtype=np.float32))  # every element must be written
    L.check(hip.fitre_hip_kfac_conv_input_factor(C.byref(shape), px, int(bias), out, ws, nb))
    got = dev.download(out, n * n).reshape(n, n)
    want = oracle64.kfac_conv_input_factor(x, N, Cin, B, A, k, p, s, bias)
    for q in (px, ws, out):
        dev.free(q)
    assert np.isfinite(got).all()
    assert rel_err(got, want) < TOL
    assert np.array_equal(got, got.T)  # the lower triangle is a copy of the upper one


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("case", FACTOR_CASES[:4])
def test_conv_input_factor_without_room_for_the_patch_rows(dev, oracle64, case, bias):
    """A workspace that only covers the product's split partials (or none at all): both operands gather their
    elements from the image; same result as with the rows written out."""
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    n = Cin * k * k + (1 if bias else 0)
    rng = np.random.default_rng(sum(case) + 7)
    x = (rng.standard_normal(Cin * N * A * B) + 0.3).astype(np.float32)
    px = dev.upload(x)
    full = hip.fitre_hip_kfac_conv_input_factor_workspace(C.byref(shape), int(bias))
    small = hip.fitre_hip_kfac_gram_workspace(n, N * shape.outA * shape.outB)
    assert small < full
    ws = dev.alloc(full)
    want = oracle64.kfac_conv_input_factor(x, N, Cin, B, A, k, p, s, bias)
    results = []
    for nb in (full, small, 0):
        out = dev.upload(np.full(n * n, np.nan, dtype=np.float32))
        L.check(hip.fitre_hip_kfac_conv_input_factor(C.byref(shape), px, int(bias), out, ws if nb else None, nb))
        got = dev.download(out, n * n).reshape(n, n)
        assert rel_err(got, want) < TOL, nb
        assert np.array_equal(got, got.T)
        results.append(got)
        dev.free(out)
    assert rel_err(results[1], results[0]) < 1e-5 and rel_err(results[2], results[0]) < 1e-5
    for q in (px, ws):
        dev.free(q)


@pytest.mark.parametrize("case", [(4, 3, 64, 32, 32, 3, 1, 1), (2, 64, 130, 16, 16, 3, 1, 1), (16, 8, 300, 2, 2, 3, 1, 1),
                                  (2, 3, 6, 32, 32, 5, 1, 0)])
def test_conv_output_factor(dev, oracle64, case):
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    M = N * shape.outA * shape.outB
    rng = np.random.default_rng(sum(case) + 8)
    d = (rng.standard_normal(Cout * M) / M).astype(np.float32)
    pd = dev.upload(d)
    nb = hip.fitre_hip_kfac_gram_workspace(Cout, M)
    ws = dev.alloc(nb)
    out = dev.upload(np.full(Cout * Cout, np.nan, dtype=np.float32))
    L.check(hip.fitre_hip_kfac_conv_output_factor(C.byref(shape), pd, out, ws, nb))
    got = dev.download(out, Cout * Cout).reshape(Cout, Cout)
    want = oracle64.kfac_conv_output_factor(d, N, shape.outB, shape.outA, Cout)
    for q in (pd, ws, out):
        dev.free(q)
    assert rel_err(got, want) < TOL
    assert np.array_equal(got, got.T)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("dims", [(512, 256), (400, 128), (84, 33), (10, 7), (1, 1), (1000, 64)])
def test_fc_factors(dev, oracle64, dims, bias):
    n_in, N = dims
    rng = np.random.default_rng(n_in + N)
    z = (rng.standard_normal(n_in * N) + 0.5).astype(np.float32)
    pz = dev.upload(z)
    n = n_in + (1 if bias else 0)
    nb = hip.fitre_hip_kfac_gram_workspace(n_in, N)
    ws = dev.alloc(nb)
    out = dev.upload(np.full(n * n, np.nan, dtype=np.float32))
    L.check(hip.fitre_hip_kfac_fc_input_factor(pz, n_in, N, int(bias), out, ws, nb))
    got = dev.download(out, n * n).reshape(n, n)
    want = oracle64.kfac_fc_input_factor(z, n_in, N, bias)
    assert rel_err(got, want) < TOL
    assert np.array_equal(got, got.T)
    if not bias:  # the output-side factor on the same data
        out2 = dev.upload(np.full(n_in * n_in, np.nan, dtype=np.float32))
        L.check(hip.fitre_hip_kfac_fc_output_factor(pz, n_in, N, out2, ws, nb))
        got2 = dev.download(out2, n_in * n_in).reshape(n_in, n_in)
        assert rel_err(got2, oracle64.kfac_fc_output_factor(z, n_in, N)) < TOL
        dev.free(out2)
    for q in (pz, ws, out):
        dev.free(q)


def test_factor_argument_errors(dev):
    shape = conv_shape(2, 3, 4, 8, 8, 3, 1, 1)
    assert hip.fitre_hip_kfac_conv_input_factor(C.byref(shape), None, 1, None, None, 0) == 2
    assert hip.fitre_hip_kfac_fc_input_factor(None, 4, 4, 1, None, None, 0) == 2
    assert hip.fitre_hip_kfac_fc_output_factor(None, 0, 4, None, None, 0) == 2


# ---------------------------------------------------------------------------- model level
def _model_cases():
    from fitre_amd.structs import AVG_POOL, CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SWISH, MAX_POOL
    from helpers import build_custom, build_lenet
    yield "lenet_bias", build_lenet(16, bias=1, bn=False), 16
    yield "small_vgg_bn", build_custom(12, 8, 8, 3, [dict(cout=6, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=True, act=CNN_ACT_RELU),
                                                      dict(cout=9, k=3, pad=1, pool=None, bn=True, act=CNN_ACT_SWISH),
                                                      dict(cout=5, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=False, act=CNN_ACT_RELU)],
                                       [(7, CNN_ACT_NONE)], bias=1), 12
    from helpers import build_vgg11
    yield "vgg11_b256", build_vgg11(256, bn=True), 256   # the benchmark's KFAC configuration at its full size
    yield "no_bias", build_custom(5, 6, 6, 2, [dict(cout=4, k=3, pad=0, pool=(AVG_POOL, 2, 2, 0), bn=False, act=CNN_ACT_SWISH)],
                                  [(6, CNN_ACT_SWISH), (3, CNN_ACT_NONE)], bias=0), 5


@pytest.mark.parametrize("name", ["lenet_bias", "small_vgg_bn", "no_bias", "vgg11_b256"])
def test_model_factor_passes(dev, oracle64, name):
    """computeOmegaZFactors / computeLambdaDeltaFactors after a forward and a backward pass: every layer's
    factor against the oracle's factor of the same z / dx contents, at the offsets of computeKFACStorageIndices."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO
    from helpers import GpuModel, batch_inputs, he_weights
    model, batch = next((m, b) for n, m, b in _model_cases() if n == name)
    rng = np.random.default_rng(sum(map(ord, name)))
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    x = x.astype(np.float32)
    gm = GpuModel(dev, model, w, x, y, batch)
    gm.forward()
    gm.backward()
    z, dxs = gm.get("z"), gm.get("dx")
    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    nc, nl = model.cLayers, model.lLayers
    tot_o, tot_l = info.OmegaZOffsets[nc + nl], info.LambdaGOffsets[nc + nl]
    omega = dev.upload(np.full(tot_o, np.nan, dtype=np.float32))
    lam = dev.upload(np.full(tot_l, np.nan, dtype=np.float32))
    ws = dev.alloc(4 * L.cnn.kfacFactorsMemRequired(C.byref(model), batch))
    L.cnn.computeOmegaZFactors(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, omega, model.zOffsets,
                               model.zztOffsets, ws)
    L.cnn.computeLambdaDeltaFactors(C.byref(info), C.byref(model), batch, gm.dx, None, lam, model.zOffsets, model.zztOffsets, ws)
    got_o, got_l = dev.download(omega, tot_o), dev.download(lam, tot_l)
    bias = model.bias != 0
    zo = model.zOffsets
    for l in range(nc):
        c = model.convLayer[l]
        if l == 0:
            src = x.reshape(-1)
        else:
            prev = model.convLayer[l - 1]
            start = zo[l] + prev.outputOffset
            src = z[start:start + c.inChannels * batch * c.height * c.width]
        n = c.inChannels * c.kSize ** 2 + (1 if bias else 0)
        want = oracle64.kfac_conv_input_factor(src, batch, c.inChannels, c.height, c.width, c.kSize, c.padding, c.stride, bias)
        got = got_o[info.OmegaZOffsets[l]:info.OmegaZOffsets[l] + n * n].reshape(n, n)
        assert rel_err(got, want) < TOL, ("omega conv", l)
        off = zo[l + 1] + (c.batchNormOffset if c.batchNorm else c.activationOffset)
        count = c.outChannels * batch * c.outHeight * c.outWidth
        want = oracle64.kfac_conv_output_factor(dxs[off:off + count], batch, c.outHeight, c.outWidth, c.outChannels)
        got = got_l[info.LambdaGOffsets[l]:info.LambdaGOffsets[l] + c.outChannels ** 2].reshape(c.outChannels, -1)
        assert rel_err(got, want) < TOL, ("lambda conv", l)
    for l in range(nl):
        f = model.fcLayer[l]
        start = zo[nc] + model.convLayer[nc - 1].outputOffset if l == 0 else zo[nc + l]
        n = f.in_ + (1 if bias else 0)
        want = oracle64.kfac_fc_input_factor(z[start:start + f.in_ * batch], f.in_, batch, bias)
        got = got_o[info.OmegaZOffsets[nc + l]:info.OmegaZOffsets[nc + l] + n * n].reshape(n, n)
        assert rel_err(got, want) < TOL, ("omega fc", l)
        start = zo[nc + l + 1]
        want = oracle64.kfac_fc_output_factor(dxs[start:start + f.out * batch], f.out, batch)
        got = got_l[info.LambdaGOffsets[nc + l]:info.LambdaGOffsets[nc + l] + f.out ** 2].reshape(f.out, -1)
        assert rel_err(got, want) < TOL, ("lambda fc", l)
    for q in (omega, lam, ws):
        dev.free(q)
    gm.release()


# ---------------------------------------------------------------------------- inverse of a factor
def _spd(n, rng, cond):
    q, _ = np.linalg.qr(rng.standard_normal((n, n)))
    ev = np.geomspace(1.0, 1.0 / cond, n)
    return ((q * ev) @ q.T).astype(np.float32)


def _spd_reflected(n, rng, cond):
    """A dense symmetric matrix with the eigenvalues geomspace(1, 1/cond, n), in O(n^2 log n): the diagonal matrix of
    the (shuffled) eigenvalues conjugated by an orthonormal cosine transform, random signs and two random Householder
    reflections — exactly known spectrum, for orders where a QR factorisation of a random matrix would dominate the
    test."""
    from scipy.fft import dct
    a = np.diag(rng.permutation(np.geomspace(1.0, 1.0 / cond, n)))
    a = dct(dct(a, axis=0, norm="ortho"), axis=1, norm="ortho")
    sign = rng.choice([-1.0, 1.0], n)
    a = sign[:, None] * a * sign[None, :]
    for _ in range(2):
        u = rng.standard_normal(n)
        u /= np.linalg.norm(u)
        au = a @ u
        a = a - 2.0 * np.outer(u, au) - 2.0 * np.outer(au, u) + 4.0 * (u @ au) * np.outer(u, u)
    return ((a + a.T) / 2).astype(np.float32)


@pytest.mark.parametrize("n", [2305, 4609])
def test_spd_inverse_at_the_largest_factor_orders(dev, n):
    """The orders of VGG-11's input-side factors (9*256+1, 9*512+1), which are the only ones that reach the upper
    levels of the halving recursion, the triangular-operand range skipping and the deep-slice products: against a
    float64 LAPACK inverse.  Spectrum geomspace(1, 1e-3) + 0.02: condition 49 after the shift; tolerance the path's
    1e-4 (max-abs error over the largest magnitude of the float64 inverse), result exactly symmetric."""
    rng = np.random.default_rng(n)
    a = _spd_reflected(n, rng, 1000.0)
    shift = 0.02
    pa = dev.upload(a.reshape(-1))
    out = dev.upload(np.full(n * n, np.nan, dtype=np.float32))
    nb = hip.fitre_hip_spd_inverse_workspace(n)
    ws = dev.alloc(nb)
    info = C.c_int(-1)
    L.check(hip.fitre_hip_spd_inverse(pa, n, shift, out, ws, nb, C.byref(info)))
    assert info.value == 0
    got = dev.download(out, n * n).reshape(n, n)
    a64 = a.astype(np.float64) + shift * np.eye(n)
    ev = np.linalg.eigvalsh(a64)
    assert 40 < ev[-1] / ev[0] < 60
    want = np.linalg.inv(a64)
    assert rel_err(got, want) < TOL
    assert np.array_equal(got, got.T)
    assert np.abs(a64 @ got.astype(np.float64) - np.eye(n)).max() < 1e-4
    for q in (pa, out, ws):
        dev.free(q)


@pytest.mark.parametrize("n", [2305, 4609])
def test_spd_inverse_batched_at_the_largest_factor_orders(dev, n):
    """Three matrices of one order through one chain of launches, as computeOmegaZ batches VGG-11's last three
    input-side factors: each against the float64 LAPACK inverse of its own matrix at 1e-4, exactly symmetric,
    strides larger than the matrices and nothing written between the results."""
    batch, shift = 3, 0.02
    rng = np.random.default_rng(7 * n)
    mats = [_spd_reflected(n, rng, 1000.0) for _ in range(batch)]
    m_stride, i_stride = n * n + 24, n * n + 64
    packed = np.zeros(batch * m_stride, np.float32)
    for b, a in enumerate(mats):
        packed[b * m_stride:b * m_stride + n * n] = a.reshape(-1)
    pa = dev.upload(packed)
    out = dev.upload(np.full(batch * i_stride, np.nan, dtype=np.float32))
    one = hip.fitre_hip_spd_inverse_workspace(n)
    ws_stride = (one + 255) // 256 * 256 + 512
    ws = dev.alloc(batch * ws_stride)
    piv = dev.upload(np.full(batch, -1, np.int32), np.int32)
    L.check(hip.fitre_hip_spd_inverse_batched_queued(batch, pa, m_stride, n, shift, out, i_stride, ws, one, ws_stride, piv))
    dev.sync()
    assert not dev.download(piv, batch, np.int32).any()
    got_all = dev.download(out, batch * i_stride)
    for b, a in enumerate(mats):
        got = got_all[b * i_stride:b * i_stride + n * n].reshape(n, n)
        want = np.linalg.inv(a.astype(np.float64) + shift * np.eye(n))
        assert rel_err(got, want) < TOL, b
        assert np.array_equal(got, got.T)
        assert np.isnan(got_all[b * i_stride + n * n:(b + 1) * i_stride]).all()
    for q in (pa, out, ws, piv):
        dev.free(q)


@pytest.mark.parametrize("n", [1, 3, 28, 64, 65, 129, 400, 577, 1153])
def test_spd_inverse(dev, oracle64, n):
    """(A + shift I)^-1 against the oracle's Cholesky inverse.  The error of an inverse computed in float32
    grows with the condition number; the matrices here have condition ~50 after the shift and the
    tolerance is the path's 1e-4."""
    rng = np.random.default_rng(n)
    a = _spd(n, rng, 1000.0)
    a = ((a + a.T) / 2).astype(np.float32)
    shift = 0.02
    pa = dev.upload(a.reshape(-1))
    out = dev.upload(np.full(n * n, np.nan, dtype=np.float32))
    nb = hip.fitre_hip_spd_inverse_workspace(n)
    ws = dev.alloc(nb)
    info = C.c_int(-1)
    L.check(hip.fitre_hip_spd_inverse(pa, n, shift, out, ws, nb, C.byref(info)))
    assert info.value == 0
    got = dev.download(out, n * n).reshape(n, n)
    oinfo, want = oracle64.matrix_inverse(a.astype(np.float64), n, shift, 0.0)
    assert oinfo == 0
    assert rel_err(got, want) < TOL
    assert np.array_equal(got, got.T)
    resid = (a.astype(np.float64) + shift * np.eye(n)) @ got.astype(np.float64) - np.eye(n)
    assert np.abs(resid).max() < 1e-4
    for q in (pa, out, ws):
        dev.free(q)


@pytest.mark.parametrize("n,batch", [(1, 2), (33, 3), (129, 4), (200, 3), (577, 2)])
def test_spd_inverse_batched(dev, oracle64, n, batch):
    """Several matrices of one order through one chain of launches: each result against the oracle's inverse of
    its own matrix, with strides larger than the matrices, and the pivot report of the one indefinite matrix of
    a second batch in its own slot."""
    rng = np.random.default_rng(100 * n + batch)
    shift = 0.02
    mats = [((lambda a: (a + a.T) / 2)(_spd(n, rng, 1000.0))).astype(np.float32) for _ in range(batch)]
    m_stride, i_stride = n * n + 24, n * n + 64
    packed = np.zeros(batch * m_stride, np.float32)
    for b, a in enumerate(mats):
        packed[b * m_stride:b * m_stride + n * n] = a.reshape(-1)
    pa = dev.upload(packed)
    out = dev.upload(np.full(batch * i_stride, np.nan, dtype=np.float32))
    one = hip.fitre_hip_spd_inverse_workspace(n)
    ws_stride = (one + 255) // 256 * 256 + 512
    ws = dev.alloc(batch * ws_stride)
    piv = dev.upload(np.full(batch, -1, np.int32), np.int32)
    L.check(hip.fitre_hip_spd_inverse_batched_queued(batch, pa, m_stride, n, shift, out, i_stride, ws, one, ws_stride, piv))
    dev.sync()
    assert not dev.download(piv, batch, np.int32).any()
    got_all = dev.download(out, batch * i_stride)
    for b, a in enumerate(mats):
        got = got_all[b * i_stride:b * i_stride + n * n].reshape(n, n)
        _, want = oracle64.matrix_inverse(a.astype(np.float64), n, shift, 0.0)
        assert rel_err(got, want) < TOL, b
        assert np.array_equal(got, got.T)
        assert np.isnan(got_all[b * i_stride + n * n:(b + 1) * i_stride]).all()    # nothing written between the results
    if n >= 33:
        bad = 1 if batch > 1 else 0
        packed[bad * m_stride + 5 * n + 5] = -7.0                                    # a negative diagonal entry
        L.check(hip.fitre_hip_copy_h2d(pa, packed.ctypes.data_as(C.c_void_p), packed.nbytes))
        L.check(hip.fitre_hip_spd_inverse_batched_queued(batch, pa, m_stride, n, shift, out, i_stride, ws, one, ws_stride, piv))
        dev.sync()
        report = dev.download(piv, batch, np.int32)
        assert report[bad] == 6 and not np.delete(report, bad).any(), report
    # argument checks: overlapping workspaces, overlapping results
    assert hip.fitre_hip_spd_inverse_batched_queued(2, pa, m_stride, n, shift, out, i_stride, ws, one, 256 if one > 256 else 0, piv) != 0
    assert hip.fitre_hip_spd_inverse_batched_queued(2, pa, m_stride, n, shift, out, n * n - 1, ws, one, ws_stride, piv) != 0
    for q in (pa, out, ws, piv):
        dev.free(q)


def test_spd_inverse_reports_indefinite_matrix(dev):
    a = np.array([[1.0, 2.0], [2.0, 1.0]], dtype=np.float32)
    pa, out = dev.upload(a.reshape(-1)), dev.zeros(4)
    nb = hip.fitre_hip_spd_inverse_workspace(2)
    ws = dev.alloc(nb)
    info = C.c_int(0)
    assert hip.fitre_hip_spd_inverse(pa, 2, 0.0, out, ws, nb, C.byref(info)) == 2
    assert info.value == 2
    assert b"positive definite" in hip.fitre_hip_last_error()
    assert hip.fitre_hip_spd_inverse(pa, 2, 0.0, out, ws, 16, C.byref(info)) == 4


@pytest.mark.parametrize("name", ["lenet_bias", "small_vgg_bn", "no_bias"])
def test_model_inverses_and_natural_gradient(dev, oracle64, name):
    """computeOmegaZ + computeLambdaDelta (factor and damped inverse per layer) and computeNaturalGradient after a
    forward and a backward pass.  The factors themselves are checked in test_model_factor_passes; here every
    inverse (stored as float pairs) is compared with the oracle's inverse of the float factor the device produced
    (computeOmegaZFactors on the same z / dx), and the natural gradient with the oracle's on those inverses.
    Tolerance of an inverse: the path's 1e-4 for condition numbers up to 50, growing linearly with the
    condition number beyond that (a float32 Cholesky cannot do better)."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO
    from helpers import GpuModel, batch_inputs, he_weights
    model, batch = next((m, b) for n, m, b in _model_cases() if n == name)
    rng = np.random.default_rng(sum(map(ord, name)) + 1)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    x = x.astype(np.float32)
    gm = GpuModel(dev, model, w, x, y, batch)
    gm.forward()
    gm.backward()
    grad = gm.get("grad")
    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    lam, gamma = 0.05, 0.15
    info.regLambda, info.dampGamma = lam, gamma
    nc, nl = model.cLayers, model.lLayers
    tot_o, tot_l = info.OmegaZOffsets[nc + nl], info.LambdaGOffsets[nc + nl]
    ofac, lfac = dev.zeros(tot_o), dev.zeros(tot_l)
    oinv, linv = dev.zeros(tot_o), dev.zeros(tot_l)
    need = max(L.cnn.kfacInverseMemRequired(C.byref(model), batch), L.cnn.kfacNaturalGradientMemRequired(C.byref(model)),
               L.cnn.kfacFactorsMemRequired(C.byref(model), batch))
    ws = dev.alloc(4 * need + 512)
    L.cnn.computeOmegaZFactors(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, ofac, model.zOffsets,
                               model.zztOffsets, ws)
    L.cnn.computeLambdaDeltaFactors(C.byref(info), C.byref(model), batch, gm.dx, None, lfac, model.zOffsets, model.zztOffsets, ws)
    L.cnn.computeOmegaZ(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, oinv, model.zOffsets,
                        model.zztOffsets, ws, None, None, None, None)
    L.cnn.computeLambdaDelta(C.byref(info), C.byref(model), batch, gm.dx, None, linv, model.zOffsets, model.zztOffsets, ws, None, None, None, None)
    fac_o, fac_l = dev.download(ofac, tot_o), dev.download(lfac, tot_l)
    got_o, got_l = dev.download(oinv, tot_o), dev.download(linv, tot_l)
    bias = model.bias != 0

    dec_o, dec_l = np.zeros(tot_o), np.zeros(tot_l)   # the inverses the pairs stand for, at the same offsets

    def check(got, factor, what, dec, at):
        n = int(round(np.sqrt(factor.size)))
        factor = factor.reshape(n, n).astype(np.float64)
        oi, want = oracle64.matrix_inverse(factor, n, lam, gamma)
        assert oi == 0
        ev = np.linalg.eigvalsh(factor + (lam + gamma) * np.eye(n))
        tol = TOL * max(1.0, (ev[-1] / ev[0]) / 50.0)
        got = stored_inverse(got, n)                      # float pairs, or the low-rank form
        dec[at:at + n * n] = got.reshape(-1)
        assert rel_err(got, want) < tol, (what, ev[-1] / ev[0])
        assert np.abs((factor + (lam + gamma) * np.eye(n)) @ got - np.eye(n)).max() < tol, what

    for l in range(nc + nl):
        if l < nc:
            c = model.convLayer[l]
            n_in, n_out = c.inChannels * c.kSize ** 2 + (1 if bias else 0), c.outChannels
        else:
            f = model.fcLayer[l - nc]
            n_in, n_out = f.in_ + (1 if bias else 0), f.out
        o0, l0 = info.OmegaZOffsets[l], info.LambdaGOffsets[l]
        check(got_o[o0:o0 + n_in * n_in], fac_o[o0:o0 + n_in * n_in], ("omega", l), dec_o, o0)
        check(got_l[l0:l0 + n_out * n_out], fac_l[l0:l0 + n_out * n_out], ("lambda", l), dec_l, l0)

    # natural gradient of the gradient the backward pass produced
    ngrad = dev.upload(np.full(model.pSize, np.nan, dtype=np.float32))
    info.OmegaZInv, info.LambdaGInv = oinv.value, linv.value
    info.gradient, info.nGradient = gm.grad.value, ngrad.value
    L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws, None)
    got = dev.download(ngrad, model.pSize)
    want = oracle64.natural_gradient(model, list(info.OmegaZOffsets), list(info.LambdaGOffsets), dec_o, dec_l, grad)
    assert np.isfinite(got).all()
    assert rel_err(got, want) < TOL
    for q in (ofac, lfac, oinv, linv, ws, ngrad):
        dev.free(q)
    gm.release()


@pytest.mark.parametrize("name", ["lenet_bias", "small_vgg_bn", "vgg11_b256"])
def test_both_inverse_passes_as_one(dev, name):
    """computeOmegaZAndLambdaDelta against computeOmegaZ followed by computeLambdaDelta on the same z / dx: the same
    matrices, whatever lanes they were dealt to."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO
    from helpers import GpuModel, batch_inputs, he_weights
    model, batch = next((m, b) for n, m, b in _model_cases() if n == name)
    rng = np.random.default_rng(sum(map(ord, name)) + 5)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
    gm.forward()
    gm.backward()
    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    info.regLambda, info.dampGamma = (1e-3, 0.0) if name == "vgg11_b256" else (0.05, 0.15)
    last = model.cLayers + model.lLayers
    tot_o, tot_l = info.OmegaZOffsets[last], info.LambdaGOffsets[last]
    o1, l1, o2, l2 = dev.zeros(tot_o), dev.zeros(tot_l), dev.zeros(tot_o), dev.zeros(tot_l)
    ws = dev.alloc(4 * L.cnn.kfacInverseMemRequired(C.byref(model), batch) + 512)
    L.cnn.computeOmegaZ(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, o1, model.zOffsets, model.zztOffsets,
                        ws, None, None, None, None)
    L.cnn.computeLambdaDelta(C.byref(info), C.byref(model), batch, gm.dx, None, l1, model.zOffsets, model.zztOffsets, ws, None, None, None, None)
    info.OmegaZInv, info.LambdaGInv = o2.value, l2.value
    L.cnn.computeOmegaZAndLambdaDelta(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, gm.dx, None,
                                      model.zOffsets, model.zztOffsets, ws)
    # the stored forms (float pairs, low-rank slots with doubles inside) word for word: a matrix does not depend on the
    # lane it was dealt to
    a, b = dev.download(o1, tot_o, dtype=np.uint32), dev.download(o2, tot_o, dtype=np.uint32)
    assert a.any() and np.array_equal(a, b)
    a, b = dev.download(l1, tot_l, dtype=np.uint32), dev.download(l2, tot_l, dtype=np.uint32)
    assert a.any() and np.array_equal(a, b)
    for q in (o1, l1, o2, l2, ws):
        dev.free(q)
    gm.release()


def _float64_natural_gradient(oracle64, model, batch, x, z, dxs, grad, lam, on_layer=None):
    """The whole leg in float64 on the host from the layer inputs (x, z), the output-side gradients (dx) and the flat
    gradient: the oracle's factors, scipy's Cholesky factorisation and solves of factor + lam I (LAPACK dpotrf / dpotrs,
    what the reference calls through cuSOLVER, solvers/kfac_inverses.cu:133-186), and Lambda^-1 * gradient * Omega^-1 per layer
    (solvers/kfac_natural_gradient.cu:36-241).  Nothing here comes from the device's factors or inverses.  Returns the
    natural gradient in the flat layout and, per layer, the condition numbers of both damped factors; on_layer(l,
    inverse of the input-side factor, inverse of the output-side factor) is called for every layer."""
    import scipy.linalg as sl
    nc, nl = model.cLayers, model.lLayers
    zo, bias = model.zOffsets, model.bias != 0
    out = np.zeros(model.pSize)
    conds = []
    for l in range(nc + nl):
        if l < nc:
            c = model.convLayer[l]
            if l == 0:
                src = x.reshape(-1)
            else:
                start = zo[l] + model.convLayer[l - 1].outputOffset
                src = z[start:start + c.inChannels * batch * c.height * c.width]
            A = oracle64.kfac_conv_input_factor(src, batch, c.inChannels, c.height, c.width, c.kSize, c.padding, c.stride, bias)
            off = zo[l + 1] + (c.batchNormOffset if c.batchNorm else c.activationOffset)
            G = oracle64.kfac_conv_output_factor(dxs[off:off + c.outChannels * batch * c.outHeight * c.outWidth], batch,
                                                 c.outHeight, c.outWidth, c.outChannels)
        else:
            f = model.fcLayer[l - nc]
            start = zo[nc] + model.convLayer[nc - 1].outputOffset if l == nc else zo[l]
            A = oracle64.kfac_fc_input_factor(z[start:start + f.in_ * batch], f.in_, batch, bias)
            start = zo[l + 1]
            G = oracle64.kfac_fc_output_factor(dxs[start:start + f.out * batch], f.out, batch)
        n_in, n_out = A.shape[0], G.shape[0]
        k = n_in - (1 if bias else 0)
        lo = model.wOffsets[l]
        g = grad[lo:lo + n_out * n_in].astype(np.float64)
        if l < nc:      # [Cout][K] weights, then Cout biases -> Cout x (K + 1)
            wb = np.concatenate([g[:n_out * k].reshape(n_out, k), g[n_out * k:].reshape(n_out, -1)], axis=1)
        else:           # column-major out x in, then out biases
            wb = np.concatenate([g[:n_out * k].reshape(k, n_out).T, g[n_out * k:].reshape(n_out, -1)], axis=1)
        A[np.diag_indices(n_in)] += lam
        G[np.diag_indices(n_out)] += lam
        ca, cg = sl.cho_factor(A), sl.cho_factor(G)
        ng = sl.cho_solve(cg, sl.cho_solve(ca, wb.T).T)
        if l < nc:
            out[lo:lo + n_out * n_in] = np.concatenate([ng[:, :k].reshape(-1), ng[:, k:].reshape(-1)])
        else:
            out[lo:lo + n_out * n_in] = np.concatenate([ng[:, :k].T.reshape(-1), ng[:, k:].reshape(-1)])
        ea, eg = np.linalg.eigvalsh(A), np.linalg.eigvalsh(G)
        conds.append((n_in, n_out, ea[-1] / ea[0], eg[-1] / eg[0]))
        if on_layer is not None:
            on_layer(l, sl.cho_solve(ca, np.eye(n_in)), sl.cho_solve(cg, np.eye(n_out)))
    return out, conds


def test_vgg11_kfac_leg_against_a_float64_pipeline(dev, oracle64):
    """Factor -> damped inverse -> natural gradient of the benchmark's KFAC configuration at its real size (VGG-11, batch
    256, damping lambda = 1e-3 and nothing else: input-side factors of order up to 4609 with 1024 patches behind them,
    condition numbers up to 7e5) as the solver runs it (computeOmegaZAndLambdaDelta, computeNaturalGradient), against the
    same leg done entirely in float64 on the host from the z / dx / gradient the device holds: the device's own factors
    and inverses are never fed to the checker.  Bounds: every stored inverse (float pairs; the low-rank form for the three
    input-side factors with at most half as many patches as their order) within 1e-7 of the largest element of LAPACK's,
    every layer block of the natural gradient within 1e-4 of its largest magnitude."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO
    from helpers import GpuModel, batch_inputs, build_vgg11, he_weights
    batch, lam = 256, float(np.float32(1e-3))     # the damping is a real (float) in the reference's struct
    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(7)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    x = x.astype(np.float32)
    gm = GpuModel(dev, model, w, x, y, batch)
    gm.forward()
    gm.backward()
    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    layers = model.cLayers + model.lLayers
    tot_o, tot_l = info.OmegaZOffsets[layers], info.LambdaGOffsets[layers]
    assert info.OmegaZOffsets[6] - info.OmegaZOffsets[5] == 4609 * 4609
    oinv, linv, ngrad = dev.zeros(tot_o), dev.zeros(tot_l), dev.zeros(model.pSize)
    need = max(L.cnn.kfacInverseMemRequired(C.byref(model), batch), L.cnn.kfacNaturalGradientMemRequired(C.byref(model)))
    ws = dev.alloc(4 * need + 512)
    info.regLambda, info.dampGamma = lam, 0.0
    info.OmegaZInv, info.LambdaGInv = oinv.value, linv.value
    info.gradient, info.nGradient = gm.grad.value, ngrad.value
    L.cnn.computeOmegaZAndLambdaDelta(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, gm.dx, None,
                                      model.zOffsets, model.zztOffsets, ws)
    L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws, None)
    got = dev.download(ngrad, model.pSize)
    z, dxs, grad = gm.get("z"), gm.get("dx"), gm.get("grad")
    inverse_errors = []

    def compare_inverses(l, omega_inverse, lambda_inverse):
        for want, ptr, offs, what in ((omega_inverse, oinv, info.OmegaZOffsets, "omega"), (lambda_inverse, linv, info.LambdaGOffsets, "lambda")):
            n = want.shape[0]
            stored = stored_inverse(dev.download(ptr, n * n, offset=offs[l]), n)
            assert np.isfinite(stored).all(), (what, l)
            inverse_errors.append((what, l, rel_err(stored, want)))

    want, conds = _float64_natural_gradient(oracle64, model, batch, x, z, dxs, grad, lam, compare_inverses)
    for q in (oinv, linv, ngrad, ws):
        dev.free(q)
    gm.release()
    assert np.isfinite(got).all()
    worst = []
    for l in range(layers):
        lo = model.wOffsets[l]
        hi = model.wOffsets[l + 1] if l + 1 < layers else model.pSize
        err = rel_err(got[lo:hi], want[lo:hi])
        print("natural gradient layer %d: orders %d / %d, condition %.3g / %.3g, error %.2e of the block's largest magnitude %.3g;"
              % ((l,) + conds[l] + (err, np.abs(want[lo:hi]).max())),
              "inverses %.1e / %.1e" % (inverse_errors[2 * l][2], inverse_errors[2 * l + 1][2]), flush=True)
        worst.append(err)
    assert max(e for _, _, e in inverse_errors) < 1e-7, inverse_errors
    assert max(worst) < TOL, worst
    # a descent direction: g' (F^-1 g) > 0 for a positive definite Fisher approximation
    assert float(np.dot(got.astype(np.float64), grad.astype(np.float64))) > 0
