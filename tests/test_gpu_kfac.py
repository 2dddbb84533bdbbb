"""Kronecker factors of the KFAC approximation (symmetric fp32-MFMA products with mirrored tiles)
against the float64 oracle, through the C boundary."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from helpers import conv_shape, rel_err

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
