"""Parity of every C-ABI kernel entry point with the float64 oracle on seeded inputs.
Tolerance: max-abs error relative to the largest reference magnitude <= 1e-4 (fp32 arithmetic);
pooling selections are bit-exact."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import (ACT_LINEAR, ACT_LOGISTIC, ACT_TANH, AVG_POOL, CNN_ACT_ELU, CNN_ACT_NONE, CNN_ACT_RELU,
                               CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, MAX_POOL, NO_POOL)
from helpers import at, conv_shape, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4
HERE = os.path.dirname(os.path.abspath(__file__))
hip = L.hip


def ok(rc):
    L.check(rc)


# ------------------------------------------------------------------ level 1 and elementwise
def test_level1(dev):
    rng = np.random.default_rng(1)
    for n in (1, 63, 1000, 262147):
        x, y = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        dx_, dy_ = dev.upload(x), dev.upload(y)
        ok(hip.fitre_hip_axpy(n, 0.75, dx_, dy_))
        np.testing.assert_allclose(dev.download(dy_, n), y + np.float32(0.75) * x, rtol=1e-6, atol=1e-6)
        ok(hip.fitre_hip_scal(n, -2.0, dx_))
        np.testing.assert_array_equal(dev.download(dx_, n), -2 * x)
        out = C.c_float()
        x2 = -2 * x.astype(np.float64)
        y2 = dev.download(dy_, n).astype(np.float64)
        ok(hip.fitre_hip_dot(n, dx_, dy_, C.byref(out)))
        assert abs(out.value - np.dot(x2, y2)) <= 1e-5 * max(1, np.abs(x2 * y2).sum())
        ok(hip.fitre_hip_nrm2(n, dx_, C.byref(out)))
        assert abs(out.value - np.linalg.norm(x2)) <= 1e-6 * np.linalg.norm(x2)
        ok(hip.fitre_hip_asum(n, dx_, C.byref(out)))
        assert abs(out.value - np.abs(x2).sum()) <= 1e-6 * np.abs(x2).sum()
        ok(hip.fitre_hip_norm_inf(n, dx_, C.byref(out)))
        assert out.value == np.float32(np.abs(x2).max())
        ok(hip.fitre_hip_sum(n, dx_, C.byref(out)))
        assert abs(out.value - x2.sum()) <= 1e-6 * np.abs(x2).sum()
        ok(hip.fitre_hip_copy(n, dx_, dy_))
        np.testing.assert_array_equal(dev.download(dy_, n), -2 * x)
        dev.free(dx_), dev.free(dy_)


def test_copy_of_a_vector_larger_than_the_caches(dev):
    """fitre_hip_copy from 64 MiB on takes a streaming kernel of its own: same bits, nothing written past the end (a
    length that is not a multiple of the 1024 vectors a workgroup moves)."""
    n = (16 << 20) + 4 * 1000
    x = np.random.default_rng(11).integers(0, 1 << 30, n + 8).astype(np.float32)
    src, dst = dev.upload(x), dev.upload(np.full(n + 8, -1.0, np.float32))
    ok(hip.fitre_hip_copy(n, src, dst))
    got = dev.download(dst, n + 8)
    np.testing.assert_array_equal(got[:n], x[:n])
    assert (got[n:] == -1.0).all()
    dev.free(src), dev.free(dst)


def test_elementwise_helpers(dev):
    rng = np.random.default_rng(2)
    n = 4099
    a, b, c, d = (rng.standard_normal(n).astype(np.float32) for _ in range(4))
    pos = np.abs(b) + np.float32(0.1)
    da, db, dc, dd, dpos, out = (dev.upload(v) for v in (a, b, c, d, pos, np.zeros(n)))
    ok(hip.fitre_hip_hadamard2(da, db, dc, dd, n, out))
    np.testing.assert_allclose(dev.download(out, n), a * b + c * d, rtol=1e-6, atol=1e-6)
    ok(hip.fitre_hip_elem_inv_scale(da, dpos, 1e-3, n, out))
    np.testing.assert_allclose(dev.download(out, n), a / (np.sqrt(pos) + np.float32(1e-3)), rtol=1e-6)
    ok(hip.fitre_hip_elem_sqr(da, n, out))
    np.testing.assert_array_equal(dev.download(out, n), a * a)
    ok(hip.fitre_hip_elem_sqr_decay(da, db, 0.8, n, out))
    np.testing.assert_allclose(dev.download(out, n), np.float32(0.8) * a + np.float32(0.2) * b * b, rtol=1e-5, atol=1e-6)
    ok(hip.fitre_hip_mat_mat_scale(da, db, n, out))
    np.testing.assert_array_equal(dev.download(out, n), a * b)
    ok(hip.fitre_hip_hadamard(da, db, n))
    np.testing.assert_array_equal(dev.download(db, n), a * b)
    ok(hip.fitre_hip_fill(out, n, 1.0))
    assert (dev.download(out, n) == 1).all()
    rows, cols = 7, 13
    m = rng.standard_normal(rows * cols).astype(np.float32)
    v = rng.standard_normal(cols).astype(np.float32)
    dm, dv, o2 = dev.upload(m), dev.upload(v), dev.zeros(rows * cols)
    ok(hip.fitre_hip_mat_row_vec_scale(dm, rows, cols, dv, o2))
    np.testing.assert_array_equal(dev.download(o2, rows * cols), (m.reshape(cols, rows) * v[:, None]).reshape(-1))
    vr = rng.standard_normal(rows).astype(np.float32)
    dvr = dev.upload(vr)
    ok(hip.fitre_hip_add_column(dm, rows, cols, dvr))
    np.testing.assert_array_equal(dev.download(dm, rows * cols), (m.reshape(cols, rows) + vr[None, :]).reshape(-1))
    x = rng.standard_normal(5 * 33).astype(np.float32)
    bias = rng.standard_normal(5).astype(np.float32)
    dxx, dbb = dev.upload(x), dev.upload(bias)
    ok(hip.fitre_hip_add_channel_bias(dxx, 5, 33, dbb))
    np.testing.assert_array_equal(dev.download(dxx, x.size), (x.reshape(5, 33) + bias[:, None]).reshape(-1))
    dsum = dev.zeros(rows)
    ok(hip.fitre_hip_row_sum(dev.upload(m), rows, cols, dsum))
    np.testing.assert_allclose(dev.download(dsum, rows), m.reshape(cols, rows).astype(np.float64).sum(0), rtol=1e-6, atol=1e-6)


def test_memset_and_copies(dev):
    n = 1003
    p = dev.upload(np.arange(n, dtype=np.float32))
    ok(hip.fitre_hip_memset(at(p, 3), 0, 4 * 500))
    got = dev.download(p, n)
    want = np.arange(n, dtype=np.float32)
    want[3:503] = 0
    np.testing.assert_array_equal(got, want)
    q = dev.zeros(n)
    ok(hip.fitre_hip_copy_d2d(q, p, 4 * n))
    np.testing.assert_array_equal(dev.download(q, n), want)


ACTS = [CNN_ACT_RELU, CNN_ACT_SWISH, CNN_ACT_SOFTPLUS, CNN_ACT_ELU, ACT_LOGISTIC, ACT_TANH, CNN_ACT_NONE, ACT_LINEAR]


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("n,misalign", [(4096, 0), (1001, 1)])
def test_activations(dev, oracle64, act, n, misalign):
    rng = np.random.default_rng(act)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    x[:4] = [25.0, -25.0, 0.0, -0.0]
    d = rng.standard_normal(n).astype(np.float32)
    buf = dev.upload(np.concatenate([np.zeros(misalign, np.float32), x]))
    px = at(buf, misalign)
    out = dev.zeros(n + misalign)
    po = at(out, misalign)
    ok(hip.fitre_hip_activation_forward(act, px, po, n))
    y = dev.download(po, n)
    want = oracle64.activation_forward(act, x.astype(np.float64))
    assert rel_err(y, want) < 1e-6
    dd = dev.upload(np.concatenate([np.zeros(misalign, np.float32), d]))
    res = dev.zeros(n + misalign)
    ok(hip.fitre_hip_activation_backward(act, at(dd, misalign), px, po, at(res, misalign), n))
    wantb = oracle64.activation_backward(act, d.astype(np.float64), x.astype(np.float64), want)
    assert rel_err(dev.download(at(res, misalign), n), wantb) < 1e-5
    for b in (buf, out, dd, res):
        dev.free(b)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("n,misalign", [(4096, 0), (1001, 1), (1000, 1)])
def test_activation_directional_derivative_backward(dev, act, n, misalign):
    """R{delta f'(x)} = R{delta} f'(x) + delta f''(x) R{x} against the closed forms of f' and f'' in float64 (16-byte
    path, which leaves out the tensors an activation does not use, and the element-wise path)."""
    rng = np.random.default_rng(100 + act)
    x = (rng.standard_normal(n) * 2).astype(np.float64)
    sg = 1.0 / (1.0 + np.exp(-x))
    if act == CNN_ACT_RELU:
        f, f1, f2 = np.maximum(x, 0), (x > 0) * 1.0, 0 * x
    elif act == CNN_ACT_SWISH:
        f, f1, f2 = x * sg, sg + x * sg * (1 - sg), sg * (1 - sg) * (2 + x * (1 - 2 * sg))
    elif act == CNN_ACT_SOFTPLUS:
        f, f1, f2 = np.log1p(np.exp(x)), sg, sg * (1 - sg)
    elif act == CNN_ACT_ELU:
        f, f1, f2 = np.where(x < 0, np.exp(x) - 1, x), np.where(x < 0, np.exp(x), 1.0), np.where(x < 0, np.exp(x), 0.0)
    elif act == ACT_LOGISTIC:
        f, f1, f2 = sg, sg * (1 - sg), sg * (1 - sg) * (1 - 2 * sg)
    elif act == ACT_TANH:
        t = np.tanh(x)
        f, f1, f2 = t, 1 - t * t, -2 * t * (1 - t * t)
    else:
        f, f1, f2 = x, 1 + 0 * x, 0 * x
    rd, d, rz = (rng.standard_normal(n) for _ in range(3))
    want = rd.astype(np.float32).astype(np.float64) * f1 + d.astype(np.float32).astype(np.float64) * f2 * rz.astype(np.float32)

    def up(v):
        buf = dev.upload(np.concatenate([np.zeros(misalign, np.float32), v.astype(np.float32)]))
        return buf, at(buf, misalign)
    bufs = [up(v) for v in (rd, d, x, f, rz)]
    out = dev.zeros(n + misalign)
    ok(hip.fitre_hip_activation_rop_backward(act, bufs[0][1], bufs[1][1], bufs[2][1], bufs[3][1], bufs[4][1], at(out, misalign), n))
    assert rel_err(dev.download(at(out, misalign), n), want) < 2e-5
    for b, _ in bufs:
        dev.free(b)
    dev.free(out)


def test_unknown_activation_code_is_an_error(dev):
    p = dev.zeros(16)
    assert hip.fitre_hip_activation_forward(99, p, p, 16) == 3
    assert b"unknown activation" in hip.fitre_hip_last_error()
    assert hip.fitre_hip_activation_backward(99, p, p, p, p, 16) == 3
    assert hip.fitre_hip_activation_forward(CNN_ACT_RELU, None, p, 16) == 2


# ------------------------------------------------------------------ pooling
POOL_GEOMS = [  # C, N, A(width), B(height), k, s, p
    (3, 2, 8, 8, 2, 2, 0),      # the 16-byte fast path
    (2, 3, 6, 10, 2, 2, 0),     # 2x2 but B % 4 != 0
    (2, 2, 7, 5, 3, 2, 1),      # the reference's 3/2/1
    (3, 2, 13, 13, 3, 2, 0),    # AlexNet 3/2/0
    (2, 2, 6, 6, 3, 1, 0),      # heavily overlapping
    (8, 1, 2, 2, 3, 2, 1),      # drivers/pool_driver.cu
    (2, 2, 5, 5, 2, 2, 0),      # odd extent: last row/column unpooled
    # maps of 64 cells and more with overlapping windows: the one-workgroup-per-map kernel
    (2, 3, 9, 11, 3, 2, 1),     # 3/2/1 on a rectangular map
    (4, 2, 55, 55, 3, 2, 0),    # AlexNet's first pool
    (2, 2, 12, 12, 3, 1, 1),    # stride 1: every cell in up to nine windows
    (3, 2, 16, 16, 2, 2, 1),    # 2x2 with padding (not the 16-byte fast path)
    # 3/2 windows through the kernel that gives a workgroup several consecutive maps and moves them in 16-byte groups
    (7, 3, 13, 13, 3, 2, 0),    # 21 maps of 169 cells: ranges that start at every alignment
    (257, 13, 13, 13, 3, 2, 0), # 3341 maps: two maps per workgroup, the last workgroup with one
    (5, 3, 27, 27, 3, 2, 0),    # AlexNet's second pool
    (3, 5, 15, 9, 3, 2, 1),     # padding 1, rectangular, odd cell count
    (3, 1367, 47, 47, 3, 2, 0), # 4101 large maps: two groups per workgroup (the second loaded while the first is
                                # worked on), the last workgroup with one
]


@pytest.mark.parametrize("geom", POOL_GEOMS)
@pytest.mark.parametrize("kind", [MAX_POOL, AVG_POOL])
def test_pool_forward_backward(dev, oracle64, geom, kind):
    Cn, N, A, B, k, s, p = geom
    oA, oB = (A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1
    rng = np.random.default_rng(k * 100 + s * 10 + p)
    x = rng.standard_normal(Cn * N * A * B).astype(np.float32)
    d = rng.standard_normal(Cn * N * oA * oB).astype(np.float32)
    px, pd = dev.upload(x), dev.upload(d)
    out, back = dev.zeros(d.size), dev.upload(np.full(x.size, 7.0))
    ok(hip.fitre_hip_pool_forward(kind, px, Cn, N, A, B, k, s, p, oA, oB, out))
    want = oracle64.pool_forward(kind, x, N, Cn, B, A, k, s, p)
    if kind == MAX_POOL:
        np.testing.assert_array_equal(dev.download(out, d.size), want.astype(np.float32))
        idx = dev.zeros(d.size, np.int32)
        ok(hip.fitre_hip_max_pool_argmax(px, Cn, N, A, B, k, s, p, oA, oB, idx))
        np.testing.assert_array_equal(dev.download(idx, d.size, np.int32), oracle64.max_pool_argmax(x, N, Cn, B, A, k, s, p))
    else:
        assert rel_err(dev.download(out, d.size), want) < 1e-6
    ok(hip.fitre_hip_pool_backward(kind, pd, px, Cn, N, A, B, k, s, p, oA, oB, back))
    wantb = oracle64.pool_backward(kind, d, x, N, Cn, B, A, k, s, p)
    got = dev.download(back, x.size)
    assert rel_err(got, wantb) < 1e-6
    if kind == MAX_POOL:  # the routing itself is exact: same zero pattern
        np.testing.assert_array_equal(got != 0, wantb != 0)


@pytest.mark.parametrize("geom", [(4, 3, 8, 8, 2, 2, 0), (3, 5, 6, 12, 2, 2, 0), (64, 16, 4, 4, 2, 2, 0), (2, 3, 6, 10, 2, 2, 0),
                                  (3, 2, 9, 11, 3, 2, 1), (2, 2, 5, 5, 2, 2, 0)])
def test_pool_forward_routed(dev, oracle64, geom):
    """What a max pool passes on of a second tensor: the value at the arg-max of z in every window (16-byte path for
    2x2 windows on rows of a multiple of four cells, the general kernel otherwise), exact."""
    Cn, N, A, B, k, s, p = geom
    oA, oB = (A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1
    rng = np.random.default_rng(A * 100 + B)
    z = rng.standard_normal(Cn * N * A * B).astype(np.float32)
    z[:16] = 0.5                                           # ties: the first cell in memory order wins
    v = rng.standard_normal(z.size).astype(np.float32)
    pz, pv, out = dev.upload(z), dev.upload(v), dev.zeros(Cn * N * oA * oB)
    ok(hip.fitre_hip_pool_forward_routed(MAX_POOL, pv, pz, Cn, N, A, B, k, s, p, oA, oB, out))
    arg = np.asarray(oracle64.max_pool_argmax(z, N, Cn, B, A, k, s, p)).reshape(Cn * N, oA * oB)
    want = np.take_along_axis(v.reshape(Cn * N, A * B), arg, axis=1)
    np.testing.assert_array_equal(dev.download(out, want.size), want.reshape(-1))
    for b in (pz, pv, out):
        dev.free(b)



def test_max_pool_ties_are_bit_exact(dev, oracle64):
    # all-equal windows (post-ReLU zeros), two-way ties, negative ties; 2x2 fast path and generic path
    for (A, B, k, s, p) in [(4, 4, 2, 2, 0), (4, 8, 2, 2, 0), (5, 5, 3, 2, 1), (6, 6, 3, 1, 0), (13, 13, 3, 2, 0), (10, 9, 3, 1, 1)]:
        rng = np.random.default_rng(A * B)
        x = rng.integers(-1, 2, size=3 * 2 * A * B).astype(np.float32)  # values in {-1, 0, 1}: ties everywhere
        oA, oB = (A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1
        d = np.arange(1, 3 * 2 * oA * oB + 1, dtype=np.float32)
        px, pd = dev.upload(x), dev.upload(d)
        idx = dev.zeros(d.size, np.int32)
        ok(hip.fitre_hip_max_pool_argmax(px, 3, 2, A, B, k, s, p, oA, oB, idx))
        np.testing.assert_array_equal(dev.download(idx, d.size, np.int32), oracle64.max_pool_argmax(x, 2, 3, B, A, k, s, p))
        back = dev.zeros(x.size)
        ok(hip.fitre_hip_pool_backward(MAX_POOL, pd, px, 3, 2, A, B, k, s, p, oA, oB, back))
        np.testing.assert_array_equal(dev.download(back, x.size), oracle64.pool_backward(0, d, x, 2, 3, B, A, k, s, p).astype(np.float32))


@pytest.mark.parametrize("geom", POOL_GEOMS[:4] + POOL_GEOMS[7:])
@pytest.mark.parametrize("act", [CNN_ACT_RELU, CNN_ACT_SWISH, CNN_ACT_SOFTPLUS, CNN_ACT_NONE])
@pytest.mark.parametrize("kind", [MAX_POOL, AVG_POOL, NO_POOL])
def test_fused_pool_activation_backward(dev, oracle64, geom, act, kind):
    Cn, N, A, B, k, s, p = geom
    oA, oB = ((A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1) if kind != NO_POOL else (A, B)
    rng = np.random.default_rng(act + kind)
    zin = rng.standard_normal(Cn * N * A * B).astype(np.float32)
    zact = oracle64.activation_forward(act, zin.astype(np.float64)).astype(np.float32)
    d = rng.standard_normal(Cn * N * oA * oB).astype(np.float32)
    pz, pa, pd = dev.upload(zin), dev.upload(zact), dev.upload(d)
    dxp, dxa = dev.zeros(zin.size), dev.zeros(zin.size)
    ok(hip.fitre_hip_pool_act_backward(kind, act, pd, pz, pa, Cn, N, A, B, k, s, p, oA, oB, dxp, dxa))
    if kind == NO_POOL:
        wantp = d.astype(np.float64)
    else:
        wantp = oracle64.pool_backward(kind, d, zact, N, Cn, B, A, k, s, p)
    wanta = oracle64.activation_backward(act, wantp, zin.astype(np.float64), zact.astype(np.float64))
    assert rel_err(dev.download(dxp, zin.size), wantp) < 1e-6
    assert rel_err(dev.download(dxa, zin.size), wanta) < 1e-5


def test_pool_shape_mismatch_is_rejected(dev):
    p = dev.zeros(64)
    assert hip.fitre_hip_pool_forward(MAX_POOL, p, 1, 1, 8, 8, 2, 2, 0, 3, 4, p) == 2
    assert hip.fitre_hip_pool_forward(5, p, 1, 1, 8, 8, 2, 2, 0, 4, 4, p) == 3


# ------------------------------------------------------------------ batch norm and reductions
def bn_ws(dev, Cn, per):
    nbytes = hip.fitre_hip_batch_norm_workspace(Cn, per)
    return dev.alloc(nbytes), nbytes


def test_bn_backward_reference_known_answer(dev):
    g = json.load(open(os.path.join(HERE, "golden", "bn_backward_known_answer.json")))
    ws, nb = bn_ws(dev, 1, 4)
    out = dev.zeros(4)
    ok(hip.fitre_hip_batch_norm_backward(dev.upload(g["err"]), dev.upload(g["zout"]), dev.upload([g["variance"]]), 1, 4,
                                         g["epsilon"], out, None, ws, nb))
    np.testing.assert_allclose(dev.download(out, 4), g["expected"], rtol=2e-5)


@pytest.mark.parametrize("Cn,N,A,B,mis", [(3, 5, 4, 6, 0), (64, 8, 32, 32, 0), (6, 37, 28, 28, 0), (5, 3, 3, 3, 1), (16, 1024, 28, 28, 0),
                                          (128, 4, 8, 8, 0), (130, 3, 5, 7, 1), (512, 256, 4, 4, 0)])  # one-workgroup-per-channel backward
def test_batch_norm_forward_backward(dev, oracle64, Cn, N, A, B, mis):
    per = N * A * B
    rng = np.random.default_rng(per % 1000)
    x = (rng.standard_normal(Cn * per) * 1.7 + 0.4).astype(np.float32)
    d = rng.standard_normal(Cn * per).astype(np.float32) * np.float32(1e-3)
    ws, nb = bn_ws(dev, Cn, per)
    xbuf = dev.upload(np.concatenate([np.zeros(mis, np.float32), x]))
    px = at(xbuf, mis)
    zh = dev.zeros(Cn * per + mis)
    pz = at(zh, mis)
    stats = dev.upload(np.concatenate([np.zeros(2 * Cn), np.full(Cn, 0.5), np.full(Cn, 2.0)]))
    mean, var, rmean, rvar = (at(stats, i * Cn) for i in range(4))
    ok(hip.fitre_hip_batch_norm_forward(px, Cn, per, pz, mean, var, rmean, rvar, 1e-5, 0.9, 1, ws, nb))
    zhat, wmean, wvar, wrm, wrv = oracle64.batch_norm_forward(x, B, A, Cn, N, running=(np.full(Cn, 0.5), np.full(Cn, 2.0)))
    got_stats = dev.download(stats, 4 * Cn)
    assert rel_err(got_stats[:Cn], wmean) < 1e-5 and rel_err(got_stats[Cn:2 * Cn], wvar) < 1e-5
    assert rel_err(got_stats[2 * Cn:3 * Cn], wrm) < 1e-5 and rel_err(got_stats[3 * Cn:], wrv) < 1e-5
    assert rel_err(dev.download(pz, Cn * per), zhat) < 1e-5
    # evaluation mode: running statistics, which the call must leave unchanged
    ok(hip.fitre_hip_batch_norm_forward(px, Cn, per, pz, mean, var, rmean, rvar, 1e-5, 0.9, 0, ws, nb))
    ze, *_ = oracle64.batch_norm_forward(x, B, A, Cn, N, train=False, running=(wrm, wrv))
    assert rel_err(dev.download(pz, Cn * per), ze) < 1e-5
    np.testing.assert_array_equal(dev.download(stats, 4 * Cn), got_stats)
    # backward on the oracle's zhat (isolates the backward kernel)
    dbuf = dev.upload(np.concatenate([np.zeros(mis, np.float32), d]))
    zbuf = dev.upload(np.concatenate([np.zeros(mis, np.float32), zhat.astype(np.float32)]))
    out = dev.zeros(Cn * per + mis)
    db_ = dev.zeros(Cn)
    ok(hip.fitre_hip_batch_norm_backward(at(dbuf, mis), at(zbuf, mis), dev.upload(wvar), Cn, per, 1e-5, at(out, mis), db_, ws, nb))
    want = oracle64.batch_norm_backward(d, zhat.astype(np.float32), wvar.astype(np.float32), B, A, Cn, N)
    got = dev.download(at(out, mis), Cn * per)
    assert rel_err(got, want) < TOL
    # bias gradient = column sums of the result; mathematically zero, so compare with the sums of what was written
    np.testing.assert_allclose(dev.download(db_, Cn), got.astype(np.float64).reshape(Cn, per).sum(1), atol=1e-5 * np.abs(got).max() * np.sqrt(per))
    for b in (xbuf, zh, dbuf, zbuf, out, ws):
        dev.free(b)


@pytest.mark.parametrize("Cn,per,mis", [(3, 4096, 0), (64, 32768, 0), (5, 1001, 0), (4, 4096, 1), (130, 64, 0)])
def test_batch_norm_backward_directional_derivative(dev, Cn, per, mis):
    """out = (R{dx} - <R{dx}> - R{zhat} <dx zhat> - zhat (<R{dx} zhat> + <dx R{zhat}>)) / s - dc <zhat R{x}> / s per channel
    (<.> the mean over the channel, s = sqrt(var + eps)) against the same formula in float64: 16-byte path and the
    element-wise one (odd channel length, misaligned tensors)."""
    rng = np.random.default_rng(Cn + per)
    names = ("rdx", "dx", "zhat", "rzhat", "rx", "dc")
    t = {k: rng.standard_normal((Cn, per)).astype(np.float32) for k in names}
    var = (rng.random(Cn) + 0.5).astype(np.float32)
    eps = 1e-5
    f = {k: v.astype(np.float64) for k, v in t.items()}
    sdev = np.sqrt(var.astype(np.float64) + eps)[:, None]
    mean = lambda v: v.mean(axis=1, keepdims=True)
    want = (f["rdx"] - mean(f["rdx"]) - f["rzhat"] * mean(f["dx"] * f["zhat"]) -
            f["zhat"] * (mean(f["rdx"] * f["zhat"]) + mean(f["dx"] * f["rzhat"]))) / sdev - f["dc"] * mean(f["zhat"] * f["rx"]) / sdev
    bufs = {k: dev.upload(np.concatenate([np.zeros(mis, np.float32), v.reshape(-1)])) for k, v in t.items()}
    p = {k: at(b, mis) for k, b in bufs.items()}
    out = dev.zeros(Cn * per + mis)
    ws, nb = bn_ws(dev, Cn, per)
    ok(hip.fitre_hip_batch_norm_rop_backward(p["rdx"], p["dx"], p["zhat"], p["rzhat"], p["rx"], p["dc"], dev.upload(var), Cn, per, eps,
                                             at(out, mis), ws, nb))
    assert rel_err(dev.download(at(out, mis), Cn * per), want.reshape(-1)) < 1e-5
    for b in list(bufs.values()) + [out, ws]:
        dev.free(b)


@pytest.mark.parametrize("act,derive", [(CNN_ACT_RELU, False), (CNN_ACT_RELU, True), (CNN_ACT_SWISH, False)])
@pytest.mark.parametrize("kind", [MAX_POOL, NO_POOL])
@pytest.mark.parametrize("geom", [(3, 40, 16, 16, 2, 2, 0), (64, 8, 32, 32, 2, 2, 0), (5, 9, 6, 12, 2, 2, 0), (160, 7, 8, 8, 2, 2, 0),
                                  (2, 4, 6, 10, 2, 2, 0), (2, 2, 7, 5, 3, 2, 1)])
def test_fused_directional_derivative_forward(dev, geom, kind, act, derive):
    """R{bn out}, R{act out} and the routed pooled values of a layer in one call against the three separate entry
    points (fused shapes and those that fall back); `derive`: without the activation output, which only ReLU allows."""
    Cn, N, A, B, k, s, p = geom
    oA, oB = (A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1
    per = N * A * B
    fusable = (kind == NO_POOL or (k == 2 and B % 4 == 0 and A % 2 == 0)) and per % 4 == 0
    rng = np.random.default_rng(Cn * 3 + A * B + act)
    rx = rng.standard_normal(Cn * per).astype(np.float32)
    zhat = rng.standard_normal(Cn * per).astype(np.float32)
    var = (rng.random(Cn) + 0.5).astype(np.float32)
    prx, pzh, pvar = dev.upload(rx), dev.upload(zhat), dev.upload(var)
    zact = dev.zeros(Cn * per)
    ok(hip.fitre_hip_activation_forward(act, pzh, zact, Cn * per))
    ws, nb = bn_ws(dev, Cn, per)
    pooled = Cn * N * oA * oB

    def run(fused):
        rbn, ract, rpool = dev.zeros(Cn * per), dev.zeros(Cn * per), dev.zeros(pooled)
        if fused:
            rc = hip.fitre_hip_bn_act_pool_rop_forward(prx, pzh, None if derive else zact, pvar, Cn, N, A, B, 1e-5, act, rbn, ract, kind, k, s,
                                                       p, oA, oB, rpool if kind != NO_POOL else None, ws, nb)
            if derive and not fusable:
                assert rc != 0                       # the separate passes need the activation output
                return None
            ok(rc)
        else:
            ok(hip.fitre_hip_batch_norm_backward(prx, pzh, pvar, Cn, per, 1e-5, rbn, None, ws, nb))
            ok(hip.fitre_hip_activation_backward(act, rbn, pzh, zact, ract, Cn * per))
            if kind != NO_POOL:
                ok(hip.fitre_hip_pool_forward_routed(kind, ract, zact, Cn, N, A, B, k, s, p, oA, oB, rpool))
        return [dev.download(b, n) for b, n in ((rbn, Cn * per), (ract, Cn * per), (rpool, pooled))]

    want, got = run(False), run(True)
    if got is not None:
        for g, w in zip(got, want):
            assert rel_err(g, w) < 1e-6
            np.testing.assert_array_equal(g == 0, w == 0)   # the same routing and the same masks
    dev.free(ws)


@pytest.mark.parametrize("act,derive", [(CNN_ACT_RELU, False), (CNN_ACT_RELU, True), (CNN_ACT_SWISH, False)])
@pytest.mark.parametrize("kind", [MAX_POOL, NO_POOL])
@pytest.mark.parametrize("geom", [(3, 40, 16, 16, 2, 2, 0), (64, 8, 32, 32, 2, 2, 0), (5, 9, 6, 12, 2, 2, 0), (160, 7, 8, 8, 2, 2, 0),
                                  (2, 4, 6, 10, 2, 2, 0), (2, 2, 7, 5, 3, 2, 1)])
def test_fused_directional_derivative_backward(dev, geom, kind, act, derive):
    """Pooling routing, R{delta f'(x)} and the batch-norm R-step of a layer in one call against the three separate entry
    points (fused shapes and those that fall back); `derive`: without the activation output, which only ReLU allows."""
    Cn, N, A, B, k, s, p = geom
    oA, oB = ((A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1) if kind != NO_POOL else (A, B)
    per = N * A * B
    fusable = (kind == NO_POOL or (k == 2 and B % 4 == 0 and A % 2 == 0)) and per % 4 == 0
    rng = np.random.default_rng(Cn * 5 + A * B + act)
    full = lambda: dev.upload(rng.standard_normal(Cn * per).astype(np.float32))
    pzh, pdelta, prz, pdx, prx, pdc = (full() for _ in range(6))
    prd = dev.upload(rng.standard_normal(Cn * N * oA * oB).astype(np.float32))
    pvar = dev.upload((rng.random(Cn) + 0.5).astype(np.float32))
    zact = dev.zeros(Cn * per)
    ok(hip.fitre_hip_activation_forward(act, pzh, zact, Cn * per))
    ws, nb = bn_ws(dev, Cn, per)

    def run(fused):
        routed, rdx, out = dev.zeros(Cn * per), dev.zeros(Cn * per), dev.zeros(Cn * per)
        if fused:
            rc = hip.fitre_hip_pool_act_bn_rop_backward(kind, act, prd, pdelta, pzh, None if derive else zact, prz, pdx, prx, pdc, pvar, Cn, N,
                                                        A, B, k, s, p, oA, oB, 1e-5, routed, rdx, out, ws, nb)
            if derive and not fusable:
                assert rc != 0                       # the separate passes need the activation output
                return None
            ok(rc)
        else:
            src = prd
            if kind != NO_POOL:
                ok(hip.fitre_hip_pool_backward(kind, prd, zact, Cn, N, A, B, k, s, p, oA, oB, routed))
                src = routed
            ok(hip.fitre_hip_activation_rop_backward(act, src, pdelta, pzh, zact, prz, rdx, Cn * per))
            ok(hip.fitre_hip_batch_norm_rop_backward(rdx, pdx, pzh, prz, prx, pdc, pvar, Cn, per, 1e-5, out, ws, nb))
        return [dev.download(b, Cn * per) for b in (rdx, out)]

    want, got = run(False), run(True)
    if got is not None:
        assert rel_err(got[0], want[0]) < 1e-6
        np.testing.assert_array_equal(got[0] == 0, want[0] == 0)   # the same routing and the same masks
        assert rel_err(got[1], want[1]) < 1e-5
    dev.free(ws)


# C, N, A, B, k, s, p: fused sums (large channels), one-workgroup-per-channel (short channels, >= 128
# of them), and shapes that fall back to the separate passes
FUSED_BN_GEOMS = [
    (3, 40, 16, 16, 2, 2, 0),    # two-launch fused path, several segments
    (64, 8, 32, 32, 2, 2, 0),
    (5, 9, 6, 12, 2, 2, 0),
    (128, 16, 4, 4, 2, 2, 0),    # short channels: one launch
    (160, 7, 8, 8, 2, 2, 0),
    (130, 2, 2, 4, 2, 2, 0),
    (512, 64, 2, 2, 2, 2, 0),    # maps with B == 2: a window is one 16-byte group
    (5, 2100, 6, 2, 2, 2, 0),    # the same on long channels
    (2, 4, 6, 10, 2, 2, 0),      # B % 4 == 2: windows moved as 8-byte rows (LeNet's 10 x 10 maps)
    (16, 32, 10, 10, 2, 2, 0),   # the same, several segments
    (130, 2, 2, 6, 2, 2, 0),     # the same on short channels (two launches)
    (2, 3, 6, 10, 2, 2, 0),      # channel length not a multiple of four: separate passes
    (3, 4, 6, 5, 2, 2, 0),       # odd B: separate passes
    (2, 2, 7, 5, 3, 2, 1),       # 3/2/1 window: separate passes
]


@pytest.mark.parametrize("bn,train", [(True, 1), (True, 0), (False, 1)])
@pytest.mark.parametrize("act", [CNN_ACT_RELU, CNN_ACT_SWISH])
@pytest.mark.parametrize("kind", [MAX_POOL, NO_POOL])
@pytest.mark.parametrize("geom", FUSED_BN_GEOMS)
def test_fused_batch_norm_activation_pool_forward(dev, oracle64, geom, kind, act, bn, train):
    """One call for the normalisation, activation and pooling of a layer's convolution output against the three
    separate entry points on the same input: the same bits in every output (fused shapes and the ones that fall back
    alike), the statistics to rounding, and zhat against the oracle."""
    Cn, N, A, B, k, s, p = geom
    oA, oB = (A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1
    per = N * A * B
    rng = np.random.default_rng(Cn * 7 + N + A * B)
    x = (rng.standard_normal(Cn * per) * 1.3 + 0.2).astype(np.float32)
    px = dev.upload(x)
    ws, nb = bn_ws(dev, Cn, per)
    running = np.concatenate([np.zeros(2 * Cn), np.full(Cn, 0.25), np.full(Cn, 1.5)]).astype(np.float32)
    pooled = Cn * N * oA * oB

    def separate():
        stats = dev.upload(running)
        mean, var, rmean, rvar = (at(stats, i * Cn) for i in range(4))
        zh, ao, po = dev.zeros(Cn * per), dev.zeros(Cn * per), dev.zeros(pooled)
        src = px
        if bn:
            ok(hip.fitre_hip_batch_norm_forward(px, Cn, per, zh, mean, var, rmean, rvar, 1e-5, 0.9, train, ws, nb))
            src = zh
        ok(hip.fitre_hip_activation_forward(act, src, ao, Cn * per))
        if kind != NO_POOL:
            ok(hip.fitre_hip_pool_forward(kind, ao, Cn, N, A, B, k, s, p, oA, oB, po))
        return [dev.download(b, n) for b, n in ((zh, Cn * per), (ao, Cn * per), (po, pooled), (stats, 4 * Cn))]

    def fused():
        stats = dev.upload(running)
        mean, var, rmean, rvar = (at(stats, i * Cn) for i in range(4))
        zh, ao, po = dev.zeros(Cn * per), dev.zeros(Cn * per), dev.zeros(pooled)
        ok(hip.fitre_hip_bn_act_pool_forward(px, Cn, N, A, B, zh if bn else None, mean if bn else None, var if bn else None,
                                             rmean if bn else None, rvar if bn else None, 1e-5, 0.9, train, act, ao, kind, k, s, p,
                                             oA, oB, po if kind != NO_POOL else None, ws, nb))
        return [dev.download(b, n) for b, n in ((zh, Cn * per), (ao, Cn * per), (po, pooled), (stats, 4 * Cn))]

    want, got = separate(), fused()
    np.testing.assert_allclose(got[3], want[3], rtol=1e-6, atol=1e-7)
    if np.array_equal(got[3], want[3]):            # the same statistics to the bit: so is everything made from them
        for g, w in zip(got[:3], want[:3]):
            np.testing.assert_array_equal(g, w)
    else:
        for g, w in zip(got[:3], want[:3]):
            assert rel_err(g, w) < 1e-6
    if bn and train:
        zhat, *_ = oracle64.batch_norm_forward(x, B, A, Cn, N, running=(np.full(Cn, 0.25), np.full(Cn, 1.5)))
        assert rel_err(got[0], zhat) < 1e-5
    dev.free(ws)


@pytest.mark.parametrize("geom", FUSED_BN_GEOMS)
@pytest.mark.parametrize("act,derive,slabs", [(CNN_ACT_RELU, True, 1), (CNN_ACT_RELU, False, 1), (CNN_ACT_SWISH, False, 1),
                                              (CNN_ACT_RELU, True, 3), (CNN_ACT_SWISH, False, 8)])
@pytest.mark.parametrize("kind", [MAX_POOL, NO_POOL, AVG_POOL])
def test_fused_pool_activation_batch_norm_backward(dev, oracle64, geom, act, derive, slabs, kind):
    """fitre_hip_pool_act_bn_backward against the oracle's three steps (functions/cnn_backward.cu:586-660).
    slabs > 1: delta arrives as unsummed split partials (the view of fitre_hip_conv_input_grad_split); the
    gradient is their sum in slab order, accumulated in double and rounded once."""
    Cn, N, A, B, k, s, p = geom
    oA, oB = ((A + 2 * p - k) // s + 1, (B + 2 * p - k) // s + 1) if kind != NO_POOL else (A, B)
    per = N * A * B
    rng = np.random.default_rng(Cn * 7 + A + act + kind)
    zhat = rng.standard_normal(Cn * per).astype(np.float32)
    zact = oracle64.activation_forward(act, zhat.astype(np.float64)).astype(np.float32)
    var = (0.5 + rng.random(Cn)).astype(np.float32)
    nd = Cn * N * oA * oB
    stride = nd + (8 - nd % 8) % 8 + 8           # slabs 16-byte aligned, with a gap
    parts = rng.standard_normal((slabs, stride)).astype(np.float32)
    d = parts[:, :nd].astype(np.float64).sum(axis=0).astype(np.float32) if slabs > 1 else parts[0, :nd].copy()
    if slabs > 1:   # sequential double accumulation, as on the device
        acc = np.zeros(nd)
        for q in range(slabs):
            acc += parts[q, :nd].astype(np.float64)
        d = acc.astype(np.float32)
    pz, pa, pd, pv = dev.upload(zhat), dev.upload(zact), dev.upload(parts.reshape(-1)), dev.upload(var)
    dxp, dxa, dxb, bias = dev.zeros(zhat.size), dev.zeros(zhat.size), dev.zeros(zhat.size), dev.zeros(Cn)
    ws, nb = bn_ws(dev, Cn, per)
    ok(hip.fitre_hip_pool_act_bn_backward(kind, act, pd, slabs, stride, pz, None if derive else pa, pv, Cn, N, A, B, k, s, p, oA,
                                          oB, 1e-5, dxp, dxa, dxb, bias, ws, nb))
    if kind == NO_POOL:
        wantp = d.astype(np.float64)
    else:
        wantp = oracle64.pool_backward(kind, d, zact, N, Cn, B, A, k, s, p)
    wanta = oracle64.activation_backward(act, wantp, zhat.astype(np.float64), zact.astype(np.float64))
    gotp, gota, gotb = (dev.download(b, zhat.size) for b in (dxp, dxa, dxb))
    assert rel_err(gotp, wantp) < 1e-6
    if kind == MAX_POOL:
        np.testing.assert_array_equal(gotp != 0, wantp != 0)  # the routing is exact
    assert rel_err(gota, wanta) < 1e-5
    # batch-norm step on the gradient the device itself wrote (isolates it from rounding of the first two)
    wantb = oracle64.batch_norm_backward(gota, zhat, var, B, A, Cn, N)
    assert rel_err(gotb, wantb) < TOL
    np.testing.assert_allclose(dev.download(bias, Cn), gotb.astype(np.float64).reshape(Cn, per).sum(1),
                               atol=1e-5 * np.abs(gotb).max() * np.sqrt(per) + 1e-7)
    for b in (pz, pa, pd, pv, dxp, dxa, dxb, bias, ws):
        dev.free(b)


@pytest.mark.parametrize("kind", [MAX_POOL, NO_POOL])
def test_fused_backward_on_a_tensor_larger_than_the_caches(dev, oracle64, kind):
    """52 MB per tensor: the pool gradient is then written with streaming stores."""
    Cn, N, A, B = 64, 200, 32, 32
    oA, oB = (A // 2, B // 2) if kind == MAX_POOL else (A, B)
    per = N * A * B
    rng = np.random.default_rng(kind + 5)
    zhat = rng.standard_normal(Cn * per).astype(np.float32)
    zact = np.maximum(zhat, 0)
    var = (0.5 + rng.random(Cn)).astype(np.float32)
    d = rng.standard_normal(Cn * N * oA * oB).astype(np.float32)
    pz, pd, pv = dev.upload(zhat), dev.upload(d), dev.upload(var)
    dxp, dxa, dxb, bias = dev.zeros(zhat.size), dev.zeros(zhat.size), dev.zeros(zhat.size), dev.zeros(Cn)
    ws, nb = bn_ws(dev, Cn, per)
    ok(hip.fitre_hip_pool_act_bn_backward(kind, CNN_ACT_RELU, pd, 1, 0, pz, None, pv, Cn, N, A, B, 2, 2, 0, oA, oB, 1e-5, dxp, dxa,
                                          dxb, bias, ws, nb))
    wantp = oracle64.pool_backward(kind, d, zact, N, Cn, B, A, 2, 2, 0) if kind == MAX_POOL else d.astype(np.float64)
    gotp, gota, gotb = (dev.download(b, zhat.size) for b in (dxp, dxa, dxb))
    np.testing.assert_array_equal(gotp, wantp.astype(np.float32))
    np.testing.assert_array_equal(gota, np.where(zhat > 0, gotp, np.float32(0)))
    wantb = oracle64.batch_norm_backward(gota, zhat, var, B, A, Cn, N)
    assert rel_err(gotb, wantb) < TOL
    for b in (pz, pd, pv, dxp, dxa, dxb, bias, ws):
        dev.free(b)


def test_fused_backward_rejects_missing_activation_output(dev):
    p = dev.zeros(256)
    ws, nb = bn_ws(dev, 1, 64)
    assert hip.fitre_hip_pool_act_bn_backward(NO_POOL, CNN_ACT_SWISH, p, 1, 0, p, None, p, 1, 1, 8, 8, 1, 1, 0, 8, 8, 1e-5, p, p, p, None, ws, nb) == 2
    assert b"ReLU only" in hip.fitre_hip_last_error()
    assert hip.fitre_hip_pool_act_bn_backward(NO_POOL, CNN_ACT_RELU, p, 2, 0, p, None, p, 1, 1, 8, 8, 1, 1, 0, 8, 8, 1e-5, p, p, p, None, ws, nb) == 2
    assert b"split view" in hip.fitre_hip_last_error()


def test_workspace_too_small_is_reported(dev):
    p = dev.zeros(4096)
    assert hip.fitre_hip_batch_norm_backward(p, p, p, 4, 1024, 1e-5, p, None, p, 8) == 4
    assert b"workspace" in hip.fitre_hip_last_error()


@pytest.mark.parametrize("Cn,per", [(6, 100352), (16, 12800), (64, 262144), (3, 17), (512, 1024)])
def test_channel_sum(dev, Cn, per):
    rng = np.random.default_rng(Cn)
    x = rng.standard_normal(Cn * per).astype(np.float32)
    nb = hip.fitre_hip_channel_sum_workspace(Cn, per)
    ws, out = dev.alloc(nb), dev.zeros(Cn)
    ok(hip.fitre_hip_channel_sum(dev.upload(x), Cn, per, out, ws, nb))
    want = x.astype(np.float64).reshape(Cn, per).sum(1)
    np.testing.assert_allclose(dev.download(out, Cn), want, atol=2e-7 * np.abs(x).astype(np.float64).reshape(Cn, per).sum(1).max())


# ------------------------------------------------------------------ softmax cross entropy
@pytest.mark.parametrize("rows,classes", [(4, 10), (256, 10), (64, 1000), (1024, 10), (3, 70)])
def test_softmax_cross_entropy(dev, oracle64, rows, classes):
    rng = np.random.default_rng(rows + classes)
    logits = (rng.standard_normal(rows * classes) * 2).astype(np.float32)
    y = rng.integers(1, classes + 1, rows).astype(np.float32)
    pl, py = dev.upload(logits), dev.upload(y)
    probs, err = dev.zeros(rows * classes), dev.zeros(rows * classes)
    loss = C.c_float()
    ok(hip.fitre_hip_softmax_cross_entropy(pl, py, rows, classes, probs, err, C.byref(loss)))
    wl, wp = oracle64.softmax_loss(logits, y, rows, classes)
    we = oracle64.cross_entropy_error(wp, y, rows, classes)
    assert abs(loss.value - wl) < 1e-5 * max(1, abs(wl))
    assert rel_err(dev.download(probs, rows * classes), wp) < 1e-5
    assert rel_err(dev.download(err, rows * classes), we) < 1e-5
    err2 = dev.zeros(rows * classes)
    ok(hip.fitre_hip_cross_entropy_error(probs, py, rows, classes, err2))
    np.testing.assert_allclose(dev.download(err2, rows * classes), dev.download(err, rows * classes), rtol=1e-6, atol=1e-9)


# ------------------------------------------------------------------ layout changes
def test_boundary_permutes(dev, oracle64):
    Cn, N, A, B = 5, 3, 4, 2
    x = np.arange(Cn * N * A * B, dtype=np.float32)
    px, out, back = dev.upload(x), dev.zeros(x.size), dev.zeros(x.size)
    ok(hip.fitre_hip_conv_to_fc(px, Cn, N, A, B, out))
    want = oracle64.transpose(oracle64.reshape(x, Cn, N, A * B), Cn * N, B, A)
    np.testing.assert_array_equal(dev.download(out, x.size), want)
    ok(hip.fitre_hip_fc_to_conv(out, Cn, N, A, B, back))
    np.testing.assert_array_equal(dev.download(back, x.size), x)
    ok(hip.fitre_hip_reshape(px, Cn, N, A * B, out))
    np.testing.assert_array_equal(dev.download(out, x.size), oracle64.reshape(x, Cn, N, A * B))
    assert hip.fitre_hip_conv_to_fc(px, Cn, N, A, B, px) == 2  # in place is refused


@pytest.mark.parametrize("rows,classes", [(4, 3), (256, 10), (1000, 1000), (1, 1)])
def test_compute_accuracy(dev, oracle64, rows, classes):
    rng = np.random.default_rng(rows + classes)
    p = rng.random((rows, classes)).astype(np.float32)
    p[0, :] = 0.25 if classes > 1 else 1.0       # a tie: the first class wins
    t = rng.integers(1, classes + 1, rows).astype(np.float32)
    pp, pt, scratch = dev.upload(p.reshape(-1)), dev.upload(t), dev.zeros(rows)
    hits = C.c_float(-1)
    pct = L.cnn.computeAccuracy(pp, pt, rows, classes, scratch, C.byref(hits))
    wpct, whits = oracle64.compute_accuracy(p.reshape(-1), t, rows, classes)
    assert hits.value == whits
    assert abs(pct - wpct) < 1e-4


def test_random_streams(dev, oracle64):
    ok(hip.fitre_hip_random_seed(4321))
    a, b = dev.zeros(1001), dev.zeros(64)
    ok(hip.fitre_hip_random_uniform(a, 1001))
    ok(hip.fitre_hip_random_uniform(b, 64))          # continues the stream
    np.testing.assert_array_equal(dev.download(a, 1001), oracle64.uniform_stream(4321, 0, 1001))
    np.testing.assert_array_equal(dev.download(b, 64), oracle64.uniform_stream(4321, 1001, 64))
    ok(hip.fitre_hip_random_seed(4321))
    ok(hip.fitre_hip_random_uniform(b, 64))          # re-seeding restarts it
    np.testing.assert_array_equal(dev.download(b, 64), oracle64.uniform_stream(4321, 0, 64))
    # normal: Box-Muller of consecutive pairs of the same stream
    n = 200001
    c = dev.zeros(n)
    ok(hip.fitre_hip_random_seed(7))
    ok(hip.fitre_hip_random_normal(c, n))
    got = dev.download(c, n)
    u = oracle64.uniform_stream(7, 0, n + 1).astype(np.float64)
    r = np.sqrt(-2 * np.log(u[0::2]))
    want = np.stack([r * np.cos(2 * np.pi * u[1::2]), r * np.sin(2 * np.pi * u[1::2])], axis=1).reshape(-1)[:n]
    assert np.abs(got - want).max() < 5e-5
    assert abs(got.mean()) < 1e-2 and abs(got.std() - 1) < 1e-2


@pytest.mark.parametrize("rows,classes", [(5, 3), (256, 10), (4096, 1000)])
def test_distribution_errors(dev, oracle64, rows, classes):
    """computeDistributionErrors: targets drawn from the predictive distribution with the seeded stream, and the
    cross-entropy errors against them; bit-exact classes given the same uniform numbers."""
    rng = np.random.default_rng(rows)
    p = rng.random((rows, classes)).astype(np.float32)
    p = (p / p.sum(1, keepdims=True)).astype(np.float32)
    pp = dev.upload(p.reshape(-1))
    tgt, err, scratch = dev.zeros(rows), dev.zeros(rows * classes), dev.zeros(rows + 1)
    ok(hip.fitre_hip_random_seed(99))
    L.cnn.computeDistributionErrors(pp, tgt, err, rows, classes, scratch, None)
    u = oracle64.uniform_stream(99, 0, rows)
    # the oracle in float32 arithmetic: the running sum must round as on the device
    import oracle.oracle as O
    want_t = O.Oracle(double=False).multinomial_classes(p.reshape(-1), u, rows, classes)
    got_t = dev.download(tgt, rows)
    np.testing.assert_array_equal(got_t, want_t)
    want_e = oracle64.cross_entropy_error(p.reshape(-1), got_t, rows, classes)
    assert rel_err(dev.download(err, rows * classes), want_e) < 1e-6
    # the empirical class frequencies follow the probabilities
    if rows >= 4096:
        assert abs(np.mean(got_t) - np.mean((p * np.arange(1, classes + 1)).sum(1))) < 0.05 * classes


def test_empty_inputs(dev):
    """Zero-length vectors are no-ops (reductions give 0), zero-sized tensors of the layer kernels are argument
    errors, negative sizes always are; nothing is launched with an empty grid."""
    p = dev.upload(np.arange(8, dtype=np.float32))
    q = dev.upload(np.full(8, 3.0, np.float32))
    res = (C.c_float * 1)(7.0)
    ok(hip.fitre_hip_axpy(0, 2.0, p, q))
    ok(hip.fitre_hip_scal(0, 2.0, q))
    ok(hip.fitre_hip_copy(0, p, q))
    ok(hip.fitre_hip_fill(q, 0, 9.0))
    ok(hip.fitre_hip_hadamard(p, q, 0))
    ok(hip.fitre_hip_activation_forward(CNN_ACT_RELU, p, q, 0))
    ok(hip.fitre_hip_activation_backward(CNN_ACT_RELU, p, p, p, q, 0))
    np.testing.assert_array_equal(dev.download(q, 8), np.full(8, 3.0, np.float32))
    for fn in (hip.fitre_hip_nrm2, hip.fitre_hip_asum, hip.fitre_hip_sum):
        res[0] = 7.0
        ok(fn(0, p, res))
        assert res[0] == 0.0
    ok(hip.fitre_hip_dot(0, p, q, res))
    assert res[0] == 0.0
    assert hip.fitre_hip_axpy(-1, 2.0, p, q) == 2
    assert hip.fitre_hip_activation_forward(CNN_ACT_RELU, p, q, -5) == 2
    assert hip.fitre_hip_pool_forward(MAX_POOL, p, 0, 1, 2, 2, 2, 2, 0, 1, 1, q) == 2
    assert hip.fitre_hip_pool_backward(MAX_POOL, p, p, 1, 0, 2, 2, 2, 2, 0, 1, 1, q) == 2
    ws, nb = bn_ws(dev, 1, 8)
    assert hip.fitre_hip_batch_norm_backward(p, p, p, 0, 8, 1e-5, q, None, ws, nb) == 2
    assert hip.fitre_hip_batch_norm_backward(p, p, p, 1, 0, 1e-5, q, None, ws, nb) == 2
    assert hip.fitre_hip_channel_sum(p, 0, 8, q, ws, nb) == 2
    assert hip.fitre_hip_softmax_cross_entropy(p, p, 0, 4, q, q, res) == 2
    from helpers import conv_shape
    s = conv_shape(0, 2, 2, 2, 2, 3, 1, 1)
    assert hip.fitre_hip_conv_weight_grad(C.byref(s), p, p, q, None, 0) == 2
    assert hip.fitre_hip_conv_input_grad(C.byref(s), p, p, q, None, 0) == 2


@pytest.mark.parametrize("m,n", [(1, 1), (5, 7), (32, 32), (33, 65), (513, 4609), (300, 10)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_geam(dev, m, n, ta, tb):
    """C = alpha op(A) + beta op(B) (the reference's cublasDgeam, solvers/kfac_natural_gradient.cu:166-170) against
    numpy on column-major operands with padded leading dimensions; the reference's own use (transpose: beta = 0, B null)
    bit for bit."""
    rng = np.random.default_rng(m * 7 + n + 2 * ta + tb)
    lda, ldb, ldc = (n if ta else m) + 3, (n if tb else m) + 1, m + 2
    a = rng.standard_normal(lda * (m if ta else n)).astype(np.float32)
    b = rng.standard_normal(ldb * (m if tb else n)).astype(np.float32)
    A = a.reshape((m if ta else n), lda).T[: (n if ta else m)]          # column-major view: A[r, c] = a[c * lda + r]
    B = b.reshape((m if tb else n), ldb).T[: (n if tb else m)]
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    pa, pb = dev.upload(a), dev.upload(b)
    pc = dev.upload(np.full(ldc * n, 9.0, np.float32))
    ok(hip.fitre_hip_geam(ta, tb, m, n, 0.75, pa, lda, -1.5, pb, ldb, pc, ldc))
    got = dev.download(pc, ldc * n).reshape(n, ldc)
    want = (np.float32(0.75) * opA + np.float32(-1.5) * opB).T                  # [c][r]
    np.testing.assert_allclose(got[:, :m], want, rtol=1e-6, atol=1e-6)
    assert (got[:, m:] == 9.0).all()                                          # the padding of C is left alone
    ok(hip.fitre_hip_geam(ta, 0, m, n, 1.0, pa, lda, 0.0, None, m, pc, ldc))    # the transpose / copy use
    np.testing.assert_array_equal(dev.download(pc, ldc * n).reshape(n, ldc)[:, :m], opA.T)
    assert hip.fitre_hip_geam(ta, tb, m, n, 1.0, pa, lda, 1.0, None, ldb, pc, ldc) == 2
    for q in (pa, pb, pc):
        dev.free(q)
