"""Backward products of one fully connected layer (fitre_hip_linear_input_grad / _weight_grad) against float64
numpy on the same float32 operands: the fused single-launch kernel for small layers and the sequence of plain
steps for large ones must both give W' * delta times the activation derivative of the layer below (optionally in
the convolution layout), dW = delta * z' and db = delta * 1."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import CNN_ACT_ELU, CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SOFTPLUS, CNN_ACT_SWISH
from helpers import rel_err

pytestmark = pytest.mark.gpu
hip = L.hip
TOL = 1e-5  # float32 products of at most 4096 terms against float64


def ok(rc):
    assert rc == 0, hip.fitre_hip_last_error().decode()


def derivative(act, zi, zo):
    """f'(.) as functions/cnn_backward.cu:100-172 applies it (ReLU and ELU decide on the activation output)."""
    sig = 1.0 / (1.0 + np.exp(-zi))
    return {CNN_ACT_RELU: (zo > 0).astype(np.float64), CNN_ACT_ELU: np.where(zo < 0, zo + 1.0, 1.0),
            CNN_ACT_SOFTPLUS: sig, CNN_ACT_SWISH: zo + sig * (1.0 - zo), CNN_ACT_NONE: np.ones_like(zi), -1: np.ones_like(zi)}[act]


def forward_act(act, zi):
    sig = 1.0 / (1.0 + np.exp(-zi))
    return {CNN_ACT_RELU: np.maximum(zi, 0), CNN_ACT_ELU: np.where(zi < 0, np.exp(zi) - 1.0, zi),
            CNN_ACT_SOFTPLUS: np.log1p(np.exp(zi)), CNN_ACT_SWISH: zi * sig, CNN_ACT_NONE: zi, -1: zi}[act]


# (in, out, samples): LeNet's tail at batch 128, ragged sizes around the 32-wide blocks and a wide, shallow product (small
# kernel); AlexNet-like layers (the engine) and long reductions over small results (ranges of the batch + a second launch)
SMALL = [(84, 10, 128), (120, 84, 128), (400, 120, 128), (33, 31, 65), (1, 1, 1), (64, 32, 32), (100, 7, 500), (4096, 100, 96)]
LARGE = [(1024, 512, 64), (400, 120, 1024), (4096, 1000, 64), (84, 10, 1024), (120, 84, 3000), (33, 7, 8192)]
# wide layers at a batch of at most 64: the weight gradient that keeps the whole reduction in registers (AlexNet's first
# linear layer at batch 64, an even batch below 64, ragged edges on either side, the smallest batch)
SKINNY = [(9216, 4096, 64), (4096, 4096, 62), (1000, 4104, 10), (4100, 1000, 2)]


@pytest.mark.parametrize("act", [CNN_ACT_RELU, CNN_ACT_SWISH, CNN_ACT_SOFTPLUS, CNN_ACT_ELU, CNN_ACT_NONE, -1])
@pytest.mark.parametrize("n_in,n_out,n", SMALL + LARGE)
def test_input_gradient_with_the_derivative_below(dev, n_in, n_out, n, act):
    assert bool(hip.fitre_hip_linear_is_small(n_in, n_out, n)) == ((n_in, n_out, n) in SMALL)
    rng = np.random.default_rng(n_in * 31 + n_out * 7 + n + (act if act > 0 else 0))
    w = rng.standard_normal(n_out * n_in).astype(np.float32)        # out x in, column-major
    d = rng.standard_normal(n_out * n).astype(np.float32)           # out x n
    zpre = rng.standard_normal(n_in * n).astype(np.float32)         # in x n
    zpost = forward_act(act, zpre.astype(np.float64)).astype(np.float32)
    W = w.reshape(n_in, n_out).T.astype(np.float64)                 # W[o, i]
    D = d.reshape(n, n_out).T.astype(np.float64)                    # D[o, s]
    want = (W.T @ D) * derivative(act, zpre.reshape(n, n_in).T.astype(np.float64), zpost.reshape(n, n_in).T.astype(np.float64))
    pw, pd, pzi, pzo = dev.upload(w), dev.upload(d), dev.upload(zpre), dev.upload(zpost)
    out = dev.upload(np.full(n_in * n, 7.0, np.float32))
    ws_bytes = hip.fitre_hip_gemm_workspace(n_in, n, n_out)
    ws = dev.alloc(ws_bytes)
    snap = dev.upload(np.full(n_out * n + 3, 9.0, np.float32))   # the copy of delta the call leaves on its way
    ok(hip.fitre_hip_linear_input_grad(n_in, n_out, n, pw, pd, act, pzi, pzo, 0, 0, out, None, ws, ws_bytes, snap))
    got = dev.download(out, n_in * n).reshape(n, n_in).T
    assert rel_err(got, want) < TOL
    copied = dev.download(snap, n_out * n + 3)
    assert np.array_equal(copied[:-3], d) and (copied[-3:] == 9.0).all()
    for p in (pw, pd, pzi, pzo, out, ws, snap):
        dev.free(p)


@pytest.mark.parametrize("channels,ext_a,ext_b,n_out,n", [(16, 5, 5, 120, 128), (3, 2, 7, 33, 40), (1, 1, 1, 5, 9),
                                                           (256, 6, 6, 512, 64), (64, 3, 2, 600, 1200)])
def test_input_gradient_in_the_convolution_layout(dev, channels, ext_a, ext_b, n_out, n):
    """Row m = (c * B + b) * A + a of the product lands at [c][sample][a][b] (fitre_hip_fc_to_conv's permutation)."""
    n_in = channels * ext_a * ext_b
    rng = np.random.default_rng(n_in + n_out + n)
    w = rng.standard_normal(n_out * n_in).astype(np.float32)
    d = rng.standard_normal(n_out * n).astype(np.float32)
    W = w.reshape(n_in, n_out).T.astype(np.float64)
    D = d.reshape(n, n_out).T.astype(np.float64)
    plain = W.T @ D                                                  # [m][s]
    want = plain.reshape(channels, ext_b, ext_a, n).transpose(0, 3, 2, 1)   # [c][s][a][b]
    pw, pd = dev.upload(w), dev.upload(d)
    out = dev.zeros(n_in * n)
    staging = dev.zeros(n_in * n)
    ws_bytes = hip.fitre_hip_gemm_workspace(n_in, n, n_out)
    ws = dev.alloc(ws_bytes)
    ok(hip.fitre_hip_linear_input_grad(n_in, n_out, n, pw, pd, -1, None, None, ext_a, ext_b, out, staging, ws, ws_bytes, None))
    got = dev.download(out, n_in * n).reshape(channels, n, ext_a, ext_b)
    assert rel_err(got, want) < TOL
    if not hip.fitre_hip_linear_is_small(n_in, n_out, n):
        # a large layer without the staging buffer is refused before anything is queued
        assert hip.fitre_hip_linear_input_grad(n_in, n_out, n, pw, pd, -1, None, None, ext_a, ext_b, out, None, ws, ws_bytes, None) == 2
    assert hip.fitre_hip_linear_input_grad(n_in, n_out, n, pw, pd, -1, None, None, ext_a + 1, ext_b, out, staging, ws, ws_bytes, None) == 2 \
        or n_in % ((ext_a + 1) * ext_b) == 0
    for p in (pw, pd, out, staging, ws):
        dev.free(p)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("n_in,n_out,n", SMALL + LARGE + SKINNY)
def test_weight_and_bias_gradient(dev, n_in, n_out, n, bias):
    rng = np.random.default_rng(n_in * 3 + n_out * 5 + n)
    d = rng.standard_normal(n_out * n).astype(np.float32)
    zin = rng.standard_normal(n_in * n).astype(np.float32)
    D = d.reshape(n, n_out).T.astype(np.float64)
    Z = zin.reshape(n, n_in).T.astype(np.float64)
    pd, pz = dev.upload(d), dev.upload(zin)
    dw = dev.upload(np.full(n_out * n_in, 3.0, np.float32))
    db = dev.upload(np.full(n_out + 4, 5.0, np.float32))
    ws_bytes = hip.fitre_hip_linear_weight_grad_workspace(n_in, n_out, n)
    ws = dev.alloc(ws_bytes)
    ok(hip.fitre_hip_linear_weight_grad(n_in, n_out, n, pd, pz, dw, db if bias else None, ws, ws_bytes))
    got = dev.download(dw, n_out * n_in).reshape(n_in, n_out).T
    assert rel_err(got, D @ Z.T) < TOL
    got_b = dev.download(db, n_out + 4)
    if bias:
        assert rel_err(got_b[:n_out], D.sum(axis=1)) < TOL
        assert (got_b[n_out:] == 5.0).all()
    else:
        assert (got_b == 5.0).all()
    for p in (pd, pz, dw, db, ws):
        dev.free(p)


def test_small_layers_are_deterministic(dev):
    """Two runs of the fused kernels give the same bits."""
    n_in, n_out, n = 400, 120, 128
    rng = np.random.default_rng(0)
    d = rng.standard_normal(n_out * n).astype(np.float32)
    zin = rng.standard_normal(n_in * n).astype(np.float32)
    pd, pz = dev.upload(d), dev.upload(zin)
    runs = []
    for _ in range(2):
        dw, db = dev.zeros(n_out * n_in), dev.zeros(n_out)
        ok(hip.fitre_hip_linear_weight_grad(n_in, n_out, n, pd, pz, dw, db, None, 0))
        runs.append((dev.download(dw, n_out * n_in), dev.download(db, n_out)))
        dev.free(dw), dev.free(db)
    assert np.array_equal(runs[0][0], runs[1][0]) and np.array_equal(runs[0][1], runs[1][1])
    dev.free(pd), dev.free(pz)


def test_linear_arguments_are_checked(dev):
    p = dev.zeros(64)
    assert hip.fitre_hip_linear_input_grad(0, 4, 4, p, p, -1, None, None, 0, 0, p, None, None, 0, None) == 2
    assert hip.fitre_hip_linear_input_grad(4, 4, 4, p, p, -1, None, None, 0, 0, p, None, None, 0, None) == 2  # result aliases delta
    assert hip.fitre_hip_linear_input_grad(4, 4, 4, None, p, -1, None, None, 0, 0, p, None, None, 0, None) == 2
    assert hip.fitre_hip_linear_weight_grad(4, 4, 0, p, p, p, None, None, 0) == 2
    assert hip.fitre_hip_linear_weight_grad(4, 4, 4, p, None, p, None, None, 0) == 2
    dev.free(p)


# layer widths bottom-up (the first is the tail's input), samples, activations per layer, (extA, extB) of the input maps
TAILS = [
    ((400, 120, 84, 10), 128, (CNN_ACT_RELU, CNN_ACT_RELU, CNN_ACT_NONE), (5, 5)),       # LeNet at batch 128
    ((400, 120, 84, 10), 1024, (CNN_ACT_RELU, CNN_ACT_RELU, CNN_ACT_NONE), (5, 5)),      # groups of eight samples
    ((36, 7), 5, (CNN_ACT_SWISH,), (3, 2)),                                                # one layer, an activation on top, ragged group
    ((64, 33, 17, 9, 3), 67, (CNN_ACT_ELU, CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, CNN_ACT_NONE), (0, 0)),   # four layers, no permutation
    ((1024, 250), 9, (-1,), (4, 4)),                                                       # the widest input: one layer in many parts
    ((300, 96, 124, 3), 777, (CNN_ACT_RELU, CNN_ACT_ELU, CNN_ACT_NONE), (5, 2)),           # a ragged batch above 512 (ranges + reduction), 12276 weights above the lowest layer
    ((1000, 3, 2), 70, (CNN_ACT_SWISH, CNN_ACT_NONE), (0, 0)),                             # very few output units under many inputs
]


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("dims,n,acts,ext", TAILS)
def test_tail_of_small_layers_in_two_launches(dev, dims, n, acts, ext, bias):
    """fitre_hip_fc_tail_backward against the chain of per-layer formulas in float64: every layer's delta, weight and bias
    gradient and the lowest layer's input gradient (in the convolution layout when the inputs are maps)."""
    from fitre_amd.structs import fitre_fc_tail_layer
    layers = len(dims) - 1
    rng = np.random.default_rng(sum(dims) + n)
    Ws = [rng.standard_normal((dims[f + 1], dims[f])) / np.sqrt(dims[f]) for f in range(layers)]
    zin0 = rng.standard_normal((dims[0], n)).astype(np.float32)
    zpre, zpost, x = [], [], zin0.astype(np.float64)
    for f in range(layers):                       # a forward pass in float64, stored as floats
        pre = (Ws[f].astype(np.float32).astype(np.float64) @ x).astype(np.float32)
        post = forward_act(acts[f], pre.astype(np.float64)).astype(np.float32)
        zpre.append(pre), zpost.append(post)
        x = post.astype(np.float64)
    top = rng.standard_normal((dims[-1], n)).astype(np.float32)
    # the reference chain
    want_delta, want_dw, want_db = [None] * layers, [None] * layers, [None] * layers
    d = top.astype(np.float64) * derivative(acts[-1], zpre[-1].astype(np.float64), zpost[-1].astype(np.float64))
    for f in range(layers - 1, -1, -1):
        want_delta[f] = d
        inp = zin0 if f == 0 else zpost[f - 1]
        want_dw[f] = d @ inp.astype(np.float64).T
        want_db[f] = d.sum(axis=1)
        below = Ws[f].astype(np.float32).astype(np.float64).T @ d
        if f > 0:
            below = below * derivative(acts[f - 1], zpre[f - 1].astype(np.float64), zpost[f - 1].astype(np.float64))
        d = below
    want_features = d                                              # dims[0] x n
    col = lambda m: np.ascontiguousarray(m.T)                      # column-major upload of a (rows x cols) matrix
    bufs = []
    def up(a):
        p = dev.upload(a)
        bufs.append(p)
        return p
    arr = (fitre_fc_tail_layer * layers)()
    slots, dws, dbs = [], [], []
    pz0 = up(col(zin0))
    pposts = [up(col(z)) for z in zpost]
    for f in range(layers):
        slots.append(up(np.full(dims[f + 1] * n, np.nan, np.float32)))
        dws.append(up(np.full(dims[f + 1] * dims[f], np.nan, np.float32)))
        dbs.append(up(np.full(dims[f + 1], np.nan, np.float32)))
        arr[f] = fitre_fc_tail_layer(dims[f], dims[f + 1], acts[f], up(col(Ws[f].astype(np.float32))).value, up(col(zpre[f])).value,
                                     pposts[f].value, (pz0 if f == 0 else pposts[f - 1]).value, slots[f].value, dws[f].value,
                                     dbs[f].value if bias else None)
    assert hip.fitre_hip_fc_tail_fits(layers, arr, n) == 1
    nb = hip.fitre_hip_fc_tail_workspace(layers, arr, n)
    ws = up(np.zeros(nb // 4 + 1, np.float32))
    ptop = up(col(top))
    feat = up(np.full(dims[0] * n, np.nan, np.float32))
    ok(hip.fitre_hip_fc_tail_backward(layers, arr, n, ptop, ext[0], ext[1], feat, ws, nb))
    for f in range(layers):
        assert rel_err(dev.download(slots[f], dims[f + 1] * n).reshape(n, dims[f + 1]).T, want_delta[f]) < TOL, ("delta", f)
        assert rel_err(dev.download(dws[f], dims[f + 1] * dims[f]).reshape(dims[f], dims[f + 1]).T, want_dw[f]) < TOL, ("dW", f)
        if bias:
            assert rel_err(dev.download(dbs[f], dims[f + 1]), want_db[f]) < TOL, ("db", f)
    got = dev.download(feat, dims[0] * n)
    if ext[0] > 0:      # row m = (c * extB + b) * extA + a of sample s -> [c][s][a][b]
        a_, b_ = ext
        c_ = dims[0] // (a_ * b_)
        want = want_features.reshape(c_, b_, a_, n).transpose(0, 3, 2, 1).reshape(-1)
    else:
        want = want_features.T.reshape(-1)
    assert rel_err(got, want) < TOL
    # a second call gives the same bits
    first = [dev.download(q, k) for q, k in zip(dws, [dims[f + 1] * dims[f] for f in range(layers)])]
    ok(hip.fitre_hip_fc_tail_backward(layers, arr, n, ptop, ext[0], ext[1], feat, ws, nb))
    for q, k, a in zip(dws, [dims[f + 1] * dims[f] for f in range(layers)], first):
        np.testing.assert_array_equal(dev.download(q, k), a)
    # and the per-layer entry points give those bits too: every sum runs in the same order
    feat_bits = dev.download(feat, dims[0] * n)
    for f in range(layers):
        dw2, db2 = up(np.zeros(dims[f + 1] * dims[f], np.float32)), up(np.zeros(dims[f + 1], np.float32))
        nb2 = hip.fitre_hip_linear_weight_grad_workspace(dims[f], dims[f + 1], n)
        ws2 = up(np.zeros(nb2 // 4 + 1, np.float32))
        ok(hip.fitre_hip_linear_weight_grad(dims[f], dims[f + 1], n, slots[f], pz0 if f == 0 else pposts[f - 1], dw2,
                                            db2 if bias else None, ws2, nb2))
        np.testing.assert_array_equal(dev.download(dw2, dims[f + 1] * dims[f]), dev.download(dws[f], dims[f + 1] * dims[f]))
        if bias:
            np.testing.assert_array_equal(dev.download(db2, dims[f + 1]), dev.download(dbs[f], dims[f + 1]))
    feat2 = up(np.zeros(dims[0] * n, np.float32))
    ok(hip.fitre_hip_linear_input_grad(dims[0], dims[1], n, arr[0].W, slots[0], -1, None, None, ext[0], ext[1], feat2, None, None, 0, None))
    np.testing.assert_array_equal(dev.download(feat2, dims[0] * n), feat_bits)
    if ext[0] > 0:
        # the input maps as the output of a 2 x 2 max pool behind an activation: the same launch takes the gradient on
        # through both, with the bits fitre_hip_pool_act_backward leaves
        from fitre_amd.structs import MAX_POOL
        a_, b_ = ext
        c_ = dims[0] // (a_ * b_)
        big = c_ * n * 4 * a_ * b_
        for act in (CNN_ACT_RELU, CNN_ACT_SWISH, CNN_ACT_NONE):
            zi = rng.standard_normal(big).astype(np.float32)
            za = forward_act(act, zi.astype(np.float64)).astype(np.float32)
            pzi, pza = up(zi), up(za)
            pool0, act0, pool1, act1 = (up(np.full(big, np.nan, np.float32)) for _ in range(4))
            ok(hip.fitre_hip_pool_act_backward(MAX_POOL, act, feat, pzi, pza, c_, n, 2 * a_, 2 * b_, 2, 2, 0, a_, b_, pool0, act0))
            feat3 = up(np.zeros(dims[0] * n, np.float32))
            ok(hip.fitre_hip_fc_tail_backward_pool_act(layers, arr, n, ptop, a_, b_, feat3, act, pzi, pza, pool1, act1, ws, nb))
            np.testing.assert_array_equal(dev.download(feat3, dims[0] * n), feat_bits)
            np.testing.assert_array_equal(dev.download(pool1, big).view(np.uint32), dev.download(pool0, big).view(np.uint32))
            np.testing.assert_array_equal(dev.download(act1, big).view(np.uint32), dev.download(act0, big).view(np.uint32))
            # without the pool's own slot
            act2 = up(np.full(big, np.nan, np.float32))
            ok(hip.fitre_hip_fc_tail_backward_pool_act(layers, arr, n, ptop, a_, b_, feat3, act, pzi, pza, None, act2, ws, nb))
            np.testing.assert_array_equal(dev.download(act2, big).view(np.uint32), dev.download(act0, big).view(np.uint32))
    for p in bufs:
        dev.free(p)


def test_tail_rejects_what_does_not_fit(dev):
    from fitre_amd.structs import fitre_fc_tail_layer
    arr = (fitre_fc_tail_layer * 2)()
    arr[0] = fitre_fc_tail_layer(9216, 4096, CNN_ACT_RELU, None, None, None, None, None, None, None)
    arr[1] = fitre_fc_tail_layer(4096, 1000, CNN_ACT_NONE, None, None, None, None, None, None, None)
    assert hip.fitre_hip_fc_tail_fits(2, arr, 64) == 0 and hip.fitre_hip_fc_tail_workspace(2, arr, 64) == 0
    arr[0] = fitre_fc_tail_layer(100, 50, CNN_ACT_RELU, None, None, None, None, None, None, None)
    arr[1] = fitre_fc_tail_layer(60, 10, CNN_ACT_NONE, None, None, None, None, None, None, None)   # 60 inputs after 50 outputs
    assert hip.fitre_hip_fc_tail_fits(2, arr, 64) == 0
    assert hip.fitre_hip_fc_tail_backward(2, arr, 64, None, 0, 0, None, None, 0) == 2
    assert hip.fitre_hip_fc_tail_backward_pool_act(2, arr, 64, None, 0, 0, None, CNN_ACT_RELU, None, None, None, None, None, 0) == 2
    # the layers above the lowest sit in LDS whole: the sum of in * (out + 1) at most 16384 floats
    arr3 = (fitre_fc_tail_layer * 3)()
    for top, fits in ((62, 1), (63, 0)):
        arr3[0] = fitre_fc_tail_layer(200, 64, CNN_ACT_RELU, None, None, None, None, None, None, None)
        arr3[1] = fitre_fc_tail_layer(64, 128, CNN_ACT_RELU, None, None, None, None, None, None, None)      # 64 * 129 = 8256
        arr3[2] = fitre_fc_tail_layer(128, top, CNN_ACT_NONE, None, None, None, None, None, None, None)     # 128 * 63 = 8064, 128 * 64 = 8192
        assert hip.fitre_hip_fc_tail_fits(3, arr3, 64) == fits, top
