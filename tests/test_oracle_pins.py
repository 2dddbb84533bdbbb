"""Pins of the CPU oracle that do not involve the HIP path: the reference's stored known answer,
closed forms, brute force on tiny inputs, adjoint identities and library routines.  Each is chosen
so that a dropped term, a wrong index or a transposed operand fails it."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fitre_amd.structs import (ACT_LOGISTIC, ACT_TANH, CNN_ACT_ELU, CNN_ACT_RELU, CNN_ACT_SOFTPLUS, CNN_ACT_SWISH)
from oracle.torchref import from_nchw, to_nchw

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------ batch norm
def test_bn_backward_reference_known_answer(oracle64):
    g = json.load(open(os.path.join(HERE, "golden", "bn_backward_known_answer.json")))
    out = oracle64.batch_norm_backward(g["err"], g["zout"], [g["variance"]], 1, 1, 1, g["m"], g["epsilon"])
    np.testing.assert_allclose(out, g["expected"], rtol=0, atol=5e-9)
    # the intermediate sums the reference printed
    assert abs(np.sum(g["err"]) - g["error_sum"]) < 1e-15
    assert abs(np.dot(g["err"], g["zout"]) - g["zerr_sum"]) < 1e-12


def test_bn_forward_backward_against_autograd_and_invariants(oracle64):
    rng = np.random.default_rng(1)
    C, N, W, H = 3, 5, 4, 6
    x = rng.standard_normal(C * N * W * H) * 2 + 0.7
    zhat, mean, var, rmean, rvar = oracle64.batch_norm_forward(x, H, W, C, N)
    xt = to_nchw(x, C, N, W, H).requires_grad_(True)
    yt = F.batch_norm(xt, None, None, training=True, eps=1e-5)
    np.testing.assert_allclose(zhat, from_nchw(yt), atol=1e-12)
    np.testing.assert_allclose(mean, xt.detach().mean(dim=(0, 2, 3)).numpy(), atol=1e-13)
    np.testing.assert_allclose(var, xt.detach().var(dim=(0, 2, 3), unbiased=False).numpy(), atol=1e-13)
    # running statistics start at zero in this call: 0.9*0 + 0.1*batch
    np.testing.assert_allclose(rmean, 0.1 * mean, atol=1e-14)
    np.testing.assert_allclose(rvar, 0.1 * var, atol=1e-14)
    d = rng.standard_normal(x.size)
    dx = oracle64.batch_norm_backward(d, zhat, var, H, W, C, N)
    yt.backward(to_nchw(d, C, N, W, H))
    np.testing.assert_allclose(dx, from_nchw(xt.grad), atol=1e-12)
    # per-channel invariants of the formula
    dxc, zc = dx.reshape(C, -1), zhat.reshape(C, -1)
    np.testing.assert_allclose(dxc.sum(1), 0, atol=1e-11)
    # sum(dx*zhat) = s2 * (m - sum(zhat^2)) / (m*sqrt(var+eps)); zero up to the eps in the denominator
    m = zc.shape[1]
    s2 = (d.reshape(C, -1) * zc).sum(1)
    np.testing.assert_allclose((dxc * zc).sum(1), s2 * (m - (zc * zc).sum(1)) / (m * np.sqrt(var + 1e-5)), atol=1e-11)


def test_bn_eval_mode_uses_running_statistics(oracle64):
    rng = np.random.default_rng(2)
    C, N, W, H = 2, 3, 2, 2
    x = rng.standard_normal(C * N * W * H)
    rm, rv = np.array([0.3, -0.2]), np.array([1.5, 0.4])
    zhat, *_ = oracle64.batch_norm_forward(x, H, W, C, N, train=False, running=(rm, rv))
    want = (x.reshape(C, -1) - rm[:, None]) / np.sqrt(rv[:, None] + 1e-5)
    np.testing.assert_allclose(zhat, want.reshape(-1), atol=1e-13)


# ------------------------------------------------------------------ convolution
def brute_conv(x, w, b, N, Cin, H, W, k, pad, stride, Cout):
    """Direct convolution on logical (n, c, h, w) indices; no patch matrix."""
    Hc, Wc = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    X = np.asarray(x).reshape(Cin, N, W, H)       # [c][n][w][h]
    Wt = np.asarray(w).reshape(Cout, Cin, k, k)   # [o][c][kw][kh]
    out = np.zeros((Cout, N, Wc, Hc))
    for o in range(Cout):
        for n in range(N):
            for wo in range(Wc):
                for ho in range(Hc):
                    s = 0.0 if b is None else b[o]
                    for c in range(Cin):
                        for kw in range(k):
                            for kh in range(k):
                                wi, hi = wo * stride - pad + kw, ho * stride - pad + kh
                                if 0 <= wi < W and 0 <= hi < H:
                                    s += X[c, n, wi, hi] * Wt[o, c, kw, kh]
                    out[o, n, wo, ho] = s
    return out.reshape(-1)


CONV_CASES = [  # N, Cin, H, W, k, pad, stride, Cout
    (2, 2, 5, 4, 3, 1, 1, 3),
    (1, 3, 6, 6, 5, 0, 1, 2),
    (2, 1, 7, 9, 3, 0, 2, 2),
    (1, 2, 9, 9, 5, 2, 4, 3),
    (3, 2, 2, 2, 3, 1, 1, 2),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_forward_brute_force_and_torch(oracle64, case):
    N, Cin, H, W, k, pad, stride, Cout = case
    rng = np.random.default_rng(hash(case) % 1000)
    x = rng.standard_normal(Cin * N * W * H)
    w = rng.standard_normal(Cout * Cin * k * k)
    b = rng.standard_normal(Cout)
    got = oracle64.conv_forward(x, w, b, N, Cin, H, W, k, pad, stride, Cout)
    np.testing.assert_allclose(got, brute_conv(x, w, b, N, Cin, H, W, k, pad, stride, Cout), atol=1e-12)
    wt = torch.tensor(w.reshape(Cout, Cin, k, k)).permute(0, 1, 3, 2)
    yt = F.conv2d(to_nchw(x, Cin, N, W, H), wt, torch.tensor(b), stride=stride, padding=pad)
    np.testing.assert_allclose(got, from_nchw(yt), atol=1e-12)


def test_conv_forward_counter_inputs_closed_form(oracle64):
    # inputs of the reference's drivers/convolution_driver.cu:158-238: image value p+1+channel,
    # every weight of filter o equal to o+1, bias 0.1*(o+1); no padding, stride 1
    N, Cin, H, W, k, Cout = 2, 3, 6, 6, 3, 4
    x = np.zeros((Cin, N, W, H))
    for p in range(N):
        for i in range(Cin):
            x[i, p] = p + 1 + i
    w = np.repeat(np.arange(1, Cout + 1), Cin * k * k).astype(float)
    b = 0.1 * np.arange(1, Cout + 1)
    got = oracle64.conv_forward(x.reshape(-1), w, b, N, Cin, H, W, k, 0, 1, Cout).reshape(Cout, N, -1)
    for o in range(Cout):
        for p in range(N):
            want = (o + 1) * k * k * sum(p + 1 + i for i in range(Cin)) + 0.1 * (o + 1)
            np.testing.assert_allclose(got[o, p], want, atol=1e-12)


def test_im2col_column_order_is_channel_then_window_column_then_row(oracle64):
    # one 3x3 single-channel image whose value encodes its position: x[w][h] = 10*w + h
    H = W = 3
    x = np.array([[10 * w + h for h in range(H)] for w in range(W)], dtype=float).reshape(-1)
    col = oracle64.im2col(x, 1, 1, H, W, 2, 0, 1).reshape(4, 4)  # [tap j*2+i][w_out*2+h_out]
    # output cell (w_out=1, h_out=0); taps (j=window column, i=window row): value 10*(1+j) + (0+i)
    np.testing.assert_array_equal(col[:, 2], [10, 11, 20, 21])


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_weight_gradient_brute_force_and_adjoint(oracle64, case):
    N, Cin, H, W, k, pad, stride, Cout = case
    rng = np.random.default_rng(7)
    Hc, Wc = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    x = rng.standard_normal(Cin * N * W * H)
    w = rng.standard_normal(Cout * Cin * k * k)
    d = rng.standard_normal(Cout * N * Wc * Hc)
    dW = oracle64.conv_weight_grad(x, d, N, Cin, H, W, k, pad, stride, Cout)
    # adjoint identity <conv(x, w), d> = <w, dW(x, d)>, conv evaluated by brute force
    lhs = np.dot(brute_conv(x, w, None, N, Cin, H, W, k, pad, stride, Cout), d)
    np.testing.assert_allclose(np.dot(w, dW), lhs, rtol=1e-11)
    # and element by element against autograd
    wt = torch.tensor(w.reshape(Cout, Cin, k, k)).permute(0, 1, 3, 2).contiguous().requires_grad_(True)
    yt = F.conv2d(to_nchw(x, Cin, N, W, H), wt, None, stride=stride, padding=pad)
    yt.backward(to_nchw(d, Cout, N, Wc, Hc))
    np.testing.assert_allclose(dW, wt.grad.permute(0, 1, 3, 2).contiguous().numpy().reshape(-1), atol=1e-11)


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[6] == 1])
def test_conv_input_gradient_adjoint_and_autograd(oracle64, case):
    N, Cin, H, W, k, pad, stride, Cout = case
    rng = np.random.default_rng(9)
    Hc, Wc = H + 2 * pad - k + 1, W + 2 * pad - k + 1
    x = rng.standard_normal(Cin * N * W * H)
    w = rng.standard_normal(Cout * Cin * k * k)
    d = rng.standard_normal(Cout * N * Wc * Hc)
    dX = oracle64.conv_input_grad(d, w, N, Cin, H, W, k, pad, Cout)
    lhs = np.dot(brute_conv(x, w, None, N, Cin, H, W, k, pad, 1, Cout), d)
    np.testing.assert_allclose(np.dot(x, dX), lhs, rtol=1e-11)
    xt = to_nchw(x, Cin, N, W, H).requires_grad_(True)
    wt = torch.tensor(w.reshape(Cout, Cin, k, k)).permute(0, 1, 3, 2)
    F.conv2d(xt, wt, None, padding=pad).backward(to_nchw(d, Cout, N, Wc, Hc))
    np.testing.assert_allclose(dX, from_nchw(xt.grad), atol=1e-11)


def test_gemm_matches_numpy_for_all_transpose_combinations(oracle64):
    rng = np.random.default_rng(3)
    M, N, K = 5, 4, 7
    for ta in (0, 1):
        for tb in (0, 1):
            A = rng.standard_normal((K, M) if ta else (M, K))
            B = rng.standard_normal((N, K) if tb else (K, N))
            C0 = rng.standard_normal((M, N))
            want = 0.5 * (A.T if ta else A) @ (B.T if tb else B) + 2.0 * C0
            got = oracle64.gemm(ta, tb, M, N, K, 0.5, A.T.reshape(-1), A.shape[0], B.T.reshape(-1), B.shape[0], 2.0,
                                C0.T.reshape(-1), M)
            np.testing.assert_allclose(got.reshape(N, M).T, want, atol=1e-12)


# ------------------------------------------------------------------ pooling
def test_max_pool_reference_driver_case(oracle64):
    # drivers/pool_driver.cu:26-38: 8 channels of 2x2, window 3, stride 2, padding 1 -> one cell
    rng = np.random.default_rng(5)
    x = rng.standard_normal(8 * 2 * 2)
    out = oracle64.pool_forward(0, x, 1, 8, 2, 2, 3, 2, 1)
    np.testing.assert_allclose(out, x.reshape(8, 4).max(1))
    idx = oracle64.max_pool_argmax(x, 1, 8, 2, 2, 3, 2, 1)
    np.testing.assert_array_equal(idx, x.reshape(8, 4).argmax(1))
    d = rng.standard_normal(8)
    back = oracle64.pool_backward(0, d, x, 1, 8, 2, 2, 3, 2, 1).reshape(8, 4)
    want = np.zeros((8, 4))
    want[np.arange(8), x.reshape(8, 4).argmax(1)] = d
    np.testing.assert_allclose(back, want)


@pytest.mark.parametrize("geom", [(6, 6, 2, 2, 0), (7, 5, 3, 2, 1), (8, 8, 3, 2, 0), (5, 5, 2, 2, 0)])
def test_pool_forward_backward_against_autograd(oracle64, geom):
    H, W, k, s, p = geom
    rng = np.random.default_rng(11)
    C, N = 2, 3
    x = rng.standard_normal(C * N * W * H)
    for kind in (0, 1):
        xt = to_nchw(x, C, N, W, H).requires_grad_(True)
        yt = F.max_pool2d(xt, k, s, p) if kind == 0 else F.avg_pool2d(xt, k, s, p, count_include_pad=True)
        got = oracle64.pool_forward(kind, x, N, C, H, W, k, s, p)
        np.testing.assert_allclose(got, from_nchw(yt), atol=1e-13)
        d = rng.standard_normal(got.size)
        yt.backward(to_nchw(d, C, N, yt.shape[3], yt.shape[2]))
        back = oracle64.pool_backward(kind, d, x, N, C, H, W, k, s, p)
        np.testing.assert_allclose(back, from_nchw(xt.grad), atol=1e-13)


def test_max_pool_tie_break_is_first_maximum_in_memory_order(oracle64):
    # one 2x2 map [w][h]; window 2, stride 2.  Scan order of the reference (dev_pool.cu:374-391):
    # window columns outer, rows inner = offsets 0,1,2,3 of the map.
    flat = lambda a: np.array(a, dtype=float)
    assert oracle64.max_pool_argmax(flat([0, 0, 0, 0]), 1, 1, 2, 2, 2, 2, 0)[0] == 0      # all equal
    assert oracle64.max_pool_argmax(flat([1, 5, 5, 2]), 1, 1, 2, 2, 2, 2, 0)[0] == 1      # two-way tie
    assert oracle64.max_pool_argmax(flat([-3, -1, -1, -1]), 1, 1, 2, 2, 2, 2, 0)[0] == 1  # negative tie
    back = oracle64.pool_backward(0, flat([2.5]), flat([1, 5, 5, 2]), 1, 1, 2, 2, 2, 2, 0)
    np.testing.assert_array_equal(back, [0, 2.5, 0, 0])
    # overlapping windows that share their maximum add up (window 3, stride 1 on 4x4 -> 2x2 cells)
    x = np.zeros(16)
    x[5] = 9.0  # cell (w=1, h=1) is inside all four windows
    back = oracle64.pool_backward(0, flat([1, 2, 3, 4]), x, 1, 1, 4, 4, 3, 1, 0)
    assert back[5] == 10.0 and np.count_nonzero(back) == 1


# ------------------------------------------------------------------ activations
@pytest.mark.parametrize("code", [CNN_ACT_RELU, CNN_ACT_SWISH, CNN_ACT_SOFTPLUS, CNN_ACT_ELU, ACT_LOGISTIC, ACT_TANH])
def test_activation_forward_backward_against_autograd(oracle64, code):
    from oracle.torchref import act_torch
    rng = np.random.default_rng(13)
    x = rng.standard_normal(257) * 3
    x[:3] = [25.0, -25.0, 0.5]
    xt = torch.tensor(x, requires_grad=True)
    yt = act_torch(code, xt)
    y = oracle64.activation_forward(code, x)
    np.testing.assert_allclose(y, yt.detach().numpy(), atol=1e-12)
    d = rng.standard_normal(x.size)
    yt.backward(torch.tensor(d))
    np.testing.assert_allclose(oracle64.activation_backward(code, d, x, y), xt.grad.numpy(), atol=1e-12)


def test_swish_closed_forms(oracle64):
    # y(0) = 0, y'(0) = 1/2 (functions/swish.cu:25-43: y' = y + s(1-y))
    assert oracle64.activation_forward(CNN_ACT_SWISH, [0.0])[0] == 0.0
    assert oracle64.activation_backward(CNN_ACT_SWISH, [1.0], [0.0], [0.0])[0] == 0.5
    assert oracle64.activation_backward(CNN_ACT_RELU, [3.0, 3.0], [0.0, 0.0], [0.0, 2.0]).tolist() == [0.0, 3.0]


def test_unknown_activation_is_rejected(oracle64):
    with pytest.raises(ValueError):
        oracle64.activation_forward(99, [1.0])


# ------------------------------------------------------------------ softmax cross entropy
def test_softmax_loss_closed_forms_and_torch(oracle64):
    rows, classes = 6, 10
    loss, probs = oracle64.softmax_loss(np.zeros(rows * classes), np.ones(rows), rows, classes)
    assert abs(loss - np.log(classes)) < 1e-8 and np.allclose(probs, 0.1)
    rng = np.random.default_rng(17)
    logits = rng.standard_normal(rows * classes) * 1.5
    y = rng.integers(1, classes + 1, rows).astype(float)
    loss, probs = oracle64.softmax_loss(logits, y, rows, classes)
    lt = torch.tensor(logits.reshape(rows, classes), requires_grad=True)
    want = F.cross_entropy(lt, torch.tensor(y.astype(np.int64) - 1))
    assert abs(loss - want.item()) < 1e-6                     # the 1e-10 floor moves each term by 1e-10/p
    # exactly: mean(-log(softmax + 1e-10)), also for large logits where the floor is visible
    big = logits * 6
    lossb, probsb = oracle64.softmax_loss(big, y, rows, classes)
    sm = torch.softmax(torch.tensor(big.reshape(rows, classes)), 1).numpy() + 1e-10
    np.testing.assert_allclose(probsb, sm.reshape(-1), rtol=1e-12)
    np.testing.assert_allclose(lossb, np.mean(-np.log(sm[np.arange(rows), y.astype(int) - 1])), rtol=1e-12)
    err = oracle64.cross_entropy_error(probs, y, rows, classes)
    want.backward()
    np.testing.assert_allclose(err, lt.grad.numpy().reshape(-1), atol=1e-9)
    np.testing.assert_allclose(err.reshape(rows, classes).sum(1), classes * 1e-10 / rows, atol=1e-15)


# ------------------------------------------------------------------ layout changes
def test_reshape_and_transposes(oracle64):
    x = np.arange(2 * 3 * 4, dtype=float)
    got = oracle64.reshape(x, 2, 3, 4).reshape(3, 2, 4)
    np.testing.assert_array_equal(got, x.reshape(2, 3, 4).transpose(1, 0, 2))
    m = np.arange(2 * 3 * 5, dtype=float)  # two maps, height 3, width 5, column-major
    t = oracle64.transpose(m, 2, 3, 5).reshape(2, 3, 5)
    np.testing.assert_array_equal(t, m.reshape(2, 5, 3).transpose(0, 2, 1))
    np.testing.assert_array_equal(oracle64.transpose(t.reshape(-1), 2, 3, 5, rc=True), m)


# ------------------------------------------------------------------ KFAC factors
def unfold_patches(x_nchw, k, pad, stride):
    """(N*L) x (C*k*k) patch matrix from the library unfold, columns re-ordered from torch's
    (c, kh, kw) to the weight layout's (c, window column, window row); pytorch/testing/test_expanded.py:13-35
    builds the same matrix and forms exp^T exp."""
    N, C = x_nchw.shape[:2]
    u = F.unfold(x_nchw, k, padding=pad, stride=stride)                    # N, C*k*k, L
    u = u.reshape(N, C, k, k, -1).permute(0, 4, 1, 3, 2).reshape(-1, C * k * k)  # rows (n, l); cols (c, kw, kh)
    return u.numpy()


@pytest.mark.parametrize("case", [(3, 2, 5, 4, 3, 1, 1, True), (2, 3, 6, 6, 3, 0, 1, False), (2, 1, 7, 5, 2, 1, 2, True),
                                  (1, 2, 4, 4, 5, 2, 1, True)])
def test_kfac_conv_input_factor_against_unfold(oracle64, case):
    N, C, H, W, k, pad, stride, bias = case
    rng = np.random.default_rng(11)
    xt = torch.from_numpy(rng.standard_normal((N, C, H, W)))
    OH, OW = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    P = unfold_patches(xt, k, pad, stride) / (OH * OW)
    if bias:
        P = np.concatenate([P, np.ones((P.shape[0], 1))], axis=1)
    want = P.T @ P / N
    got = oracle64.kfac_conv_input_factor(from_nchw(xt), N, C, H, W, k, pad, stride, bias)
    np.testing.assert_allclose(got, want, atol=1e-13)
    np.testing.assert_allclose(got, got.T, atol=0)
    assert np.linalg.eigvalsh(got).min() > -1e-12
    if bias:
        assert abs(got[-1, -1] - OH * OW) < 1e-12  # ones^T ones / N


def test_kfac_conv_input_factor_closed_form_for_constant_image(oracle64):
    # x = 1 without padding: every patch entry is 1, so each patch-patch entry is
    # (1/L)^2 * N*L / N = 1/L, each patch-bias entry is 1 and the corner is L  (L = OH*OW)
    N, C, H, W, k = 3, 2, 6, 5, 3
    L = (H - k + 1) * (W - k + 1)
    got = oracle64.kfac_conv_input_factor(np.ones(N * C * H * W), N, C, H, W, k, 0, 1, True)
    K = C * k * k
    np.testing.assert_allclose(got[:K, :K], 1.0 / L, atol=1e-14)
    np.testing.assert_allclose(got[K, :K], 1.0, atol=1e-14)
    assert abs(got[K, K] - L) < 1e-12


def test_kfac_output_and_fc_factors_against_numpy(oracle64):
    rng = np.random.default_rng(12)
    N, Cout, OH, OW = 3, 4, 2, 5
    d = rng.standard_normal((Cout, N * OH * OW))               # [Cout][N][OW][OH] flattened
    got = oracle64.kfac_conv_output_factor(d.reshape(-1), N, OH, OW, Cout)
    np.testing.assert_allclose(got, d @ d.T * (N * OH * OW), atol=1e-11)
    n_in, n_out = 5, 3
    z = rng.standard_normal((N, n_in))                         # column-major in x N: sample-major memory
    for bias in (False, True):
        Z = np.concatenate([z, np.ones((N, 1))], axis=1) if bias else z
        got = oracle64.kfac_fc_input_factor(z.reshape(-1), n_in, N, bias)
        np.testing.assert_allclose(got, Z.T @ Z / N, atol=1e-13)
    dl = rng.standard_normal((N, n_out))
    got = oracle64.kfac_fc_output_factor(dl.reshape(-1), n_out, N)
    np.testing.assert_allclose(got, dl.T @ dl * N, atol=1e-12)


# ------------------------------------------------------------------ matrix inverse
def spd_matrix(n, rng, cond=50.0):
    q, _ = np.linalg.qr(rng.standard_normal((n, n)))
    ev = np.geomspace(1.0, 1.0 / cond, n)
    return (q * ev) @ q.T


@pytest.mark.parametrize("n", [1, 2, 7, 64, 65, 200])
def test_matrix_inverse_against_scipy_cholesky(oracle64, n):
    import scipy.linalg
    rng = np.random.default_rng(n)
    a = spd_matrix(n, rng)
    lam, gamma = 1e-3, 2e-2
    info, inv = oracle64.matrix_inverse(a, n, lam, gamma)
    assert info == 0
    shifted = a + (lam + gamma) * np.eye(n)
    want = scipy.linalg.cho_solve(scipy.linalg.cho_factor(shifted, lower=True), np.eye(n))
    np.testing.assert_allclose(inv, want, rtol=0, atol=1e-11 * np.abs(want).max())
    np.testing.assert_allclose(shifted @ inv, np.eye(n), atol=1e-11)
    np.testing.assert_allclose(inv, inv.T, atol=1e-12 * np.abs(inv).max())


def test_matrix_inverse_closed_form_and_failure(oracle64):
    # diagonal matrix: the damping enters every pivot
    d = np.array([4.0, 1.0, 0.25])
    info, inv = oracle64.matrix_inverse(np.diag(d), 3, 0.5, 0.25)
    assert info == 0
    np.testing.assert_allclose(inv, np.diag(1.0 / (d + 0.75)), atol=1e-15)
    # 2x2 with a known inverse
    info, inv = oracle64.matrix_inverse(np.array([[2.0, 1.0], [1.0, 2.0]]), 2, 0.0, 0.0)
    np.testing.assert_allclose(inv, np.array([[2.0, -1.0], [-1.0, 2.0]]) / 3.0, atol=1e-15)
    # indefinite: the second pivot is 1 - 4 < 0, reported 1-based like cusolver's devInfo
    info, _ = oracle64.matrix_inverse(np.array([[1.0, 2.0], [2.0, 1.0]]), 2, 0.0, 0.0)
    assert info == 2


def test_natural_gradient_against_kron_solve(oracle64):
    """Per layer the natural gradient is Lambda^-1 G Omega^-1 with G the layer's gradient as a Cout x (K+1)
    matrix; vec(A G B) = (B' kron A) vec(G), so it must equal the solution of the Kronecker-factored system."""
    from fitre_amd.structs import CNN_ACT_NONE, CNN_ACT_SWISH, MAX_POOL
    from helpers import build_custom
    model = build_custom(3, 6, 6, 2, [dict(cout=3, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), bn=False, act=CNN_ACT_SWISH)],
                         [(4, CNN_ACT_NONE)], bias=1)
    rng = np.random.default_rng(5)
    g = rng.standard_normal(model.pSize)
    dims = [(2 * 9 + 1, 3), (3 * 3 * 3 + 1, 4)]          # (K+1, Cout) of the conv layer, (in+1, out) of the FC layer
    oo, lo, om, la = [0], [0], [], []
    for k1, o in dims:
        a, b = rng.standard_normal((k1, k1)), rng.standard_normal((o, o))
        om.append(a @ a.T + np.eye(k1))
        la.append(b @ b.T + np.eye(o))
        oo.append(oo[-1] + k1 * k1)
        lo.append(lo[-1] + o * o)
    got = oracle64.natural_gradient(model, oo, lo, np.concatenate([m.reshape(-1) for m in om]),
                                    np.concatenate([m.reshape(-1) for m in la]), g)
    # conv layer: flat layout [W (Cout x K, K fastest) | b (Cout)]
    K, O = 18, 3
    G = np.concatenate([g[:O * K].reshape(O, K), g[O * K:O * K + O, None]], axis=1)        # Cout x (K+1)
    want = la[0] @ G @ om[0]
    np.testing.assert_allclose(got[:O * K].reshape(O, K), want[:, :K], atol=1e-11)
    np.testing.assert_allclose(got[O * K:O * K + O], want[:, K], atol=1e-11)
    # FC layer: [W | b] column-major out x (in+1)
    off, n_in, n_out = model.wOffsets[1], 27, 4
    Gf = g[off:off + n_out * (n_in + 1)].reshape(n_in + 1, n_out).T
    wantf = la[1] @ Gf @ om[1]
    np.testing.assert_allclose(got[off:off + n_out * (n_in + 1)].reshape(n_in + 1, n_out).T, wantf, atol=1e-11)
    # the Kronecker identity on the conv block
    vecG = G.reshape(-1, order="F")
    np.testing.assert_allclose(np.kron(om[0].T, la[0]) @ vecG, want.reshape(-1, order="F"), atol=1e-10)


def test_compute_accuracy_counts_first_maximum(oracle64):
    probs = np.array([[0.1, 0.7, 0.2],     # class 2
                      [0.4, 0.4, 0.2],     # tie: first maximum, class 1
                      [0.0, 0.0, 0.0],     # nothing exceeds 0: class 1 by default
                      [0.2, 0.3, 0.5]])    # class 3
    target = np.array([2.0, 2.0, 1.0, 1.0])
    pct, hits = oracle64.compute_accuracy(probs.reshape(-1), target, 4, 3)
    assert hits == 2 and pct == 50.0
    rng = np.random.default_rng(0)
    p = rng.random((100, 10))
    t = rng.integers(1, 11, 100).astype(np.float64)
    pct, hits = oracle64.compute_accuracy(p.reshape(-1), t, 100, 10)
    assert hits == float(np.sum(p.argmax(1) + 1 == t)) and abs(pct - hits) < 1e-12


def test_multinomial_classes_inverse_cdf(oracle64):
    probs = np.array([[0.2, 0.5, 0.3], [0.2, 0.5, 0.3], [0.2, 0.5, 0.3], [0.2, 0.5, 0.3], [0.25, 0.25, 0.25]])
    u = np.array([0.1, 0.2, 0.2000001, 0.95, 0.9])      # boundary included in the lower class (c >= u)
    got = oracle64.multinomial_classes(probs.reshape(-1), u, 5, 3)
    np.testing.assert_array_equal(got, [1, 1, 2, 3, 4])  # last row: the total stays below the draw -> classes + 1
    rng = np.random.default_rng(3)
    p = rng.random((2000, 7))
    p /= p.sum(1, keepdims=True)
    uu = rng.random(2000)
    want = 1 + (np.cumsum(p, axis=1) >= uu[:, None]).argmax(1)
    np.testing.assert_array_equal(oracle64.multinomial_classes(p.reshape(-1), uu, 2000, 7), want)


def test_uniform_stream_known_values_and_statistics(oracle64):
    # splitmix64 with seed 0 produces the published first outputs when hashed position by position
    def splitmix(seed, g):
        m = (1 << 64) - 1
        z = (seed + (g + 1) * 0x9E3779B97F4A7C15) & m
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        return z ^ (z >> 31)
    assert splitmix(0, 0) == 0xE220A8397B1DCDAF and splitmix(0, 1) == 0x6E789E6AA1B965F4  # reference vectors of SplitMix64
    got = oracle64.uniform_stream(1234, 5, 1000)
    want = np.array([((splitmix(1234, 5 + i) >> 40) + 1) / 16777216.0 for i in range(1000)], dtype=np.float32)
    np.testing.assert_array_equal(got, want)
    big = oracle64.uniform_stream(99, 0, 200000)
    assert big.min() > 0 and big.max() <= 1
    assert abs(big.mean() - 0.5) < 3e-3 and abs(big.var() - 1 / 12) < 2e-3
    # continuing the stream equals one long draw
    np.testing.assert_array_equal(np.concatenate([oracle64.uniform_stream(7, 0, 10), oracle64.uniform_stream(7, 10, 6)]),
                                  oracle64.uniform_stream(7, 0, 16))


# ------------------------------------------------------------------ input pipeline
def _images(rng, C, N, W, H):
    """[C][N][W][H] flat (H fastest) and the same data as an array indexed [c][n][col][row]."""
    x = rng.integers(0, 256, size=C * N * W * H).astype(np.float64)
    return x, x.reshape(C, N, W, H)


def test_extract_columns_is_fancy_indexing(oracle64):
    rng = np.random.default_rng(3)
    rows, cols = 7, 20
    src = rng.standard_normal(rows * cols)
    idx = rng.integers(0, cols, size=9)
    want = src.reshape(cols, rows)[idx].reshape(-1)   # column-major features x columns: column j is a contiguous run
    np.testing.assert_array_equal(oracle64.extract_columns(src, idx, rows), want)


def test_crop_shifts_known_values(oracle64):
    # trunc(u * 100) mod 9 - 4 for padding 4 (augmentation/dev_crop.cu:57)
    u = [0.0, 0.004, 0.01, 0.37, 0.44, 0.45, 0.99, 0.089999]
    want = [-4, -4, -3, 37 % 9 - 4, 44 % 9 - 4, 45 % 9 - 4, 99 % 9 - 4, 8 % 9 - 4]
    np.testing.assert_array_equal(oracle64.crop_shifts(u, 4, 4), want)
    rng = np.random.default_rng(0)
    s = oracle64.crop_shifts(rng.random(2000), 1000, 4)
    assert s.min() == -4 and s.max() == 4
    # padding 2: values in [-2, 2]
    s2 = oracle64.crop_shifts(rng.random(2000), 1000, 2)
    assert s2.min() == -2 and s2.max() == 2


def test_random_crop_is_a_zero_filled_shift(oracle64):
    rng = np.random.default_rng(5)
    C, N, W, H = 3, 6, 5, 7   # rectangular: a swapped axis would show
    x, img = _images(rng, C, N, W, H)
    sr = np.array([0, 2, -3, 4, -1, 6])
    sc = np.array([0, -1, 2, 0, 4, -4])
    got = oracle64.random_crop(x, N, H, W, C, sr, sc, default=-9.0).reshape(C, N, W, H)
    for n in range(N):
        # out[col][row] = in[col + sc][row + sr]: pad by the largest shift, then slice
        P = 8
        padded = np.pad(img[:, n], ((0, 0), (P, P), (P, P)), constant_values=-9.0)
        want = padded[:, P + sc[n]:P + sc[n] + W, P + sr[n]:P + sr[n] + H]
        np.testing.assert_array_equal(got[:, n], want)
    # zero shift is the identity
    np.testing.assert_array_equal(oracle64.random_crop(x, N, H, W, C, np.zeros(N), np.zeros(N)), x)


def test_random_flip_mirrors_the_column_axis(oracle64):
    rng = np.random.default_rng(6)
    C, N, W, H = 2, 5, 6, 4
    x, img = _images(rng, C, N, W, H)
    probs = np.array([0.1, 0.5, 0.49999, 0.9, 0.0])
    got = oracle64.random_flip(x, N, C, H, W, probs).reshape(C, N, W, H)
    for n in range(N):
        want = np.flip(img[:, n], axis=1) if probs[n] < 0.5 else img[:, n]
        np.testing.assert_array_equal(got[:, n], want)
    # an involution
    np.testing.assert_array_equal(oracle64.random_flip(got.reshape(-1), N, C, H, W, probs), x)


def test_normalize_closed_form(oracle64):
    rng = np.random.default_rng(7)
    C, N, W, H = 3, 4, 3, 5
    x, img = _images(rng, C, N, W, H)
    mean, std = np.array([0.4914, 0.4822, 0.4465]), np.array([0.2470, 0.2435, 0.2616])
    want = (img / 255.0 - mean[:, None, None, None]) / std[:, None, None, None]
    np.testing.assert_allclose(oracle64.normalize(x, N, H, W, C, mean, std).reshape(C, N, W, H), want, rtol=1e-15)


def test_augment_data_composition(oracle64):
    """solvers/kfac_da.cu:22-89: sample-major -> channel-major, crop, flip, normalise."""
    rng = np.random.default_rng(8)
    C, N, W, H = 3, 7, 8, 8
    sampled = rng.integers(0, 256, size=N * C * W * H).astype(np.float64)      # [N][C][W][H]
    cu, fu = rng.random(2 * N), rng.random(N)
    mean, std = np.array([0.5071, 0.4865, 0.4409]), np.array([0.2673, 0.2564, 0.2762])
    img = sampled.reshape(N, C, W, H).transpose(1, 0, 2, 3)                     # [C][N][W][H]
    shifts = (np.trunc(cu * 100).astype(int) % 9) - 4
    out = np.empty_like(img)
    for n in range(N):
        padded = np.pad(img[:, n], ((0, 0), (4, 4), (4, 4)))
        sr, sc = shifts[n], shifts[N + n]
        v = padded[:, 4 + sc:4 + sc + W, 4 + sr:4 + sr + H]
        out[:, n] = np.flip(v, axis=1) if fu[n] < 0.5 else v
    want = (out / 255.0 - mean[:, None, None, None]) / std[:, None, None, None]
    got = oracle64.augment_data(sampled, N, C, H, W, 1, cu, fu, mean, std).reshape(C, N, W, H)
    np.testing.assert_allclose(got, want, rtol=1e-15)
    # without augmentation: layout change and normalisation only
    plain = oracle64.augment_data(sampled, N, C, H, W, 0, cu, fu, mean, std).reshape(C, N, W, H)
    np.testing.assert_allclose(plain, (img / 255.0 - mean[:, None, None, None]) / std[:, None, None, None], rtol=1e-15)
