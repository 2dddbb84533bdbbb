"""The float64 products on the matrix pipes (fitre_hip_gemm_f64), the float64 inverse built from them and the float64
Kronecker factors, against numpy / LAPACK / the float64 oracle, through the C boundary."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import (FITRE_GEMM_A_LOWER, FITRE_GEMM_A_UPPER, FITRE_GEMM_B_LOWER, FITRE_GEMM_B_UPPER, FITRE_GEMM_SYMMETRIC,
                               FITRE_MAT_F32, FITRE_MAT_F64, FITRE_MAT_SYM_PAIR, fitre_matrix)
from helpers import conv_shape, pair_decode, pair_encode, rel_err

pytestmark = pytest.mark.gpu
hip = L.hip


def mat(ptr, rs, cs, kind, ones_row=-1, ones_col=-1, ones_value=0.0):
    return fitre_matrix(ptr.value if hasattr(ptr, "value") else ptr, rs, cs, kind, ones_row, ones_col, ones_value)


GEMM_CASES = [
    # M, N, K, kind A, kind B, trans A, trans B, kind C, C column-major?
    (1, 1, 1, "f32", "f32", 0, 0, "f64", True),
    (17, 33, 5, "f32", "f64", 0, 0, "f64", True),
    (130, 70, 129, "f64", "f32", 1, 0, "f32", True),
    (64, 64, 64, "f64", "f64", 0, 1, "f64", False),
    (200, 300, 1000, "f32", "f32", 1, 1, "f64", True),
    (513, 10, 513, "f32", "f64", 0, 0, "f32", False),
    (300, 257, 4100, "f32", "f32", 0, 1, "f64", True),      # split reduction
    (1200, 1100, 70, "f64", "f64", 0, 0, "f64", True),      # 128-tiles
]


@pytest.mark.parametrize("case", GEMM_CASES)
def test_gemm_f64(dev, case):
    M, N, K, ka, kb, ta, tb, kc, colmajor = case
    rng = np.random.default_rng(sum(map(lambda v: v if isinstance(v, int) else len(v), case)))
    A = rng.standard_normal((M, K))
    B = rng.standard_normal((K, N))
    Cold = rng.standard_normal((M, N))
    dt = {"f32": np.float32, "f64": np.float64}
    kinds = {"f32": FITRE_MAT_F32, "f64": FITRE_MAT_F64}
    A, B, Cold = A.astype(dt[ka]), B.astype(dt[kb]), Cold.astype(dt[kc])
    # storage: trans = 1 keeps the transposed matrix in memory (row-major storage of the logical matrix)
    sa = np.ascontiguousarray(A.T if not ta else A)      # column-major A when not transposed
    sb = np.ascontiguousarray(B.T if not tb else B)
    pa, pb = dev.upload(sa, dtype=dt[ka]), dev.upload(sb, dtype=dt[kb])
    sc = np.ascontiguousarray(Cold.T if colmajor else Cold)
    pc = dev.upload(sc, dtype=dt[kc])
    ma = mat(pa, 1, M, kinds[ka]) if not ta else mat(pa, K, 1, kinds[ka])
    mb = mat(pb, 1, K, kinds[kb]) if not tb else mat(pb, N, 1, kinds[kb])
    mc = mat(pc, 1, M, kinds[kc]) if colmajor else mat(pc, N, 1, kinds[kc])
    nb = hip.fitre_hip_gemm_f64_workspace(M, N, K, 0)
    ws = dev.alloc(nb)
    alpha, beta = 0.75, -0.5
    L.check(hip.fitre_hip_gemm_f64(M, N, K, alpha, C.byref(ma), C.byref(mb), beta, C.byref(mc), 0.0, 0, ws, nb))
    got = dev.download(pc, M * N, dtype=dt[kc])
    got = got.reshape(N, M).T if colmajor else got.reshape(M, N)
    want = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * Cold.astype(np.float64)
    for q in (pa, pb, pc, ws):
        dev.free(q)
    assert rel_err(got, want) < (1e-6 if kc == "f32" else 1e-13)


@pytest.mark.parametrize("n,k", [(5, 3), (64, 200), (129, 77), (300, 1500), (1300, 260)])
def test_gemm_f64_symmetric_with_a_constant_row(dev, n, k):
    """R R^T * alpha + shift I with a row of R that is not in memory (the bias row of a KFAC factor), as doubles (both
    triangles) and as float pairs."""
    rng = np.random.default_rng(n + k)
    R = rng.standard_normal((n - 1, k)).astype(np.float32)
    full = np.concatenate([R.astype(np.float64), np.full((1, k), 2.5)], axis=0)
    want = 0.3 * full @ full.T + 0.125 * np.eye(n)
    pr = dev.upload(R)
    a = mat(pr, k, 1, FITRE_MAT_F32, ones_row=n - 1, ones_value=2.5)
    b = mat(pr, 1, k, FITRE_MAT_F32, ones_col=n - 1, ones_value=2.5)
    nb = hip.fitre_hip_gemm_f64_workspace(n, n, k, FITRE_GEMM_SYMMETRIC)
    ws = dev.alloc(nb)
    out = dev.upload(np.full(n * n, np.nan), dtype=np.float64)
    c = mat(out, 1, n, FITRE_MAT_F64)
    L.check(hip.fitre_hip_gemm_f64(n, n, k, 0.3, C.byref(a), C.byref(b), 0.0, C.byref(c), 0.125, FITRE_GEMM_SYMMETRIC, ws, nb))
    got = dev.download(out, n * n, dtype=np.float64).reshape(n, n)
    assert rel_err(got, want) < 1e-13
    np.testing.assert_array_equal(got, got.T)
    outp = dev.upload(np.full(n * n, np.nan, dtype=np.float32))
    c = mat(outp, n, n, FITRE_MAT_SYM_PAIR)
    L.check(hip.fitre_hip_gemm_f64(n, n, k, 0.3, C.byref(a), C.byref(b), 0.0, C.byref(c), 0.125, FITRE_GEMM_SYMMETRIC, ws, nb))
    pair = dev.download(outp, n * n).reshape(n, n).T      # column-major on the device
    assert rel_err(pair_decode(pair), want) < 1e-9       # 32 significant bits on the diagonal and beside it, 48 elsewhere
    off = ~(np.eye(n, dtype=bool) | np.eye(n, k=1, dtype=bool) | np.eye(n, k=-1, dtype=bool))
    off[0, n - 1] = off[n - 1, 0] = False
    assert np.abs((pair_decode(pair) - want)[off]).max(initial=0.0) < 1e-13 * np.abs(want).max()
    np.testing.assert_array_equal(np.triu(pair), np.triu(got.astype(np.float32)))   # the upper triangle alone is the float matrix
    for q in (pr, ws, out, outp):
        dev.free(q)


@pytest.mark.parametrize("n,m", [(70, 9), (257, 130), (513, 10)])
def test_gemm_f64_float_pair_operand(dev, n, m):
    """A symmetric float-pair matrix on either side of a product."""
    rng = np.random.default_rng(n * m)
    q = rng.standard_normal((n, n))
    S = q @ q.T * 1e3
    G = rng.standard_normal((m, n)).astype(np.float32)
    ps, pg = dev.upload(pair_encode(S).T.copy()), dev.upload(np.ascontiguousarray(G.T))   # column-major uploads
    S = pair_decode(pair_encode(S))
    nb = max(hip.fitre_hip_gemm_f64_workspace(m, n, n, 0), hip.fitre_hip_gemm_f64_workspace(n, m, n, 0))
    ws = dev.alloc(nb)
    out = dev.upload(np.zeros(m * n), dtype=np.float64)
    sm, gm, cm = mat(ps, n, n, FITRE_MAT_SYM_PAIR), mat(pg, 1, m, FITRE_MAT_F32), mat(out, 1, m, FITRE_MAT_F64)
    L.check(hip.fitre_hip_gemm_f64(m, n, n, 1.0, C.byref(gm), C.byref(sm), 0.0, C.byref(cm), 0.0, 0, ws, nb))
    got = dev.download(out, m * n, dtype=np.float64).reshape(n, m).T
    assert rel_err(got, G.astype(np.float64) @ S) < 1e-13
    gt, ct = mat(pg, m, 1, FITRE_MAT_F32), mat(out, 1, n, FITRE_MAT_F64)      # G^T (n x m)
    L.check(hip.fitre_hip_gemm_f64(n, m, n, 1.0, C.byref(sm), C.byref(gt), 0.0, C.byref(ct), 0.0, 0, ws, nb))
    got = dev.download(out, m * n, dtype=np.float64).reshape(m, n).T
    assert rel_err(got, S @ G.astype(np.float64).T) < 1e-13
    for p in (ps, pg, ws, out):
        dev.free(p)


@pytest.mark.parametrize("n", [1, 2, 3, 31, 33, 100, 577])
def test_float_pair_decoded_on_the_device(dev, n):
    """fitre_hip_pair_to_f64 gives, bit for bit, the doubles the host decoder reads out of the same words (both triangles,
    the shared words beside the diagonal included), into a result with a leading dimension of its own."""
    rng = np.random.default_rng(n)
    q = rng.standard_normal((n, n))
    words = pair_encode(q @ q.T * 1e3 + np.eye(n))
    ld = n + 3
    pp = dev.upload(words.T.copy())                              # column-major
    out = dev.upload(np.full(ld * n, -7.0), dtype=np.float64)
    L.check(hip.fitre_hip_pair_to_f64(pp, n, n, out, ld))
    got = dev.download(out, ld * n, dtype=np.float64).reshape(n, ld)
    np.testing.assert_array_equal(got[:, :n].T, pair_decode(words))
    assert (got[:, n:] == -7.0).all()
    assert hip.fitre_hip_pair_to_f64(pp, n - 1, n, out, ld) == 2
    dev.free(pp), dev.free(out)


@pytest.mark.parametrize("flag", ["a_lower", "a_upper", "b_lower", "b_upper", "both"])
@pytest.mark.parametrize("n", [100, 333])
def test_gemm_f64_triangular_ranges(dev, flag, n):
    """Products with a triangular operand: the reduction skips the zero part and gives the plain product."""
    rng = np.random.default_rng(n)
    A, B = rng.standard_normal((n, n)), rng.standard_normal((n, n))
    flags = 0
    if flag in ("a_lower",):
        A, flags = np.tril(A), FITRE_GEMM_A_LOWER
    if flag in ("a_upper", "both"):
        A, flags = np.triu(A), flags | FITRE_GEMM_A_UPPER
    if flag in ("b_lower", "both"):
        B, flags = np.tril(B), flags | FITRE_GEMM_B_LOWER
    if flag == "b_upper":
        B, flags = np.triu(B), FITRE_GEMM_B_UPPER
    # the zero triangle holds garbage where the kernel may not look: NaN outside the 16-aligned margin it may still read
    pa, pb = dev.upload(np.ascontiguousarray(A.T), dtype=np.float64), dev.upload(np.ascontiguousarray(B.T), dtype=np.float64)
    out = dev.upload(np.zeros(n * n), dtype=np.float64)
    nb = hip.fitre_hip_gemm_f64_workspace(n, n, n, flags)
    ws = dev.alloc(nb)
    for colmajor in (True, False):
        ma, mb = mat(pa, 1, n, FITRE_MAT_F64), mat(pb, 1, n, FITRE_MAT_F64)
        mc = mat(out, 1, n, FITRE_MAT_F64) if colmajor else mat(out, n, 1, FITRE_MAT_F64)
        L.check(hip.fitre_hip_gemm_f64(n, n, n, 1.0, C.byref(ma), C.byref(mb), 0.0, C.byref(mc), 0.0, flags, ws, nb))
        got = dev.download(out, n * n, dtype=np.float64).reshape(n, n)
        got = got.T if colmajor else got
        assert rel_err(got, A @ B) < 1e-13, colmajor
    for p in (pa, pb, out, ws):
        dev.free(p)


def _spd_with_condition(n, rng, cond):
    q, _ = np.linalg.qr(rng.standard_normal((n, n)))
    ev = np.geomspace(1.0, 1.0 / cond, n)
    s = (q * ev) @ q.T
    return (s + s.T) / 2


@pytest.mark.parametrize("n", [1, 2, 37, 64, 65, 128, 200, 577, 1153])
@pytest.mark.parametrize("kind", ["f64", "pair", "f32"])
def test_spd_inverse_f64(dev, n, kind):
    """The float64 inverse against LAPACK at condition 1e6: 1e-9 of the largest element as doubles or float pairs, float
    rounding as floats."""
    import scipy.linalg as sl
    if kind != "pair" and n not in (37, 200, 1153):
        pytest.skip("the other result kinds share everything but the last store")
    rng = np.random.default_rng(n)
    S = _spd_with_condition(n, rng, 1e6)
    want = sl.cho_solve(sl.cho_factor(S), np.eye(n))
    pm = dev.upload(S.reshape(-1), dtype=np.float64)
    nb = hip.fitre_hip_spd_inverse_f64_workspace(n)
    ws = dev.alloc(nb)
    pivot = dev.upload(np.array([7], dtype=np.int32), dtype=np.int32)
    k, dt = {"f64": (FITRE_MAT_F64, np.float64), "pair": (FITRE_MAT_SYM_PAIR, np.float32), "f32": (FITRE_MAT_F32, np.float32)}[kind]
    out = dev.upload(np.full(n * n, np.nan).astype(dt), dtype=dt)
    L.check(hip.fitre_hip_spd_inverse_f64_queued(pm, n, out, k, ws, nb, pivot))
    dev.sync()
    assert dev.download(pivot, 1, dtype=np.int32)[0] == 0
    got = dev.download(out, n * n, dtype=dt).reshape(n, n)
    for p in (pm, ws, pivot, out):
        dev.free(p)
    if kind == "pair":
        got = pair_decode(got.T)                              # column-major on the device
    assert np.isfinite(got).all()
    # a float pair has 32 significant bits on the diagonal from order 3 on, 24 below that
    assert rel_err(got, want) < (1e-6 if kind == "f32" or (kind == "pair" and n < 3) else 1e-9)
    if kind != "pair":
        np.testing.assert_array_equal(got, got.T)


def test_spd_inverse_f64_reports_the_pivot(dev):
    n = 150
    S = _spd_with_condition(n, np.random.default_rng(3), 10.0)
    S[100, 100] = -1.0
    pm = dev.upload(S.reshape(-1), dtype=np.float64)
    nb = hip.fitre_hip_spd_inverse_f64_workspace(n)
    ws = dev.alloc(nb)
    pivot = dev.upload(np.array([0], dtype=np.int32), dtype=np.int32)
    out = dev.upload(np.zeros(n * n), dtype=np.float64)
    L.check(hip.fitre_hip_spd_inverse_f64_queued(pm, n, out, FITRE_MAT_F64, ws, nb, pivot))
    dev.sync()
    assert dev.download(pivot, 1, dtype=np.int32)[0] == 101
    for p in (pm, ws, pivot, out):
        dev.free(p)


def test_compute_matrix_inverse(dev):
    """computeMatrixInverse: float matrix in, float inverse of matrix + (lambda + gamma) I out, float64 in between."""
    import scipy.linalg as sl
    n, lam, gamma = 300, 1e-3, 2e-3
    rng = np.random.default_rng(11)
    p = rng.standard_normal((n, 40))
    S = (p @ p.T).astype(np.float32)          # rank 40: the damping alone makes it definite
    S = np.maximum(S, S.T)
    pm, out = dev.upload(S.reshape(-1)), dev.upload(np.full(n * n, np.nan, dtype=np.float32))
    ws = dev.alloc(4 * L.cnn.matrixInverseMemRequired(n))
    L.cnn.computeMatrixInverse(pm, out, n, ws, lam, gamma)
    got = dev.download(out, n * n).reshape(n, n)
    shift = float(np.float32(lam)) + float(np.float32(gamma))
    want = sl.cho_solve(sl.cho_factor(S.astype(np.float64) + shift * np.eye(n)), np.eye(n))
    for q in (pm, out, ws):
        dev.free(q)
    assert rel_err(got, want) < 1e-6


FACTOR_CASES = [
    (2, 3, 6, 32, 32, 5, 1, 0),
    (2, 64, 128, 16, 16, 3, 1, 1),
    (16, 128, 8, 4, 4, 3, 1, 1),
    (2, 3, 8, 67, 67, 11, 4, 2),
    (3, 5, 7, 9, 6, 3, 1, 1),
]


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("case", FACTOR_CASES)
def test_factors_f64(dev, oracle64, case, bias):
    """The four Kronecker factors accumulated in float64, damping on the diagonal, against the oracle."""
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    rng = np.random.default_rng(sum(case))
    x = (rng.standard_normal(Cin * N * A * B) + 0.3).astype(np.float32)
    n = Cin * k * k + (1 if bias else 0)
    px = dev.upload(x)
    nb = hip.fitre_hip_kfac_conv_input_factor_f64_workspace(C.byref(shape), int(bias))
    ws = dev.alloc(nb)
    out = dev.upload(np.full(n * n, np.nan), dtype=np.float64)
    L.check(hip.fitre_hip_kfac_conv_input_factor_f64(C.byref(shape), px, int(bias), 0.25, out, ws, nb))
    got = dev.download(out, n * n, dtype=np.float64).reshape(n, n)
    want = oracle64.kfac_conv_input_factor(x, N, Cin, B, A, k, p, s, bias) + 0.25 * np.eye(n)
    assert rel_err(got, want) < 1e-12
    np.testing.assert_array_equal(got, got.T)
    for q in (px, ws, out):
        dev.free(q)
    R = N * shape.outA * shape.outB
    d = rng.standard_normal(Cout * R).astype(np.float32)
    pd = dev.upload(d)
    nb = hip.fitre_hip_gemm_f64_workspace(Cout, Cout, R, FITRE_GEMM_SYMMETRIC)
    ws = dev.alloc(nb)
    out = dev.upload(np.full(Cout * Cout, np.nan), dtype=np.float64)
    L.check(hip.fitre_hip_kfac_conv_output_factor_f64(C.byref(shape), pd, 0.5, out, ws, nb))
    got = dev.download(out, Cout * Cout, dtype=np.float64).reshape(Cout, Cout)
    want = oracle64.kfac_conv_output_factor(d, N, shape.outB, shape.outA, Cout) + 0.5 * np.eye(Cout)
    assert rel_err(got, want) < 1e-12
    for q in (pd, ws, out):
        dev.free(q)
    # fully connected: in = Cin * 7, samples = N * 5
    fin, fout, samples = Cin * 7, Cout, N * 5
    z, d = rng.standard_normal(fin * samples).astype(np.float32), rng.standard_normal(fout * samples).astype(np.float32)
    pz, pd = dev.upload(z), dev.upload(d)
    n = fin + (1 if bias else 0)
    nb = max(hip.fitre_hip_gemm_f64_workspace(n, n, samples, FITRE_GEMM_SYMMETRIC), hip.fitre_hip_gemm_f64_workspace(fout, fout, samples, FITRE_GEMM_SYMMETRIC))
    ws = dev.alloc(nb)
    out = dev.upload(np.full(n * n, np.nan), dtype=np.float64)
    L.check(hip.fitre_hip_kfac_fc_input_factor_f64(pz, fin, samples, int(bias), 1e-3, out, ws, nb))
    got = dev.download(out, n * n, dtype=np.float64).reshape(n, n)
    assert rel_err(got, oracle64.kfac_fc_input_factor(z, fin, samples, bias) + 1e-3 * np.eye(n)) < 1e-12
    out2 = dev.upload(np.full(fout * fout, np.nan), dtype=np.float64)
    L.check(hip.fitre_hip_kfac_fc_output_factor_f64(pd, fout, samples, 1e-3, out2, ws, nb))
    got = dev.download(out2, fout * fout, dtype=np.float64).reshape(fout, fout)
    assert rel_err(got, oracle64.kfac_fc_output_factor(d, fout, samples) + 1e-3 * np.eye(fout)) < 1e-12
    for q in (pz, pd, ws, out, out2):
        dev.free(q)
