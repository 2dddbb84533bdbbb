"""fp32-MFMA contractions against the float64 oracle: convolution forward, weight gradient, input
gradient and the column-major GEMM, over tile-edge, split-K and layout edge cases."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L
from helpers import conv_shape, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4
hip = L.hip

# N, Cin, Cout, A(width), B(height), k, stride, pad
CONV_CASES = [
    (2, 3, 6, 32, 32, 5, 1, 0),      # LeNet conv1
    (2, 6, 16, 14, 14, 5, 1, 0),     # LeNet conv2
    (4, 3, 64, 32, 32, 3, 1, 1),     # VGG conv1
    (2, 64, 128, 16, 16, 3, 1, 1),   # VGG conv2
    (4, 130, 70, 8, 8, 3, 1, 1),     # channel counts off the tile grid
    (8, 256, 256, 4, 4, 3, 1, 1),    # deep reduction, small map
    (16, 96, 200, 2, 2, 3, 1, 1),    # 2x2 maps (VGG conv8 shape class)
    (2, 3, 8, 67, 67, 11, 4, 2),     # AlexNet conv1 (strided)
    (2, 8, 12, 13, 13, 5, 1, 2),     # AlexNet conv2
    (3, 5, 7, 9, 6, 3, 1, 1),        # rectangular
    (1, 1, 1, 5, 5, 3, 1, 0),        # degenerate
    (2, 4, 5, 7, 7, 1, 1, 0),        # 1x1 window
    (2, 4, 6, 9, 9, 3, 2, 1),        # stride 2
    # 65..96 channel rows on the general engine: the 96-row tile (AlexNet's 96-channel layers)
    (2, 96, 40, 13, 13, 5, 1, 2),    # input gradient with 96 rows
    (2, 20, 96, 13, 13, 5, 1, 2),    # forward and weight gradient with 96 rows
    (2, 80, 72, 9, 9, 5, 1, 2),      # 80 and 72 rows: partial 96-row tiles
    # 3x3 / stride 1 / pad 1 fast paths: tile edges in every dimension
    (3, 8, 16, 8, 8, 3, 1, 1),       # 192 positions: not a multiple of the 128-position tile
    (2, 16, 40, 6, 10, 3, 1, 1),     # rectangular maps, 40 output channels
    (5, 24, 136, 4, 4, 3, 1, 1),     # 136 channels: one full and one partial channel tile
    (2, 32, 32, 32, 32, 3, 1, 1),    # 32-wide rows
    (1, 8, 8, 64, 64, 3, 1, 1),      # widest row the LDS window holds
    (1, 8, 8, 66, 66, 3, 1, 1),      # one wider: general engine
    (7, 48, 64, 3, 5, 3, 1, 1),      # odd extents, 105 positions
    (64, 64, 64, 2, 2, 3, 1, 1),     # 2x2 maps: the dense-product form of both gradients
    (40, 68, 200, 2, 2, 3, 1, 1),    # the same with partial tiles in every dimension (272 x 800 x 40)
    (96, 128, 192, 2, 2, 3, 1, 1),   # split reduction of the input gradient
    (24, 64, 64, 2, 2, 3, 1, 1),     # too few images for the dense form: nine-tap kernels
    # 4x4 maps: the kernels that leave out the taps outside the image (whole stages of four images)
    (32, 32, 128, 4, 4, 3, 1, 1),    # one tile each way
    (36, 40, 72, 4, 4, 3, 1, 1),     # partial channel tiles, nine stages
    (64, 96, 160, 4, 4, 3, 1, 1),    # split reduction
    (32, 40, 72, 4, 4, 3, 1, 1),     # whole image tiles with partial channel tiles in the input gradient's cell form
    (6, 16, 32, 4, 4, 3, 1, 1),      # six images: not whole stages, nine-tap kernels
    # 8x8 maps: the weight gradient's stages are half maps of two images
    (6, 32, 128, 8, 8, 3, 1, 1),     # one tile, six stages
    (18, 48, 160, 8, 8, 3, 1, 1),    # partial tiles, split reduction
    (3, 16, 32, 8, 8, 3, 1, 1),      # an odd number of images: nine-tap kernel
    # weight-gradient stages whose window starts in a different column every stage (64 % B != 0)
    (64, 16, 32, 3, 5, 3, 1, 1),     # B = 5, 960 positions
    (16, 24, 40, 4, 6, 3, 1, 1),     # B = 6, partial channel tiles
    (8, 16, 32, 2, 24, 3, 1, 1),     # B = 24: the wide-row instantiation
    (128, 16, 32, 1, 1, 3, 1, 1),    # 1x1 maps: only the centre tap sees data
    (32, 16, 32, 2, 1, 3, 1, 1),     # single-column maps
    (4, 16, 32, 1, 16, 3, 1, 1),     # single-row maps
    # weight gradient with at most three input channels (the first layer's kernel): chunks of whole image rows
    (6, 3, 64, 32, 32, 3, 1, 1),     # the benchmark's first layer at a small batch
    (5, 3, 64, 8, 16, 3, 1, 1),      # eight rows per chunk
    (3, 2, 40, 32, 4, 3, 1, 1),      # 32 rows per chunk, partial output-channel block
    (2, 1, 7, 2, 64, 3, 1, 1),       # one input channel, two rows per chunk
    (3, 3, 64, 1, 128, 3, 1, 1),     # one row per chunk: nothing above or below
    (2, 3, 16, 12, 32, 3, 1, 1),     # A not a multiple of the rows per chunk... 12 % 4 == 0: eligible
    (2, 3, 16, 6, 32, 3, 1, 1),      # 6 % 4 != 0: general engine
    # few channels, the vector kernels: bands of output rows, several images per workgroup, borders, strides
    (128, 3, 6, 32, 32, 5, 1, 0),    # LeNet conv1 at batch 128: two bands per image
    (128, 6, 16, 14, 14, 5, 1, 0),   # LeNet conv2 at batch 128
    (600, 6, 16, 14, 14, 5, 1, 0),   # more images than workgroups: two units per workgroup, a ragged last one
    (5, 6, 16, 14, 14, 5, 1, 2),     # padded: the zero border of both kernels
    (3, 4, 12, 11, 9, 3, 1, 1),      # rectangular, 3x3 window, bands of uneven height
    (7, 2, 5, 13, 13, 4, 1, 3),      # even window, border of the full window minus one
    (9, 5, 10, 15, 15, 5, 2, 1),     # strided weight gradient
    (2, 16, 16, 9, 9, 5, 1, 0),      # sixteen channels each side
]


def run_conv(dev, oracle64, case, which):
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    oA, oB = shape.outA, shape.outB
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal(Cin * N * A * B).astype(np.float32)
    w = (rng.standard_normal(Cout * Cin * k * k) / np.sqrt(Cin * k * k)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    d = rng.standard_normal(Cout * N * oA * oB).astype(np.float32)
    px, pw, pb, pd = dev.upload(x), dev.upload(w), dev.upload(b), dev.upload(d)
    bufs = [px, pw, pb, pd]
    if which == "fwd":
        nb = hip.fitre_hip_conv_forward_workspace(C.byref(shape))
        ws, out = dev.alloc(nb), dev.zeros(d.size)
        L.check(hip.fitre_hip_conv_forward(C.byref(shape), px, pw, pb, out, ws, nb))
        got, want = dev.download(out, d.size), oracle64.conv_forward(x, w, b, N, Cin, B, A, k, p, s, Cout)
    elif which == "dw":
        nb = hip.fitre_hip_conv_weight_grad_workspace(C.byref(shape))
        ws, out = dev.alloc(nb), dev.zeros(w.size)
        L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px, pd, out, ws, nb))
        got, want = dev.download(out, w.size), oracle64.conv_weight_grad(x, d, N, Cin, B, A, k, p, s, Cout)
    else:
        nb = hip.fitre_hip_conv_input_grad_workspace(C.byref(shape))
        ws, out = dev.alloc(nb), dev.zeros(x.size)
        L.check(hip.fitre_hip_conv_input_grad(C.byref(shape), pd, pw, out, ws, nb))
        got, want = dev.download(out, x.size), oracle64.conv_input_grad(d, w, N, Cin, B, A, k, p, Cout)
    for q in bufs + [ws, out]:
        dev.free(q)
    return got, want


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_forward(dev, oracle64, case):
    got, want = run_conv(dev, oracle64, case, "fwd")
    assert rel_err(got, want) < TOL


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_weight_gradient(dev, oracle64, case):
    got, want = run_conv(dev, oracle64, case, "dw")
    assert rel_err(got, want) < TOL


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[6] == 1])
def test_conv_input_gradient(dev, oracle64, case):
    got, want = run_conv(dev, oracle64, case, "dx")
    assert rel_err(got, want) < TOL


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[1] <= 16 and c[2] <= 16 or c in CONV_CASES[2:5]])
def test_conv_weight_and_bias_gradient(dev, oracle64, case):
    """dW and db = sum of delta per output channel in one call: the fused kernel of thin layers and the two-step path of
    the others, against the float64 oracle and numpy; the bias slot's neighbours stay untouched."""
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    oA, oB = shape.outA, shape.outB
    rng = np.random.default_rng(sum(case) + 5)
    x = rng.standard_normal(Cin * N * A * B).astype(np.float32)
    d = rng.standard_normal(Cout * N * oA * oB).astype(np.float32)
    px, pd = dev.upload(x), dev.upload(d)
    nb = hip.fitre_hip_conv_weight_bias_grad_workspace(C.byref(shape))
    assert nb >= hip.fitre_hip_conv_weight_grad_workspace(C.byref(shape))
    ws = dev.alloc(nb)
    dw = dev.upload(np.full(Cout * Cin * k * k + 2, 3.0, np.float32))
    db = dev.upload(np.full(Cout + 2, 5.0, np.float32))
    L.check(hip.fitre_hip_conv_weight_bias_grad(C.byref(shape), px, pd, dw, db, ws, nb))
    got_w, got_b = dev.download(dw, Cout * Cin * k * k + 2), dev.download(db, Cout + 2)
    assert rel_err(got_w[:-2], oracle64.conv_weight_grad(x, d, N, Cin, B, A, k, p, s, Cout)) < TOL
    assert rel_err(got_b[:Cout], d.astype(np.float64).reshape(Cout, -1).sum(axis=1)) < TOL
    assert (got_w[-2:] == 3.0).all() and (got_b[Cout:] == 5.0).all()
    # without a bias slot: the plain weight gradient
    L.check(hip.fitre_hip_memset(dw, 0, 4 * Cout * Cin * k * k))
    L.check(hip.fitre_hip_conv_weight_bias_grad(C.byref(shape), px, pd, dw, None, ws, nb))
    assert rel_err(dev.download(dw, Cout * Cin * k * k), oracle64.conv_weight_grad(x, d, N, Cin, B, A, k, p, s, Cout)) < TOL
    for q in (px, pd, ws, dw, db):
        dev.free(q)


PAIR_CASES = [c for c in CONV_CASES if c[5] == 3 and c[6] == 1 and c[7] == 1] + [(256, 64, 128, 16, 16, 3, 1, 1),
                                                                                 (64, 512, 512, 2, 2, 3, 1, 1)]


@pytest.mark.parametrize("case", PAIR_CASES)
def test_sums_of_two_products_in_one_launch(dev, oracle64, case):
    """conv(x1,w1) + conv(x2,w2) + bias, dX(d1,w1) + dX(d2,w2) and dW(x1,d1) + dW(x2,d2) through the pair entry points,
    for every shape the specialised 3x3 kernels take, against the oracle's two products added in float64 (and, at the
    two benchmark-sized shapes, against the device's own two products added)."""
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
    rng = np.random.default_rng(sum(case) + 11)
    big = N * A * B * max(Cin, Cout) > 2_000_000
    xs = [rng.standard_normal(Cin * N * A * B).astype(np.float32) for _ in range(2)]
    ws_ = [(rng.standard_normal(Cout * Cin * 9) / np.sqrt(Cin * 9)).astype(np.float32) for _ in range(2)]
    ds = [rng.standard_normal(Cout * N * A * B).astype(np.float32) for _ in range(2)]
    b = rng.standard_normal(Cout).astype(np.float32)
    px, pw, pd, pb = [dev.upload(v) for v in xs], [dev.upload(v) for v in ws_], [dev.upload(v) for v in ds], dev.upload(b)

    def single(which, i):
        """the device's single product (reference when the oracle would take too long)"""
        if which == 0:
            nb = hip.fitre_hip_conv_forward_workspace(C.byref(shape)); w_ = dev.alloc(nb); out = dev.zeros(ds[0].size)
            L.check(hip.fitre_hip_conv_forward(C.byref(shape), px[i], pw[i], pb if i == 0 else None, out, w_, nb)); n = ds[0].size
        elif which == 1:
            nb = hip.fitre_hip_conv_input_grad_workspace(C.byref(shape)); w_ = dev.alloc(nb); out = dev.zeros(xs[0].size)
            L.check(hip.fitre_hip_conv_input_grad(C.byref(shape), pd[i], pw[i], out, w_, nb)); n = xs[0].size
        else:
            nb = hip.fitre_hip_conv_weight_grad_workspace(C.byref(shape)); w_ = dev.alloc(nb); out = dev.zeros(ws_[0].size)
            L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px[i], pd[i], out, w_, nb)); n = ws_[0].size
        got = dev.download(out, n).astype(np.float64)
        dev.free(w_), dev.free(out)
        return got

    for kind in (0, 1, 2):
        if not hip.fitre_hip_conv_pair_supported(C.byref(shape), kind):
            assert hip.fitre_hip_conv_pair_workspace(C.byref(shape), kind) == 0
            continue
        nb = hip.fitre_hip_conv_pair_workspace(C.byref(shape), kind)
        wsp = dev.alloc(nb)
        if kind == 0:
            out = dev.upload(np.full(ds[0].size, np.nan, np.float32))
            L.check(hip.fitre_hip_conv_forward_pair(C.byref(shape), px[0], pw[0], px[1], pw[1], pb, out, wsp, nb))
            got = dev.download(out, ds[0].size)
            want = single(0, 0) + single(0, 1) if big else (oracle64.conv_forward(xs[0], ws_[0], b, N, Cin, B, A, 3, 1, 1, Cout) +
                                                           oracle64.conv_forward(xs[1], ws_[1], 0 * b, N, Cin, B, A, 3, 1, 1, Cout))
        elif kind == 1:
            out = dev.upload(np.full(xs[0].size, np.nan, np.float32))
            L.check(hip.fitre_hip_conv_input_grad_pair(C.byref(shape), pd[0], pw[0], pd[1], pw[1], out, wsp, nb))
            got = dev.download(out, xs[0].size)
            want = single(1, 0) + single(1, 1) if big else (oracle64.conv_input_grad(ds[0], ws_[0], N, Cin, B, A, 3, 1, Cout) +
                                                           oracle64.conv_input_grad(ds[1], ws_[1], N, Cin, B, A, 3, 1, Cout))
        else:
            out = dev.upload(np.full(ws_[0].size, np.nan, np.float32))
            L.check(hip.fitre_hip_conv_weight_grad_pair(C.byref(shape), px[0], pd[0], px[1], pd[1], out, wsp, nb))
            got = dev.download(out, ws_[0].size)
            want = single(2, 0) + single(2, 1) if big else (oracle64.conv_weight_grad(xs[0], ds[0], N, Cin, B, A, 3, 1, 1, Cout) +
                                                           oracle64.conv_weight_grad(xs[1], ds[1], N, Cin, B, A, 3, 1, 1, Cout))
        assert rel_err(got, want) < TOL, kind
        dev.free(wsp), dev.free(out)
    for q in px + pw + pd + [pb]:
        dev.free(q)


def test_conv3x3_with_unaligned_weight_and_delta_pointers(dev, oracle64):
    """Flat parameter vectors put weight blocks at arbitrary offsets: the fast paths must fall back to
    4-byte accesses when a pointer is not 16-byte aligned."""
    from helpers import at
    N, Cin, Cout, A, B = 4, 16, 32, 8, 8
    shape = conv_shape(N, Cin, Cout, A, B, 3, 1, 1)
    rng = np.random.default_rng(77)
    x = rng.standard_normal(Cin * N * A * B).astype(np.float32)
    w = rng.standard_normal(Cout * Cin * 9).astype(np.float32)
    d = rng.standard_normal(Cout * N * A * B).astype(np.float32)
    pw = at(dev.upload(np.concatenate([np.zeros(3, np.float32), w])), 3)
    pd = at(dev.upload(np.concatenate([np.zeros(1, np.float32), d])), 1)
    px = dev.upload(x)
    ws = dev.alloc(1 << 24)
    out = dev.zeros(max(d.size, x.size, w.size))
    L.check(hip.fitre_hip_conv_forward(C.byref(shape), px, pw, None, out, ws, 1 << 24))
    assert rel_err(dev.download(out, d.size), oracle64.conv_forward(x, w, None, N, Cin, B, A, 3, 1, 1, Cout)) < TOL
    L.check(hip.fitre_hip_conv_input_grad(C.byref(shape), pd, pw, out, ws, 1 << 24))
    assert rel_err(dev.download(out, x.size), oracle64.conv_input_grad(d, w, N, Cin, B, A, 3, 1, Cout)) < TOL
    L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px, pd, out, ws, 1 << 24))
    assert rel_err(dev.download(out, w.size), oracle64.conv_weight_grad(x, d, N, Cin, B, A, 3, 1, 1, Cout)) < TOL


def test_conv_input_gradient_refuses_stride(dev):
    shape = conv_shape(2, 4, 6, 9, 9, 3, 2, 1)
    p = dev.zeros(4096)
    assert hip.fitre_hip_conv_input_grad(C.byref(shape), p, p, p, p, 4096) == 3
    assert b"stride" in hip.fitre_hip_last_error()


def test_conv_shape_is_validated(dev):
    shape = conv_shape(2, 4, 6, 9, 9, 3, 1, 1)
    shape.outA = 5
    p = dev.zeros(4096)
    assert hip.fitre_hip_conv_forward(C.byref(shape), p, p, None, p, p, 4096) == 2


def test_split_k_is_deterministic_and_workspace_independent(dev, oracle64):
    # long reduction, one output tile: planned with many splits; a tiny workspace forces fewer
    case = (32, 3, 16, 32, 32, 3, 1, 1)
    N, Cin, Cout, A, B, k, s, p = case
    shape = conv_shape(*case)
    rng = np.random.default_rng(3)
    x = rng.standard_normal(Cin * N * A * B).astype(np.float32)
    d = rng.standard_normal(Cout * N * A * B).astype(np.float32)
    px, pd = dev.upload(x), dev.upload(d)
    nb = hip.fitre_hip_conv_weight_grad_workspace(C.byref(shape))
    assert nb > 0
    ws, out = dev.alloc(nb), dev.zeros(Cout * Cin * k * k)
    res = []
    for _ in range(3):
        L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px, pd, out, ws, nb))
        res.append(dev.download(out, Cout * Cin * k * k))
    np.testing.assert_array_equal(res[0], res[1])
    np.testing.assert_array_equal(res[0], res[2])
    want = oracle64.conv_weight_grad(x, d, N, Cin, B, A, k, p, s, Cout)
    assert rel_err(res[0], want) < TOL
    small = 3 * Cout * Cin * k * k * 4  # room for three partial tiles only
    L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px, pd, out, ws, small))
    assert rel_err(dev.download(out, Cout * Cin * k * k), want) < TOL
    L.check(hip.fitre_hip_conv_weight_grad(C.byref(shape), px, pd, out, None, 0))  # unsplit
    assert rel_err(dev.download(out, Cout * Cin * k * k), want) < TOL


@pytest.mark.parametrize("case", [(256, 256, 512, 4, 4), (64, 512, 512, 2, 2), (96, 200, 520, 4, 4), (4, 16, 32, 8, 8), (2, 4, 6, 9, 9)])
def test_input_gradient_left_as_split_partials(dev, case):
    """fitre_hip_conv_input_grad_split: the slabs of the view, summed in order in double, are what
    fitre_hip_conv_input_grad writes -- bit for bit; an unsplit product reports one slab at dx."""
    from fitre_amd.structs import fitre_split_view
    N, Cin, Cout, A, B = case
    shape = conv_shape(N, Cin, Cout, A, B, 3, 1, 1)
    rng = np.random.default_rng(Cin + A)
    w = (rng.standard_normal(Cout * Cin * 9) / np.sqrt(Cin * 9)).astype(np.float32)
    d = rng.standard_normal(Cout * N * A * B).astype(np.float32)
    n = Cin * N * A * B
    pw, pd = dev.upload(w), dev.upload(d)
    nb = hip.fitre_hip_conv_input_grad_workspace(C.byref(shape))
    ws, ref, out = dev.alloc(nb), dev.zeros(n), dev.upload(np.full(n, 7.0, np.float32))
    L.check(hip.fitre_hip_conv_input_grad(C.byref(shape), pd, pw, ref, ws, nb))
    want = dev.download(ref, n)
    view = fitre_split_view()
    L.check(hip.fitre_hip_conv_input_grad_split(C.byref(shape), pd, pw, out, ws, nb, C.byref(view)))
    if view.splits == 1:
        assert view.base == out.value
        np.testing.assert_array_equal(dev.download(out, n), want)
    else:
        # the slabs lie inside the workspace (behind the rearranged weights for 2 x 2 maps)
        assert ws.value <= view.base and view.base + 4 * n * view.splits <= ws.value + nb and view.stride == n
        acc = np.zeros(n)
        for q in range(view.splits):
            acc += dev.download(C.c_void_p(view.base), n, offset=q * view.stride).astype(np.float64)
        np.testing.assert_array_equal(acc.astype(np.float32), want)
        np.testing.assert_array_equal(dev.download(out, n), np.full(n, 7.0, np.float32))   # dx itself is left alone
    for q in (pw, pd, ws, ref, out):
        dev.free(q)


GEMM_CASES = [  # M, N, K
    (10, 256, 512), (512, 256, 10), (120, 7, 400), (84, 128, 120), (1, 1, 1), (129, 65, 33), (300, 200, 64), (64, 64, 4096),
]


@pytest.mark.parametrize("M,N,K", GEMM_CASES)
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm(dev, oracle64, M, N, K, ta, tb):
    rng = np.random.default_rng(M + N + K)
    lda = (K if ta else M) + 3
    ldb = (N if tb else K) + 1
    ldc = M + 2
    A = rng.standard_normal(lda * (M if ta else K)).astype(np.float32)
    Bm = rng.standard_normal(ldb * (K if tb else N)).astype(np.float32)
    C0 = rng.standard_normal(ldc * N).astype(np.float32)
    pa, pb, pc = dev.upload(A), dev.upload(Bm), dev.upload(C0)
    nb = hip.fitre_hip_gemm_workspace(M, N, K)
    ws = dev.alloc(nb)
    L.check(hip.fitre_hip_gemm(ta, tb, M, N, K, 0.5, pa, lda, pb, ldb, 2.0, pc, ldc, None, ws, nb))
    want = oracle64.gemm(ta, tb, M, N, K, 0.5, A, lda, Bm, ldb, 2.0, C0, ldc)
    got = dev.download(pc, ldc * N)
    assert rel_err(got, want) < TOL
    # padding rows of C (ldc > M) are untouched
    np.testing.assert_array_equal(got.reshape(N, ldc)[:, M:], C0.reshape(N, ldc)[:, M:])
    # beta = 0 with a bias column added
    bias = rng.standard_normal(M).astype(np.float32)
    L.check(hip.fitre_hip_gemm(ta, tb, M, N, K, 1.0, pa, lda, pb, ldb, 0.0, pc, ldc, dev.upload(bias), ws, nb))
    want = oracle64.gemm(ta, tb, M, N, K, 1.0, A, lda, Bm, ldb, 0.0, np.zeros(ldc * N), ldc).reshape(N, ldc)[:, :M] + bias[None, :]
    assert rel_err(dev.download(pc, ldc * N).reshape(N, ldc)[:, :M], want) < TOL
    for q in (pa, pb, pc, ws):
        dev.free(q)


# N, Cin, Cout, A, B, k, pad, whether it is one launch: the input gradient of this layer taken on through the 2 x 2 max pool and the activation of
# the layer below (maps of 2A x 2B)
FOLD_CASES = [
    (2, 6, 16, 14, 14, 5, 0, 1),     # LeNet conv2 above conv1's pool: 14 = three groups of four cells and a half one
    (3, 4, 8, 6, 10, 5, 2, 1),       # rectangular, padded
    (3, 4, 8, 6, 10, 3, 1, 0),       # a shape the 3 x 3 kernels take: the two steps one after the other
    (5, 3, 5, 3, 2, 3, 1, 1),        # a row is half a group
    (2, 16, 16, 12, 12, 5, 2, 1),    # the most channels the kernel takes
    (2, 3, 5, 7, 7, 3, 1, 0),        # odd extent: the two steps one after the other
    (2, 64, 128, 8, 8, 3, 1, 0),     # a layer of the 3 x 3 kernels: likewise
]


@pytest.mark.parametrize("case", FOLD_CASES)
@pytest.mark.parametrize("act", [1, 3, 6, 0])  # filled in below: codes from fitre_amd.structs
def test_input_gradient_through_pool_and_activation(dev, case, act):
    """fitre_hip_conv_input_grad_pool_act against fitre_hip_conv_input_grad followed by
    fitre_hip_pool_act_backward: dx, dxPool and dxAct bit for bit, also without dxPool."""
    from fitre_amd.structs import ACT_LOGISTIC, CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SWISH, MAX_POOL
    act = {1: CNN_ACT_RELU, 3: CNN_ACT_SWISH, 6: ACT_LOGISTIC, 0: CNN_ACT_NONE}[act]
    N, Cin, Cout, A, B, k, p, one_launch = case
    shape = conv_shape(N, Cin, Cout, A, B, k, 1, p)
    rng = np.random.default_rng(sum(case) + 31 * act)
    w = (rng.standard_normal(Cout * Cin * k * k) / np.sqrt(Cin * k * k)).astype(np.float32)
    d = rng.standard_normal(Cout * N * shape.outA * shape.outB).astype(np.float32)
    big = Cin * N * 4 * A * B
    z_in = rng.standard_normal(big).astype(np.float32)
    if act == CNN_ACT_RELU:
        z_act = np.maximum(z_in, 0).astype(np.float32)  # whole windows of equal zeros: the first cell takes the gradient
    elif act == ACT_LOGISTIC:
        z_act = (1.0 / (1.0 + np.exp(-z_in.astype(np.float64)))).astype(np.float32)
    elif act == CNN_ACT_SWISH:
        z_act = (z_in.astype(np.float64) / (1.0 + np.exp(-z_in.astype(np.float64)))).astype(np.float32)
    else:
        z_act = z_in.copy()
    pw, pd, pzi, pza = dev.upload(w), dev.upload(d), dev.upload(z_in), dev.upload(z_act)
    nb = hip.fitre_hip_conv_input_grad_workspace(C.byref(shape))
    ws = dev.alloc(max(nb, 256))
    small = Cin * N * A * B
    dx0, pool0, act0 = dev.zeros(small), dev.zeros(big), dev.zeros(big)
    L.check(hip.fitre_hip_conv_input_grad(C.byref(shape), pd, pw, dx0, ws, nb))
    L.check(hip.fitre_hip_pool_act_backward(MAX_POOL, act, dx0, pzi, pza, Cin, N, 2 * A, 2 * B, 2, 2, 0, A, B, pool0, act0))
    want = [dev.download(dx0, small), dev.download(pool0, big), dev.download(act0, big)]
    folds = hip.fitre_hip_conv_input_grad_folds_pool(C.byref(shape))
    assert folds == one_launch
    for with_pool in (True, False):
        dx1, pool1, act1 = dev.zeros(small), dev.zeros(big), dev.zeros(big)
        L.check(hip.fitre_hip_conv_input_grad_pool_act(C.byref(shape), pd, pw, dx1, act, pzi, pza, pool1 if with_pool else None, act1, ws, nb))
        got = [dev.download(dx1, small), dev.download(pool1, big), dev.download(act1, big)]
        assert np.array_equal(got[0], want[0])
        assert np.array_equal(got[2], want[2])
        if with_pool:
            assert np.array_equal(got[1], want[1])
        else:
            assert not got[1].any()
        for q in (dx1, pool1, act1):
            dev.free(q)
    assert want[2].any()
    for q in (pw, pd, pzi, pza, ws, dx0, pool0, act0):
        dev.free(q)


def test_input_gradient_through_pool_refuses_bad_arguments(dev):
    shape = conv_shape(2, 6, 16, 14, 14, 5, 1, 0)
    p = dev.zeros(64)
    assert hip.fitre_hip_conv_input_grad_pool_act(C.byref(shape), p, p, p, 1, None, None, None, p, None, 0) == 2   # no z_act
    assert hip.fitre_hip_conv_input_grad_pool_act(C.byref(shape), p, p, p, 12345, None, p, None, p, None, 0) == 2  # unknown activation
    assert hip.fitre_hip_conv_input_grad_folds_pool(None) == 0
    dev.free(p)


@pytest.mark.parametrize("eighths", [8, 7, 6, 4])
def test_weight_gradient_planned_for_a_share_of_the_chip(dev, oracle64, eighths):
    """fitre_hip_weight_grad_share: the 3 x 3 weight gradients cut for fewer compute units (another split of the
    reduction) stay within the tolerance of the float64 oracle; the setting is refused outside 4 to 8 eighths."""
    try:
        L.check(hip.fitre_hip_weight_grad_share(eighths))
        for case in [(64, 128, 256, 8, 8, 3, 1, 1), (32, 64, 128, 16, 16, 3, 1, 1), (32, 256, 512, 4, 4, 3, 1, 1)]:
            got, want = run_conv(dev, oracle64, case, "dw")
            assert rel_err(got, want) < TOL, case
    finally:
        L.check(hip.fitre_hip_weight_grad_share(8))
    assert hip.fitre_hip_weight_grad_share(3) == 2 and hip.fitre_hip_weight_grad_share(9) == 2


def test_held_back_reductions_of_small_layers_are_one_launch_with_the_same_bits(dev):
    """fitre_hip_thin_reduce_defer / _flush: the weight and bias gradients of two LeNet-sized layers with their reductions
    held back and made together equal, bit for bit, what the two calls write on their own; nothing is written before the
    flush; shapes of other kernels report no bytes to keep."""
    cases = [(8, 3, 6, 32, 32, 5, 1, 0), (8, 6, 16, 14, 14, 5, 1, 0)]
    rng = np.random.default_rng(99)
    data = []
    for N, Cin, Cout, A, B, k, s, p in cases:
        shape = conv_shape(N, Cin, Cout, A, B, k, s, p)
        keep = hip.fitre_hip_thin_reduce_bytes(C.byref(shape))
        assert keep > 0
        x = rng.standard_normal(Cin * N * A * B).astype(np.float32)
        d = rng.standard_normal(Cout * N * shape.outA * shape.outB).astype(np.float32)
        nb = hip.fitre_hip_conv_weight_bias_grad_workspace(C.byref(shape))
        assert nb >= 0 and keep <= max(nb, keep)
        data.append((shape, dev.upload(x), dev.upload(d), Cout * Cin * k * k, Cout, max(nb, keep)))
    assert hip.fitre_hip_thin_reduce_bytes(C.byref(conv_shape(4, 64, 128, 8, 8, 3, 1, 1))) == 0
    want = []
    for shape, px, pd, nw, nbias, nb in data:
        ws, dw, db = dev.alloc(nb), dev.zeros(nw), dev.zeros(nbias)
        L.check(hip.fitre_hip_conv_weight_bias_grad(C.byref(shape), px, pd, dw, db, ws, nb))
        want.append((dev.download(dw, nw).view(np.uint32), dev.download(db, nbias).view(np.uint32)))
        for q in (ws, dw, db):
            dev.free(q)
    held = []
    L.check(hip.fitre_hip_thin_reduce_defer(1))
    try:
        for shape, px, pd, nw, nbias, nb in data:
            ws, dw, db = dev.alloc(nb), dev.upload(np.full(nw, 7.0, np.float32)), dev.upload(np.full(nbias, 7.0, np.float32))
            L.check(hip.fitre_hip_conv_weight_bias_grad(C.byref(shape), px, pd, dw, db, ws, nb))
            held.append((ws, dw, db, nw, nbias))
        dev.sync()
        for ws, dw, db, nw, nbias in held:
            assert (dev.download(dw, nw) == 7.0).all() and (dev.download(db, nbias) == 7.0).all()
        L.check(hip.fitre_hip_thin_reduce_flush())
    finally:
        L.check(hip.fitre_hip_thin_reduce_defer(0))
    for (ws, dw, db, nw, nbias), (wdw, wdb) in zip(held, want):
        np.testing.assert_array_equal(dev.download(dw, nw).view(np.uint32), wdw)
        np.testing.assert_array_equal(dev.download(db, nbias).view(np.uint32), wdb)
        for q in (ws, dw, db):
            dev.free(q)
    for shape, px, pd, nw, nbias, nb in data:
        dev.free(px), dev.free(pd)
