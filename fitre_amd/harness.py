"""Host harness over the C boundary: model construction, seeded inputs, device buffers and the
per-model device state that drives cnnForward / cnnBackward / computeCNNGradient through ctypes.
Used by the benchmark, the smoke entry and the tests; nothing here computes on the CPU."""
import ctypes as C

import numpy as np

from fitre_amd import lib as L
from fitre_amd.structs import (AVG_POOL, CNN_ACT_NONE, CNN_ACT_RELU, CNN_MODEL, DEVICE_DATASET, MAX_POOL, NO_POOL,
                               PERFORM_BATCH_NORM, PERFORM_NO_BATCH_NORM, SCRATCH_AREA, fitre_conv_shape)


# ---------------------------------------------------------------- models
def build_custom(batch, height, width, in_channels, convs, fcs, bias=1):
    """convs: list of dict(cout, k, stride, pad, pool=(type, k, s, p) or None, bn=bool, act=code)
    fcs: list of (out, act).  Returns a finalised CNN_MODEL (slab scheme of nn/read_vgg.c:25-120)."""
    m = CNN_MODEL()
    h, w, cin = height, width, in_channels
    oh, ow = C.c_int(), C.c_int()
    for i, cv in enumerate(convs):
        pool = cv.get("pool")
        ptype, pk, ps, pp = pool if pool else (NO_POOL, 2, 2, 0)
        m.actFuns[i] = cv.get("act", CNN_ACT_RELU)
        L.cnn.fitre_make_conv_layer(C.byref(m.convLayer[i]), C.byref(m.poolLayer[i]), cin, cv["cout"], h, w, cv["k"],
                                    cv.get("stride", 1), cv.get("pad", 0), ptype, pk, ps, pp, batch,
                                    PERFORM_BATCH_NORM if cv.get("bn") else PERFORM_NO_BATCH_NORM, C.byref(oh),
                                    C.byref(ow))
        h, w, cin = oh.value, ow.value, cv["cout"]
    m.cLayers = len(convs)
    fan_in = cin * h * w
    for i, (out, act) in enumerate(fcs):
        m.fcLayer[i].in_ = fan_in
        m.fcLayer[i].out = out
        m.fcLayer[i].actFun = act
        m.fcLayer[i].batchNorm = 0
        m.fcLayer[i].offset = batch * out
        fan_in = out
    m.lLayers = len(fcs)
    m.bias = bias
    m.enableBatchNorm = int(any(cv.get("bn") for cv in convs))
    L.cnn.fitre_finalize_model(C.byref(m), height, width, batch)
    return m


def build_lenet(batch, bn=False, act=CNN_ACT_RELU, fc_act=CNN_ACT_RELU, bias=1, classes=10):
    m = CNN_MODEL()
    L.cnn.fitre_build_lenet(C.byref(m), batch, 32, 32, 3, classes, bias, int(bn), act, fc_act)
    return m


def build_vgg11(batch, bn=True, act=CNN_ACT_RELU, bias=1, classes=10):
    m = CNN_MODEL()
    L.cnn.fitre_build_vgg11(C.byref(m), batch, 32, 32, 3, classes, bias, int(bn), act)
    return m


def build_alexnet(batch, act=CNN_ACT_RELU, fc_act=CNN_ACT_RELU, bias=1, classes=1000, size=224):
    m = CNN_MODEL()
    L.cnn.fitre_build_alexnet(C.byref(m), batch, size, size, 3, classes, bias, act, fc_act)
    return m


def input_dims(model):
    c0 = model.convLayer[0]
    return c0.inChannels, c0.height, c0.width


def num_classes(model):
    return model.fcLayer[model.lLayers - 1].out


# ---------------------------------------------------------------- seeded inputs
def he_weights(model, rng, bias_scale=0.0):
    """He-normal weights N(0, 2/fan_in) in the flat layout; biases zero unless bias_scale > 0."""
    w = np.zeros(model.pSize, dtype=np.float64)
    for l in range(model.cLayers):
        c = model.convLayer[l]
        fan_in = c.inChannels * c.kSize * c.kSize
        n = fan_in * c.outChannels
        w[model.wOffsets[l]:model.wOffsets[l] + n] = rng.standard_normal(n) * np.sqrt(2.0 / fan_in)
        if model.bias:
            w[model.bOffsets[l]:model.bOffsets[l] + c.outChannels] = bias_scale * rng.standard_normal(c.outChannels)
    for f in range(model.lLayers):
        fc = model.fcLayer[f]
        l = model.cLayers + f
        n = fc.in_ * fc.out
        w[model.wOffsets[l]:model.wOffsets[l] + n] = rng.standard_normal(n) * np.sqrt(2.0 / fc.in_)
        if model.bias:
            w[model.bOffsets[l]:model.bOffsets[l] + fc.out] = bias_scale * rng.standard_normal(fc.out)
    return w


def batch_inputs(model, batch, rng):
    """x ~ N(0,1) in [C][N][W][H]; labels uniform, 1-based, as floats."""
    c, h, w = input_dims(model)
    x = rng.standard_normal(c * batch * h * w)
    y = rng.integers(1, num_classes(model) + 1, size=batch).astype(np.float64)
    return x, y


def rel_err(a, b):
    """max-abs error relative to the largest magnitude of the reference b."""
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    scale = np.max(np.abs(b))
    return float(np.max(np.abs(a - b)) / (scale if scale > 0 else 1.0))


# ---------------------------------------------------------------- float-pair matrices
def _diagonal_words(n):
    """Float-pair matrices (FITRE_MAT_SYM_PAIR, include/fitre_hip.h): (row, column) of the word that carries the remainder of diagonal element k in its lower 16 bits."""
    return [(k + 1, k) if k + 1 < n else (n - 1, 0) for k in range(n)]


def pair_decode(a):
    """The symmetric matrix a float-pair array stands for (a[r][c] = element (r, c) of the device's column-major array)."""
    n = a.shape[0]
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).copy()
    diag_lo = np.zeros(n)
    if n >= 3:
        for k, (r, c) in enumerate(_diagonal_words(n)):
            diag_lo[k] = np.uint32((int(bits[r, c]) & 0xFFFF) << 16).view(np.float32)
            bits[r, c] &= np.uint32(0xFFFF0000)
    a = bits.view(np.float32).astype(np.float64)
    full = np.triu(a) + np.tril(a, -1).T
    full = full + np.triu(full, 1).T
    full[np.diag_indices(n)] += diag_lo
    return full


def pair_encode(s):
    n = s.shape[0]
    hi = s.astype(np.float32)
    lo = (s - hi.astype(np.float64)).astype(np.float32)
    out = (np.triu(hi) + np.tril(lo, -1)).astype(np.float32)
    if n >= 3:
        bits = out.view(np.uint32)
        dl = np.diag(lo).copy().view(np.uint32)
        for k, (r, c) in enumerate(_diagonal_words(n)):
            bits[r, c] = (int(bits[r, c]) & 0xFFFF0000) | (int(dl[k]) >> 16)
    return out


KFAC_LOWRANK_TAG, KFAC_LOWRANK_HEADER = 0xF15EED12, 64


def stored_inverse(words, n):
    """The dense float64 inverse that the n * n floats of a KFAC slot stand for: a float-pair matrix (column-major), or --
    input-side factors with few positions behind them -- the low-rank form of kfac_path.c: a header (tag, positions,
    order, strides of R, alpha and the damping s as doubles, the word at which S^-1 starts), R and S^-1 as doubles, for
    (alpha R R^T + s I)^-1 = (I - alpha R S^-1 R^T) / s."""
    words = np.ascontiguousarray(words, dtype=np.float32)
    head = words[:16].view(np.uint32)
    if n * n >= 16 and int(head[0]) == KFAC_LOWRANK_TAG:
        m, order, rs, cs = int(head[1]), int(head[2]), int(head[3]), int(head[4])
        assert order == n
        alpha, shift = head[5:9].view(np.float64)
        body = words[KFAC_LOWRANK_HEADER:]
        r = np.lib.stride_tricks.as_strided(body, shape=(n, m), strides=(4 * rs, 4 * cs)).astype(np.float64)
        at = int(head[9])                                    # doubles, at an 8-byte boundary of the device array
        sinv = words[at:at + 2 * m * m].view(np.float64).reshape(m, m)
        return (np.eye(n) - alpha * (r @ sinv @ r.T)) / shift
    return pair_decode(words[:n * n].reshape(n, n).T)


# ---------------------------------------------------------------- device buffers
class Device:
    """Owns device buffers through the C-ABI (no torch involved)."""

    def __init__(self, index=0):
        L.check(L.hip.fitre_hip_init(index), "fitre_hip_init")
        self.bufs = []

    def close(self):
        for p in self.bufs:
            L.hip.fitre_hip_free(p)
        self.bufs = []

    def alloc(self, nbytes):
        p = C.c_void_p()
        L.check(L.hip.fitre_hip_malloc(C.byref(p), max(int(nbytes), 16)), "fitre_hip_malloc")
        self.bufs.append(p)
        return p

    def free(self, p):
        self.bufs = [b for b in self.bufs if b.value != p.value]
        L.check(L.hip.fitre_hip_free(p), "fitre_hip_free")

    def upload(self, arr, dtype=np.float32):
        a = np.ascontiguousarray(arr, dtype=dtype)
        p = self.alloc(a.nbytes)
        if a.nbytes:
            L.check(L.hip.fitre_hip_copy_h2d(p, a.ctypes.data_as(C.c_void_p), a.nbytes), "h2d")
        return p

    def zeros(self, n, dtype=np.float32):
        nbytes = int(n) * np.dtype(dtype).itemsize
        p = self.alloc(nbytes)
        L.check(L.hip.fitre_hip_memset(p, 0, max(nbytes, 16)), "memset")
        return p

    def download(self, p, n, dtype=np.float32, offset=0):
        out = np.empty(int(n), dtype=dtype)
        src = C.c_void_p(p.value + int(offset) * np.dtype(dtype).itemsize)
        if out.nbytes:
            L.check(L.hip.fitre_hip_copy_d2h(out.ctypes.data_as(C.c_void_p), src, out.nbytes), "d2h")
        return out

    def sync(self):
        L.check(L.hip.fitre_hip_sync(), "sync")


def at(p, offset_elems, itemsize=4):
    return C.c_void_p(p.value + int(offset_elems) * itemsize)


class GpuModel:
    """Device-side state for one model: weights, batch, labels, z, dx, gradient, scratch arena."""

    def __init__(self, dev, model, weights, x, y, batch):
        self.dev, self.model, self.batch = dev, model, batch
        self.classes = num_classes(model)
        self.w = dev.upload(weights)
        self.x = dev.upload(x)
        self.y = dev.upload(y)
        self.z = dev.zeros(model.zSize)
        self.dx = dev.zeros(model.zSize)
        self.grad = dev.zeros(model.pSize)
        self.probs = dev.zeros(self.classes * batch)
        self.errors = dev.zeros(max(self.classes * batch, model.maxDeltaSize))
        need = 2 * model.maxDeltaSize + max(L.cnn.cnnForwardMemRequired(C.byref(model)),
                                            L.cnn.cnnBackwardMemRequired(C.byref(model))) + 1024
        self.arena = dev.zeros(need)
        self.arena_reals = need
        self.data = DEVICE_DATASET()
        self.data.weights = self.w.value
        self.data.currentBatch = self.x.value
        self.data.sampledTrainY = self.y.value
        self.data.numClasses = self.classes
        c, h, w = input_dims(model)
        self.data.features = c * h * w
        self.data.height, self.data.width = h, w
        self.scratch = SCRATCH_AREA()
        self.scratch.devWorkspace = self.arena.value
        self.scratch.nextDevPtr = self.arena.value

    def forward(self, mode=10):
        return L.cnn.cnnForward(C.byref(self.model), C.byref(self.data), C.byref(self.scratch), self.z, self.probs,
                                self.errors, 0, self.batch, mode)

    def backward(self):
        """cnnBackward on a copy of errors (delta buffers are clobbered)."""
        m = self.model
        delta = self.arena
        delta_new = at(self.arena, m.maxDeltaSize)
        ws = at(self.arena, 2 * m.maxDeltaSize)
        L.check(L.hip.fitre_hip_copy_d2d(delta, self.errors, 4 * self.classes * self.batch), "d2d")
        L.cnn.cnnBackward(C.byref(m), C.byref(self.data), ws, self.z, self.grad, self.dx, delta, delta_new, 0,
                          self.batch, None)

    def gradient(self, weight_decay=0.0):
        return L.cnn.computeCNNGradient(C.byref(self.model), C.byref(self.data), C.byref(self.scratch), self.z, self.dx,
                                        self.probs, self.errors, self.grad, 0, self.batch, weight_decay)

    def get(self, name, n=None):
        m = self.model
        sizes = dict(z=m.zSize, dx=m.zSize, grad=m.pSize, probs=self.classes * self.batch,
                     errors=self.classes * self.batch)
        return self.dev.download(getattr(self, name), sizes[name] if n is None else n)

    def release(self):
        for p in (self.w, self.x, self.y, self.z, self.dx, self.grad, self.probs, self.errors, self.arena):
            self.dev.free(p)


def conv_shape(samples, cin, cout, in_a, in_b, k, stride, pad):
    s = fitre_conv_shape()
    s.samples, s.inChannels, s.outChannels = samples, cin, cout
    s.inA, s.inB = in_a, in_b
    s.outA = (in_a + 2 * pad - k) // stride + 1
    s.outB = (in_b + 2 * pad - k) // stride + 1
    s.ksize, s.stride, s.padding = k, stride, pad
    return s
