"""ctypes front end of the CPU oracle (oracle/fitre_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py; never by the fitre_amd package.

Two builds of the same C file: float64 (`f64`, the parity checker) and float32
(`f32`, the timed CPU baseline).  Arrays are numpy arrays in the reference's
flat layouts; see the C file for the reference lines each function follows.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from fitre_amd.structs import CNN_MODEL

_DIR = os.path.dirname(os.path.abspath(__file__))


def build():
    """Compiles both oracle libraries with the Makefile next to this file."""
    subprocess.run(["make", "-s", "-C", _DIR, "all"], check=True)


class Oracle:
    def __init__(self, double=True):
        name = "libfitre_oracle_f64.so" if double else "libfitre_oracle_f32.so"
        path = os.path.join(_DIR, name)
        if not os.path.exists(path):
            build()
        self.lib = C.CDLL(path)
        self.dtype = np.float64 if double else np.float32
        self.creal = C.c_double if double else C.c_float
        assert self.lib.oracle_sizeof_real() == np.dtype(self.dtype).itemsize
        self.lib.oracle_cnn_forward.restype = self.creal
        self.lib.oracle_cnn_gradient.restype = self.creal
        self.lib.oracle_softmax_loss.restype = self.creal

    # ---- helpers -------------------------------------------------------
    def arr(self, a):
        return np.ascontiguousarray(a, dtype=self.dtype)

    def zeros(self, n):
        return np.zeros(int(n), dtype=self.dtype)

    @staticmethod
    def p(a):
        return a.ctypes.data_as(C.c_void_p)

    def r(self, v):
        return self.creal(v)

    # ---- whole model ---------------------------------------------------
    def forward(self, model: CNN_MODEL, weights, x, y, classes, batch, mode=10, z=None):
        """Returns (loss, z, probs, errors).  Pass z to carry running batch-norm statistics."""
        weights, x, y = self.arr(weights), self.arr(x), self.arr(y)
        z = self.zeros(model.zSize) if z is None else z
        probs, errors = self.zeros(classes * batch), self.zeros(classes * batch)
        loss = self.lib.oracle_cnn_forward(C.byref(model), self.p(weights), self.p(x), self.p(y), classes,
                                           self.p(z), self.p(probs), self.p(errors), batch, mode)
        return float(loss), z, probs, errors

    def backward(self, model: CNN_MODEL, weights, x, z, errors, batch):
        """Returns (gradient, dx)."""
        weights, x = self.arr(weights), self.arr(x)
        grad, dx = self.zeros(model.pSize), self.zeros(model.zSize)
        delta = self.zeros(model.maxDeltaSize)
        delta[:errors.size] = errors
        delta_new = self.zeros(model.maxDeltaSize)
        rc = self.lib.oracle_cnn_backward(C.byref(model), self.p(weights), self.p(x), self.p(z), self.p(grad),
                                          self.p(dx), self.p(delta), self.p(delta_new), batch)
        if rc != 0:
            raise ValueError("oracle_cnn_backward: unknown activation or pooling code")
        return grad, dx

    def gradient(self, model: CNN_MODEL, weights, x, y, classes, batch, weight_decay=0.0):
        """computeCNNGradient: returns dict(loss, gradient, z, dx, probs, errors)."""
        weights, x, y = self.arr(weights), self.arr(x), self.arr(y)
        z, dx = self.zeros(model.zSize), self.zeros(model.zSize)
        probs, errors = self.zeros(classes * batch), self.zeros(classes * batch)
        grad = self.zeros(model.pSize)
        loss = self.lib.oracle_cnn_gradient(C.byref(model), self.p(weights), self.p(x), self.p(y), classes,
                                            self.p(z), self.p(dx), self.p(probs), self.p(errors), self.p(grad),
                                            batch, self.r(weight_decay))
        return dict(loss=float(loss), gradient=grad, z=z, dx=dx, probs=probs, errors=errors)

    def hessian_vector(self, model: CNN_MODEL, weights, x, z, probs, errors, dx, vector, classes, batch):
        """H * vector of the mean loss at `weights` (no weight-decay term), from the z / probs / errors / dx of a
        gradient call on the same batch."""
        arrs = [self.arr(a) for a in (weights, x, z, probs, errors, dx, vector)]
        hv = self.zeros(model.pSize)
        rc = self.lib.oracle_cnn_hv(C.byref(model), self.p(arrs[0]), self.p(arrs[1]), self.p(arrs[2]), self.p(arrs[3]),
                                    self.p(arrs[4]), self.p(arrs[5]), self.p(arrs[6]), self.p(hv), batch, classes)
        if rc != 0:
            raise ValueError("oracle_cnn_hv failed (unknown activation or pool code)")
        return hv

    # ---- single operations ------------------------------------------------
    def gemm(self, ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc):
        A, B, Cm = self.arr(A), self.arr(B), self.arr(Cm).copy()
        self.lib.oracle_gemm(ta, tb, M, N, K, self.r(alpha), self.p(A), lda, self.p(B), ldb, self.r(beta),
                             self.p(Cm), ldc)
        return Cm

    def im2col(self, x, samples, channels, height, width, k, pad, stride):
        x = self.arr(x)
        hc, wc = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        col = self.zeros(hc * wc * samples * channels * k * k)
        self.lib.oracle_im2col(self.p(x), samples, channels, height, width, k, pad, stride, self.p(col))
        return col

    def conv_forward(self, x, w, bias, samples, cin, height, width, k, pad, stride, cout):
        """Convolution output only ([Cout][N][Wc][Hc])."""
        x, w = self.arr(x), self.arr(w)
        hc, wc = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        M, K = hc * wc * samples, k * k * cin
        col = self.im2col(x, samples, cin, height, width, k, pad, stride)
        out = self.gemm(0, 0, M, cout, K, 1.0, col, M, w, K, 0.0, self.zeros(M * cout), M)
        if bias is not None:
            out = (out.reshape(cout, M) + self.arr(bias)[:, None]).reshape(-1)
        return out

    def conv_weight_grad(self, x, delta, samples, cin, height, width, k, pad, stride, cout):
        x, delta = self.arr(x), self.arr(delta)
        hc, wc = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        dW = self.zeros(cout * cin * k * k)
        scratch = self.zeros(hc * wc * samples * cin * k * k)
        self.lib.oracle_conv_weight_gradient(self.p(x), self.p(delta), samples, cin, height, width, k, pad, stride,
                                             cout, self.p(dW), self.p(scratch))
        return dW

    def conv_input_grad(self, delta, w, samples, cin, height, width, k, pad, cout):
        delta, w = self.arr(delta), self.arr(w)
        dh, dw = height + 2 * pad - k + 1, width + 2 * pad - k + 1
        out = self.zeros(samples * height * width * cin)
        scratch = self.zeros(samples * height * width * k * k * cout + cout * cin * k * k)
        self.lib.oracle_conv_input_gradient(self.p(delta), dh, dw, cout, self.p(w), k, k, height, width, pad, cin,
                                            samples, self.p(out), self.p(scratch))
        return out

    # ---- KFAC factors ---------------------------------------------------
    def kfac_conv_input_factor(self, x, samples, cin, height, width, k, pad, stride, bias):
        x = self.arr(x)
        hc, wc = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        n = cin * k * k + (1 if bias else 0)
        factor = self.zeros(n * n)
        scratch = self.zeros(hc * wc * samples * n)
        self.lib.oracle_kfac_conv_input_factor(self.p(x), samples, cin, height, width, k, pad, stride, int(bool(bias)),
                                               self.p(factor), self.p(scratch))
        return factor.reshape(n, n)

    def kfac_conv_output_factor(self, delta, samples, out_height, out_width, cout):
        delta = self.arr(delta)
        factor = self.zeros(cout * cout)
        self.lib.oracle_kfac_conv_output_factor(self.p(delta), samples, out_height, out_width, cout, self.p(factor))
        return factor.reshape(cout, cout)

    def kfac_fc_input_factor(self, z, n_in, samples, bias):
        z = self.arr(z)
        n = n_in + (1 if bias else 0)
        factor = self.zeros(n * n)
        scratch = self.zeros(2 * n * samples)
        self.lib.oracle_kfac_fc_input_factor(self.p(z), n_in, samples, int(bool(bias)), self.p(factor), self.p(scratch))
        return factor.reshape(n, n)

    def kfac_fc_output_factor(self, delta, n_out, samples):
        delta = self.arr(delta)
        factor = self.zeros(n_out * n_out)
        self.lib.oracle_kfac_fc_output_factor(self.p(delta), n_out, samples, self.p(factor))
        return factor.reshape(n_out, n_out)

    def matrix_inverse(self, matrix, n, lam, gamma):
        """(info, inverse) of matrix + (lam + gamma) I."""
        matrix = self.arr(matrix)
        inverse, scratch = self.zeros(n * n), self.zeros(n * n)
        info = self.lib.oracle_matrix_inverse(self.p(matrix), self.p(inverse), n, self.r(lam), self.r(gamma), self.p(scratch))
        return info, inverse.reshape(n, n)

    def natural_gradient(self, model, omega_offsets, lambda_offsets, omega_inv, lambda_inv, vec):
        omega_inv, lambda_inv, vec = self.arr(omega_inv), self.arr(lambda_inv), self.arr(vec)
        oo = (C.c_int * len(omega_offsets))(*omega_offsets)
        lo = (C.c_int * len(lambda_offsets))(*lambda_offsets)
        out = self.zeros(model.pSize)
        big = 1
        for i in range(model.cLayers):
            c = model.convLayer[i]
            big = max(big, (c.inChannels * c.kSize ** 2 + 1) * c.outChannels)
        for i in range(model.lLayers):
            f = model.fcLayer[i]
            big = max(big, (f.in_ + 1) * f.out)
        scratch = self.zeros(3 * big)
        self.lib.oracle_natural_gradient(C.byref(model), oo, lo, self.p(omega_inv), self.p(lambda_inv), self.p(vec),
                                         self.p(out), self.p(scratch))
        return out

    def compute_accuracy(self, probs, target, rows, classes):
        probs, target = self.arr(probs), self.arr(target)
        hits = self.creal(0)
        self.lib.oracle_compute_accuracy.restype = self.creal
        pct = self.lib.oracle_compute_accuracy(self.p(probs), self.p(target), rows, classes, C.byref(hits))
        return float(pct), float(hits.value)

    def multinomial_classes(self, probs, uniforms, samples, classes):
        probs, uniforms = self.arr(probs), self.arr(uniforms)
        out = self.zeros(samples)
        self.lib.oracle_multinomial_classes(self.p(probs), samples, classes, self.p(uniforms), self.p(out))
        return out

    def uniform_stream(self, seed, first, n):
        out = np.zeros(int(n), dtype=np.float32)
        self.lib.oracle_uniform_stream(C.c_ulonglong(seed), C.c_ulonglong(first), C.c_long(n), self.p(out))
        return out

    # ---- fully connected model family -----------------------------------
    def nn_gradient(self, model, weights, dataset, target, n):
        """(ll, model_error, gradient, z, dx) for an NN_MODEL whose z / rZ offsets were built for n points."""
        weights, dataset, target = self.arr(weights), self.arr(dataset), self.arr(target)
        big = max(model.layerSizes[i] for i in range(model.numLayers + 1)) * n
        z, dx, grad = self.zeros(model.zSize + big), self.zeros(model.rFullSize + big), self.zeros(model.pSize)
        err, scratch = self.zeros(big), self.zeros(big)
        merr = self.creal(0)
        self.lib.oracle_nn_gradient.restype = self.creal
        ll = self.lib.oracle_nn_gradient(C.byref(model), self.p(weights), self.p(dataset), self.p(target), n, model.zOffsets,
                                         model.rZOffsets, self.p(z), self.p(dx), self.p(grad), C.byref(merr), self.p(err),
                                         self.p(scratch))
        return float(ll), float(merr.value), grad, z[:model.zSize], dx[:model.rFullSize]

    def nn_hessian_vec(self, model, weights, vec, dataset, n, z, dx, gauss_newton=False, top_layer_term=True):
        """Hessian (or Gauss-Newton) times vec for an NN_MODEL, from z and dx of nn_gradient at the same point."""
        weights, vec, dataset, z, dx = (self.arr(a) for a in (weights, vec, dataset, z, dx))
        out = self.zeros(model.pSize)
        rc = self.lib.oracle_nn_hessian_vec(C.byref(model), self.p(weights), self.p(vec), self.p(dataset), n, model.zOffsets,
                                            model.rZOffsets, self.p(z), self.p(dx), int(gauss_newton), int(top_layer_term),
                                            self.p(out))
        if rc:
            raise ValueError("unsupported head or activation")
        return out

    def nn_forward(self, model, weights, dataset, target, n_cols, n_cols_target):
        weights, dataset, target = self.arr(weights), self.arr(dataset), self.arr(target)
        big = max(model.layerSizes[i] for i in range(model.numLayers + 1)) * max(n_cols, n_cols_target)
        z, err, scratch = self.zeros(model.zSize + big), self.zeros(big), self.zeros(big)
        merr = self.creal(0)
        self.lib.oracle_nn_forward.restype = self.creal
        ll = self.lib.oracle_nn_forward(C.byref(model), self.p(weights), self.p(dataset), self.p(target), n_cols,
                                        n_cols_target, model.zOffsets, self.p(z), self.p(err), C.byref(merr), self.p(scratch))
        return float(ll), float(merr.value), z[:model.zSize], err[:model.layerSizes[model.numLayers] * n_cols_target]

    def activation_forward(self, act, x):
        x = self.arr(x).copy()
        rc = self.lib.oracle_activation_forward(act, self.p(x), C.c_size_t(x.size))
        if rc:
            raise ValueError("unknown activation %d" % act)
        return x

    def activation_backward(self, act, delta, z_in, z_out):
        d = self.arr(delta).copy()
        z_in, z_out = self.arr(z_in), self.arr(z_out)
        rc = self.lib.oracle_activation_backward(act, self.p(d), self.p(z_in), self.p(z_out), C.c_size_t(d.size))
        if rc:
            raise ValueError("unknown activation %d" % act)
        return d

    def pool_forward(self, kind, x, samples, channels, height, width, k, stride, pad):
        x = self.arr(x)
        ph, pw = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        out = self.zeros(ph * pw * samples * channels)
        fn = self.lib.oracle_max_pool_forward if kind == 0 else self.lib.oracle_avg_pool_forward
        fn(self.p(x), samples, channels, height, width, k, stride, pad, ph, pw, self.p(out))
        return out

    def max_pool_argmax(self, x, samples, channels, height, width, k, stride, pad):
        x = self.arr(x)
        ph, pw = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        idx = np.zeros(ph * pw * samples * channels, dtype=np.int32)
        self.lib.oracle_max_pool_argmax(self.p(x), samples, channels, height, width, k, stride, pad, ph, pw,
                                        idx.ctypes.data_as(C.c_void_p))
        return idx

    def pool_backward(self, kind, delta, z_in, samples, channels, height, width, k, stride, pad):
        delta = self.arr(delta)
        ph, pw = (height + 2 * pad - k) // stride + 1, (width + 2 * pad - k) // stride + 1
        out = self.zeros(height * width * samples * channels)
        if kind == 0:
            z_in = self.arr(z_in)
            self.lib.oracle_max_pool_backward(self.p(delta), self.p(z_in), channels, height, width, k, stride, pad,
                                              ph, pw, samples, self.p(out))
        else:
            self.lib.oracle_avg_pool_backward(self.p(delta), channels, height, width, k, stride, pad, ph, pw,
                                              samples, self.p(out))
        return out

    def batch_norm_forward(self, x, height, width, channels, samples, eps=1e-5, train=True, momentum=0.9,
                           running=None):
        """Returns (zhat, mean, var, running_mean, running_var)."""
        x = self.arr(x)
        n = height * width * samples * channels
        out = self.zeros(n + 4 * channels)
        if running is not None:
            out[n + 2 * channels:n + 3 * channels] = running[0]
            out[n + 3 * channels:] = running[1]
        self.lib.oracle_batch_norm_forward(self.p(x), height, width, channels, samples, self.p(out), n, n + channels,
                                           self.r(eps), 10 if train else 20, self.r(momentum), n + 2 * channels,
                                           n + 3 * channels)
        c = channels
        return out[:n], out[n:n + c], out[n + c:n + 2 * c], out[n + 2 * c:n + 3 * c], out[n + 3 * c:]

    def batch_norm_backward(self, delta, zhat, variance, height, width, channels, samples, eps=1e-5):
        delta, zhat, variance = self.arr(delta), self.arr(zhat), self.arr(variance)
        out = self.zeros(delta.size)
        self.lib.oracle_batch_norm_backward(self.p(delta), height, width, channels, samples, self.p(variance),
                                            self.p(out), self.p(zhat), self.r(eps))
        return out

    def softmax_loss(self, logits, target, rows, classes):
        logits, target = self.arr(logits), self.arr(target)
        probs = self.zeros(rows * classes)
        loss = self.lib.oracle_softmax_loss(self.p(logits), self.p(target), rows, classes, self.p(probs))
        return float(loss), probs

    def cross_entropy_error(self, probs, target, rows, classes):
        probs, target = self.arr(probs), self.arr(target)
        err = self.zeros(rows * classes)
        self.lib.oracle_cross_entropy_error(self.p(probs), rows, classes, self.p(target), self.p(err))
        return err

    def reshape(self, x, right, left, chunk):
        x = self.arr(x)
        out = self.zeros(x.size)
        self.lib.oracle_reshape(self.p(x), right, left, chunk, self.p(out))
        return out

    def transpose(self, x, maps, height, width, rc=False):
        x = self.arr(x)
        out = self.zeros(x.size)
        (self.lib.oracle_transpose_rc if rc else self.lib.oracle_transpose)(self.p(x), maps, height, width, self.p(out))
        return out

    # ---- input pipeline
    def extract_columns(self, src, indices, rows):
        src = self.arr(src)
        idx = np.ascontiguousarray(indices, dtype=np.int32)
        out = self.zeros(rows * idx.size)
        self.lib.oracle_extract_columns(self.p(out), self.p(src), idx.ctypes.data_as(C.c_void_p), rows, C.c_long(rows * idx.size))
        return out

    def crop_shifts(self, uniforms, samples, padding):
        u = self.arr(uniforms)
        out = np.zeros(2 * samples, dtype=np.int32)
        self.lib.oracle_crop_shifts(self.p(u), samples, padding, out.ctypes.data_as(C.c_void_p))
        return out

    def random_crop(self, x, samples, height, width, channels, shift_row, shift_col, default=0.0):
        x = self.arr(x)
        sr = np.ascontiguousarray(shift_row, dtype=np.int32)
        sc = np.ascontiguousarray(shift_col, dtype=np.int32)
        out = self.zeros(x.size)
        self.lib.oracle_random_crop(self.p(x), samples, height, width, channels, sr.ctypes.data_as(C.c_void_p),
                                    sc.ctypes.data_as(C.c_void_p), self.r(default), self.p(out))
        return out

    def random_flip(self, x, samples, channels, height, width, probs):
        x, probs = self.arr(x), self.arr(probs)
        out = self.zeros(x.size)
        self.lib.oracle_random_flip(self.p(x), samples, channels, height, width, self.p(probs), self.p(out))
        return out

    def normalize(self, x, samples, height, width, channels, means, std, scale=255.0):
        x = self.arr(x).copy()
        means, std = self.arr(means), self.arr(std)
        self.lib.oracle_normalize(self.p(x), samples, height, width, channels, self.p(means), self.p(std), self.r(scale))
        return x

    def augment_data(self, sampled, samples, channels, height, width, enable, crop_uniforms, flip_uniforms, means, std):
        sampled = self.arr(sampled)
        cu, fu, means, std = self.arr(crop_uniforms), self.arr(flip_uniforms), self.arr(means), self.arr(std)
        scratch, out = self.zeros(sampled.size), self.zeros(sampled.size)
        self.lib.oracle_augment_data(self.p(sampled), samples, channels, height, width, int(enable), self.p(cu), self.p(fu),
                                     self.p(means), self.p(std), self.p(scratch), self.p(out))
        return out
