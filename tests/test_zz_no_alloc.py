"""fitre_hip_batch_norm_backward_static: the batch-norm backward step with its partial sums in the library's static
device array (no workspace argument, no allocation) against fitre_hip_batch_norm_backward on the same inputs —
bit for bit, on two calls in a row, the second with a smaller input (the array keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

from fitre_amd import lib as L

pytestmark = pytest.mark.gpu
hip = L.hip

STATIC_BYTES = 1 << 20   # FITRE_HIP_STATIC_SCRATCH_BYTES of include/fitre_hip.h


def both(dev, channels, per, seed, with_bias=True):
    rng = np.random.default_rng(seed)
    n = channels * per
    delta = dev.upload(rng.standard_normal(n).astype(np.float32))
    zhat = dev.upload(rng.standard_normal(n).astype(np.float32))
    var = dev.upload(rng.uniform(0.5, 2.0, channels).astype(np.float32))
    out_ws, out_st = dev.upload(np.full(n, np.nan, np.float32)), dev.upload(np.full(n, np.nan, np.float32))
    bias_ws, bias_st = dev.upload(np.full(channels, np.nan, np.float32)), dev.upload(np.full(channels, np.nan, np.float32))
    nb = hip.fitre_hip_batch_norm_workspace(channels, per)
    assert nb <= STATIC_BYTES
    ws = dev.alloc(nb)
    L.check(hip.fitre_hip_batch_norm_backward(delta, zhat, var, channels, per, 1e-5, out_ws, bias_ws if with_bias else None, ws, nb))
    L.check(hip.fitre_hip_batch_norm_backward_static(delta, zhat, var, channels, per, 1e-5, out_st, bias_st if with_bias else None))
    dev.sync()
    a, b = dev.download(out_ws, n), dev.download(out_st, n)
    assert np.isfinite(a).all()
    np.testing.assert_array_equal(a, b)
    if with_bias:
        np.testing.assert_array_equal(dev.download(bias_ws, channels), dev.download(bias_st, channels))
    for q in (delta, zhat, var, out_ws, out_st, bias_ws, bias_st, ws):
        dev.free(q)


def test_static_scratch_entry_point_matches_the_workspace_one(dev):
    both(dev, 64, 256 * 32 * 32 // 4, seed=1)          # segmented path: 32 segments per channel
    both(dev, 16, 4096 + 37, seed=2, with_bias=False)  # smaller, ragged, right after: stale sums of call 1 in the array
    both(dev, 256, 1024, seed=3)                       # one workgroup per channel (no partial sums at all)
    both(dev, 3, 5, seed=4)


def _free_bytes():
    free = C.c_size_t(0)
    L.check(hip.fitre_hip_device_info(None, None, None, None, C.byref(free), None, 0))
    return free.value


def test_static_scratch_entry_point_allocates_nothing(dev):
    """The device's free memory is the same before and after calls of the entry point (segmented and single-workgroup
    shapes), with every buffer of the test allocated beforehand; the workspace entry point's partial sums stay out of it."""
    channels, per = 64, 65536
    n = channels * per
    rng = np.random.default_rng(9)
    delta, zhat = dev.upload(rng.standard_normal(n).astype(np.float32)), dev.upload(rng.standard_normal(n).astype(np.float32))
    var, out, bias = dev.upload(rng.uniform(0.5, 2.0, channels).astype(np.float32)), dev.zeros(n), dev.zeros(channels)
    L.check(hip.fitre_hip_batch_norm_backward_static(delta, zhat, var, channels, per, 1e-5, out, bias))   # first call on the device
    dev.sync()
    before = _free_bytes()
    for c, p in ((channels, per), (16, 4133), (channels, 1024)):
        L.check(hip.fitre_hip_batch_norm_backward_static(delta, zhat, var, c, p, 1e-5, out, bias))
    dev.sync()
    assert _free_bytes() == before
    for q in (delta, zhat, var, out, bias):
        dev.free(q)


def test_static_scratch_entry_point_rejects_what_does_not_fit(dev):
    channels, per = 20000, 8                           # 20000 slots of 64 bytes > 1 MiB
    assert hip.fitre_hip_batch_norm_workspace(channels, per) > STATIC_BYTES
    p = dev.zeros(channels * per)
    v = dev.zeros(channels)
    rc = hip.fitre_hip_batch_norm_backward_static(p, p, v, channels, per, 1e-5, p, None)
    assert rc == 4 and b"static" in hip.fitre_hip_last_error()
    assert hip.fitre_hip_batch_norm_backward_static(None, p, v, 4, 8, 1e-5, p, None) == 2
    dev.free(p)
    dev.free(v)
