"""Hessian-vector product (R-operator passes): the oracle against float64 double backward, symmetry and the
second-order Taylor remainder (CPU), and the HIP path against the oracle through the C boundary (GPU)."""
import ctypes as C

import numpy as np
import pytest

import torchref
from fitre_amd.structs import (ACT_TANH, AVG_POOL, CNN_ACT_NONE, CNN_ACT_RELU, CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, MAX_POOL)
from helpers import batch_inputs, build_custom, he_weights, rel_err


def models():
    yield "swish_maxpool_fc", build_custom(6, 8, 8, 2, [dict(cout=4, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_SWISH),
                                                        dict(cout=5, k=3, pad=1, pool=(MAX_POOL, 2, 2, 0), act=CNN_ACT_SWISH)],
                                           [(7, CNN_ACT_SWISH), (4, CNN_ACT_NONE)]), 6
    yield "bn_softplus_avgpool", build_custom(5, 6, 6, 3, [dict(cout=4, k=3, pad=1, pool=(AVG_POOL, 2, 2, 0), bn=True, act=CNN_ACT_SOFTPLUS),
                                                           dict(cout=3, k=3, pad=1, pool=None, bn=True, act=CNN_ACT_SWISH)],
                                              [(5, CNN_ACT_NONE)]), 5
    yield "bn_relu_maxpool", build_custom(7, 8, 8, 1, [dict(cout=3, k=5, pad=2, pool=(MAX_POOL, 2, 2, 0), bn=True, act=CNN_ACT_RELU),
                                                       dict(cout=4, k=3, pad=0, pool=None, bn=False, act=CNN_ACT_SWISH)],
                                          [(6, ACT_TANH), (3, CNN_ACT_NONE)]), 7
    yield "no_bias_unpooled_last", build_custom(4, 5, 5, 2, [dict(cout=3, k=3, pad=1, pool=None, act=CNN_ACT_SWISH)],
                                                [(3, CNN_ACT_NONE)], bias=0), 4


MODELS = {name: (m, b) for name, m, b in models()}


def setup(name, rng):
    model, batch = MODELS[name]
    w = he_weights(model, rng) * 1.5
    x, y = batch_inputs(model, batch, rng)
    v = rng.standard_normal(model.pSize)
    return model, batch, w, x, y, v


def classes_of(model):
    return model.fcLayer[model.lLayers - 1].out


@pytest.mark.parametrize("name", list(MODELS))
def test_oracle_hv_against_double_backward(oracle64, name):
    rng = np.random.default_rng(sum(map(ord, name)))
    model, batch, w, x, y, v = setup(name, rng)
    k = classes_of(model)
    ref = oracle64.gradient(model, w, x, y, k, batch)
    hv = oracle64.hessian_vector(model, w, x, ref["z"], ref["probs"], ref["errors"], ref["dx"], v, k, batch)
    want = torchref.hessian_vector(model, w, x, y, batch, v)
    assert rel_err(hv, want) < 1e-8, name


@pytest.mark.parametrize("name", ["swish_maxpool_fc", "bn_softplus_avgpool"])
def test_oracle_hv_symmetry_and_taylor(oracle64, name):
    rng = np.random.default_rng(7)
    model, batch, w, x, y, v = setup(name, rng)
    k = classes_of(model)
    u = rng.standard_normal(model.pSize)
    ref = oracle64.gradient(model, w, x, y, k, batch)
    args = (model, w, x, ref["z"], ref["probs"], ref["errors"], ref["dx"])
    hv, hu = oracle64.hessian_vector(*args, v, k, batch), oracle64.hessian_vector(*args, u, k, batch)
    assert abs(u @ hv - v @ hu) < 1e-9 * max(1.0, abs(u @ hv))
    if name == "bn_softplus_avgpool":   # smooth everywhere: the remainder of the quadratic model decays like t^3
        g, f0 = ref["gradient"], ref["loss"]
        d = v / np.linalg.norm(v)
        hd = oracle64.hessian_vector(*args, d, k, batch)
        rem = []
        for t in (1e-2, 5e-3, 2.5e-3):
            ft = oracle64.gradient(model, w + t * d, x, y, k, batch)["loss"]
            rem.append(abs(ft - f0 - t * (g @ d) - 0.5 * t * t * (d @ hd)))
        assert rem[0] / rem[1] > 6 and rem[1] / rem[2] > 6, rem   # 8 for an exact Hessian, 4 for a wrong one
