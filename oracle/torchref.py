"""float64 autograd model of the textbook layers, driven by a CNN_MODEL record.

This is the library-routine check of the oracle: torch's conv2d / batch_norm /
max_pool2d / linear / cross_entropy and their autograd, fed through converters
between the reference's flat layouts and torch's NCHW / (out, in) layouts:

  activations  [C][N][W][H] (H fastest)      <->  x.permute(1, 0, 3, 2)
  conv weights [Cout][Cin][kw][kh]           <->  weight.permute(0, 1, 3, 2)
  FC weights   column-major out x in          <->  weight.t()

(layout evidence: functions/dev_image.cu:24-48, functions/eval_gradient.cu:63-67,
pytorch/testing/readWeights.py:4-41 of the reference)
"""
import numpy as np
import torch
import torch.nn.functional as F

from fitre_amd.structs import (ACT_LINEAR, ACT_LOGISTIC, ACT_TANH, AVG_POOL, CNN_ACT_ELU, CNN_ACT_NONE, CNN_ACT_RELU,
                               CNN_ACT_SOFTPLUS, CNN_ACT_SWISH, MAX_POOL, NO_POOL, PERFORM_NO_BATCH_NORM)

torch.set_grad_enabled(True)


def act_torch(code, x):
    if code == CNN_ACT_RELU:
        return torch.relu(x)
    if code == CNN_ACT_SWISH:
        return x * torch.sigmoid(x)
    if code == CNN_ACT_SOFTPLUS:
        return F.softplus(x, threshold=20.0)
    if code == CNN_ACT_ELU:
        return F.elu(x)
    if code == ACT_LOGISTIC:
        return torch.sigmoid(x)
    if code == ACT_TANH:
        return torch.tanh(x)
    if code in (CNN_ACT_NONE, ACT_LINEAR):
        return x
    raise ValueError(code)


def to_nchw(flat, C, N, W, H, dtype=torch.float64):
    return torch.tensor(np.asarray(flat, dtype=np.float64).reshape(C, N, W, H), dtype=dtype).permute(1, 0, 3, 2).contiguous()


def from_nchw(t):
    return t.detach().permute(1, 0, 3, 2).contiguous().numpy().reshape(-1)


def unpack(model, wflat, dtype=torch.float64):
    """Returns (conv list of (W, b), fc list of (W, b)) as leaf tensors requiring grad."""
    wflat = np.asarray(wflat, dtype=np.float64)
    convs, fcs = [], []
    for l in range(model.cLayers):
        c = model.convLayer[l]
        n = c.outChannels * c.inChannels * c.kSize * c.kSize
        W = torch.tensor(wflat[model.wOffsets[l]:model.wOffsets[l] + n].reshape(c.outChannels, c.inChannels, c.kSize, c.kSize),
                         dtype=dtype).permute(0, 1, 3, 2).contiguous().requires_grad_(True)
        b = None
        if model.bias:
            b = torch.tensor(wflat[model.bOffsets[l]:model.bOffsets[l] + c.outChannels], dtype=dtype).requires_grad_(True)
        convs.append((W, b))
    for f in range(model.lLayers):
        fc = model.fcLayer[f]
        l = model.cLayers + f
        n = fc.in_ * fc.out
        W = torch.tensor(wflat[model.wOffsets[l]:model.wOffsets[l] + n].reshape(fc.in_, fc.out), dtype=dtype).t().contiguous().requires_grad_(True)
        b = None
        if model.bias:
            b = torch.tensor(wflat[model.bOffsets[l]:model.bOffsets[l] + fc.out], dtype=dtype).requires_grad_(True)
        fcs.append((W, b))
    return convs, fcs


def pack_grads(model, convs, fcs):
    g = np.zeros(model.pSize, dtype=np.float64)
    for l, (W, b) in enumerate(convs):
        gw = W.grad.permute(0, 1, 3, 2).contiguous().numpy().reshape(-1)
        g[model.wOffsets[l]:model.wOffsets[l] + gw.size] = gw
        if b is not None:
            g[model.bOffsets[l]:model.bOffsets[l] + b.numel()] = b.grad.numpy()
    for f, (W, b) in enumerate(fcs):
        l = model.cLayers + f
        gw = W.grad.t().contiguous().numpy().reshape(-1)
        g[model.wOffsets[l]:model.wOffsets[l] + gw.size] = gw
        if b is not None:
            g[model.bOffsets[l]:model.bOffsets[l] + b.numel()] = b.grad.numpy()
    return g


def run(model, wflat, x_flat, y, batch, dtype=torch.float64, want_intermediates=True):
    """Forward + backward.  Returns dict(loss, gradient, stages) where stages[l] holds, for conv
    layer l, the tensors conv / bn / act / pool and their gradients in the reference layout."""
    convs, fcs = unpack(model, wflat, dtype)
    c0 = model.convLayer[0]
    h = to_nchw(x_flat, c0.inChannels, batch, c0.width, c0.height, dtype)
    stages = []
    for l in range(model.cLayers):
        c, p = model.convLayer[l], model.poolLayer[l]
        W, b = convs[l]
        st = {}
        conv = F.conv2d(h, W, b, stride=c.stride, padding=c.padding)
        st["conv"] = conv
        pre = conv
        if c.batchNorm != PERFORM_NO_BATCH_NORM:
            pre = F.batch_norm(conv, None, None, training=True, eps=1e-5)
            st["bn"] = pre
        act = act_torch(model.actFuns[l], pre)
        st["act"] = act
        h = act
        if p.type == MAX_POOL:
            h = F.max_pool2d(act, p.pSize, p.stride, p.padding)
            st["pool"] = h
        elif p.type == AVG_POOL:
            h = F.avg_pool2d(act, p.pSize, p.stride, p.padding, count_include_pad=True)
            st["pool"] = h
        if want_intermediates:
            for t in st.values():
                t.retain_grad()
        stages.append(st)
    h = h.reshape(batch, -1)
    fc_stages = []
    for f in range(model.lLayers):
        W, b = fcs[f]
        pre = F.linear(h, W, b)
        h = act_torch(model.fcLayer[f].actFun, pre)
        if want_intermediates:
            pre.retain_grad()
        fc_stages.append(dict(pre=pre, out=h))
    target = torch.tensor(np.asarray(y, dtype=np.int64) - 1)
    loss = F.cross_entropy(h, target)
    loss.backward()
    return dict(loss=loss.item(), gradient=pack_grads(model, convs, fcs), stages=stages, fc_stages=fc_stages,
                logits=h.detach().numpy())


def forward_loss(model, convs, fcs, x_flat, y, batch, dtype=torch.float64):
    c0 = model.convLayer[0]
    h = to_nchw(x_flat, c0.inChannels, batch, c0.width, c0.height, dtype)
    for l in range(model.cLayers):
        c, p = model.convLayer[l], model.poolLayer[l]
        W, b = convs[l]
        pre = F.conv2d(h, W, b, stride=c.stride, padding=c.padding)
        if c.batchNorm != PERFORM_NO_BATCH_NORM:
            pre = F.batch_norm(pre, None, None, training=True, eps=1e-5)
        h = act_torch(model.actFuns[l], pre)
        if p.type == MAX_POOL:
            h = F.max_pool2d(h, p.pSize, p.stride, p.padding)
        elif p.type == AVG_POOL:
            h = F.avg_pool2d(h, p.pSize, p.stride, p.padding, count_include_pad=True)
    h = h.reshape(batch, -1)
    for f in range(model.lLayers):
        W, b = fcs[f]
        h = act_torch(model.fcLayer[f].actFun, F.linear(h, W, b))
    return F.cross_entropy(h, torch.tensor(np.asarray(y, dtype=np.int64) - 1))


def time_gradient(model, wflat, x_flat, y, batch, dtype=torch.float32, warmup=3, repeats=10):
    """Wall time of the autograd gradient on the host cores, the way pytorch/gradtest times its models
    (alexnet_cifar.py:48-62 forward, :88-101 loss.backward()): `warmup` untimed passes, then `repeats` timed
    ones; returns the medians in seconds of forward + backward and of backward alone (loss.backward() with the
    forward pass done beforehand)."""
    import time
    convs, fcs = unpack(model, wflat, dtype)
    params = [t for pair in convs + fcs for t in pair if t is not None]
    x_flat = np.asarray(x_flat, dtype=np.float64)
    both, back = [], []
    for i in range(warmup + repeats):
        for t in params:
            t.grad = None
        t0 = time.perf_counter()
        loss = forward_loss(model, convs, fcs, x_flat, y, batch, dtype)
        t1 = time.perf_counter()
        loss.backward()
        t2 = time.perf_counter()
        if i >= warmup:
            both.append(t2 - t0)
            back.append(t2 - t1)
    return float(np.median(both)), float(np.median(back))


def hessian_vector(model, wflat, x_flat, y, batch, vflat):
    """H * v of the mean cross-entropy loss by double backward, in the flat parameter layout."""
    convs, fcs = unpack(model, wflat)
    vconvs, vfcs = unpack(model, vflat)
    params = [t for pair in convs + fcs for t in pair if t is not None]
    vs = [t.detach() for pair in vconvs + vfcs for t in pair if t is not None]
    loss = forward_loss(model, convs, fcs, x_flat, y, batch)
    grads = torch.autograd.grad(loss, params, create_graph=True)
    dot = sum((g * v).sum() for g, v in zip(grads, vs))
    hv = torch.autograd.grad(dot, params, allow_unused=True)
    it = iter(hv)
    for pair in convs + fcs:
        for t in pair:
            if t is not None:
                g = next(it)
                t.grad = torch.zeros_like(t) if g is None else g
    return pack_grads(model, convs, fcs)
