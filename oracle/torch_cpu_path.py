"""TEST INFRASTRUCTURE ONLY -- the reference's CPU algorithm for quaternion Conv2D with the scalar
convolutions supplied by oneDNN as embedded in PyTorch's CPU backend.

The reference's CPU backend runs 8 (factorized, default) or 16 (memory-optimized) scalar oneDNN
convolutions plus elementwise lane passes (src/conv2d.hpp:167-275, 433-562;
src/backend/onednn/tensor.hpp:61-170).  Its own binary cannot be built here (oneDNN is an empty
submodule), so this module restates that algorithm step for step -- same lanes, same temporaries,
same accumulate passes -- and calls torch.nn.functional.conv2d / torch.nn.grad on CPU tensors for
each scalar primitive.  Used as bench.py's cpu_baseline ("port") and cross-checked against the C
oracle in tests/test_oracle_torch_path.py.
"""
import torch
import torch.nn.functional as F
from torch.nn import grad as nn_grad

from . import product_terms, QUATERNION


def _conv(x, w, b, g):
    if g.pt != g.pb or g.pl != g.pr:
        x = F.pad(x, (g.pl, g.pr, g.pt, g.pb))
        pad = (0, 0)
    else:
        pad = (g.pt, g.pl)
    return F.conv2d(x, w, b, stride=(g.sh, g.sw), padding=pad, dilation=(g.dh, g.dw))


def _conv_bwd(x, w, gr, g, need_dx):
    if g.pt != g.pb or g.pl != g.pr:
        raise NotImplementedError("asymmetric padding is not timed on this path")
    kw = dict(stride=(g.sh, g.sw), padding=(g.pt, g.pl), dilation=(g.dh, g.dw))
    dw = nn_grad.conv2d_weight(x, w.shape, gr, **kw)
    dx = nn_grad.conv2d_input(x.shape, w, gr, **kw) if need_dx else None
    return dw, dx


def decompose_left(x):
    a, b, c, d = x
    return [d + b, a - c, a + c, d - b, d - c, b + a, a - b, d + c]


def decompose_right(w):
    a, b, c, d = w
    return [b + c, a + d, a - d, b - c, c - d, b + a, c + d, a - b]


def decompose_grad(g):
    t1, t3, t2, t4 = g[0] + g[1], g[0] - g[1], g[2] + g[3], g[2] - g[3]
    return [0.5 * (t2 - t1), 0.5 * (t3 - t4), 0.5 * (t3 + t4), 0.5 * (t1 + t2), g[0], g[1], g[2], g[3]]


def conv2d_fwd(geom, x, w, bias=None, mode="factorized"):
    """x [4n,ci,h,w], w [4,co,ci,kh,kw], bias [4,co] or None (CPU float32 tensors)."""
    n = geom.n
    xs = [x[p * n:(p + 1) * n] for p in range(4)]
    ws = [w[p] for p in range(4)]
    if mode == "factorized":
        L, R = decompose_left(xs), decompose_right(ws)
        P = [_conv(L[i], R[i], bias[i - 4] if (bias is not None and i >= 4) else None, geom) for i in range(8)]
        a2 = P[0] + P[1] + P[2]
        a5 = 0.5 * (a2 + P[3])
        return torch.cat([a5 - P[0] + P[4], a5 - a2 + P[5], a5 - P[1] + P[6], a5 - P[2] + P[7]])
    y = [None] * 4
    for left, right, dim, positive, fill in product_terms(QUATERNION):
        if fill:
            y[dim] = _conv(xs[left], ws[right], bias[dim] if bias is not None else None, geom)
        else:
            buf = _conv(xs[left], ws[right], None, geom)
            if positive:
                y[dim] += buf
            else:
                y[dim] -= buf
    return torch.cat(y)


def conv2d_bwd(geom, x, w, grad, mode="factorized", need_dx=True):
    n = geom.n
    xs = [x[p * n:(p + 1) * n] for p in range(4)]
    ws = [w[p] for p in range(4)]
    gs = [grad[p * n:(p + 1) * n] for p in range(4)]
    if mode == "factorized":
        L, R, G = decompose_left(xs), decompose_right(ws), decompose_grad(gs)
        dR, dL = zip(*[_conv_bwd(L[i], R[i], G[i], geom, need_dx) for i in range(8)])
        dw = torch.stack([dR[1] + dR[2] + dR[5] + dR[7], dR[0] + dR[3] + dR[5] - dR[7],
                          dR[0] - dR[3] + dR[4] + dR[6], dR[1] - dR[2] - dR[4] + dR[6]])
        dx = None
        if need_dx:
            dx = torch.cat([dL[1] + dL[2] + dL[5] + dL[6], dL[0] - dL[3] + dL[5] - dL[6],
                            dL[2] - dL[1] - dL[4] + dL[7], dL[0] + dL[3] + dL[4] + dL[7]])
        return dw, dx
    dws, dxs = [None] * 4, [None] * 4
    for left, right, dim, positive, fill in product_terms(QUATERNION, backprop=True):
        bw, bx = _conv_bwd(xs[left], ws[right], gs[dim], geom, need_dx)
        if fill:
            dws[right], dxs[left] = bw, bx
        elif positive:
            dws[right] += bw
            if need_dx:
                dxs[left] += bx
        else:
            dws[right] -= bw
            if need_dx:
                dxs[left] -= bx
    return torch.stack(dws), (torch.cat(dxs) if need_dx else None)


def _dense(x, w, b):
    """Scalar Dense of the CPU backend: one matmul Y[N,O] = X[N,I] . W[I,O] (+ bias)
    (src/backend/onednn/dense.hpp:53-93); torch.nn.functional.linear takes the filter as [O,I]."""
    return F.linear(x, w.t(), b)


def _dense_bwd(x, w, gr, need_dx):
    """dW = X^T . G and dX = G . W^T through transposed views (src/backend/onednn/dense.hpp:166-181, 203-210)."""
    dw = F.linear(x.t(), gr.t())
    dx = F.linear(gr, w) if need_dx else None
    return dw, dx


def dense_fwd(x, w, bias=None, mode="factorized"):
    """Quaternion Dense forward (src/dense.hpp:77-140 factorized, :143-180 generic).
    x [4n,i], w [4,i,o] (layout IO), bias [4,o] or None (CPU float32 tensors)."""
    n = x.shape[0] // 4
    xs = [x[p * n:(p + 1) * n] for p in range(4)]
    ws = [w[p] for p in range(4)]
    if mode == "factorized":
        L, R = decompose_left(xs), decompose_right(ws)
        P = [_dense(L[i], R[i], bias[i - 4] if (bias is not None and i >= 4) else None) for i in range(8)]
        a2 = P[0] + P[1] + P[2]
        a5 = 0.5 * (a2 + P[3])
        return torch.cat([a5 - P[0] + P[4], a5 - a2 + P[5], a5 - P[1] + P[6], a5 - P[2] + P[7]])
    y = [None] * 4
    for left, right, dim, positive, fill in product_terms(QUATERNION):
        if fill:
            y[dim] = _dense(xs[left], ws[right], bias[dim] if bias is not None else None)
        else:
            buf = _dense(xs[left], ws[right], None)
            if positive:
                y[dim] += buf
            else:
                y[dim] -= buf
    return torch.cat(y)


def dense_bwd(x, w, grad, mode="factorized", need_dx=True):
    """Quaternion Dense backward (src/dense.hpp:252-335 factorized, :338-377 generic): returns (dw, dx)."""
    n = x.shape[0] // 4
    xs = [x[p * n:(p + 1) * n] for p in range(4)]
    ws = [w[p] for p in range(4)]
    gs = [grad[p * n:(p + 1) * n] for p in range(4)]
    if mode == "factorized":
        L, R, G = decompose_left(xs), decompose_right(ws), decompose_grad(gs)
        dR, dL = zip(*[_dense_bwd(L[i], R[i], G[i], need_dx) for i in range(8)])
        dw = torch.stack([dR[1] + dR[2] + dR[5] + dR[7], dR[0] + dR[3] + dR[5] - dR[7],
                          dR[0] - dR[3] + dR[4] + dR[6], dR[1] - dR[2] - dR[4] + dR[6]])
        dx = None
        if need_dx:
            dx = torch.cat([dL[1] + dL[2] + dL[5] + dL[6], dL[0] - dL[3] + dL[5] - dL[6],
                            dL[2] - dL[1] - dL[4] + dL[7], dL[0] + dL[3] + dL[4] + dL[7]])
        return dw, dx
    dws, dxs = [None] * 4, [None] * 4
    for left, right, dim, positive, fill in product_terms(QUATERNION, backprop=True):
        bw, bx = _dense_bwd(xs[left], ws[right], gs[dim], need_dx)
        if fill:
            dws[right], dxs[left] = bw, bx
        elif positive:
            dws[right] += bw
            if need_dx:
                dxs[left] += bx
        else:
            dws[right] -= bw
            if need_dx:
                dxs[left] -= bx
    return torch.stack(dws), (torch.cat(dxs) if need_dx else None)
