"""Oracle for the local convolution on the halo-padded tile: forward, dgrad,
wgrad and bias gradient, through the same torch CPU operators the reference
calls. Test infrastructure only."""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch.nn import grad as G

_CONV = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}
_CONV_INPUT = {1: G.conv1d_input, 2: G.conv2d_input, 3: G.conv3d_input}
_CONV_WEIGHT = {1: G.conv1d_weight, 2: G.conv2d_weight, 3: G.conv3d_weight}


def forward(x_aug, w, b, stride, local_padding, dilation, groups=1):
    """Local conv on the padded tile (jigsaw/modules/convolution/_conv/channel_comm.py:155-158;
    primitive table config.py:27, 82-83). ``local_padding`` is zero on split axes
    (_common/spatial_split.py:75-82)."""
    n = w.dim() - 2
    return _CONV[n](x_aug, w, b, stride=stride, padding=local_padding, dilation=dilation, groups=groups)


def dgrad(x_aug_shape, w, g, stride, local_padding, dilation, groups=1):
    """Gradient w.r.t. the PADDED tile (distributed.py:346-355)."""
    n = w.dim() - 2
    return _CONV_INPUT[n](x_aug_shape, w, g.to(w.dtype), stride=stride, padding=local_padding, dilation=dilation, groups=groups)


def wgrad(x_aug, w_shape, g, stride, local_padding, dilation, groups=1):
    """Gradient w.r.t. the weight (distributed.py:359-368)."""
    n = len(w_shape) - 2
    return _CONV_WEIGHT[n](x_aug, w_shape, g.to(x_aug.dtype), stride=stride, padding=local_padding, dilation=dilation, groups=groups)


def grad_bias(g, n_spatial):
    """Sum over batch and spatial axes (config.py:117-120)."""
    return g.sum(dim=(-(n_spatial + 2), *range(-n_spatial, 0)))


def brute_forward(x, w, b, stride, padding, dilation):
    """Direct 7-loop convolution for tiny shapes (pins the torch operator choice and
    argument order; cross-correlation, zero padding, NCHW / OIHW)."""
    n, cin, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho = (h + 2 * padding[0] - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    wo = (wd + 2 * padding[1] - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    y = torch.zeros(n, cout, ho, wo, dtype=torch.float64)
    for ni in range(n):
        for co in range(cout):
            for i in range(ho):
                for j in range(wo):
                    acc = float(b[co]) if b is not None else 0.0
                    for ci in range(cin):
                        for a in range(kh):
                            for c in range(kw):
                                ii = i * stride[0] - padding[0] + a * dilation[0]
                                jj = j * stride[1] - padding[1] + c * dilation[1]
                                if 0 <= ii < h and 0 <= jj < wd:
                                    acc += float(x[ni, ci, ii, jj]) * float(w[co, ci, a, c])
                    y[ni, co, i, j] = acc
    return y
