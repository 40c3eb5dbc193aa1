"""TimeEncoder with the constructor, parameters and state_dict keys of the
reference's starrygl/nn/model/time_encoder.py:7-31; forward runs the fused
cos(w*dt + b) kernel of libsgl_hot.so."""
import math

import numpy as np
import torch
import torch.nn as nn

from ...lib import _abi, hot_path


class _TimeEncode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, t, weight, bias):
        hp = hot_path(weight.device)
        if t.dtype == torch.int64:
            dt, code = t.reshape(-1).contiguous(), _abi.DT_I64
        else:
            dt, code = t.reshape(-1).float().contiguous(), _abi.DT_F32
        w = weight.detach().reshape(-1).contiguous()
        b = bias.detach().contiguous()
        dt = dt.to(weight.device)          # the copy the kernel read is the one backward multiplies with
        out = hp.time_encode(dt, w, b, dt_dtype=code)
        ctx.save_for_backward(dt, weight, bias)
        ctx.t_shape, ctx.t_device, ctx.t_dtype = t.shape, t.device, t.dtype
        return out

    @staticmethod
    def backward(ctx, grad):
        # d cos(a)/da = -sin(a), a = w * x + b
        dt, weight, bias = ctx.saved_tensors
        x = dt.float().reshape(-1, 1)
        a = x * weight.reshape(1, -1) + bias.reshape(1, -1)
        g = -torch.sin(a) * grad
        gw = (g * x).sum(0).reshape(weight.shape) if ctx.needs_input_grad[1] else None
        gb = g.sum(0) if ctx.needs_input_grad[2] else None
        gt = None
        if ctx.needs_input_grad[0]:        # a floating-point t: d/dt cos(w t + b) summed over the frequencies
            gt = (g * weight.reshape(1, -1)).sum(1).reshape(ctx.t_shape).to(device=ctx.t_device, dtype=ctx.t_dtype)
        return gt, gw, gb


class TimeEncoder(nn.Module):
    """cos(w * t + b) over `dimension` frequencies; w = 1 / 10^linspace(0, 9, dim)
    (or 1 / alpha^linspace(0, dim/beta, dim) with frozen parameters), b = 0."""

    def __init__(self, dimension, alpha=None, beta=None, parameter_requires_grad: bool = True):
        super().__init__()
        self.dimension = dimension
        self.w = nn.Linear(1, dimension)
        if not parameter_requires_grad:
            alpha = math.sqrt(dimension) if alpha is None else alpha
            beta = math.sqrt(dimension) if beta is None else beta
            freq = 1.0 / alpha ** np.linspace(0, dimension / beta, dimension, dtype=np.float32)
        else:
            freq = 1.0 / 10 ** np.linspace(0, 9, dimension, dtype=np.float32)
        self.w.weight = nn.Parameter(torch.from_numpy(freq.astype(np.float32)).reshape(dimension, -1),
                                     requires_grad=parameter_requires_grad)
        self.w.bias = nn.Parameter(torch.zeros(dimension), requires_grad=parameter_requires_grad)

    def forward(self, t):
        if not self.w.weight.is_cuda:
            raise RuntimeError("TimeEncoder runs on a HIP device: move the module to the GPU first")
        return _TimeEncode.apply(t, self.w.weight, self.w.bias)
