"""RMSNorm, fused with the addition into the residual stream.

Formula as the reference computes it (/root/reference/src/models/norm.cpp:30-62,
CUDA form /root/reference/src/cuda/ops/self_attn_detail.cuh:385-418):
ss = sum_j x_j^2 in float32, inv = 1 / sqrt(ss / H + eps), y_j = x_j * inv * w_j.
The reference fixes eps = 1e-6 in code (norm.cpp:41); here it is a parameter.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Norm, register_part
from .spec import ParamSpec


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, eps: float):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        h = self.hidden_size
        return [ParamSpec(self.prefix + "weight", (h,), role="norm_scale", alt_shapes=((h, 1),))]

    def load(self, get, dtype, device):
        self.weight = self._to(get(self.prefix + "weight").reshape(self.hidden_size), "compute", dtype, device)

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, h, delta):
        out = torch.empty(h.shape, dtype=self.weight.dtype, device=h.device)
        kernels.backend().add_rmsnorm(h, delta, self.weight, self.eps, out)
        return out

    def forward_rows(self, h, delta, rows):
        out = torch.empty((rows.shape[0], h.shape[1]), dtype=self.weight.dtype, device=h.device)
        kernels.backend().rows_add_rmsnorm(h, delta, rows, self.weight, self.eps, out)
        return out


class ScalarRMSNorm(RMSNorm):
    """RMS norm with one gain for all coordinates: y = x / sqrt(mean(x^2) + eps) * g.  The gain is a tensor with a
    single number (`prefix + name`); on the device it is repeated over the width, so the kernels of the norm with a
    weight per coordinate run it, and parts that fold a norm into their first kernel see an ordinary weight."""

    def __init__(self, prefix: str, hidden_size: int, eps: float, name: str = "weight"):
        super().__init__(prefix, hidden_size, eps)
        self.name = name

    def param_specs(self):
        return [ParamSpec(self.prefix + self.name, (), role="norm_scale", alt_shapes=((1,),))]

    def load(self, get, dtype, device):
        gain = get(self.prefix + self.name).reshape(1).to(dtype)
        self.weight = gain.expand(self.hidden_size).to(device).contiguous()


class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * weight + bias, var the mean of the squared deviations; statistics in float32,
    fused with the addition into the residual stream like the RMS norm.  The weight is the tensor `prefix + name`, the
    bias `prefix + bias_name` (None: the norm has no bias).  The stream it norms is float32."""

    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, eps: float, name: str = "weight", bias_name: str | None = "bias"):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.name, self.bias_name = name, bias_name
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def param_specs(self):
        h = self.hidden_size
        specs = [ParamSpec(self.prefix + self.name, (h,), role="norm_scale")]
        if self.bias_name is not None:
            specs.append(ParamSpec(self.prefix + self.bias_name, (h,), role="bias"))
        return specs

    def load(self, get, dtype, device):
        self.weight = self._to(get(self.prefix + self.name), "compute", dtype, device)
        if self.bias_name is not None:
            self.bias = self._to(get(self.prefix + self.bias_name), "compute", dtype, device)

    def forward(self, h, delta):
        out = torch.empty(h.shape, dtype=self.weight.dtype, device=h.device)
        kernels.backend().add_layernorm(h, delta, None, self.weight, self.bias, self.eps, out)
        return out

    def forward_rows(self, h, delta, rows):
        out = torch.empty((rows.shape[0], h.shape[1]), dtype=self.weight.dtype, device=h.device)
        kernels.backend().add_layernorm(h, delta, rows, self.weight, self.bias, self.eps, out)
        return out


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
register_part("norm", "rmsnorm_scalar", ScalarRMSNorm)
