"""Residual streams with learned read / write / mixing weights (hyper-connections), and the one-gain RMS norm
that reads them.

A model with ``n`` streams keeps ``xs`` [n, T, W] in fp32 instead of one residual row per token.  Sub-layer q
    reads   u = sum_s w_in[s] xs[s]         -> h = u / sqrt(mean(u^2) + eps) * gain   (gain: one number per norm)
    writes  xs[t] <- sum_s mix[s, t] xs[s] + w_out[t] * sublayer(h)                     (mix indexed [from, to])
and the model's output is the sum of the streams.  ``n = 1`` with all weights 1 is the plain pre-norm residual,
kept in fp32.  The write of one sub-layer and the read of the next are one kernel (``ops.stream_step``), which is
why ``StreamPort`` bundles what a reader needs.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from .linear import set_weight_attrs


def _fp32_param(shape, fill: float = 1.0) -> nn.Parameter:
    p = nn.Parameter(torch.full(shape, fill, dtype=torch.float32), requires_grad=False)

    def load(param, t, *_):
        param.data.copy_(t.to(torch.float32).reshape(param.shape))
    set_weight_attrs(p, {"weight_loader": load})
    return p


class ScalarRMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * g with a single learned number g (kept in fp32)."""

    def __init__(self, eps: float):
        super().__init__()
        self.eps = float(eps)
        self.weight = _fp32_param((1,))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        f = x.float()
        return (f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight).to(x.dtype)


class StreamPort(nn.Module):
    """Read, write and mixing weights of one sub-layer.  ``learned=False``: the plain residual (weights fixed at 1;
    with several streams every one receives the sub-layer's output and the reader sums them)."""

    def __init__(self, streams: int, learned: bool = True):
        super().__init__()
        self.streams = streams
        if learned:
            self.w_in, self.w_out = _fp32_param((streams,)), _fp32_param((streams,))
            self.mix = _fp32_param((streams, streams), 0.0)
        else:
            self.register_buffer("w_in", torch.ones(streams, dtype=torch.float32), persistent=False)
            self.register_buffer("w_out", torch.ones(streams, dtype=torch.float32), persistent=False)
            self.register_buffer("mix", torch.eye(streams, dtype=torch.float32), persistent=False)


def read_streams(xs: torch.Tensor, port: StreamPort, norm: ScalarRMSNorm, dtype: torch.dtype) -> torch.Tensor:
    return ops.stream_step(xs, w_in=port.w_in, gain=norm.weight, eps=norm.eps, out_dtype=dtype)


def write_read_streams(xs: torch.Tensor, y: torch.Tensor, port: StreamPort, nxt: Optional[StreamPort],
                       nxt_norm: Optional[ScalarRMSNorm]) -> Optional[torch.Tensor]:
    """Write sub-layer output ``y`` through ``port`` and read for the next sub-layer in the same pass."""
    if nxt is None:
        return ops.stream_step(xs, y, port.mix, port.w_out)
    return ops.stream_step(xs, y, port.mix, port.w_out, w_in=nxt.w_in, gain=nxt_norm.weight, eps=nxt_norm.eps,
                           out_dtype=y.dtype)
