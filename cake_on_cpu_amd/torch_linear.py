"""PyTorch operator over the C-ABI: the linear layer of the reference's only
framework binding (src/linear.cpp:12-107, python/cake.py:18-49), with the same
names -- forward / backward, cake_linear_function, cake_linear.

Tensors on a ROCm device are used in place through their device pointers on
torch's current stream; CPU tensors are staged by the library.  torch only
provides memory, streams and autograd bookkeeping; every product, transpose and
reduction runs in libcake_hip.so."""
from __future__ import annotations

import torch
from torch import nn

from . import api


def _f32c(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.float32:
        raise TypeError(f"{what} must be float32, got {t.dtype}")
    return t.detach().contiguous()


def forward(cache_sz, input, weight, bias=None, weight_t=None):
    """output[M][N] = input[M][K] . weight[N][K]^T (+ bias).  `cache_sz` (the
    reference passes the host's L2/L3 sizes, src/linear.cpp:37) is accepted and
    unused: block sizes come from the device.  weight_t: the weights already
    transposed ([K][N]), from a caller that holds them that way; the library itself reads
    `weight` as it lies and needs no such copy."""
    if input.dim() != 2 or weight.dim() != 2 or input.size(1) != weight.size(1):
        raise ValueError(f"linear forward: input {tuple(input.shape)} does not match weight {tuple(weight.shape)}")
    M, K = input.shape
    N = weight.size(0)
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError(f"linear forward: bias {tuple(bias.shape)} does not match {N} outputs")
    x = _f32c(input, "input")
    b = None if bias is None else _f32c(bias, "bias")
    out = torch.empty((M, N), dtype=torch.float32, device=input.device)
    # device tensors: no event timing, so the call only enqueues work on torch's current stream
    timed = not input.is_cuda
    if weight_t is not None:
        if tuple(weight_t.shape) != (K, N):
            raise ValueError(f"linear forward: weight_t {tuple(weight_t.shape)} is not {(K, N)}")
        api.linear_forward_wt(x, _f32c(weight_t, "weight_t"), b, out, M, N, K, timed=timed)
    else:
        api.linear_forward(x, _f32c(weight, "weight"), b, out, M, N, K, timed=timed)
    return out


def backward(cache_sz, grad_output, input, weight, bias=None, needs=(True, True, True)):
    """(grad_input, grad_weight, grad_bias) for grad_output[M][N]; entries whose
    `needs` flag is false (or grad_bias when bias is None) are returned as None."""
    M, K = input.shape
    N = weight.size(0)
    if tuple(grad_output.shape) != (M, N):
        raise ValueError(f"linear backward: grad_output {tuple(grad_output.shape)} is not {(M, N)}")
    g = _f32c(grad_output, "grad_output")
    x, w = _f32c(input, "input"), _f32c(weight, "weight")
    dev = grad_output.device
    gx = torch.empty((M, K), dtype=torch.float32, device=dev) if needs[0] else None
    gw = torch.empty((N, K), dtype=torch.float32, device=dev) if needs[1] else None
    gb = torch.empty((N,), dtype=torch.float32, device=dev) if (needs[2] and bias is not None) else None
    api.linear_backward(g, x if gw is not None else None, w if gx is not None else None, gx, gw, gb, M, N, K,
                        timed=not grad_output.is_cuda)
    return gx, gw, gb


class cake_linear_function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, weight, bias=None, weight_t=None):
        ctx.save_for_backward(data, weight, bias)
        return forward(None, data, weight, bias, weight_t)

    @staticmethod
    def backward(ctx, grad_output):
        data, weight, bias = ctx.saved_tensors
        return (*backward(None, grad_output, data, weight, bias, ctx.needs_input_grad[:3]), None)


class cake_linear(nn.Module):
    """Drop-in for the reference's cake_linear (python/cake.py:33-49): weight
    [output_features][input_features] and bias drawn from U(-0.1, 0.1)."""

    def __init__(self, input_features, output_features, bias=True):
        super().__init__()
        self.input_features = input_features
        self.output_features = output_features
        self.weight = nn.Parameter(torch.empty(output_features, input_features).uniform_(-0.1, 0.1))
        if bias:
            self.bias = nn.Parameter(torch.empty(output_features).uniform_(-0.1, 0.1))
        else:
            self.register_parameter("bias", None)

    def forward(self, data):
        lead = data.shape[:-1]
        flat = data.reshape(-1, self.input_features)
        out = cake_linear_function.apply(flat, self.weight, self.bias)
        return out.reshape(*lead, self.output_features)

    def extra_repr(self):
        return f"input_features={self.input_features}, output_features={self.output_features}, bias={self.bias is not None}"
