"""The oracle's restatement of the linear layer (src/linear.cpp) pinned against a
library routine: torch.nn.functional.linear and its autograd on the CPU, and
against fp64 numpy.  A transposed operand or a dropped bias fails these."""
import numpy as np
import pytest
import torch

import oracle

SHAPES = [(1, 1, 1), (7, 5, 3), (64, 96, 48), (33, 130, 257), (128, 10, 960)]  # M (batch), K (in), N (out)


def _data(M, K, N):
    return (oracle.uniform((M, K), 11), oracle.uniform((N, K), 12), oracle.uniform((N,), 13),
            oracle.uniform((M, N), 14))


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("with_bias", [True, False])
def test_forward_matches_torch_and_fp64(shape, with_bias):
    M, K, N = shape
    x, w, b, _ = _data(M, K, N)
    bias = b if with_bias else None
    y = oracle.linear_forward(x, w, bias)
    ref = torch.nn.functional.linear(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                                     torch.from_numpy(b).double() if with_bias else None).numpy()
    S = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T + (np.abs(b)[None, :] if with_bias else 0)
    assert np.max(np.abs(y - ref) / np.maximum(S, 1e-30)) <= 2e-6
    y32 = torch.nn.functional.linear(torch.from_numpy(x), torch.from_numpy(w),
                                     torch.from_numpy(b) if with_bias else None).numpy()
    assert np.max(np.abs(y - y32) / np.maximum(S, 1e-30)) <= 4e-6


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_backward_matches_torch_autograd(shape):
    M, K, N = shape
    x, w, b, g = _data(M, K, N)
    tx = torch.from_numpy(x).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    tb = torch.from_numpy(b).double().requires_grad_()
    torch.nn.functional.linear(tx, tw, tb).backward(torch.from_numpy(g).double())
    gx, gw, gb = oracle.linear_backward(g, x, w, b)
    Sx = np.abs(g).astype(np.float64) @ np.abs(w).astype(np.float64)
    Sw = np.abs(g).astype(np.float64).T @ np.abs(x).astype(np.float64)
    assert np.max(np.abs(gx - tx.grad.numpy()) / np.maximum(Sx, 1e-30)) <= 2e-6
    assert np.max(np.abs(gw - tw.grad.numpy()) / np.maximum(Sw, 1e-30)) <= 2e-6
    assert np.allclose(gb, tb.grad.numpy(), rtol=0, atol=1e-12 * M)
    assert oracle.linear_backward(g, x, w, None)[2] is None


def test_a_transposed_weight_is_caught():
    M, K, N = 16, 24, 24   # square weight: a missing transpose keeps the shapes legal
    x, w, _, _ = _data(M, K, N)
    wrong = oracle.cake_sgemm(x, np.ascontiguousarray(w), 10)
    right = oracle.linear_forward(x, w)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.max(np.abs(right - ref)) < 1e-4 < np.max(np.abs(wrong - ref))
