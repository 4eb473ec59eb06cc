"""Pins oracle/mlp.py, the hand-written float64 forward / backward of the deformation MLP that the GPU parity test of
the MFMA backward kernels uses as its checker: without the bf16 roundings it must equal torch.autograd of the same
network (network.py:1757-1776 as plain F.linear / relu / cat) for every parameter and for the encoded input, on the
four shapes the GPU test runs (partial 32-row block, single row, a skip layer in different places)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import mlp as M


def _network(D, Din, n_out, seed):
    g = torch.Generator().manual_seed(seed)
    skip = D // 2
    K = lambda l: Din if l == 0 else (Din + 256 if l == skip + 1 else 256)
    weights = [(torch.randn(256, K(l), generator=g, dtype=torch.float64) * (2.0 / K(l)) ** 0.5).requires_grad_()
               for l in range(D)]
    biases = [(0.05 * torch.randn(256, generator=g, dtype=torch.float64)).requires_grad_() for _ in range(D)]
    head_w = (0.05 * torch.randn(n_out, 256, generator=g, dtype=torch.float64)).requires_grad_()
    head_b = (0.05 * torch.randn(n_out, generator=g, dtype=torch.float64)).requires_grad_()
    return weights, biases, head_w, head_b, skip, g


def _torch_network(x, weights, biases, head_w, head_b, skip):
    h = x
    for l, (W, b) in enumerate(zip(weights, biases)):
        h = torch.relu(F.linear(h, W, b))
        if l == skip:
            h = torch.cat([x, h], -1)
    return F.linear(h, head_w, head_b)


@pytest.mark.parametrize("B,D,Din,n_out", [(512, 8, 84, 10), (500, 8, 76, 14), (70, 4, 32, 10), (1, 3, 18, 10)])
def test_backward_without_rounding_is_autograd(B, D, Din, n_out):
    weights, biases, head_w, head_b, skip, g = _network(D, Din, n_out, seed=B + D)
    x = torch.randn(B, Din, generator=g, dtype=torch.float64).requires_grad_()
    g_out = torch.randn(B, n_out, generator=g, dtype=torch.float64)
    out = _torch_network(x, weights, biases, head_w, head_b, skip)
    want = torch.autograd.grad((out * g_out).sum(), [x, head_w, head_b] + weights + biases)
    with torch.no_grad():
        o, hidden = M.mlp_forward(x, weights, biases, head_w, head_b, skip)
        assert float((o - out).abs().max()) <= 1e-12 * max(float(out.abs().max()), 1.0)
        got = M.mlp_backward(x, weights, head_w, skip, g_out, hidden)
    flat = [got['x'], got['head_w'], got['head_b']] + got['weights'] + got['biases']
    assert len(flat) == len(want)
    for a, b in zip(flat, want):
        assert a.shape == b.shape
        assert float((a - b).abs().max()) <= 1e-10 * max(float(b.abs().max()), 1e-30)
    assert float(got['x'].abs().max()) > 0 and all(float(w.abs().max()) > 0 for w in got['weights'])


def test_rounding_switch_only_perturbs():
    """With the kernels' bf16 roundings switched on the same function stays within bf16 accuracy of the exact gradients
    (the states are the exact forward's here, so no ReLU unit flips): the switch changes roundings, not the formula."""
    B, D, Din, n_out = 96, 4, 40, 10
    weights, biases, head_w, head_b, skip, g = _network(D, Din, n_out, seed=5)
    x = torch.randn(B, Din, generator=g, dtype=torch.float64)
    g_out = torch.randn(B, n_out, generator=g, dtype=torch.float64)
    with torch.no_grad():
        _, hidden = M.mlp_forward(x, weights, biases, head_w, head_b, skip)
        exact = M.mlp_backward(x, weights, head_w, skip, g_out, hidden)
        rounded = M.mlp_backward(x, weights, head_w, skip, g_out, hidden, round_bf16=True)
    for key in ('x', 'head_w', 'head_b'):
        a, b = rounded[key], exact[key]
        assert 0 < float((a - b).abs().max()) <= 3e-2 * float(b.abs().max())
    for a, b in zip(rounded['weights'] + rounded['biases'], exact['weights'] + exact['biases']):
        assert float((a - b).abs().max()) <= 3e-2 * float(b.abs().max())
