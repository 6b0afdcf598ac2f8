"""Portable PyTorch paths of the RG-LRU: gate chain, sequential loop and associative scan.

These are the ``scan_mode="sequential"`` / ``"associative"`` backends of the module (CPU tensors,
dtypes or devices the HIP kernels do not cover, and the fallback of ``"auto"``).  Behaviour follows
griffin/griffin.py:237-306 of the reference; autograd differentiates them.
"""

from __future__ import annotations

import torch
from torch import Tensor
import torch.nn.functional as F

_SQRT_GRADIENT_CAP = 1000.0


class _CappedSqrt(torch.autograd.Function):
    """sqrt with d/dx = 1 / sqrt(max(4x, cap^-2)) (reference: griffin/griffin.py:48-65)."""

    @staticmethod
    def forward(ctx, value: Tensor) -> Tensor:
        ctx.save_for_backward(value)
        return value.sqrt()

    @staticmethod
    def backward(ctx, grad: Tensor):
        (value,) = ctx.saved_tensors
        return grad * torch.rsqrt((4.0 * value).clamp_min(_SQRT_GRADIENT_CAP ** -2))


def block_diagonal_project(x: Tensor, weight: Tensor, bias: Tensor) -> Tensor:
    """Apply ``weight[k]`` (out, in) to the k-th slice of the last axis (griffin/griffin.py:149-154)."""
    blocks, width = weight.shape[0], weight.shape[1]
    grouped = x.unflatten(-1, (blocks, width))
    out = (grouped.unsqueeze(-2) * weight).sum(-1) if width <= 2 else torch.einsum("...ki,koi->...ko", grouped, weight)
    return (out + bias).flatten(-2)


def decay_and_input(x, w_a, b_a, w_x, b_x, lam, c, reset_mask, active_mask, state_dtype):
    """Return (a, z) of the recurrence in ``state_dtype`` (griffin/griffin.py:237-258)."""
    gate_r = torch.sigmoid(block_diagonal_project(x, w_a, b_a))
    gate_i = torch.sigmoid(block_diagonal_project(x, w_x, b_x))
    log_a = (c * gate_r) * F.logsigmoid(lam).to(x.dtype)
    a = torch.exp(log_a)
    scale = _CappedSqrt.apply((-torch.expm1(2.0 * log_a)).clamp_min(0.0))
    reset = reset_mask.unsqueeze(-1)
    a = a.masked_fill(reset, 0.0)
    scale = scale.masked_fill(reset, 1.0)
    z = scale * gate_i * x
    idle = ~active_mask.unsqueeze(-1)
    a = a.masked_fill(idle, 1.0)
    z = z.masked_fill(idle, 0.0)
    return a.to(state_dtype), z.to(state_dtype)


def causal_depthwise_conv(projected: Tensor, conv_state: Tensor, weight: Tensor, bias: Tensor | None,
                          segment_pos: Tensor):
    """All-tokens-active temporal convolution of the recurrent block (griffin/griffin.py:474-487):
    ``weight`` [W, 1, K] of a depthwise Conv1d, taps masked per document through ``segment_pos``.
    Returns the convolved sequence and the last K-1 rows of the padded input."""
    taps = weight[:, 0, :]
    history = taps.size(1) - 1
    steps = projected.size(1)
    padded = torch.cat((conv_state.to(projected), projected), dim=1)
    out = projected.new_zeros(projected.shape)
    if bias is not None:
        out = out + bias
    for lag in range(history + 1):
        window = padded[:, history - lag: history - lag + steps]
        same_document = (segment_pos >= lag).to(window.dtype).unsqueeze(-1)
        out = out + window * same_document * taps[:, history - lag]
    return out, (padded[:, padded.size(1) - history:] if history else padded[:, :0])


def sequential_scan(a: Tensor, z: Tensor, state: Tensor) -> Tensor:
    """One step per token (griffin/griffin.py:279-284)."""
    steps = []
    for a_t, z_t in zip(a.unbind(1), z.unbind(1)):
        state = a_t * state + z_t
        steps.append(state)
    return torch.stack(steps, dim=1)


def associative_scan(a: Tensor, z: Tensor, state: Tensor) -> Tensor:
    """Log-depth composition of the affine maps h -> a h + z (griffin/griffin.py:291-306)."""
    length = a.shape[1]
    shift = 1
    while shift < length:
        head_a, head_z = a[:, :shift], z[:, :shift]
        tail_a = a[:, shift:] * a[:, :-shift]
        tail_z = z[:, shift:] + a[:, shift:] * z[:, :-shift]
        a = torch.cat((head_a, tail_a), dim=1)
        z = torch.cat((head_z, tail_z), dim=1)
        shift *= 2
    return z + a * state.unsqueeze(1)
