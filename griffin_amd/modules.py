"""Host-side mirror of the reference's RG-LRU module interface with a ``scan_mode="hip"`` backend.

Constructor signatures, parameter names and shapes, argument validation, error types and the
dispatch rules follow griffin/griffin.py:119-306 (RG_LRU, BlockDiagonalLinear) and :309-529
(RecurrentBlock and its cache), so that callers, state_dicts and tests of the reference carry
over.  What differs is the accelerator path: ``"hip"`` (explicit, fails loudly) and ``"auto"`` on
GPU tensors (after a one-time parity self-test, with a warning and the portable scan as fallback)
run the hand-written gfx950 kernels; the Triton backend is gone and ``"fused"`` is kept as an
alias of ``"hip"``.
"""

from __future__ import annotations

from dataclasses import dataclass
import math
from typing import Literal

import torch
from torch import Tensor
import torch.nn as nn
import torch.nn.functional as F

from . import hip_block_ops, hip_scan, portable

ScanMode = Literal["auto", "sequential", "associative", "hip", "fused"]
SCAN_MODES = ("auto", "sequential", "associative", "hip", "fused")


@dataclass
class RecurrentBlockCache:
    """State that lets a recurrent block continue on a later chunk (griffin/griffin.py:26-32)."""

    rnn_state: Tensor
    conv_state: Tensor
    segment_position: Tensor


def _compatible_block_count(width: int, requested_blocks: int) -> int:
    """Largest block count <= requested that divides width (griffin/griffin.py:119-126)."""
    if width <= 0 or requested_blocks <= 0:
        raise ValueError("width and requested_blocks must be positive")
    count = min(width, requested_blocks)
    while width % count:
        count -= 1
    return count


class BlockDiagonalLinear(nn.Module):
    """Block-diagonal projection: weight [blocks, out, in], bias [blocks, out] (griffin/griffin.py:129-154)."""

    def __init__(self, width: int, num_blocks: int = 16):
        super().__init__()
        self.width = width
        self.num_blocks = _compatible_block_count(width, num_blocks)
        self.block_width = width // self.num_blocks
        self.weight = nn.Parameter(torch.empty(self.num_blocks, self.block_width, self.block_width))
        self.bias = nn.Parameter(torch.empty(self.num_blocks, self.block_width))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0.0, std=math.sqrt(1.0 / self.block_width))
        nn.init.zeros_(self.bias)

    def forward(self, x: Tensor) -> Tensor:
        return portable.block_diagonal_project(x, self.weight, self.bias)


class RG_LRU(nn.Module):
    """Real-Gated Linear Recurrent Unit (griffin/griffin.py:157-306) with a HIP scan backend."""

    def __init__(self, rnn_width: int, c: float = 8.0, gate_blocks: int = 16, scan_mode: ScanMode = "auto"):
        super().__init__()
        self.rnn_width = rnn_width
        self.c = c
        if scan_mode not in SCAN_MODES:
            raise ValueError(f"Unknown RG-LRU scan mode: {scan_mode}")
        self.scan_mode = scan_mode
        self.recurrence_gate = BlockDiagonalLinear(rnn_width, gate_blocks)
        self.input_gate = BlockDiagonalLinear(rnn_width, gate_blocks)
        self.Lambda = nn.Parameter(torch.empty(rnn_width))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        self.recurrence_gate.reset_parameters()
        self.input_gate.reset_parameters()
        with torch.no_grad():
            decay_to_the_c = torch.empty_like(self.Lambda).uniform_(0.9, 0.999)
            self.Lambda.copy_(torch.logit(decay_to_the_c.pow(1.0 / self.c)))

    # -- dispatch ---------------------------------------------------------------------------
    def _hip_covers(self, xt: Tensor) -> bool:
        return (
            xt.dtype in hip_scan.SUPPORTED_DTYPES
            and self.recurrence_gate.block_width <= 512
            and xt.numel() > 0
        )

    def _gate_parameters(self):
        return (self.recurrence_gate.weight, self.recurrence_gate.bias, self.input_gate.weight,
                self.input_gate.bias, self.Lambda)

    def _needs_grad(self, xt: Tensor, ht_minus_1: Tensor | None) -> bool:
        if not torch.is_grad_enabled():
            return False
        tensors = (xt, ht_minus_1) + self._gate_parameters()
        return any(t is not None and t.requires_grad for t in tensors)

    def _prepared(self, dtype: torch.dtype, device: torch.device):
        """Kernel-side parameter image for inference, rebuilt when a parameter is replaced or updated
        in place (every in-place update bumps the tensor's version counter)."""
        params = self._gate_parameters()
        key = (dtype, device, float(self.c)) + tuple((q.data_ptr(), q._version) for q in params)
        if getattr(self, "_prep_key", None) != key:
            prep = hip_scan.PreparedParams(*params, self.c, dtype)
            if device.type == "cuda" and torch.cuda.is_current_stream_capturing():
                return prep                                  # allocated by the graph being captured: this call only
            self._prep = prep
            self._prep_key = key
        return self._prep

    def invalidate_caches(self) -> None:
        """Forget the kernel-side parameter image.  It is rebuilt by itself when a parameter is replaced or
        updated in place through PyTorch operators; writes that bypass the version counter (``p.data.copy_()``,
        ``p.data.mul_()``) need this call.  ``module.to()``/``.cuda()``, ``train()``/``eval()`` and
        ``load_state_dict`` call it."""
        self._prep = None
        self._prep_key = None

    def _apply(self, fn, *args, **kwargs):
        self.invalidate_caches()
        return super()._apply(fn, *args, **kwargs)

    def train(self, mode: bool = True):
        self.invalidate_caches()
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_caches()
        return super()._load_from_state_dict(*args, **kwargs)

    def forward(
        self,
        xt: Tensor,
        ht_minus_1: Tensor | None = None,
        *,
        reset_mask: Tensor | None = None,
        active_mask: Tensor | None = None,
        return_state: bool = False,
    ):
        if xt.dim() != 3:
            raise ValueError(f"RG_LRU expects [batch, sequence, width], got {tuple(xt.shape)}")
        batch, steps, width = xt.shape
        if width != self.rnn_width:
            raise ValueError(f"Expected width {self.rnn_width}, got {width}")
        for name, mask in (("reset_mask", reset_mask), ("active_mask", active_mask)):
            if mask is not None and mask.shape != (batch, steps):
                raise ValueError(f"{name} must have shape ({batch}, {steps}), got {tuple(mask.shape)}")
        if ht_minus_1 is not None and ht_minus_1.shape != (batch, width):
            raise ValueError(f"ht_minus_1 must have shape ({batch}, {width}), got {tuple(ht_minus_1.shape)}")
        state_dtype = torch.float32 if xt.dtype in (torch.float16, torch.bfloat16) else xt.dtype
        if reset_mask is not None:
            reset_mask = reset_mask.to(device=xt.device, dtype=torch.bool)
        if active_mask is not None:
            active_mask = active_mask.to(device=xt.device, dtype=torch.bool)
        if ht_minus_1 is not None:
            ht_minus_1 = ht_minus_1.to(device=xt.device, dtype=state_dtype)

        mode = self.scan_mode
        if mode not in SCAN_MODES:
            raise ValueError(f"Unknown RG-LRU scan mode: {mode}")
        explicit_hip = mode in ("hip", "fused")
        auto_hip = (
            mode == "auto"
            and xt.is_cuda
            and self._hip_covers(xt)
            and hip_scan.hip_scan_is_usable(xt.device)
        )
        if explicit_hip or auto_hip:
            if explicit_hip and not xt.is_cuda:
                raise RuntimeError(
                    f'scan_mode="{mode}" requires CUDA/HIP tensors and the RG-LRU HIP library; '
                    f"got a {xt.device.type} tensor"
                )
            if steps == 1 and not self._needs_grad(xt, ht_minus_1):
                # decode: the single-step kernel on a prepared parameter image kept between calls
                prep = self._prepared(xt.dtype, xt.device)
                state = (torch.zeros(batch, width, device=xt.device, dtype=torch.float32) if ht_minus_1 is None
                         else ht_minus_1.to(torch.float32).clone(memory_format=torch.contiguous_format))
                flags = hip_scan.pack_flags(reset_mask, active_mask)
                y = hip_scan.hip_rglru_step(xt[:, 0], prep, state, None if flags is None else flags.reshape(batch))
                y = y.unsqueeze(1)
                return (y, state) if return_state else y
            # the reset mask of the default positions (a document start at token 0 of every row, nothing else)
            # is known by identity: the kernels then need no per-token flags at all
            default = _DEFAULT_POSITIONS.get((batch, steps, xt.device))
            first_only = default is not None and reset_mask is default[1] and active_mask is None
            y, state = hip_scan.hip_rglru(
                xt, self.recurrence_gate.weight, self.recurrence_gate.bias, self.input_gate.weight,
                self.input_gate.bias, self.Lambda, self.c, ht_minus_1, None if first_only else reset_mask, active_mask,
                first_token_reset=first_only,
            )
            return (y, state) if return_state else y

        if reset_mask is None:
            reset_mask = torch.zeros(batch, steps, device=xt.device, dtype=torch.bool)
        if active_mask is None:
            active_mask = torch.ones(batch, steps, device=xt.device, dtype=torch.bool)
        state = (
            torch.zeros(batch, width, device=xt.device, dtype=state_dtype) if ht_minus_1 is None else ht_minus_1
        )
        a, z = portable.decay_and_input(
            xt, self.recurrence_gate.weight, self.recurrence_gate.bias, self.input_gate.weight,
            self.input_gate.bias, self.Lambda, self.c, reset_mask, active_mask, state_dtype,
        )
        use_associative = mode == "associative" or (mode == "auto" and xt.is_cuda and steps > 1)
        if use_associative:
            states = portable.associative_scan(a, z, state)
        else:
            states = portable.sequential_scan(a, z, state)
        y = states.to(xt.dtype)
        return (y, states[:, -1]) if return_state else y

    _associative_scan = staticmethod(portable.associative_scan)


# Positions 0 .. T-1 for every row and their "document starts here" mask: what a call without cache,
# explicit positions or padding resolves to.  They depend only on (batch, steps, device), so they are
# built once (a training step would otherwise spend six small launches per block on them) and must
# not be modified in place by anyone.
_DEFAULT_POSITIONS: dict = {}


def _default_positions(batch: int, steps: int, device: torch.device):
    key = (batch, steps, device)
    hit = _DEFAULT_POSITIONS.get(key)
    if hit is None:
        # Built outside inference mode whatever the caller's mode: an inference tensor cannot be saved for a
        # backward pass, and an evaluation pass followed by a training step at the same shape is the normal loop.
        with torch.inference_mode(False):
            pos = torch.arange(steps, device=device, dtype=torch.long).expand(batch, steps).contiguous()
            hit = (pos, pos == 0)
        # tensors made while a graph is being captured live in that graph's memory and hold nothing until
        # it is replayed: they are used for this call only
        if not (device.type == "cuda" and torch.cuda.is_current_stream_capturing()):
            if len(_DEFAULT_POSITIONS) >= 16:
                _DEFAULT_POSITIONS.clear()
            _DEFAULT_POSITIONS[key] = hit
    return hit


def _resolve_segment_positions(x, segment_pos, previous_position=None, active_mask=None) -> Tensor:
    """Explicit positions, or previous + running count of active tokens (griffin/griffin.py:309-338)."""
    batch, steps = x.shape[:2]
    if steps == 0:
        raise ValueError("Empty token sequences are not supported")
    if segment_pos is None and previous_position is None and active_mask is None:
        return _default_positions(batch, steps, x.device)[0]
    if segment_pos is not None:
        if segment_pos.shape != (batch, steps):
            raise ValueError(f"segment_pos must have shape ({batch}, {steps}), got {tuple(segment_pos.shape)}")
        return segment_pos.to(device=x.device, dtype=torch.long)
    if previous_position is None:
        start = torch.full((batch,), -1, device=x.device, dtype=torch.long)
    else:
        if previous_position.shape != (batch,):
            raise ValueError("Cached segment positions have an incompatible shape")
        start = previous_position.to(device=x.device, dtype=torch.long)
    if active_mask is None:
        counts = torch.arange(1, steps + 1, device=x.device, dtype=torch.long).expand(batch, steps)
    else:
        counts = active_mask.to(torch.long).cumsum(dim=1)
    return start[:, None] + counts


def _last_active_position(segment_pos: Tensor, active_mask: Tensor, previous_position: Tensor | None) -> Tensor:
    """Position of each row's last active token, or the previous one when the row is all padding
    (griffin/griffin.py:341-358), computed without a per-row host loop."""
    batch, steps = segment_pos.shape
    if previous_position is None:
        fallback = torch.full((batch,), -1, device=segment_pos.device, dtype=torch.long)
    else:
        fallback = previous_position.to(device=segment_pos.device, dtype=torch.long)
    index = torch.arange(steps, device=segment_pos.device).expand(batch, steps)
    last = torch.where(active_mask, index, torch.full_like(index, -1)).max(dim=1).values
    picked = segment_pos.gather(1, last.clamp_min(0)[:, None])[:, 0]
    return torch.where(last >= 0, picked, fallback)


class RMSNorm(nn.Module):
    """Root-mean-square normalisation with a learned per-channel scale (griffin/griffin.py:68-80), the
    layer in front of the recurrent block.  GPU tensors the HIP library covers go through its kernels
    (after the same per-device self-test as ``scan_mode="auto"``); everything else through PyTorch."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.g = nn.Parameter(torch.zeros(dim))

    def _hip_covers(self, x: Tensor) -> bool:
        if not x.is_cuda or x.dtype not in hip_scan.SUPPORTED_DTYPES or x.numel() == 0:
            return False
        if not hip_scan.hip_scan_is_usable(x.device):
            return False
        aligned = x.size(-1) % (8 if x.dtype == torch.bfloat16 else 4) == 0
        return x.size(-1) <= hip_block_ops.rmsnorm_max_width(x.dtype, aligned)

    def forward(self, x: Tensor) -> Tensor:
        if self._hip_covers(x):
            return hip_block_ops.hip_rmsnorm(x, self.g, self.eps)
        normalized = x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return normalized * (1.0 + self.g)


class RecurrentBlock(nn.Module):
    """Linear -> causal depthwise conv -> RG-LRU, gated by GeLU(Linear), then Linear out
    (griffin/griffin.py:361-529).  The RG-LRU inside honours ``scan_mode`` unchanged."""

    def __init__(self, input_dim: int, rnn_width: int, conv_kernel_size: int = 4, gate_blocks: int = 16,
                 final_w_init_variance_scale: float = 1.0, scan_mode: ScanMode = "auto"):
        super().__init__()
        if conv_kernel_size <= 0:
            raise ValueError("conv_kernel_size must be positive")
        self.rnn_width = rnn_width
        self.conv_kernel_size = conv_kernel_size
        self.linear_x = nn.Linear(input_dim, rnn_width)
        self.linear_y = nn.Linear(input_dim, rnn_width)
        self.temporal_conv = nn.Conv1d(rnn_width, rnn_width, kernel_size=conv_kernel_size, padding=0,
                                       groups=rnn_width)
        self.rg_lru = RG_LRU(rnn_width, gate_blocks=gate_blocks, scan_mode=scan_mode)
        self.linear_out = nn.Linear(rnn_width, input_dim)
        self.final_w_init_variance_scale = final_w_init_variance_scale
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.linear_x.weight, std=math.sqrt(1.0 / self.linear_x.in_features))
        nn.init.normal_(self.linear_y.weight, std=math.sqrt(1.0 / self.linear_y.in_features))
        nn.init.normal_(self.linear_out.weight,
                        std=math.sqrt(self.final_w_init_variance_scale / self.linear_out.in_features))
        nn.init.normal_(self.temporal_conv.weight, std=math.sqrt(0.01 / self.conv_kernel_size))
        for layer in (self.linear_x, self.linear_y, self.linear_out, self.temporal_conv):
            nn.init.zeros_(layer.bias)

    def invalidate_caches(self) -> None:
        """Forget the stacked decode projection (and the RG-LRU's parameter image).  Both are rebuilt by
        themselves when a parameter is replaced or updated in place through PyTorch operators; writes that
        bypass the version counter (``p.data.copy_()``) need this call.  ``module.to()``, ``train()``/``eval()``
        and ``load_state_dict`` call it."""
        self._stacked_projection = None
        self.rg_lru.invalidate_caches()

    def _apply(self, fn, *args, **kwargs):
        self._stacked_projection = None
        return super()._apply(fn, *args, **kwargs)

    def train(self, mode: bool = True):
        self._stacked_projection = None
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self._stacked_projection = None
        return super()._load_from_state_dict(*args, **kwargs)

    def _empty_conv_state(self, x: Tensor) -> Tensor:
        return x.new_zeros(x.size(0), self.conv_kernel_size - 1, self.rnn_width)

    def _hip_block_ops_covers(self, projected: Tensor) -> bool:
        """The HIP convolution runs wherever the RG-LRU inside takes its HIP path."""
        mode = self.rg_lru.scan_mode
        if not projected.is_cuda or projected.dtype not in hip_scan.SUPPORTED_DTYPES or projected.numel() == 0:
            return False
        if mode == "auto":
            if not (self.rg_lru._hip_covers(projected) and hip_scan.hip_scan_is_usable(projected.device)):
                return False
        elif mode not in ("hip", "fused"):
            return False
        return self.conv_kernel_size <= hip_block_ops.max_kernel_size()

    def _hip_block_forward_covers(self, projected: Tensor, gate_input: Tensor, cache: RecurrentBlockCache | None) -> bool:
        """The one-launch forward (convolution, RG-LRU, output gate) exists for this shape and these types."""
        if gate_input.dtype != projected.dtype or gate_input.shape != projected.shape:
            return False
        if cache is not None and cache.rnn_state is not None and cache.rnn_state.shape != (projected.size(0), self.rnn_width):
            return False                                     # the RG-LRU reports the shape error
        return hip_block_ops.hip_block_forward_covers(self.rnn_width, self.rg_lru.recurrence_gate.weight.shape[0],
                                                      self.conv_kernel_size, projected.dtype)

    def _hip_decode_covers(self, x: Tensor, cache: RecurrentBlockCache | None) -> bool:
        """Single-token inference takes the two-launch decode path of the HIP library."""
        if not x.is_cuda or x.dtype not in hip_scan.SUPPORTED_DTYPES or x.numel() == 0:
            return False
        if torch.is_grad_enabled():
            tensors = [x, *self.parameters()]
            if cache is not None:
                tensors += [cache.rnn_state, cache.conv_state]
            if any(t.requires_grad for t in tensors):
                return False
        if self.linear_x.weight.dtype != x.dtype or self.linear_y.weight.dtype != x.dtype:
            return False
        mode = self.rg_lru.scan_mode
        if mode == "auto":
            probe = x.new_empty(x.size(0), 1, self.rnn_width)
            return self._hip_block_ops_covers(probe)
        return mode in ("hip", "fused") and self.conv_kernel_size <= hip_block_ops.max_kernel_size()

    def _hip_decode(self, x: Tensor, cache: RecurrentBlockCache | None, segment_pos: Tensor | None,
                    active_mask: Tensor | None, return_cache: bool):
        """One token per row (griffin/griffin.py:459-528 with T == 1): positions, convolution, RG-LRU
        step and output gate in two kernel launches around the three projections."""
        batch = x.size(0)
        width = self.rnn_width
        history = self.conv_kernel_size - 1
        if segment_pos is not None:
            if segment_pos.shape != (batch, 1):
                raise ValueError(f"segment_pos must have shape ({batch}, 1), got {tuple(segment_pos.shape)}")
            segment_pos = segment_pos.to(device=x.device, dtype=torch.long)[:, 0].contiguous()
        conv_state = prev_pos = rnn_state = None
        if cache is not None:
            conv_state, prev_pos, rnn_state = cache.conv_state, cache.segment_position, cache.rnn_state
            if conv_state.shape != (batch, history, width):
                raise ValueError("Recurrent convolution cache has an incompatible shape")
            if prev_pos.shape != (batch,):
                raise ValueError("Cached segment positions have an incompatible shape")
            if rnn_state is not None and rnn_state.shape != (batch, width):
                raise ValueError(f"ht_minus_1 must have shape ({batch}, {width}), got {tuple(rnn_state.shape)}")
            prev_pos = prev_pos.to(device=x.device, dtype=torch.long).contiguous()
        active = None
        if active_mask is not None and not bool(active_mask.all()):
            active = active_mask[:, 0].to(torch.uint8).contiguous()
        projected, gate_input = self._decode_projections(x[:, 0])
        prep = self.rg_lru._prepared(projected.dtype, projected.device)
        gated, new_rnn_state, new_conv_state, new_pos = hip_block_ops.hip_block_decode_step(
            projected, gate_input, conv_state, self.temporal_conv.weight, self.temporal_conv.bias,
            prev_pos, segment_pos, active, prep, rnn_state)
        output = self.linear_out(gated).unsqueeze(1)
        if active is not None:
            output = output.masked_fill(~active_mask.unsqueeze(-1), 0.0)
        if return_cache:
            return output, RecurrentBlockCache(new_rnn_state, new_conv_state, new_pos)
        return output

    def _decode_projections(self, token: Tensor):
        """``linear_x`` and ``linear_y`` of one token per row as ONE GEMM against the two weights stacked
        (the decode kernels take the halves of its output as strided rows).  The stacked copy is kept
        until a weight or bias changes (storage or version counter)."""
        layers = (self.linear_x, self.linear_y)
        tensors = [t for layer in layers for t in (layer.weight, layer.bias) if t is not None]
        key = tuple((t.data_ptr(), t._version, t.dtype, t.device) for t in tensors)
        cached = getattr(self, "_stacked_projection", None)
        if cached is None or cached[0] != key:
            if len(tensors) != 4 or (token.is_cuda and torch.cuda.is_current_stream_capturing()):
                # nothing allocated during a graph capture may outlive it: two GEMMs this time
                return self.linear_x(token), self.linear_y(token)
            with torch.no_grad():
                weight = torch.cat([self.linear_x.weight, self.linear_y.weight], 0).contiguous()
                bias = torch.cat([self.linear_x.bias, self.linear_y.bias], 0).contiguous()
            cached = (key, weight, bias)
            self._stacked_projection = cached
        both = torch.nn.functional.linear(token, cached[1], cached[2])
        return both[:, :self.rnn_width], both[:, self.rnn_width:]

    def _linear(self, layer: nn.Linear, x: Tensor) -> Tensor:
        """A Linear layer of the block; in training on the HIP path its bias gradient is summed by a
        kernel of the library instead of a generic reduction (the GEMMs are the BLAS library's either way)."""
        if self._linear_on_hip(layer, x):
            return hip_block_ops.hip_linear(x, layer.weight, layer.bias)
        return layer(x)

    def _linear_on_hip(self, layer: nn.Linear, x: Tensor) -> bool:
        return (torch.is_grad_enabled() and layer.bias is not None and layer.bias.requires_grad
                and x.is_cuda and x.dtype in hip_scan.SUPPORTED_DTYPES and layer.weight.dtype == x.dtype
                and self.rg_lru.scan_mode in ("hip", "fused", "auto") and x.numel() > 0
                and (self.rg_lru.scan_mode != "auto" or hip_scan.hip_scan_is_usable(x.device)))

    def _dense_conv(self, projected: Tensor, conv_state: Tensor | None, segment_pos: Tensor, need_state: bool = True):
        """All-tokens-active path (griffin/griffin.py:476-487): taps are masked per document."""
        if self._hip_block_ops_covers(projected):
            return hip_block_ops.hip_causal_conv(projected, conv_state, self.temporal_conv.weight,
                                                 self.temporal_conv.bias, segment_pos, need_state)
        return portable.causal_depthwise_conv(projected, conv_state, self.temporal_conv.weight,
                                              self.temporal_conv.bias, segment_pos)

    def _padded_conv(self, projected: Tensor, conv_state: Tensor, segment_pos: Tensor, active_mask: Tensor):
        """Right-padded batches (griffin/griffin.py:488-510): padding never enters the history."""
        if self._hip_block_ops_covers(projected):
            return hip_block_ops.hip_causal_conv_padded(projected, conv_state, self.temporal_conv.weight,
                                                        self.temporal_conv.bias, segment_pos, active_mask)
        taps = self.temporal_conv.weight[:, 0, :]
        history = self.conv_kernel_size - 1
        window = conv_state.to(projected)
        rows = []
        for t in range(projected.size(1)):
            live = active_mask[:, t, None]
            fresh = (segment_pos[:, t] == 0)[:, None, None] & live[:, :, None]
            window = window.masked_fill(fresh, 0.0)
            now = projected[:, t]
            value = now * taps[:, -1] + self.temporal_conv.bias
            if history:
                value = value + (window * taps[:, :history].T).sum(dim=1)
            rows.append(value.masked_fill(~live, 0.0))
            if history:
                advanced = torch.cat((window[:, 1:], now[:, None]), dim=1)
                window = torch.where(live[:, :, None], advanced, window)
        return torch.stack(rows, dim=1), window

    def forward(self, x: Tensor, cache: RecurrentBlockCache | None = None, segment_pos: Tensor | None = None,
                *, active_mask: Tensor | None = None, return_cache: bool = False):
        if x.dim() != 3:
            raise ValueError(f"RecurrentBlock expects [batch, sequence, width], got {tuple(x.shape)}")
        batch, steps = x.shape[:2]
        everything_active = active_mask is None
        if not everything_active:
            if active_mask.shape != (batch, steps):
                raise ValueError("active_mask must match the input [batch, sequence] dimensions")
            active_mask = active_mask.to(device=x.device, dtype=torch.bool)
        previous_position = None if cache is None else cache.segment_position
        if steps == 1 and self._hip_decode_covers(x, cache):
            return self._hip_decode(x, cache, segment_pos, active_mask, return_cache)
        segment_pos = _resolve_segment_positions(
            x, segment_pos, previous_position, None if everything_active else active_mask)

        if self._linear_on_hip(self.linear_x, x) and self._linear_on_hip(self.linear_y, x):
            projected, gate_input = hip_block_ops.hip_linear_pair(
                x, self.linear_x.weight, self.linear_x.bias, self.linear_y.weight, self.linear_y.bias)
        else:
            gate_input = self._linear(self.linear_y, x)
            projected = self._linear(self.linear_x, x)
        on_hip = self._hip_block_ops_covers(projected)
        # the HIP convolution takes "no carried state" as such; the portable path wants the zeros
        conv_state = (None if on_hip else self._empty_conv_state(projected)) if cache is None else cache.conv_state
        if conv_state is not None and conv_state.shape != (batch, self.conv_kernel_size - 1, self.rnn_width):
            raise ValueError("Recurrent convolution cache has an incompatible shape")
        dense = everything_active or bool(active_mask.all())
        default = _DEFAULT_POSITIONS.get((batch, steps, x.device))
        if dense and on_hip and self._hip_block_forward_covers(projected, gate_input, cache):
            # convolution, RG-LRU and output gate in one forward launch
            rnn_state = None if cache is None else cache.rnn_state
            needs_grad = torch.is_grad_enabled() and any(
                t is not None and t.requires_grad
                for t in (projected, gate_input, conv_state, rnn_state, self.temporal_conv.weight,
                          self.temporal_conv.bias, *self.rg_lru._gate_parameters()))
            gated, new_rnn_state, new_conv_state = hip_block_ops.hip_block_forward(
                projected, gate_input, conv_state, self.temporal_conv.weight, self.temporal_conv.bias, segment_pos,
                hip_scan.FIRST_TOKEN_RESET if (cache is None and default is not None and segment_pos is default[0]) else None,
                *self.rg_lru._gate_parameters(), rnn_state, self.rg_lru.c,
                None if needs_grad else self.rg_lru._prepared(projected.dtype, projected.device))
        else:
            if dense:
                recurrent_in, new_conv_state = self._dense_conv(projected, conv_state, segment_pos, return_cache)
            else:
                recurrent_in, new_conv_state = self._padded_conv(projected, conv_state, segment_pos, active_mask)
            recurrent_out, new_rnn_state = self.rg_lru(
                recurrent_in,
                None if cache is None else cache.rnn_state,
                reset_mask=default[1] if (default is not None and segment_pos is default[0]) else segment_pos == 0,
                active_mask=None if everything_active else active_mask,
                return_state=True,
            )
            if on_hip and gate_input.dtype == recurrent_out.dtype:
                gated = hip_block_ops.hip_gelu_gate(recurrent_out, gate_input)
            else:
                gated = recurrent_out * F.gelu(gate_input, approximate="tanh")
        output = self._linear(self.linear_out, gated)
        if not everything_active:
            output = output.masked_fill(~active_mask.unsqueeze(-1), 0.0)
        if return_cache:
            if everything_active:
                last_position = segment_pos[:, -1].clone()   # every token is active: the last one's position
            else:
                last_position = _last_active_position(segment_pos, active_mask, previous_position)
            return output, RecurrentBlockCache(new_rnn_state, new_conv_state, last_position)
        return output
