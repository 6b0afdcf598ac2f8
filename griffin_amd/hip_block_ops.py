"""PyTorch operators for the two elementwise stages around the RG-LRU inside the recurrent block: the
causal depthwise convolution that feeds it (griffin/griffin.py:474-487, the all-tokens-active path)
over ``rglru_hip_conv_fwd`` / ``rglru_hip_conv_bwd``, and the output gate ``h * gelu_tanh(v)``
(griffin/griffin.py:464, :520) over ``rglru_hip_gelu_gate_fwd`` / ``_bwd`` of librglru_hip.so.

There is no CPU fallback here: the operator raises when the library or a GPU is missing.
"""

from __future__ import annotations

import torch
from torch import Tensor
from torch.autograd.function import once_differentiable

from . import _lib
from .hip_scan import (FIRST_TOKEN_RESET, _DTYPE_CODES, _dtype_code, _flags_ptr, _on_device, _parameter_operands,
                       _prep_bytes, _ptr, _require_gpu, _stream_ptr, rglru_backward)


def max_kernel_size() -> int:
    """Largest convolution kernel size the HIP kernels cover."""
    return int(_lib.load().rglru_hip_conv_max_kernel_size())


def _parameter_operand(t: Tensor | None, like: torch.dtype) -> Tensor | None:
    """A parameter as the library reads it: its own type when that is fp32 or bf16, else converted."""
    if t is None:
        return None
    if t.dtype not in _DTYPE_CODES:
        t = t.to(like)
    return t.contiguous()


class _HipCausalConv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, u: Tensor, state: Tensor | None, weight: Tensor, bias: Tensor | None, segment_pos: Tensor):
        _require_gpu("hip_causal_conv", u, state, weight, bias, segment_pos)
        if u.dim() != 3:
            raise ValueError(f"hip_causal_conv expects [batch, sequence, width], got {tuple(u.shape)}")
        batch, steps, width = u.shape
        if weight.dim() != 3 or weight.size(0) != width or weight.size(1) != 1:
            raise ValueError("weight must be that of a depthwise Conv1d: [width, 1, kernel_size]")
        taps_count = weight.size(2)
        if bias is not None and bias.shape != (width,):
            raise ValueError("bias must have shape [width]")
        if state is not None and state.shape != (batch, taps_count - 1, width):
            raise ValueError("state must have shape [batch, kernel_size - 1, width]")
        if segment_pos.shape != (batch, steps):
            raise ValueError("segment_pos must have shape [batch, sequence]")
        code = _dtype_code(u.dtype)
        u_c = u.contiguous()
        state_c = None if state is None or taps_count == 1 else state.to(u.dtype).contiguous()
        taps = _parameter_operand(weight, u.dtype)
        if bias is not None and bias.dtype != taps.dtype:
            bias = bias.to(taps.dtype)
        bias_c = _parameter_operand(bias, u.dtype)
        pos = segment_pos.to(device=u.device, dtype=torch.int64).contiguous()
        out = torch.empty_like(u_c)
        lib = _lib.load()
        with _on_device(u.device):
            _lib.check(lib.rglru_hip_conv_fwd(
                _ptr(u_c), _ptr(state_c), _ptr(taps), _ptr(bias_c), _ptr(pos), _ptr(out), None,
                batch, steps, width, taps_count, code, _DTYPE_CODES[taps.dtype], _stream_ptr(u.device)),
                "rglru_hip_conv_fwd")
        ctx.save_for_backward(u_c, state_c, taps, pos)
        ctx.meta = (None if state is None else state.dtype, weight.dtype, None if bias is None else bias.dtype, weight.shape)
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dout: Tensor | None):
        if dout is None:
            return None, None, None, None, None
        u, state, taps, pos = ctx.saved_tensors
        return (*_conv_backward(u, state, taps, pos, dout, ctx.meta, ctx.needs_input_grad[:4]), None)


def _conv_backward(u: Tensor, state: Tensor | None, taps: Tensor, pos: Tensor, dout: Tensor, meta, needs,
                   du_out: Tensor | None = None):
    """Reverse mode of the dense convolution on contiguous operands: (du, dstate, dweight, dbias) in the types
    of the forward's arguments; ``meta`` = (state dtype, weight dtype, bias dtype, weight shape).  ``du_out``:
    where to write du instead of a new tensor -- [B, T, W] with unit stride along W and rows a common distance
    apart (a column range of a wider matrix)."""
    state_dtype, weight_dtype, bias_dtype, weight_shape = meta
    batch, steps, width = u.shape
    taps_count = weight_shape[2]
    code = _dtype_code(u.dtype)
    dout_c = dout.to(u.dtype).contiguous()
    lib = _lib.load()
    need_u, need_state, need_w, need_b = needs
    grad_dtype = taps.dtype
    du = torch.empty_like(u) if du_out is None else du_out
    dstate = torch.empty_like(state) if (need_state and state is not None) else None
    dtaps = torch.empty(width, taps_count, device=u.device, dtype=grad_dtype) if need_w else None
    dbias = torch.empty(width, device=u.device, dtype=grad_dtype) if (need_b and bias_dtype is not None) else None
    scratch = torch.empty(lib.rglru_hip_conv_scratch_bytes(batch, steps, width, taps_count),
                          device=u.device, dtype=torch.uint8)
    with _on_device(u.device):
        _lib.check(lib.rglru_hip_conv_bwd(
            _ptr(u), _ptr(state), _ptr(taps), _ptr(pos), _ptr(dout_c), _ptr(scratch), _ptr(du), du.stride(1),
            _ptr(dstate), _ptr(dtaps), _ptr(dbias),
            batch, steps, width, taps_count, code, _DTYPE_CODES[taps.dtype], _DTYPE_CODES[grad_dtype],
            _stream_ptr(u.device)), "rglru_hip_conv_bwd")
    dweight = None if dtaps is None else dtaps.view(weight_shape).to(weight_dtype)
    if dbias is not None:
        dbias = dbias.to(bias_dtype)
    if need_state and state_dtype is not None:
        dstate = (u.new_zeros(batch, taps_count - 1, width) if dstate is None else dstate).to(state_dtype)
    return (du if need_u else None), dstate, dweight, dbias


def hip_causal_conv(u: Tensor, state: Tensor | None, weight: Tensor, bias: Tensor | None,
                    segment_pos: Tensor, need_state: bool = True) -> tuple[Tensor, Tensor | None]:
    """Depthwise causal convolution with per-document tap masking.

    ``u`` [B, T, W]; ``state`` [B, K-1, W] or None (zeros); ``weight`` [W, 1, K] and ``bias`` [W] of a
    depthwise ``nn.Conv1d``; ``segment_pos`` [B, T] integer positions (a tap reaching back ``lag`` tokens
    contributes only where ``segment_pos >= lag``).  Returns ``(out [B, T, W], new_state [B, K-1, W])``;
    ``new_state`` is the last K-1 rows of ``cat(state, u)`` (griffin/griffin.py:487), or None when the
    caller says it does not need it (a training step that returns no cache).
    """
    out = _HipCausalConv.apply(u, state, weight, bias, segment_pos)
    if not need_state:
        return out, None
    history = weight.size(2) - 1
    steps = u.size(1)
    if steps >= history:
        new_state = u[:, steps - history:].clone()
    else:
        previous = u.new_zeros(u.size(0), history, u.size(2)) if state is None else state.to(u.dtype)
        new_state = torch.cat((previous[:, steps:], u), dim=1)
    return out, new_state


class _HipCausalConvPadded(torch.autograd.Function):
    @staticmethod
    def forward(ctx, u: Tensor, state: Tensor | None, weight: Tensor, bias: Tensor | None,
                segment_pos: Tensor, active_mask: Tensor):
        _require_gpu("hip_causal_conv_padded", u, state, weight, bias, segment_pos, active_mask)
        if u.dim() != 3:
            raise ValueError(f"hip_causal_conv_padded expects [batch, sequence, width], got {tuple(u.shape)}")
        batch, steps, width = u.shape
        if weight.dim() != 3 or weight.size(0) != width or weight.size(1) != 1:
            raise ValueError("weight must be that of a depthwise Conv1d: [width, 1, kernel_size]")
        taps_count = weight.size(2)
        if state is not None and state.shape != (batch, taps_count - 1, width):
            raise ValueError("state must have shape [batch, kernel_size - 1, width]")
        if segment_pos.shape != (batch, steps) or active_mask.shape != (batch, steps):
            raise ValueError("segment_pos and active_mask must have shape [batch, sequence]")
        code = _dtype_code(u.dtype)
        u_c = u.contiguous()
        state_c = None if state is None or taps_count == 1 else state.to(u.dtype).contiguous()
        taps = _parameter_operand(weight, u.dtype)
        bias_c = None if bias is None else _parameter_operand(bias.to(taps.dtype), u.dtype)
        pos = segment_pos.to(device=u.device, dtype=torch.int64).contiguous()
        live = active_mask.to(device=u.device, dtype=torch.uint8).contiguous()
        lib = _lib.load()
        with _on_device(u.device):
            out = torch.empty_like(u_c)
            new_state = u.new_empty(batch, taps_count - 1, width)
            scratch = torch.empty(lib.rglru_hip_conv_padded_scratch_bytes(batch, steps), dtype=torch.uint8, device=u.device)
            _lib.check(lib.rglru_hip_conv_padded_fwd(
                _ptr(u_c), _ptr(state_c), _ptr(taps), _ptr(bias_c), _ptr(pos), _ptr(live), _ptr(scratch), _ptr(out),
                _ptr(new_state) if taps_count > 1 else None,
                batch, steps, width, taps_count, code, _DTYPE_CODES[taps.dtype], _stream_ptr(u.device)),
                "rglru_hip_conv_padded_fwd")
        ctx.save_for_backward(u_c, state_c, taps, pos, live)
        ctx.meta = (None if state is None else state.dtype, weight.dtype, None if bias is None else bias.dtype, weight.shape)
        ctx.mark_non_differentiable(new_state)
        ctx.set_materialize_grads(False)
        return out, new_state

    @staticmethod
    @once_differentiable
    def backward(ctx, dout: Tensor | None, _dstate_out):
        u, state, taps, pos, live = ctx.saved_tensors
        state_dtype, weight_dtype, bias_dtype, weight_shape = ctx.meta
        if dout is None:
            return None, None, None, None, None, None
        batch, steps, width = u.shape
        taps_count = weight_shape[2]
        dout_c = dout.to(u.dtype).contiguous()
        lib = _lib.load()
        need_u, need_state, need_w, need_b = ctx.needs_input_grad[:4]
        grad_dtype = taps.dtype
        with _on_device(u.device):
            du = torch.empty_like(u)
            dstate = u.new_empty(batch, taps_count - 1, width) if (need_state and taps_count > 1) else None
            dtaps = torch.empty(width, taps_count, device=u.device, dtype=grad_dtype) if need_w else None
            dbias = torch.empty(width, device=u.device, dtype=grad_dtype) if (need_b and bias_dtype is not None) else None
            index = torch.empty(lib.rglru_hip_conv_padded_scratch_bytes(batch, steps), dtype=torch.uint8, device=u.device)
            scratch = torch.empty(lib.rglru_hip_conv_scratch_bytes(batch, steps, width, taps_count),
                                  device=u.device, dtype=torch.uint8)
            _lib.check(lib.rglru_hip_conv_padded_bwd(
                _ptr(u), _ptr(state), _ptr(taps), _ptr(pos), _ptr(live), _ptr(dout_c), _ptr(index), _ptr(scratch),
                _ptr(du), _ptr(dstate), _ptr(dtaps), _ptr(dbias),
                batch, steps, width, taps_count, _dtype_code(u.dtype), _DTYPE_CODES[taps.dtype],
                _DTYPE_CODES[grad_dtype], _stream_ptr(u.device)), "rglru_hip_conv_padded_bwd")
        dweight = None if dtaps is None else dtaps.view(weight_shape).to(weight_dtype)
        if dbias is not None:
            dbias = dbias.to(bias_dtype)
        if need_state and state_dtype is not None:
            dstate = (u.new_zeros(batch, taps_count - 1, width) if dstate is None else dstate).to(state_dtype)
        else:
            dstate = None
        return (du if need_u else None), dstate, dweight, dbias, None, None


def hip_causal_conv_padded(u: Tensor, state: Tensor | None, weight: Tensor, bias: Tensor | None,
                           segment_pos: Tensor, active_mask: Tensor) -> tuple[Tensor, Tensor]:
    """The convolution over right-padded batches (griffin/griffin.py:488-510): inactive tokens give zeros
    and stay out of the window of previous inputs, an active token at position 0 clears the window.
    Returns ``(out [B, T, W], new_state [B, K-1, W])``.  ``out`` is differentiable in ``u``, ``state``,
    ``weight`` and ``bias``; ``new_state`` (the cache handed to the next call) carries no gradient."""
    return _HipCausalConvPadded.apply(u, state, weight, bias, segment_pos, active_mask)


class _HipGeluGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h: Tensor, v: Tensor) -> Tensor:
        _require_gpu("hip_gelu_gate", h, v)
        if h.shape != v.shape:
            raise ValueError(f"hip_gelu_gate expects equal shapes, got {tuple(h.shape)} and {tuple(v.shape)}")
        if h.dtype != v.dtype:
            raise TypeError(f"hip_gelu_gate expects equal dtypes, got {h.dtype} and {v.dtype}")
        code = _dtype_code(h.dtype)
        h_c, v_c = h.contiguous(), v.contiguous()
        out = torch.empty_like(h_c)
        if h_c.numel():
            with _on_device(h.device):
                _lib.check(_lib.load().rglru_hip_gelu_gate_fwd(
                    _ptr(h_c), _ptr(v_c), _ptr(out), h_c.numel(), code, _stream_ptr(h.device)),
                    "rglru_hip_gelu_gate_fwd")
        ctx.save_for_backward(h_c, v_c)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dout: Tensor):
        h, v = ctx.saved_tensors
        dout_c = dout.to(h.dtype).contiguous()
        dh, dv = torch.empty_like(h), torch.empty_like(v)
        if h.numel():
            with _on_device(h.device):
                _lib.check(_lib.load().rglru_hip_gelu_gate_bwd(
                    _ptr(dout_c), _ptr(h), _ptr(v), _ptr(dh), _ptr(dv), h.numel(), h.size(-1), 0, _dtype_code(h.dtype),
                    _stream_ptr(h.device)), "rglru_hip_gelu_gate_bwd")
        return dh, dv


def hip_gelu_gate(h: Tensor, v: Tensor) -> Tensor:
    """``h * gelu(v, approximate="tanh")`` in one pass, differentiable in both arguments."""
    return _HipGeluGate.apply(h, v)


def hip_block_forward_covers(width: int, blocks: int, taps_count: int, dtype: torch.dtype) -> bool:
    """Whether ``hip_block_forward`` has a kernel for this shape (rglru_hip_block_fwd_path)."""
    if dtype not in _DTYPE_CODES or blocks <= 0 or width % blocks:
        return False
    return bool(_lib.load().rglru_hip_block_fwd_path(width, blocks, taps_count, _DTYPE_CODES[dtype]))


def _row_view(t: Tensor) -> Tensor:
    """[B, T, W] as the library addresses it: channels contiguous, one row stride for all tokens."""
    batch, steps, width = t.shape
    if t.stride(2) == 1 and t.stride(1) >= width and (batch == 1 or t.stride(0) == steps * t.stride(1)) \
            and (t.stride(1) * t.element_size()) % 16 == 0 and t.data_ptr() % 16 == 0:
        return t
    return t.contiguous()


class _HipBlockForward(torch.autograd.Function):
    """conv -> RG-LRU -> output gate of the recurrent block in one forward launch (rglru_hip_block_fwd); the
    backward pass runs the three reverse kernels one after the other on the x and y the forward kept."""

    @staticmethod
    def forward(ctx, u, v, conv_state, weight, bias, segment_pos, flags, w_a, b_a, w_x, b_x, lam, h0, c, prep):
        _require_gpu("hip_block_forward", u, v, conv_state, weight, bias, segment_pos, w_a, b_a, w_x, b_x, lam, h0)
        if u.dim() != 3 or u.shape != v.shape or u.dtype != v.dtype:
            raise ValueError("hip_block_forward expects two [batch, sequence, width] tensors of one dtype")
        B, T, W = u.shape
        nb = w_a.shape[0]
        taps_count = weight.size(2)
        if weight.dim() != 3 or weight.size(0) != W or weight.size(1) != 1:
            raise ValueError("weight must be that of a depthwise Conv1d: [width, 1, kernel_size]")
        if conv_state is not None and conv_state.shape != (B, taps_count - 1, W):
            raise ValueError("conv_state must have shape [batch, kernel_size - 1, width]")
        if segment_pos.shape != (B, T):
            raise ValueError("segment_pos must have shape [batch, sequence]")
        if h0 is not None and h0.shape != (B, W):
            raise ValueError(f"initial state must have shape ({B}, {W}), got {tuple(h0.shape)}")
        first_reset = flags is FIRST_TOKEN_RESET
        if flags is not None and not first_reset and (
                flags.shape != (B, T) or flags.dtype != torch.uint8 or not flags.is_contiguous()):
            raise ValueError("flags must be a contiguous uint8 tensor of shape [batch, sequence]")
        code = _dtype_code(u.dtype)
        lib = _lib.load()
        training = any(ctx.needs_input_grad)
        u_r, v_r = _row_view(u), _row_view(v)
        state_c = None if conv_state is None or taps_count == 1 else conv_state.to(u.dtype).contiguous()
        taps = _parameter_operand(weight.detach(), u.dtype)
        bias_c = None if bias is None else _parameter_operand(bias.detach().to(taps.dtype), u.dtype)
        pos = segment_pos.to(device=u.device, dtype=torch.int64).contiguous()
        h0c = None if h0 is None else h0.detach().to(torch.float32).contiguous()
        device = u.device
        with _on_device(device):
            stream = _stream_ptr(device)
            if flags is None:
                flags = hip_block_flags(pos)
            gated = u.new_empty(B, T, W)
            x_conv = u.new_empty(B, T, W) if training else None
            y = u.new_empty(B, T, W) if training else None
            new_conv = u.new_empty(B, taps_count - 1, W)
            h_last = torch.empty(B, W, dtype=torch.float32, device=device)
            ws = torch.empty(lib.rglru_hip_workspace_bytes(B, T, W, nb), dtype=torch.uint8, device=device)
            tail = (_ptr(h0c), _flags_ptr(flags), _ptr(x_conv), _ptr(y), _ptr(gated), _ptr(new_conv) if taps_count > 1 else None,
                    _ptr(h_last), _ptr(ws), B, T, W, nb, code, stream)
            if training or prep is None:
                operands, vec_code = _parameter_operands(w_a, b_a, w_x, b_x, lam, u.dtype)
                image = torch.empty(_prep_bytes(W, nb, code), dtype=torch.uint8, device=device)
                _lib.check(lib.rglru_hip_prepare_block_fwd(
                    *(t.data_ptr() for t in operands), float(c), vec_code, image.data_ptr(),
                    _ptr(u_r), u_r.stride(1), _ptr(v_r), v_r.stride(1), _ptr(state_c), _ptr(taps), _ptr(bias_c), taps_count,
                    *tail), "rglru_hip_prepare_block_fwd")
            else:
                image = prep.image
                _lib.check(lib.rglru_hip_block_fwd(
                    _ptr(u_r), u_r.stride(1), _ptr(v_r), v_r.stride(1), _ptr(state_c), _ptr(taps), _ptr(bias_c), taps_count,
                    _DTYPE_CODES[taps.dtype], image.data_ptr(), *tail), "rglru_hip_block_fwd")
        if training:
            ctx.save_for_backward(u_r, v_r, state_c, taps, pos, x_conv, y, w_a, w_x, h0c, None if first_reset else flags, ws, image)
            ctx.first_reset = first_reset
            ctx.conv_meta = (None if conv_state is None else conv_state.dtype, weight.dtype,
                             None if bias is None else bias.dtype, weight.shape)
            ctx.param_dtypes = (w_a.dtype, b_a.dtype, w_x.dtype, b_x.dtype, lam.dtype)
            ctx.h0_dtype = None if h0 is None else h0.dtype
        ctx.mark_non_differentiable(new_conv)
        ctx.set_materialize_grads(False)
        return gated, h_last, new_conv

    @staticmethod
    @once_differentiable
    def backward(ctx, dgated, dh_last, _dnew_conv):
        u, v, state, taps, pos, x_conv, y, w_a, w_x, h0c, flags, ws, image = ctx.saved_tensors
        if ctx.first_reset:
            flags = FIRST_TOKEN_RESET
        need = ctx.needs_input_grad
        lib = _lib.load()
        dy = dv = du_out = None
        if dgated is not None:
            dout_c = dgated.to(y.dtype).contiguous()
            v_c = v.contiguous()
            B, T, W = y.shape
            dy = torch.empty_like(y)
            if need[0] and need[1] and (W * y.element_size()) % 16 == 0 and B * T * 2 * W * y.element_size() < 2 ** 31:
                # The gradients of the two projections as the halves of ONE [B, T, 2 W] matrix: the Linear layers'
                # backward then runs one GEMM each for dx and dW and one column sum (hip_linear_pair).
                both = y.new_empty(B, T, 2 * W)
                du_out, dv = both[..., :W], both[..., W:]
            else:
                dv = torch.empty_like(v_c)
            with _on_device(y.device):
                _lib.check(lib.rglru_hip_gelu_gate_bwd(
                    _ptr(dout_c), _ptr(y), _ptr(v_c), _ptr(dy), _ptr(dv), y.numel(), W, dv.stride(1), _dtype_code(y.dtype),
                    _stream_ptr(y.device)), "rglru_hip_gelu_gate_bwd")
        dx, dw_a, db_a, dw_x, db_x, dlam, dh0 = rglru_backward(
            x_conv, y, w_a, w_x, h0c, flags, ws, image, dy, dh_last, ctx.param_dtypes, need[12])
        u_c = u.contiguous()
        du, dstate, dweight, dbias = _conv_backward(u_c, state, taps, pos, dx, ctx.conv_meta, (need[0], need[2], need[3], need[4]),
                                                    du_out)
        return (du, dv if need[1] else None, dstate, dweight, dbias, None, None, dw_a, db_a, dw_x, db_x, dlam,
                None if dh0 is None else dh0.to(ctx.h0_dtype), None, None)


def hip_block_flags(segment_pos: Tensor) -> Tensor:
    """Per-token flag bytes of ``hip_block_forward`` for integer positions [B, T] (rglru_hip_block_flags):
    reset where a document starts (position 0) and, in bits 2-3, how many convolution lags reach in front
    of the token's document."""
    _require_gpu("hip_block_flags", segment_pos)
    pos = segment_pos.to(torch.int64).contiguous()
    flags = torch.empty(pos.shape, dtype=torch.uint8, device=pos.device)
    if pos.numel():
        with _on_device(pos.device):
            _lib.check(_lib.load().rglru_hip_block_flags(_ptr(pos), _ptr(flags), pos.numel(), _stream_ptr(pos.device)),
                       "rglru_hip_block_flags")
    return flags


def hip_block_forward(u: Tensor, v: Tensor, conv_state: Tensor | None, weight: Tensor, bias: Tensor | None,
                      segment_pos: Tensor, flags: Tensor | None, w_a: Tensor, b_a: Tensor, w_x: Tensor, b_x: Tensor,
                      lam: Tensor, h0: Tensor | None, c: float = 8.0, prep=None):
    """``gelu_tanh(v) * RG_LRU(conv(u))`` for whole sequences with every token active, one forward launch.

    ``u``, ``v`` [B, T, W]: the block's two projections; ``conv_state`` [B, K-1, W] or None; ``weight``
    [W, 1, K], ``bias`` [W] of the depthwise ``nn.Conv1d`` (K <= 4); ``segment_pos`` [B, T]; ``flags``:
    ``hip_block_flags(segment_pos)`` if the caller has it already, ``hip_scan.FIRST_TOKEN_RESET`` when the
    positions are 0 .. T-1 in every row (no flag tensor is needed then), else None; the five RG-LRU parameters, ``h0`` [B, W] or None; ``prep``: a prepared parameter image to use
    when no gradient is asked for.  Returns ``(gated [B, T, W], final state [B, W] fp32, new_conv_state
    [B, K-1, W])``; differentiable in u, v, the parameters, conv_state and h0.
    """
    gated, h_last, new_conv = _HipBlockForward.apply(u, v, conv_state, weight, bias, segment_pos, flags,
                                                     w_a, b_a, w_x, b_x, lam, h0, c, prep)
    if torch.is_grad_enabled() and (u.requires_grad or (conv_state is not None and conv_state.requires_grad)):
        # the carried rows as a differentiable function of u and conv_state (the kernel's copy carries no gradient)
        history, steps = weight.size(2) - 1, u.size(1)
        if steps >= history:
            new_conv = u[:, steps - history:].clone()
        else:
            previous = u.new_zeros(u.size(0), history, u.size(2)) if conv_state is None else conv_state.to(u.dtype)
            new_conv = torch.cat((previous[:, steps:], u), dim=1)
    return gated, h_last, new_conv


def hip_block_decode_step(u: Tensor, v: Tensor, conv_state: Tensor | None, weight: Tensor, bias: Tensor | None,
                          prev_pos: Tensor | None, segment_pos: Tensor | None, active: Tensor | None,
                          prep, rnn_state: Tensor | None):
    """One token per row through conv -> RG-LRU step -> output gate (no autograd), two kernel launches.

    ``u``, ``v`` [B, W]: the block's two projections of the token (rows may be strided views of one wider
    buffer); ``conv_state`` [B, K-1, W] or None;
    ``prev_pos`` [B] (None: -1) or explicit ``segment_pos`` [B]; ``active`` [B] uint8 or None (all
    active); ``prep`` the prepared RG-LRU parameters; ``rnn_state`` [B, W] fp32 or None (zeros).
    Returns ``(gated [B, W], new_rnn_state, new_conv_state, new_pos)``; the inputs are left untouched.
    """
    _require_gpu("hip_block_decode_step", u, v, conv_state, weight, bias, prev_pos, segment_pos, active, rnn_state)
    if u.dim() != 2 or u.shape != v.shape or u.dtype != v.dtype:
        raise ValueError("hip_block_decode_step expects two [batch, width] tensors of one dtype")
    batch, width = u.shape
    if width != prep.width or u.dtype != prep.dtype:
        raise ValueError("the prepared RG-LRU parameters do not match the activations")
    taps_count = weight.size(2)
    code = _dtype_code(u.dtype)
    # rows may be views into a wider buffer (the two halves of one fused projection)
    u_c = u if u.stride(1) == 1 and u.stride(0) >= width else u.contiguous()
    v_c = v if v.stride(1) == 1 and v.stride(0) >= width else v.contiguous()
    state_c = None if conv_state is None or taps_count == 1 else conv_state.to(u.dtype).contiguous()
    taps = _parameter_operand(weight.detach(), u.dtype)
    bias_c = None if bias is None else _parameter_operand(bias.detach().to(taps.dtype), u.dtype)
    device = u.device
    lib = _lib.load()
    with _on_device(device):
        x_conv = u.new_empty(batch, width)
        new_conv = u.new_empty(batch, taps_count - 1, width)
        new_pos = torch.empty(batch, dtype=torch.int64, device=device)
        flags = torch.empty(batch, dtype=torch.uint8, device=device)
        h_in = (torch.zeros(batch, width, dtype=torch.float32, device=device) if rnn_state is None
                else rnn_state.to(torch.float32).contiguous())
        h_out = torch.empty_like(h_in)
        out = u.new_empty(batch, width)
        stream = _stream_ptr(device)
        _lib.check(lib.rglru_hip_decode_prepare(
            _ptr(u_c), u_c.stride(0), _ptr(state_c), _ptr(taps), _ptr(bias_c), _ptr(prev_pos), _ptr(segment_pos), _ptr(active),
            _ptr(x_conv), _ptr(new_conv) if taps_count > 1 else None, _ptr(new_pos), _ptr(flags),
            batch, width, taps_count, code, _DTYPE_CODES[taps.dtype], stream), "rglru_hip_decode_prepare")
        _lib.check(lib.rglru_hip_step_gated(
            _ptr(x_conv), prep.image.data_ptr(), _ptr(h_in), _ptr(h_out), _ptr(flags), _ptr(v_c), v_c.stride(0),
            _ptr(out), batch, width, prep.blocks, code, stream), "rglru_hip_step_gated")
    return out, h_out, new_conv, new_pos


class _HipLinear(torch.autograd.Function):
    """``F.linear`` whose bias gradient is summed by ``rglru_hip_colsum`` (the two GEMMs of the backward
    pass stay with the BLAS library, as in ``nn.Linear``)."""

    @staticmethod
    def forward(ctx, x: Tensor, weight: Tensor, bias: Tensor | None) -> Tensor:
        ctx.save_for_backward(x, weight)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    @once_differentiable
    def backward(ctx, dy: Tensor):
        x, weight = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad
        dx = torch.matmul(dy, weight.to(dy.dtype)) if need_x else None
        dw, db = _linear_parameter_grads(x, weight, dy, need_w, ctx.bias_dtype if need_b else None)
        return dx, dw, db


def _sum_sets(sets: Tensor) -> Tensor:
    """``sets.sum(0)`` for a contiguous [sets, ...] tensor on the GPU by a kernel of the library (one pass over the
    sets, 16-byte accesses; the generic reduction takes about three times as long for eight sets of a weight
    gradient); anything else goes to ``sum``."""
    if not sets.is_cuda or sets.dtype not in _DTYPE_CODES or not sets.is_contiguous() or sets.numel() == 0:
        return sets.sum(0)
    lib = _lib.load()
    with _on_device(sets.device):
        out = torch.empty(sets.shape[1:], dtype=sets.dtype, device=sets.device)
        _lib.check(lib.rglru_hip_sum_sets(_ptr(sets), _ptr(out), sets.size(0), out.numel(), _dtype_code(sets.dtype),
                                          _stream_ptr(sets.device)), "rglru_hip_sum_sets")
    return out


def _linear_parameter_grads(x: Tensor, weight: Tensor, dy: Tensor, need_w: bool, bias_dtype):
    """(dW, db) of ``y = x W^T + b`` for the incoming ``dy``; ``bias_dtype`` None skips db."""
    dy2 = dy.reshape(-1, dy.size(-1))
    dw = db = None
    if need_w:
        x2 = x.reshape(-1, x.size(-1)).to(dy.dtype)
        rows = dy2.size(0)
        # dW = dy^T x contracts over all tokens: one GEMM with K = rows runs at a fraction of the rate of
        # the same work as a batch of GEMMs with K = 2048 whose results are added (100 us against 43 us
        # for 16384 x 1024 x 768 in bf16 on this library), so long contractions are split
        chunks = rows // 2048 if (rows % 2048 == 0 and dy2.is_contiguous() and x2.is_contiguous()) else 1
        while chunks > 16 and chunks % 2 == 0:
            chunks //= 2
        if chunks > 1:
            per = rows // chunks
            dw = _sum_sets(torch.bmm(dy2.view(chunks, per, -1).transpose(1, 2), x2.view(chunks, per, -1)))
        else:
            dw = torch.mm(dy2.t(), x2)
        dw = dw.to(weight.dtype)
    if bias_dtype is not None:
        rows, width = dy2.shape
        dy_c = dy2.contiguous()
        out_dtype = bias_dtype if bias_dtype in _DTYPE_CODES else torch.float32
        lib = _lib.load()
        with _on_device(dy.device):
            db = torch.empty(width, dtype=out_dtype, device=dy.device)
            scratch = torch.empty(lib.rglru_hip_colsum_scratch_bytes(rows, width), dtype=torch.uint8, device=dy.device)
            _lib.check(lib.rglru_hip_colsum(_ptr(dy_c), _ptr(scratch), _ptr(db), rows, width, _dtype_code(dy.dtype),
                                            _DTYPE_CODES[out_dtype], _stream_ptr(dy.device)), "rglru_hip_colsum")
        db = db.to(bias_dtype)
    return dw, db


def _stacked_halves(a: Tensor | None, b: Tensor | None) -> Tensor | None:
    """The [rows, 2 W] matrix whose column halves ``a`` and ``b`` ([..., W] each) are, or None if they are not
    laid out that way (same storage, b starts W elements behind a, rows 2 W elements apart)."""
    if a is None or b is None or a.shape != b.shape or a.dtype != b.dtype or a.dim() < 2 or a.numel() == 0:
        return None
    width = a.size(-1)
    if a.stride() != b.stride() or a.stride(-1) != 1 or b.storage_offset() != a.storage_offset() + width:
        return None
    if a.untyped_storage().data_ptr() != b.untyped_storage().data_ptr():
        return None
    expect = 2 * width                                       # every leading axis must continue the rows of the one before
    for size, stride in zip(reversed(a.shape[:-1]), reversed(a.stride()[:-1])):
        if size != 1 and stride != expect:
            return None
        expect *= size
    rows = a.numel() // width
    return torch.as_strided(a, (rows, 2 * width), (2 * width, 1), a.storage_offset())


class _HipLinearPair(torch.autograd.Function):
    """Two Linear layers on one input (the block's two branches).  Their input gradients are one GEMM that
    accumulates into the other's result instead of two results and an addition."""

    @staticmethod
    def forward(ctx, x: Tensor, w1: Tensor, b1: Tensor | None, w2: Tensor, b2: Tensor | None):
        ctx.save_for_backward(x, w1, w2)
        ctx.bias_dtypes = (None if b1 is None else b1.dtype, None if b2 is None else b2.dtype)
        ctx.set_materialize_grads(False)
        return torch.nn.functional.linear(x, w1, b1), torch.nn.functional.linear(x, w2, b2)

    @staticmethod
    @once_differentiable
    def backward(ctx, dy1: Tensor | None, dy2: Tensor | None):
        x, w1, w2 = ctx.saved_tensors
        need_x, need_w1, need_b1, need_w2, need_b2 = ctx.needs_input_grad
        both = _stacked_halves(dy1, dy2)
        if (both is not None and w1.dtype == w2.dtype and w1.shape == w2.shape and need_w1 == need_w2 and need_b1 == need_b2
                and ctx.bias_dtypes[0] == ctx.bias_dtypes[1]):
            # dy1 | dy2 are the column halves of one matrix (hip_block_forward's backward writes them so): one
            # GEMM for dx against the stacked weights, one for both weight gradients, one column sum.  At 16384
            # rows, 768 -> 2 x 1024: 49 against 65 us (dx), 60 against 83 us (dW), two launches instead of four (db).
            n = w1.size(0)
            dx = torch.mm(both, torch.cat((w1, w2)).to(both.dtype)).view(x.shape) if need_x else None
            dw, db = _linear_parameter_grads(x, w1, both, need_w1, ctx.bias_dtypes[0] if need_b1 else None)
            return (dx, None if dw is None else dw[:n], None if db is None else db[:n],
                    None if dw is None else dw[n:], None if db is None else db[n:])
        dx = None
        if need_x:
            for dy, w in ((dy1, w1), (dy2, w2)):
                if dy is None:
                    continue
                flat = dy.reshape(-1, dy.size(-1))
                if dx is None:
                    dx = torch.mm(flat, w.to(dy.dtype))
                else:
                    dx.addmm_(flat, w.to(dy.dtype))
            dx = None if dx is None else dx.view(x.shape)
        dw1 = db1 = dw2 = db2 = None
        if dy1 is not None:
            dw1, db1 = _linear_parameter_grads(x, w1, dy1, need_w1, ctx.bias_dtypes[0] if need_b1 else None)
        if dy2 is not None:
            dw2, db2 = _linear_parameter_grads(x, w2, dy2, need_w2, ctx.bias_dtypes[1] if need_b2 else None)
        return dx, dw1, db1, dw2, db2


def hip_linear(x: Tensor, weight: Tensor, bias: Tensor | None) -> Tensor:
    """``x @ weight.T + bias`` (griffin/griffin.py:379-389, the block's Linear layers) with the bias
    gradient reduced by a kernel of this library; differentiable in all three arguments."""
    _require_gpu("hip_linear", x, weight, bias)
    _dtype_code(x.dtype)
    return _HipLinear.apply(x, weight, bias)


def hip_linear_pair(x: Tensor, w1: Tensor, b1: Tensor | None, w2: Tensor, b2: Tensor | None) -> tuple[Tensor, Tensor]:
    """``(x @ w1.T + b1, x @ w2.T + b2)``: two ``hip_linear`` calls whose backward passes share the input
    gradient (the second GEMM accumulates into the first one's result)."""
    _require_gpu("hip_linear_pair", x, w1, b1, w2, b2)
    _dtype_code(x.dtype)
    return _HipLinearPair.apply(x, w1, b1, w2, b2)


class _HipRMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, g: Tensor, eps: float) -> Tensor:
        _require_gpu("hip_rmsnorm", x, g)
        if g.dim() != 1 or x.dim() < 1 or x.size(-1) != g.numel():
            raise ValueError(f"hip_rmsnorm expects a scale of shape [{x.size(-1) if x.dim() else '?'}], got {tuple(g.shape)}")
        code = _dtype_code(x.dtype)
        width = x.size(-1)
        x_c = x.contiguous()
        rows = x_c.numel() // width
        scale = _parameter_operand(g.detach(), x.dtype)
        lib = _lib.load()
        with _on_device(x.device):
            y = torch.empty_like(x_c)
            inv = torch.empty(rows, dtype=torch.float32, device=x.device)
            if rows:
                _lib.check(lib.rglru_hip_rmsnorm_fwd(_ptr(x_c), _ptr(scale), _ptr(y), _ptr(inv), rows, width, float(eps), code,
                                                     _DTYPE_CODES[scale.dtype], _stream_ptr(x.device)), "rglru_hip_rmsnorm_fwd")
        ctx.save_for_backward(x_c, scale, inv)
        ctx.scale_dtype = g.dtype
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy: Tensor):
        x, scale, inv = ctx.saved_tensors
        width = x.size(-1)
        rows = x.numel() // width
        dy_c = dy.to(x.dtype).contiguous()
        lib = _lib.load()
        need_g = ctx.needs_input_grad[1]
        with _on_device(x.device):
            dx = torch.empty_like(x)
            dg = torch.empty(width, dtype=scale.dtype, device=x.device) if need_g else None
            if rows:
                scratch = torch.empty(lib.rglru_hip_rmsnorm_scratch_bytes(rows, width), dtype=torch.uint8, device=x.device)
                _lib.check(lib.rglru_hip_rmsnorm_bwd(_ptr(x), _ptr(scale), _ptr(inv), _ptr(dy_c), _ptr(scratch), _ptr(dx), _ptr(dg),
                                                     rows, width, _dtype_code(x.dtype), _DTYPE_CODES[scale.dtype],
                                                     _DTYPE_CODES[scale.dtype], _stream_ptr(x.device)), "rglru_hip_rmsnorm_bwd")
            elif dg is not None:
                dg.zero_()
        return dx, (None if dg is None else dg.to(ctx.scale_dtype)), None


def rmsnorm_max_width(dtype: torch.dtype, aligned: bool = True) -> int:
    return int(_lib.load().rglru_hip_rmsnorm_max_width(_dtype_code(dtype), 1 if aligned else 0))


def hip_rmsnorm(x: Tensor, g: Tensor, eps: float = 1e-6) -> Tensor:
    """``x * rsqrt(mean(x^2, -1) + eps) * (1 + g)`` (griffin/griffin.py:68-80), differentiable in x and g."""
    return _HipRMSNorm.apply(x, g, eps)
