"""PyTorch operators over the C ABI of librglru_hip.so, and the one-time device self-test.

Mirrors the reference's operator module (griffin/triton_scan.py): ``hip_rglru_scan`` has the
contract of ``fused_rglru_scan`` (:274-276), ``hip_scan_available`` / ``hip_scan_is_usable`` those of
``triton_scan_available`` / ``triton_scan_is_usable`` (:125-127, :180-204).  ``hip_rglru`` is one
fusion level higher: it takes x and the RG-LRU parameters and runs gates + scan in one kernel.

There is no CPU fallback in this file: every operator raises when the library or a GPU is missing.
"""

from __future__ import annotations

import weakref

import threading
import warnings

import torch
from torch import Tensor
from torch.autograd.function import once_differentiable

from . import _lib

_VALIDATION_LOCK = threading.Lock()
_VALIDATED: dict[int, bool] = {}

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16)


def hip_scan_available() -> bool:
    """Whether the HIP library is built and loads (reference: triton_scan_available)."""
    return _lib.available()


def set_reproducible(enable: bool) -> bool:
    """Bit-reproducible results from run to run (rglru_hip_set_reproducible): every chunk of a sequence then
    takes its carry from the finished chunk before it instead of combining whatever its neighbours have
    published so far.  Slower, mostly for long sequences; off by default.  Returns the previous setting."""
    return bool(_lib.load().rglru_hip_set_reproducible(1 if enable else 0))


def set_chain_forward(mode: int) -> int:
    """Choice of the forward kernel for bf16 storage and gate blocks of 32, 64 or 128 channels
    (rglru_hip_set_chain_forward): 0 = by shape (default), 1 = always tiles with a look-back between
    workgroups, 2 = one workgroup per chain whenever that kernel covers the shape.  Returns the previous mode."""
    return int(_lib.load().rglru_hip_set_chain_forward(int(mode)))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_ptr(device: torch.device) -> int:
    """The current stream of ``device`` as a raw hipStream_t (the C ABI takes it as void*)."""
    index = device.index
    if _raw_stream is not None and index is not None:
        return _raw_stream(index)                        # no Stream object: a fraction of a microsecond
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device: torch.device):
    """``torch.cuda.device(device)`` without the cost of the guard when ``device`` is current already
    (the usual case; the guard costs several microseconds per call, as much as a decode step's kernel)."""
    if _raw_device is not None and device.index is not None and _raw_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


class _FirstTokenReset:
    """In place of a flag tensor: token 0 of every sequence starts a document, no other token carries a flag
    (RGLRU_FLAGS_FIRST_RESET of the C ABI).  The kernels then run their variants without per-token flags."""

    def __repr__(self):
        return "FIRST_TOKEN_RESET"


FIRST_TOKEN_RESET = _FirstTokenReset()


def _flags_ptr(flags) -> int | None:
    return 1 if flags is FIRST_TOKEN_RESET else _ptr(flags)


def _ptr(t: Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


_gpu_seen = False


def _require_gpu(name: str, *tensors: Tensor) -> None:
    global _gpu_seen
    if not _gpu_seen:
        _lib.load()  # raises RuntimeError when the extension is missing
        if not torch.cuda.is_available():
            raise RuntimeError(f"{name} requires a CUDA/HIP device, none is available")
        _gpu_seen = True                                 # both facts hold for the life of the process
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(f"{name} requires CUDA/HIP tensors, got a {t.device.type} tensor")


# ----------------------------------------------------------------------------------------------
# scan-only operator: h_t = a_t h_{t-1} + z_t
# ----------------------------------------------------------------------------------------------
class _HipScan(torch.autograd.Function):
    @staticmethod
    def forward(ctx, decay: Tensor, current_input: Tensor, initial_state: Tensor) -> Tensor:
        _require_gpu("hip_rglru_scan", decay, current_input, initial_state)
        if decay.dim() != 3 or decay.shape != current_input.shape:
            raise ValueError("decay and current_input must share shape [batch, sequence, width]")
        if initial_state.shape != (decay.size(0), decay.size(2)):
            raise ValueError("initial_state must have shape [batch, width]")
        if decay.dtype != torch.float32 or current_input.dtype != torch.float32:
            raise TypeError("hip_rglru_scan expects fp32 decay and normalized input")
        if initial_state.dtype != torch.float32:
            raise TypeError("hip_rglru_scan expects fp32 recurrent state")
        lib = _lib.load()
        decay = decay.contiguous()
        current_input = current_input.contiguous()
        initial_state = initial_state.contiguous()
        B, T, W = decay.shape
        out = torch.empty_like(current_input)
        if out.numel() == 0:
            ctx.save_for_backward(decay, initial_state, out)
            return out
        with _on_device(decay.device):
            ws = torch.empty(lib.rglru_hip_scan_workspace_bytes(B, T, W), dtype=torch.uint8, device=decay.device)
            _lib.check(lib.rglru_hip_scan_fwd(decay.data_ptr(), current_input.data_ptr(), initial_state.data_ptr(),
                                              out.data_ptr(), ws.data_ptr(), B, T, W, _stream_ptr(decay.device)),
                       "rglru_hip_scan_fwd")
        ctx.save_for_backward(decay, initial_state, out)
        # the forward call has cleared the backward part of the workspace too: the first backward call over this
        # forward finds it clear (a repeated one clears its part itself)
        ctx.workspace = [ws]
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out: Tensor):
        decay, initial_state, out = ctx.saved_tensors
        lib = _lib.load()
        grad_out = grad_out.contiguous()
        B, T, W = decay.shape
        d_decay = torch.empty_like(decay)
        d_input = torch.empty_like(decay)
        d_state = torch.empty_like(initial_state)
        if decay.numel() == 0:
            return d_decay, d_input, d_state.zero_()
        with _on_device(decay.device):
            held = getattr(ctx, "workspace", None)
            fresh = bool(held)
            ws = held.pop() if fresh else torch.empty(lib.rglru_hip_scan_workspace_bytes(B, T, W), dtype=torch.uint8,
                                                      device=decay.device)
            _lib.check(lib.rglru_hip_scan_bwd(decay.data_ptr(), initial_state.data_ptr(), out.data_ptr(),
                                              grad_out.data_ptr(), d_decay.data_ptr(), d_input.data_ptr(),
                                              d_state.data_ptr(), ws.data_ptr(), 1 if fresh else 0, B, T, W,
                                              _stream_ptr(decay.device)),
                       "rglru_hip_scan_bwd")
        return d_decay, d_input, d_state


def hip_rglru_scan(decay: Tensor, current_input: Tensor, initial_state: Tensor) -> Tensor:
    """Differentiable linear recurrence on the GPU (contract of griffin/triton_scan.py:274-276)."""
    return _HipScan.apply(decay, current_input, initial_state)


# ----------------------------------------------------------------------------------------------
# fused operator: gates + scan
# ----------------------------------------------------------------------------------------------
_DTYPE_CODES = {torch.float32: _lib.RGLRU_F32, torch.bfloat16: _lib.RGLRU_BF16}


def _dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _lib.RGLRU_F32
    if dtype == torch.bfloat16:
        return _lib.RGLRU_BF16
    raise TypeError(f"hip RG-LRU supports float32 and bfloat16 activations, got {dtype}")


_PACKED_FLAGS: dict = {}       # id(mask) -> (weak reference to the mask, its version, the packed bytes)


def pack_flags(reset_mask: Tensor | None, active_mask: Tensor | None) -> Tensor | None:
    """One byte per token: bit 0 = reset, bit 1 = inactive.  None when no token is flagged.  The bytes
    of a reset mask that comes without an activity mask are remembered for as long as that tensor lives
    and is not written to (a module that passes the same mask every step pays for them once)."""
    if reset_mask is not None and active_mask is None and reset_mask.dtype == torch.bool:
        hit = _PACKED_FLAGS.get(id(reset_mask))
        if hit is not None and hit[0]() is reset_mask and hit[1] == reset_mask._version:
            return hit[2]
        # outside inference mode whatever the caller's mode: the bytes outlive this call, and an inference tensor
        # cannot be saved for the backward pass of a later training step that finds them here
        with torch.inference_mode(False):
            flags = reset_mask.to(torch.uint8).contiguous()
        if not (reset_mask.is_cuda and torch.cuda.is_current_stream_capturing()):   # made under capture: valid inside that graph only
            if len(_PACKED_FLAGS) >= 64:
                _PACKED_FLAGS.clear()
            _PACKED_FLAGS[id(reset_mask)] = (weakref.ref(reset_mask), reset_mask._version, flags)
        return flags
    flags = None
    if reset_mask is not None:
        flags = reset_mask.to(torch.uint8)
    if active_mask is not None:
        idle = (~active_mask.to(torch.bool)).to(torch.uint8) * 2
        flags = idle if flags is None else flags + idle
    return None if flags is None else flags.contiguous()


def _parameter_operands(w_a: Tensor, b_a: Tensor, w_x: Tensor, b_x: Tensor, lam: Tensor, dtype: torch.dtype):
    """The five parameters as the library reads them: gate weights in the storage type; biases and
    Lambda in their own type when the library knows it (fp32 or bf16), so the usual cases launch no
    conversion kernels.  Returns the tensors (kept alive by the caller) and the vector dtype code."""
    vec_dtype = b_a.dtype if (b_a.dtype == b_x.dtype == lam.dtype and b_a.dtype in _DTYPE_CODES) else torch.float32
    tensors = (w_a.detach().to(dtype).contiguous(), b_a.detach().to(vec_dtype).contiguous(),
               w_x.detach().to(dtype).contiguous(), b_x.detach().to(vec_dtype).contiguous(),
               lam.detach().to(vec_dtype).contiguous())
    return tensors, _DTYPE_CODES[vec_dtype]


def _prep_bytes(width: int, blocks: int, code: int) -> int:
    size = _lib.load().rglru_hip_prep_bytes(width, blocks, code)
    if size == 0:
        _lib.check(2, "rglru_hip_prep_bytes")
    return size


class PreparedParams:
    """Kernel-side image of the RG-LRU parameters (see rglru_hip_prepare)."""

    def __init__(self, w_a: Tensor, b_a: Tensor, w_x: Tensor, b_x: Tensor, lam: Tensor, c: float, dtype: torch.dtype):
        lib = _lib.load()
        nb, bw, _ = w_a.shape
        self.width = nb * bw
        self.blocks = nb
        self.dtype = dtype
        self.c = float(c)
        code = _dtype_code(dtype)
        size = _prep_bytes(self.width, nb, code)
        device = w_a.device
        operands, vec_code = _parameter_operands(w_a, b_a, w_x, b_x, lam, dtype)
        with _on_device(device):
            self.image = torch.empty(size, dtype=torch.uint8, device=device)
            _lib.check(lib.rglru_hip_prepare(*(t.data_ptr() for t in operands), self.c, self.width, nb, code, vec_code,
                                             self.image.data_ptr(), _stream_ptr(device)), "rglru_hip_prepare")


def _check_fused_inputs(x: Tensor, w_a: Tensor, h0: Tensor | None, flags: Tensor | None) -> None:
    if x.dim() != 3:
        raise ValueError(f"hip RG-LRU expects [batch, sequence, width], got {tuple(x.shape)}")
    B, T, W = x.shape
    nb, bw, bw2 = w_a.shape
    if bw != bw2 or nb * bw != W:
        raise ValueError(f"gate weights {tuple(w_a.shape)} do not match width {W}")
    if h0 is not None and h0.shape != (B, W):
        raise ValueError(f"initial state must have shape ({B}, {W}), got {tuple(h0.shape)}")
    if flags is not None and flags is not FIRST_TOKEN_RESET and flags.shape != (B, T):
        raise ValueError(f"token flags must have shape ({B}, {T}), got {tuple(flags.shape)}")
    if T == 0 or B == 0:
        raise ValueError("hip RG-LRU does not accept empty batches or sequences")
    _dtype_code(x.dtype)


def _aligned(t: Tensor) -> Tensor:
    """``t`` itself when its storage starts on a 16-byte boundary (what every fresh allocation does), else a
    copy that does: a view at an odd offset costs one copy instead of sending the whole call to the portable
    kernels, which are several times slower."""
    return t if t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)


def kernel_path(B: int, T: int, W: int, nb: int, dtype: torch.dtype, *tensors: Tensor) -> int:
    """Which kernel family of the library serves this configuration (rglru_hip_backward_path): one of
    ``_lib.PATH_*``.  ``tensors``: the activation tensors of the call; one that is not 16-byte aligned
    sends the call to the portable kernels."""
    aligned = all(t is None or t.data_ptr() % 16 == 0 for t in tensors)
    path = _lib.load().rglru_hip_backward_path(B, T, W, nb, _dtype_code(dtype), 1 if aligned else 0)
    if path < 0:
        _lib.check(2, "rglru_hip_backward_path")
    return path


class _HipRGLRU(torch.autograd.Function):
    """y, h_T = RG-LRU(x; W_a, b_a, W_x, b_x, Lambda) with a recomputing backward."""

    @staticmethod
    def forward(ctx, x, w_a, b_a, w_x, b_x, lam, h0, flags, c):
        first_reset = flags is FIRST_TOKEN_RESET
        _require_gpu("hip RG-LRU", x, w_a, b_a, w_x, b_x, lam, h0, None if first_reset else flags)
        _check_fused_inputs(x, w_a, h0, flags)
        lib = _lib.load()
        x = _aligned(x.contiguous())
        B, T, W = x.shape
        nb = w_a.shape[0]
        code = _dtype_code(x.dtype)
        operands, vec_code = _parameter_operands(w_a, b_a, w_x, b_x, lam, x.dtype)
        h0c = None if h0 is None else h0.detach().to(torch.float32).contiguous()
        device = x.device
        with _on_device(device):
            y = torch.empty_like(x)
            h_last = torch.empty(B, W, dtype=torch.float32, device=device)
            image = torch.empty(_prep_bytes(W, nb, code), dtype=torch.uint8, device=device)
            ws = torch.empty(lib.rglru_hip_workspace_bytes(B, T, W, nb), dtype=torch.uint8, device=device)
            if kernel_path(B, T, W, nb, x.dtype, x) == _lib.PATH_PRE:
                pre = torch.empty(nb, B * T, 2 * (W // nb), dtype=x.dtype, device=device)   # scratch of the call
                _lib.check(lib.rglru_hip_prepare(*(t.data_ptr() for t in operands), float(c), W, nb, code, vec_code,
                                                 image.data_ptr(), _stream_ptr(device)), "rglru_hip_prepare")
                _lib.check(lib.rglru_hip_fwd_pre(x.data_ptr(), pre.data_ptr(), image.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                                 y.data_ptr(), h_last.data_ptr(), ws.data_ptr(), B, T, W, nb, code,
                                                 _stream_ptr(device)), "rglru_hip_fwd_pre")
                del pre
            else:
                # parameter conversion, workspace clearing and the forward kernel: two launches, or one where the
                # forward kernel does all three (batch-rich shapes)
                _lib.check(lib.rglru_hip_prepare_fwd(*(t.data_ptr() for t in operands), float(c), vec_code,
                                                     image.data_ptr(), x.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                                     y.data_ptr(), h_last.data_ptr(), ws.data_ptr(), B, T, W, nb, code,
                                                     _stream_ptr(device)), "rglru_hip_prepare_fwd")
        ctx.save_for_backward(x, w_a, w_x, h0c, None if first_reset else flags, ws, image, y)
        ctx.first_reset = first_reset
        ctx.param_dtypes = (w_a.dtype, b_a.dtype, w_x.dtype, b_x.dtype, lam.dtype)
        ctx.h0_dtype = None if h0 is None else h0.dtype
        ctx.set_materialize_grads(False)      # an unused output arrives as None, not as a tensor of zeros
        return y, h_last

    @staticmethod
    @once_differentiable
    def backward(ctx, dy, dh_last):
        x, w_a, w_x, h0c, flags, ws, image, y = ctx.saved_tensors
        if ctx.first_reset:
            flags = FIRST_TOKEN_RESET
        dx, dw_a, db_a, dw_x, db_x, dlam, dh0 = rglru_backward(
            x, y, w_a, w_x, h0c, flags, ws, image, dy, dh_last, ctx.param_dtypes, ctx.needs_input_grad[6])
        return (dx, dw_a, db_a, dw_x, db_x, dlam, None if dh0 is None else dh0.to(ctx.h0_dtype), None, None)


def rglru_backward(x, y, w_a, w_x, h0c, flags, ws, image, dy, dh_last, param_dtypes, need_dh0):
    """Backward pass of the RG-LRU on what its forward kept (the workspace with checkpoints and records, the
    parameter image): returns (dx, dW_a, db_a, dW_x, db_x, dLambda, dh0 in fp32 or None), the parameter
    gradients in the parameters' types."""
    lib = _lib.load()
    B, T, W = x.shape
    nb, bw, _ = w_a.shape
    code = _dtype_code(x.dtype)
    device = x.device
    dy = torch.zeros_like(x) if dy is None else _aligned(dy.to(x.dtype).contiguous())
    dhl = None if dh_last is None else dh_last.to(torch.float32).contiguous()
    # parameter gradients come back in the parameters' own type when all five share one the
    # library writes (fp32 or bf16); otherwise in fp32, converted below
    pd = param_dtypes
    gdt = pd[0] if (len(set(pd)) == 1 and pd[0] in _DTYPE_CODES) else torch.float32
    gcode = _DTYPE_CODES[gdt]
    with _on_device(device):
        dx = torch.empty_like(x)
        db_a = torch.empty(nb, bw, dtype=gdt, device=device)
        db_x = torch.empty(nb, bw, dtype=gdt, device=device)
        dlam = torch.empty(W, dtype=gdt, device=device)
        dh0 = torch.empty(B, W, dtype=torch.float32, device=device) if need_dh0 else None
        # scratch of this call only (the workspace kept since forward holds just checkpoints and records)
        scratch = torch.empty(lib.rglru_hip_bwd_scratch_bytes(B, T, W, nb, code), dtype=torch.uint8, device=device)
        path = kernel_path(B, T, W, nb, x.dtype, x, y, dy, dx)
        if path in (_lib.PATH_FAST_CHAIN, _lib.PATH_FAST_TILED):
            # everything in hand-written kernels, including the two gate GEMMs
            dw_a = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            dw_x = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            _lib.check(lib.rglru_hip_bwd_full(x.data_ptr(), y.data_ptr(), image.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                              dy.data_ptr(), _ptr(dhl), ws.data_ptr(), scratch.data_ptr(), dx.data_ptr(), dw_a.data_ptr(),
                                              dw_x.data_ptr(), db_a.data_ptr(), db_x.data_ptr(), dlam.data_ptr(),
                                              _ptr(dh0), B, T, W, nb, code, gcode, _stream_ptr(device)),
                       "rglru_hip_bwd_full")
        elif path == _lib.PATH_WIDE:
            # blocks of 160 .. 384 channels: scan and gate math, then the two gate GEMMs, all hand-written
            dw_a = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            dw_x = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            _lib.check(lib.rglru_hip_bwd_wide(x.data_ptr(), image.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                              dy.data_ptr(), _ptr(dhl), ws.data_ptr(), scratch.data_ptr(), dx.data_ptr(), dw_a.data_ptr(),
                                              dw_x.data_ptr(), db_a.data_ptr(), db_x.data_ptr(), dlam.data_ptr(),
                                              _ptr(dh0), B, T, W, nb, code, gcode, _stream_ptr(device)),
                       "rglru_hip_bwd_wide")
        elif path == _lib.PATH_PRE:
            # bf16 blocks of 416 .. 512 channels: a GEMM kernel for the gate projections, the scan and all gate math
            # in the scan kernel, then the two GEMM kernels of the gate gradients
            dw_a = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            dw_x = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            pre = torch.empty(nb, B * T, 2 * bw, dtype=x.dtype, device=device)
            du = torch.empty_like(pre)
            _lib.check(lib.rglru_hip_bwd_pre(x.data_ptr(), pre.data_ptr(), image.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                             dy.data_ptr(), _ptr(dhl), ws.data_ptr(), scratch.data_ptr(), dx.data_ptr(),
                                             du.data_ptr(), dw_a.data_ptr(), dw_x.data_ptr(), db_a.data_ptr(), db_x.data_ptr(),
                                             dlam.data_ptr(), _ptr(dh0), B, T, W, nb, code, gcode, _stream_ptr(device)),
                       "rglru_hip_bwd_pre")
        else:
            # any storage type, width and alignment: the scan kernel leaves the gradients at the gate
            # pre-activations in du_a, du_x; two GEMM kernels of the library finish dW and dx
            dw_a = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            dw_x = torch.empty(nb, bw, bw, dtype=gdt, device=device)
            du_a = torch.empty_like(x)
            du_x = torch.empty_like(x)
            _lib.check(lib.rglru_hip_bwd(x.data_ptr(), image.data_ptr(), _ptr(h0c), _flags_ptr(flags),
                                         dy.data_ptr(), _ptr(dhl), ws.data_ptr(), scratch.data_ptr(), dx.data_ptr(), du_a.data_ptr(),
                                         du_x.data_ptr(), dw_a.data_ptr(), dw_x.data_ptr(), db_a.data_ptr(), db_x.data_ptr(),
                                         dlam.data_ptr(), _ptr(dh0), B, T, W, nb, code, gcode, _stream_ptr(device)), "rglru_hip_bwd")
    return dx, dw_a.to(pd[0]), db_a.to(pd[1]), dw_x.to(pd[2]), db_x.to(pd[3]), dlam.to(pd[4]), dh0


def hip_rglru(x: Tensor, w_a: Tensor, b_a: Tensor, w_x: Tensor, b_x: Tensor, lam: Tensor, c: float = 8.0,
              h0: Tensor | None = None, reset_mask: Tensor | None = None,
              active_mask: Tensor | None = None, first_token_reset: bool = False) -> tuple[Tensor, Tensor]:
    """Fused RG-LRU on the GPU: returns (y in x.dtype, final state in fp32).  Differentiable in
    x, the five parameters and h0 (first order).  ``first_token_reset`` stands for the reset mask that is True
    at token 0 of every row and nowhere else (rows that each hold one document from its beginning), without
    building it: the kernels then run without per-token flags."""
    if first_token_reset:
        if reset_mask is not None or active_mask is not None:
            raise ValueError("first_token_reset replaces the masks; pass one or the other")
        flags = FIRST_TOKEN_RESET
    else:
        flags = pack_flags(reset_mask, active_mask)
    return _HipRGLRU.apply(x, w_a, b_a, w_x, b_x, lam, h0, flags, c)


def hip_rglru_step(x: Tensor, prep: PreparedParams, state: Tensor, flags: Tensor | None = None) -> Tensor:
    """One decode step: ``state`` [B, W] fp32 is updated in place; returns y [B, W] in x.dtype."""
    _require_gpu("hip RG-LRU step", x, state, flags)
    if x.dim() != 2 or x.shape[1] != prep.width:
        raise ValueError(f"step expects x of shape [batch, {prep.width}], got {tuple(x.shape)}")
    if state.shape != x.shape or state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("step expects a contiguous fp32 state of the same shape as x")
    if x.dtype != prep.dtype:
        raise TypeError(f"parameters were prepared for {prep.dtype}, got activations in {x.dtype}")
    lib = _lib.load()
    x = x.contiguous()
    with _on_device(x.device):
        y = torch.empty_like(x)
        _lib.check(lib.rglru_hip_step(x.data_ptr(), prep.image.data_ptr(), state.data_ptr(), _ptr(flags),
                                      y.data_ptr(), x.shape[0], prep.width, prep.blocks, _dtype_code(x.dtype),
                                      _stream_ptr(x.device)), "rglru_hip_step")
    return y


def hip_rglru_steps(xs: Tensor, prep: PreparedParams, state: Tensor, flags: Tensor | None = None) -> Tensor:
    """K decode steps in one launch for inputs known in advance: ``xs`` [K, B, W]; ``state`` [B, W] fp32
    is updated in place to the state after the last step; returns y [K, B, W] in xs.dtype (the result
    of K calls of ``hip_rglru_step``)."""
    _require_gpu("hip RG-LRU steps", xs, state, flags)
    if xs.dim() != 3 or xs.shape[2] != prep.width:
        raise ValueError(f"steps expects x of shape [steps, batch, {prep.width}], got {tuple(xs.shape)}")
    if state.shape != xs.shape[1:] or state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("steps expects a contiguous fp32 state of shape [batch, width]")
    if flags is not None and (flags.shape != xs.shape[:2] or flags.dtype != torch.uint8):
        raise ValueError("flags must be uint8 of shape [steps, batch]")
    if xs.dtype != prep.dtype:
        raise TypeError(f"parameters were prepared for {prep.dtype}, got activations in {xs.dtype}")
    lib = _lib.load()
    xs = xs.contiguous()
    K, B, _ = xs.shape
    with _on_device(xs.device):
        ys = torch.empty_like(xs)
        if K > 0 and B > 0:
            _lib.check(lib.rglru_hip_steps(xs.data_ptr(), prep.image.data_ptr(), state.data_ptr(),
                                           None if flags is None else flags.contiguous().data_ptr(), ys.data_ptr(),
                                           K, B, prep.width, prep.blocks, _dtype_code(xs.dtype), _stream_ptr(xs.device)),
                       "rglru_hip_steps")
    return ys


# ----------------------------------------------------------------------------------------------
# one-time self-test (reference: griffin/triton_scan.py:130-204)
# ----------------------------------------------------------------------------------------------
def _loop_scan(decay: Tensor, current_input: Tensor, state: Tensor) -> Tensor:
    rows = []
    for t in range(decay.size(1)):
        state = decay[:, t] * state + current_input[:, t]
        rows.append(state)
    return torch.stack(rows, dim=1)


def _validate_hip_scan(device: torch.device) -> None:
    """Forward/backward parity of both operators against autograd through a plain loop, on the
    seed-free inputs of the reference self-test (width 257 = one partial tile, 7 steps) and on a
    second case long enough to cross chunk boundaries."""
    from . import portable

    for width, steps in ((257, 7), (96, 75)):
        k = torch.arange(width * steps, device=device, dtype=torch.float32)
        decay = (0.9 + 0.05 * torch.sin(k / 97.0)).reshape(1, steps, width)
        inp = (0.1 * torch.cos(k / 53.0)).reshape(1, steps, width)
        state = torch.sin(torch.arange(width, device=device) / 31.0)[None]
        upstream = torch.cos(k / 71.0).reshape(1, steps, width)
        ref_in = [t.detach().clone().requires_grad_(True) for t in (decay, inp, state)]
        hip_in = [t.detach().clone().requires_grad_(True) for t in (decay, inp, state)]
        ref_out = _loop_scan(*ref_in)
        hip_out = hip_rglru_scan(*hip_in)
        ref_g = torch.autograd.grad(ref_out, ref_in, upstream)
        hip_g = torch.autograd.grad(hip_out, hip_in, upstream)
        torch.cuda.synchronize(device)
        torch.testing.assert_close(hip_out, ref_out, atol=2e-5, rtol=2e-5)
        for got, want in zip(hip_g, ref_g):
            torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5)

    # fused operator on a small closed-form module: W = 48 in 3 blocks, 70 steps, reset + padding
    B, T, W, nb = 2, 70, 48, 3
    bw = W // nb
    k = torch.arange(B * T * W, device=device, dtype=torch.float32)
    x = torch.sin(k / 37.0).reshape(B, T, W)
    kw = torch.arange(nb * bw * bw, device=device, dtype=torch.float32)
    w_a = (0.3 * torch.cos(kw / 11.0)).reshape(nb, bw, bw)
    w_x = (0.3 * torch.sin(kw / 13.0)).reshape(nb, bw, bw)
    kb = torch.arange(W, device=device, dtype=torch.float32)
    b_a = (0.1 * torch.sin(kb / 5.0)).reshape(nb, bw)
    b_x = (0.1 * torch.cos(kb / 7.0)).reshape(nb, bw)
    lam = 4.0 + 3.0 * torch.sin(kb / 9.0) ** 2
    h0 = torch.cos(torch.arange(B * W, device=device, dtype=torch.float32) / 17.0).reshape(B, W)
    reset = torch.zeros(B, T, dtype=torch.bool, device=device)
    reset[:, 40] = True
    active = torch.ones(B, T, dtype=torch.bool, device=device)
    active[1, -5:] = False
    upstream = torch.cos(k / 29.0).reshape(B, T, W)

    def run(use_hip):
        leaves = [t.detach().clone().requires_grad_(True) for t in (x, w_a, b_a, w_x, b_x, lam, h0)]
        if use_hip:
            y, _ = hip_rglru(*leaves[:6], 8.0, leaves[6], reset, active)
        else:
            a, z = portable.decay_and_input(*leaves[:6], 8.0, reset, active, torch.float32)
            y = _loop_scan(a, z, leaves[6])
        return y, torch.autograd.grad(y, leaves, upstream)

    ref_y, ref_g = run(False)
    hip_y, hip_g = run(True)
    torch.cuda.synchronize(device)
    torch.testing.assert_close(hip_y, ref_y, atol=2e-5, rtol=2e-5)
    for got, want in zip(hip_g, ref_g):
        scale = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(got, want, atol=3e-5 * scale, rtol=3e-5)

    # the caller's temporal convolution: 4 taps, carried state, a document boundary inside
    from .hip_block_ops import hip_causal_conv

    taps = (0.2 * torch.cos(torch.arange(W * 4, device=device, dtype=torch.float32) / 3.0)).reshape(W, 1, 4)
    conv_bias = 0.1 * torch.sin(kb / 4.0)
    conv_state = torch.cos(torch.arange(B * 3 * W, device=device, dtype=torch.float32) / 19.0).reshape(B, 3, W)
    positions = torch.arange(T, device=device).repeat(B, 1)
    positions[1, 33:] -= 33

    def run_conv(use_hip):
        leaves = [t.detach().clone().requires_grad_(True) for t in (x, conv_state, taps, conv_bias)]
        fn = hip_causal_conv if use_hip else (lambda u, s, w, b, pos: portable.causal_depthwise_conv(u, s, w, b, pos))
        out, carried = fn(*leaves, positions)
        return out, carried, torch.autograd.grad(out, leaves, upstream)

    ref_o, ref_c, ref_g = run_conv(False)
    hip_o, hip_c, hip_g = run_conv(True)
    torch.cuda.synchronize(device)
    torch.testing.assert_close(hip_o, ref_o, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(hip_c, ref_c, atol=0.0, rtol=0.0)
    for got, want in zip(hip_g, ref_g):
        scale = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(got, want, atol=3e-5 * scale, rtol=3e-5)

    # the block's output gate h * gelu_tanh(v)
    from .hip_block_ops import hip_gelu_gate

    def run_gate(use_hip):
        leaves = [t.detach().clone().requires_grad_(True) for t in (x, 4.0 * upstream)]
        out = hip_gelu_gate(*leaves) if use_hip else leaves[0] * torch.nn.functional.gelu(leaves[1], approximate="tanh")
        return out, torch.autograd.grad(out, leaves, upstream)

    ref_o, ref_g = run_gate(False)
    hip_o, hip_g = run_gate(True)
    torch.cuda.synchronize(device)
    torch.testing.assert_close(hip_o, ref_o, atol=2e-5, rtol=2e-5)
    for got, want in zip(hip_g, ref_g):
        torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5)

    # RMSNorm in front of the block
    from .hip_block_ops import hip_rmsnorm

    def run_norm(use_hip):
        leaves = [t.detach().clone().requires_grad_(True) for t in (x, conv_bias)]
        if use_hip:
            out = hip_rmsnorm(*leaves, 1e-6)
        else:
            out = leaves[0] * torch.rsqrt(leaves[0].pow(2).mean(dim=-1, keepdim=True) + 1e-6) * (1.0 + leaves[1])
        return out, torch.autograd.grad(out, leaves, upstream)

    ref_o, ref_g = run_norm(False)
    hip_o, hip_g = run_norm(True)
    torch.cuda.synchronize(device)
    torch.testing.assert_close(hip_o, ref_o, atol=2e-5, rtol=2e-5)
    for got, want in zip(hip_g, ref_g):
        scale = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(got, want, atol=3e-5 * scale, rtol=3e-5)


    # 16-bit storage: the kernels with register-held weights, the convolution, the RG-LRU and the output gate
    # in one forward launch and their backward, against the same computation in fp32 on the rounded operands
    from .hip_block_ops import hip_block_forward, hip_block_forward_covers

    if hip_block_forward_covers(W * 2, nb, 4, torch.bfloat16):
        bf = torch.bfloat16
        W2, bw2 = W * 2, 2 * bw                                    # 96 channels in 3 blocks of 32
        k2 = torch.arange(B * T * W2, device=device, dtype=torch.float32)
        u16 = torch.sin(k2 / 37.0).reshape(B, T, W2).to(bf)
        v16 = torch.cos(k2 / 23.0).reshape(B, T, W2).to(bf)
        kw2 = torch.arange(nb * bw2 * bw2, device=device, dtype=torch.float32)
        params16 = [(0.2 * torch.cos(kw2 / 11.0)).reshape(nb, bw2, bw2).to(bf), torch.cat((b_a, b_a), 1).to(bf),
                    (0.2 * torch.sin(kw2 / 13.0)).reshape(nb, bw2, bw2).to(bf), torch.cat((b_x, b_x), 1).to(bf),
                    torch.cat((lam, lam)).to(bf)]
        taps16 = torch.cat((taps, taps)).to(bf)
        cbias16 = torch.cat((conv_bias, conv_bias)).to(bf)
        up16 = torch.cos(k2 / 29.0).reshape(B, T, W2).to(bf)

        def run_block(use_hip):
            dtype = bf if use_hip else torch.float32
            leaves = [t.detach().to(dtype).clone().requires_grad_(True) for t in (u16, v16, taps16, cbias16, *params16)]
            uu, vv, tt, cb, *prm = leaves
            if use_hip:
                out, _, _ = hip_block_forward(uu, vv, None, tt, cb, positions, None, *prm, None, 8.0)
            else:
                xc, _ = portable.causal_depthwise_conv(uu, torch.zeros(B, 3, W2, device=device), tt, cb, positions)
                a, z = portable.decay_and_input(xc, *prm, 8.0, positions == 0,
                                                torch.ones(B, T, dtype=torch.bool, device=device), torch.float32)
                out = _loop_scan(a, z, torch.zeros(B, W2, device=device)) * torch.nn.functional.gelu(vv, approximate="tanh")
            return out, torch.autograd.grad(out, leaves, up16.to(dtype))

        ref_o, ref_g = run_block(False)
        hip_o, hip_g = run_block(True)
        torch.cuda.synchronize(device)
        for got, want in zip((hip_o, *hip_g), (ref_o, *ref_g)):
            got, want = got.detach().float(), want.detach()
            err = float((got - want).norm() / want.norm().clamp_min(1e-30))
            if not err < 2e-2:
                raise AssertionError(f"16-bit block forward self-test: relative error {err:.3e}")


def hip_scan_is_usable(device: torch.device | str) -> bool:
    """Validate the HIP kernels once per device before ``scan_mode="auto"`` may use them."""
    resolved = torch.device(device)
    if resolved.type != "cuda" or not torch.cuda.is_available() or not hip_scan_available():
        return False
    index = torch.cuda.current_device() if resolved.index is None else resolved.index
    with _VALIDATION_LOCK:
        if index in _VALIDATED:
            return _VALIDATED[index]
        try:
            with torch.enable_grad(), torch.cuda.device(index):
                _validate_hip_scan(torch.device("cuda", index))
        except Exception as error:  # launch failures and numerical mismatches both fall back
            _VALIDATED[index] = False
            warnings.warn(
                "HIP RG-LRU scan failed its CUDA/HIP self-test; using the portable scan instead. "
                f"Original error: {error}",
                RuntimeWarning,
                stacklevel=2,
            )
        else:
            _VALIDATED[index] = True
        return _VALIDATED[index]
