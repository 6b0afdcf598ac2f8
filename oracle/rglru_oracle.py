"""CPU oracle for the RG-LRU (Real-Gated Linear Recurrent Unit) hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``griffin_amd/`` may import this file; it is the
checker that the HIP kernels are compared against (tests, the smoke check and the CPU-baseline
leg of the benchmark), never the thing that is shipped or measured as the product.

It restates, in plain PyTorch CPU ops (fp32 or fp64), the algorithm of the reference
implementation.  Every function names the reference lines it follows:

* ``block_diagonal_gate``      - griffin/griffin.py:149-154 (einsum "...bi,boi->...bo" + bias)
* ``BoundedSqrt``              - griffin/griffin.py:48-65 (sqrt, derivative capped at 1000)
* ``gate_math``                - griffin/griffin.py:237-258 (r, i, log-space decay, masks, upcast)
* ``sequential_scan``          - griffin/griffin.py:279-284 and griffin/triton_scan.py:130-137
* ``rglru_forward``            - griffin/griffin.py:190-289 (whole forward, accumulation dtype rule :226)
* ``rglru_backward_explicit``  - reverse recurrence of griffin/triton_scan.py:63-122 plus the chain
                                 rule through griffin/griffin.py:237-255, written out by hand so
                                 that it is independent of autograd
* ``selftest_inputs``          - griffin/triton_scan.py:142-153 (seed-free sin/cos inputs)
* ``lambda_init`` / ``gate_init`` - griffin/griffin.py:146-147, 183-188
* ``causal_conv``, ``recurrent_block_forward`` - griffin/griffin.py:309-338, 439-529

Pinning status (what checks each function independently of its own formula):
  sequential_scan   brute-force closed form in fp64, scipy.signal.lfilter for constant decay,
                    cumsum for a == 1, identity for a == 0, chunk-split == whole
  block_diagonal_gate   dense matmul with torch.block_diag
  BoundedSqrt       closed-form derivative, cap value, finite at zero
  gate_math         a^2 + g^2 == 1 off reset, exp(c r log sigma) == sigma^(c r), mask semantics
  rglru_backward_explicit   autograd over rglru_forward in fp64 and torch.autograd.gradcheck
  rglru_forward / recurrent_block_forward (composite behaviour)   golden vectors under
                    tests/golden/ written once from the reference implementation
"""

from __future__ import annotations

import math
from typing import NamedTuple, Optional

import torch
from torch import Tensor

MAX_SQRT_GRADIENT = 1000.0  # griffin/griffin.py:51


def accumulation_dtype(dtype: torch.dtype) -> torch.dtype:
    """fp32 state for half-precision inputs, otherwise the input dtype (griffin/griffin.py:226)."""
    return torch.float32 if dtype in (torch.float16, torch.bfloat16) else dtype


def block_diagonal_gate(x: Tensor, weight: Tensor, bias: Tensor) -> Tensor:
    """y[..., k, o] = sum_i x[..., k, i] * weight[k, o, i] + bias[k, o] (griffin/griffin.py:149-154)."""
    nb, bw, _ = weight.shape
    lead = x.shape[:-1]
    xb = x.reshape(-1, nb, bw).transpose(0, 1)            # [nb, N, bw]
    out = torch.bmm(xb, weight.transpose(1, 2))            # [nb, N, bw_out]
    out = out.transpose(0, 1) + bias
    return out.reshape(*lead, nb * bw)


class BoundedSqrt(torch.autograd.Function):
    """sqrt(x) whose derivative is 1/sqrt(max(4x, 1/1000^2)) (griffin/griffin.py:48-65)."""

    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return x.sqrt()

    @staticmethod
    def backward(ctx, g):
        (x,) = ctx.saved_tensors
        floor = 1.0 / (MAX_SQRT_GRADIENT * MAX_SQRT_GRADIENT)
        return g / (4.0 * x).clamp(min=floor).sqrt()


class Gates(NamedTuple):
    r: Tensor       # recurrence gate
    i: Tensor       # input gate
    log_a: Tensor   # c * r * logsigmoid(Lambda), before masks
    a: Tensor       # decay after masks, accumulation dtype
    g: Tensor       # input scale after the reset mask (1 at reset)
    z: Tensor       # gated, normalised input after masks, accumulation dtype


def gate_math(x, w_a, b_a, w_x, b_x, lam, c=8.0, reset_mask=None, active_mask=None) -> Gates:
    """Gate and decay math of griffin/griffin.py:237-258, in x.dtype, then upcast."""
    B, T, W = x.shape
    r = torch.sigmoid(block_diagonal_gate(x, w_a, b_a))                   # :237
    i = torch.sigmoid(block_diagonal_gate(x, w_x, b_x))                   # :238
    log_base = torch.nn.functional.logsigmoid(lam).to(x.dtype)            # :239
    log_a = c * r * log_base                                              # :240
    a = log_a.exp()                                                       # :241
    g2 = (-torch.expm1(2.0 * log_a)).clamp(min=0.0)                       # :244
    g = BoundedSqrt.apply(g2)                                             # :245
    if reset_mask is not None:
        rm = reset_mask.to(torch.bool)[..., None]
        a = torch.where(rm, torch.zeros_like(a), a)                       # :248
        g = torch.where(rm, torch.ones_like(g), g)                        # :249
    z = g * i * x                                                         # :250
    if active_mask is not None:
        am = active_mask.to(torch.bool)[..., None]
        a = torch.where(am, a, torch.ones_like(a))                        # :252
        z = torch.where(am, z, torch.zeros_like(z))                       # :253-255
    acc = accumulation_dtype(x.dtype)
    return Gates(r, i, log_a, a.to(acc), g, z.to(acc))                    # :257-258


def sequential_scan(a: Tensor, z: Tensor, h0: Tensor) -> Tensor:
    """h_t = a_t * h_{t-1} + z_t, one step at a time (griffin/griffin.py:279-284)."""
    h = h0
    rows = []
    for t in range(a.shape[1]):
        h = a[:, t] * h + z[:, t]
        rows.append(h)
    return torch.stack(rows, dim=1)


def rglru_forward(x, w_a, b_a, w_x, b_x, lam, c=8.0, h0=None, reset_mask=None, active_mask=None):
    """Whole RG-LRU forward (griffin/griffin.py:190-289): returns (y in x.dtype, h_T in accumulation dtype)."""
    B, T, W = x.shape
    acc = accumulation_dtype(x.dtype)
    state = torch.zeros(B, W, dtype=acc) if h0 is None else h0.to(acc)
    gates = gate_math(x, w_a, b_a, w_x, b_x, lam, c, reset_mask, active_mask)
    h = sequential_scan(gates.a, gates.z, state)
    return h.to(x.dtype), h[:, -1]


def rglru_backward_explicit(x, w_a, b_a, w_x, b_x, lam, dy, c=8.0, h0=None, reset_mask=None,
                            active_mask=None, dh_last=None):
    """Hand-derived gradients of ``rglru_forward`` (no autograd).

    delta_t = dy_t + a_{t+1} delta_{t+1};  dz = delta;  da = delta * h_{t-1};  dh0 = a_0 delta_0
    (griffin/triton_scan.py:86-122), then the chain rule through griffin/griffin.py:237-255 with the
    bounded square-root derivative of :59-65.  Returns a dict of gradients.
    """
    B, T, W = x.shape
    nb, bw, _ = w_a.shape
    dt = x.dtype
    state = torch.zeros(B, W, dtype=dt) if h0 is None else h0.to(dt)
    gates = gate_math(x, w_a, b_a, w_x, b_x, lam, c, reset_mask, active_mask)
    r, i, log_a, a, z = gates.r, gates.i, gates.log_a, gates.a, gates.z
    h = sequential_scan(a, z, state)
    h_prev = torch.cat([state[:, None], h[:, :-1]], dim=1)

    delta = torch.zeros_like(h)
    carry = torch.zeros(B, W, dtype=dt) if dh_last is None else dh_last.to(dt).clone()
    for t in range(T - 1, -1, -1):
        d = dy[:, t] + carry
        delta[:, t] = d
        carry = a[:, t] * d
    dh0 = carry
    dz = delta
    da = delta * h_prev

    live = torch.ones(B, T, 1, dtype=torch.bool) if active_mask is None else active_mask.to(torch.bool)[..., None]
    rst = torch.zeros(B, T, 1, dtype=torch.bool) if reset_mask is None else reset_mask.to(torch.bool)[..., None]
    zero = torch.zeros_like(x)
    dz = torch.where(live, dz, zero)
    da = torch.where(live & ~rst, da, zero)          # a is a constant at reset / padding

    a_raw = log_a.exp()
    g2 = (-torch.expm1(2.0 * log_a)).clamp(min=0.0)
    g_raw = g2.sqrt()
    g_used = torch.where(rst, torch.ones_like(g_raw), g_raw)
    dg = torch.where(rst, zero, dz * i * x)
    di = dz * g_used * x
    dx = dz * g_used * i
    floor = 1.0 / (MAX_SQRT_GRADIENT * MAX_SQRT_GRADIENT)
    dg2 = dg / (4.0 * g2).clamp(min=floor).sqrt()
    dlog_a = da * a_raw - 2.0 * torch.exp(2.0 * log_a) * dg2
    s = torch.nn.functional.logsigmoid(lam)
    dr = dlog_a * c * s
    ds = (dlog_a * c * r).sum(dim=(0, 1))
    dlam = ds * torch.sigmoid(-lam)
    du_a = dr * r * (1.0 - r)
    du_x = di * i * (1.0 - i)

    def gate_grads(du, w):
        dub = du.reshape(B * T, nb, bw).transpose(0, 1)          # [nb, N, o]
        xb = x.reshape(B * T, nb, bw).transpose(0, 1)            # [nb, N, j]
        dw = torch.bmm(dub.transpose(1, 2), xb)                  # [nb, o, j]
        db = dub.sum(dim=1)
        dxg = torch.bmm(dub, w).transpose(0, 1).reshape(B, T, W)
        return dw, db, dxg

    dwa, dba, dxa = gate_grads(du_a, w_a)
    dwx, dbx, dxx = gate_grads(du_x, w_x)
    return {"x": dx + dxa + dxx, "w_a": dwa, "b_a": dba, "w_x": dwx, "b_x": dbx,
            "lam": dlam, "h0": dh0, "du_a": du_a, "du_x": du_x}


def rglru_autograd(x, w_a, b_a, w_x, b_x, lam, dy, c=8.0, h0=None, reset_mask=None, active_mask=None,
                   dh_last=None):
    """Forward + autograd backward of the restatement; returns (y, h_T, grads dict)."""
    leaves = [t.detach().clone().requires_grad_(True) for t in (x, w_a, b_a, w_x, b_x, lam)]
    acc = accumulation_dtype(x.dtype)
    h0_leaf = (torch.zeros(x.shape[0], x.shape[2], dtype=acc) if h0 is None else h0.detach().clone().to(acc))
    h0_leaf.requires_grad_(True)
    y, h_last = rglru_forward(*leaves, c=c, h0=h0_leaf, reset_mask=reset_mask, active_mask=active_mask)
    outs, gouts = [y], [dy.to(y.dtype)]
    if dh_last is not None:
        outs.append(h_last)
        gouts.append(dh_last.to(h_last.dtype))
    grads = torch.autograd.grad(outs, leaves + [h0_leaf], gouts)
    names = ("x", "w_a", "b_a", "w_x", "b_x", "lam", "h0")
    return y.detach(), h_last.detach(), dict(zip(names, grads))


def scan_autograd(a, z, h0, dh):
    """Scan-only contract of griffin/triton_scan.py:207-271: returns (h, da, dz, dh0) by autograd."""
    leaves = [t.detach().clone().requires_grad_(True) for t in (a, z, h0)]
    h = sequential_scan(*leaves)
    return (h.detach(),) + tuple(torch.autograd.grad(h, leaves, dh))


def selftest_inputs(dtype=torch.float32):
    """Seed-free closed-form inputs of the reference self-test (griffin/triton_scan.py:142-153)."""
    width, steps = 257, 7
    k = torch.arange(width * steps, dtype=torch.float32)
    a = (0.9 + 0.05 * torch.sin(k / 97.0)).reshape(1, steps, width).to(dtype)
    z = (0.1 * torch.cos(k / 53.0)).reshape(1, steps, width).to(dtype)
    h0 = torch.sin(torch.arange(width, dtype=torch.float32) / 31.0)[None].to(dtype)
    up = torch.cos(k / 71.0).reshape(1, steps, width).to(dtype)
    return a, z, h0, up


def gate_init(nb: int, bw: int, gen: torch.Generator, dtype=torch.float32):
    """LeCun-normal block weights, zero bias (griffin/griffin.py:146-147)."""
    w = torch.randn(nb, bw, bw, generator=gen, dtype=torch.float32) * math.sqrt(1.0 / bw)
    return w.to(dtype), torch.zeros(nb, bw, dtype=dtype)


def lambda_init(width: int, gen: torch.Generator, lo=0.9, hi=0.999, c=8.0, dtype=torch.float32):
    """Lambda with sigmoid(Lambda)^c uniform in [lo, hi] (griffin/griffin.py:183-188)."""
    u = torch.rand(width, generator=gen, dtype=torch.float64) * (hi - lo) + lo
    base = u.pow(1.0 / c)
    return torch.logit(base).to(dtype)


def make_case(B, T, W, nb, seed=0, lo=0.9, hi=0.999, c=8.0, h0_std=0.0, bias_std=0.0):
    """Synthetic inputs of the benchmark configurations: fp32 tensors on the CPU.  The gate biases
    are zero, as the reference initialises them, unless bias_std > 0 (parity cases: a trained model
    does not keep them at zero); they come from a generator of their own, so the other tensors do
    not depend on bias_std."""
    gen = torch.Generator().manual_seed(seed)
    bw = W // nb
    x = torch.randn(B, T, W, generator=gen)
    w_a, b_a = gate_init(nb, bw, gen)
    w_x, b_x = gate_init(nb, bw, gen)
    lam = lambda_init(W, gen, lo, hi, c)
    dy = torch.randn(B, T, W, generator=gen)
    h0 = torch.randn(B, W, generator=gen) * h0_std if h0_std > 0 else None
    if bias_std > 0:
        gen_b = torch.Generator().manual_seed(seed + 7919)
        b_a = bias_std * torch.randn(nb, bw, generator=gen_b)
        b_x = bias_std * torch.randn(nb, bw, generator=gen_b)
    return {"x": x, "w_a": w_a, "b_a": b_a, "w_x": w_x, "b_x": b_x, "lam": lam, "dy": dy, "h0": h0}


# ----------------------------------------------------------------------------------------------
# Caller side: causal depthwise convolution and the recurrent block (griffin/griffin.py:309-529)
# ----------------------------------------------------------------------------------------------

def segment_positions(B, T, prev=None, active_mask=None):
    """Default per-sequence positions: prev + cumsum(active) (griffin/griffin.py:327-338)."""
    act = torch.ones(B, T, dtype=torch.long) if active_mask is None else active_mask.to(torch.long)
    start = torch.full((B,), -1, dtype=torch.long) if prev is None else prev.to(torch.long)
    return start[:, None] + act.cumsum(dim=1)


def causal_conv(px, conv_w, conv_b, conv_state, seg_pos):
    """Dense-path depthwise causal conv with document mask (griffin/griffin.py:474-487).

    px [B,T,W]; conv_w [W,K] (tap K-1 multiplies the current token); conv_state [B,K-1,W].
    out_t = b + sum_lag w[:, K-1-lag] * px_{t-lag} * [seg_pos_t >= lag].  Returns (out, new_state).
    """
    B, T, W = px.shape
    K = conv_w.shape[1]
    hist = K - 1
    full = torch.cat([conv_state.to(px.dtype), px], dim=1)
    out = conv_b[None, None, :].expand(B, T, W).clone()
    for lag in range(K):
        src = full[:, hist - lag: hist - lag + T]
        keep = (seg_pos >= lag).to(px.dtype)[..., None]
        out = out + src * keep * conv_w[:, K - 1 - lag][None, None, :]
    new_state = full[:, full.shape[1] - hist:] if hist else full[:, :0]
    return out, new_state


def causal_conv_padded(px, conv_w, conv_b, conv_state, seg_pos, active):
    """Padded-path depthwise causal conv (griffin/griffin.py:488-510): a running window of the last
    K-1 active inputs, cleared where an active token has position 0; inactive tokens yield zeros and
    leave the window alone.  Shapes as in ``causal_conv``; ``active`` [B,T] bool.  Returns (out, window)."""
    B, T, W = px.shape
    K = conv_w.shape[1]
    window = conv_state.to(px.dtype).clone()
    rows = []
    for t in range(T):
        live = active[:, t]
        fresh = live & (seg_pos[:, t] == 0)
        window = torch.where(fresh[:, None, None], torch.zeros_like(window), window)
        value = px[:, t] * conv_w[:, K - 1] + conv_b
        for j in range(K - 1):
            value = value + window[:, j] * conv_w[:, j]
        rows.append(torch.where(live[:, None], value, torch.zeros_like(value)))
        if K > 1:
            moved = torch.cat([window[:, 1:], px[:, t][:, None]], dim=1)
            window = torch.where(live[:, None, None], moved, window)
    return torch.stack(rows, dim=1), window


def rmsnorm(x, g, eps=1e-6):
    """RMSNorm in front of the block (griffin/griffin.py:68-80): x * rsqrt(mean(x^2) + eps) * (1 + g)."""
    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps) * (1.0 + g)


def gelu_tanh(v):
    """tanh approximation of GeLU, the activation of the block's second branch (griffin/griffin.py:464,
    ``F.gelu(..., approximate="tanh")``): v/2 * (1 + tanh(sqrt(2/pi) * (v + 0.044715 v^3)))."""
    return 0.5 * v * (1.0 + torch.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))


def gelu_gate(h, v):
    """Output gate of the block: RG-LRU output times the GeLU branch (griffin/griffin.py:520)."""
    return h * gelu_tanh(v)


def recurrent_block_forward(x, p, c=8.0, cache=None):
    """All-active path of RecurrentBlock.forward (griffin/griffin.py:439-529).

    ``p`` holds linear_x.{w,b}, linear_y.{w,b}, conv.{w,b}, gate params, lam, linear_out.{w,b}.
    ``cache`` is (rnn_state, conv_state, segment_position) or None.  Returns (out, new_cache).
    """
    B, T, _ = x.shape
    prev = None if cache is None else cache[2]
    seg = segment_positions(B, T, prev)
    gate_in = x @ p["ly_w"].T + p["ly_b"]
    px = x @ p["lx_w"].T + p["lx_b"]
    K = p["conv_w"].shape[1]
    cstate = torch.zeros(B, K - 1, px.shape[2], dtype=px.dtype) if cache is None else cache[1]
    xb, new_cstate = causal_conv(px, p["conv_w"], p["conv_b"], cstate, seg)
    h0 = None if cache is None else cache[0]
    yr, h_last = rglru_forward(xb, p["w_a"], p["b_a"], p["w_x"], p["b_x"], p["lam"], c, h0,
                               reset_mask=(seg == 0), active_mask=None)
    out = gelu_gate(yr, gate_in) @ p["lo_w"].T + p["lo_b"]
    return out, (h_last, new_cstate, seg[:, -1].clone())
