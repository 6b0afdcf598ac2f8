"""Pins the CPU oracle: closed forms, library routines, invariants and the golden vectors."""

import os

import numpy as np
import pytest
import scipy.signal
import torch

from oracle import rglru_oracle as orc

torch.set_default_dtype(torch.float32)


def _load(golden_dir, name):
    data = np.load(os.path.join(golden_dir, name + ".npz"))
    return {k: torch.from_numpy(data[k]) for k in data.files}


# ---------------------------------------------------------------- scan

def test_scan_matches_bruteforce_closed_form():
    gen = torch.Generator().manual_seed(0)
    B, T, W = 2, 9, 3
    a = torch.rand(B, T, W, generator=gen, dtype=torch.float64)
    z = torch.randn(B, T, W, generator=gen, dtype=torch.float64)
    h0 = torch.randn(B, W, generator=gen, dtype=torch.float64)
    h = orc.sequential_scan(a, z, h0)
    for t in range(T):
        want = h0 * a[:, : t + 1].prod(dim=1)
        for s in range(t + 1):
            want = want + z[:, s] * a[:, s + 1: t + 1].prod(dim=1)
        torch.testing.assert_close(h[:, t], want, atol=1e-12, rtol=1e-12)


def test_scan_constant_decay_is_an_iir_filter():
    gen = torch.Generator().manual_seed(1)
    z = torch.randn(1, 64, 1, generator=gen, dtype=torch.float64)
    a = torch.full_like(z, 0.83)
    h = orc.sequential_scan(a, z, torch.zeros(1, 1, dtype=torch.float64))
    want = scipy.signal.lfilter([1.0], [1.0, -0.83], z[0, :, 0].numpy())
    np.testing.assert_allclose(h[0, :, 0].numpy(), want, atol=1e-12)


def test_scan_special_decays():
    gen = torch.Generator().manual_seed(2)
    z = torch.randn(2, 12, 4, generator=gen, dtype=torch.float64)
    h0 = torch.randn(2, 4, generator=gen, dtype=torch.float64)
    ones = orc.sequential_scan(torch.ones_like(z), z, h0)
    torch.testing.assert_close(ones, h0[:, None] + z.cumsum(dim=1))
    zeros = orc.sequential_scan(torch.zeros_like(z), z, h0)
    torch.testing.assert_close(zeros, z)


def test_scan_chunk_split_equals_whole():
    gen = torch.Generator().manual_seed(3)
    a = torch.rand(2, 20, 5, generator=gen, dtype=torch.float64)
    z = torch.randn(2, 20, 5, generator=gen, dtype=torch.float64)
    h0 = torch.randn(2, 5, generator=gen, dtype=torch.float64)
    whole = orc.sequential_scan(a, z, h0)
    first = orc.sequential_scan(a[:, :7], z[:, :7], h0)
    second = orc.sequential_scan(a[:, 7:], z[:, 7:], first[:, -1])
    torch.testing.assert_close(torch.cat([first, second], dim=1), whole, atol=1e-13, rtol=1e-13)


def test_scan_gradients_match_reverse_recurrence():
    gen = torch.Generator().manual_seed(4)
    a = torch.rand(2, 7, 3, generator=gen, dtype=torch.float64)
    z = torch.randn(2, 7, 3, generator=gen, dtype=torch.float64)
    h0 = torch.randn(2, 3, generator=gen, dtype=torch.float64)
    dh = torch.randn(2, 7, 3, generator=gen, dtype=torch.float64)
    h, da, dz, dh0 = orc.scan_autograd(a, z, h0, dh)
    delta = torch.zeros_like(dh)
    carry = torch.zeros(2, 3, dtype=torch.float64)
    for t in range(6, -1, -1):
        delta[:, t] = dh[:, t] + carry
        carry = a[:, t] * delta[:, t]
    h_prev = torch.cat([h0[:, None], h[:, :-1]], dim=1)
    torch.testing.assert_close(dz, delta)
    torch.testing.assert_close(da, delta * h_prev)
    torch.testing.assert_close(dh0, carry)


# ---------------------------------------------------------------- gates

def test_block_diagonal_gate_equals_dense_block_diag_matmul():
    gen = torch.Generator().manual_seed(5)
    nb, bw = 3, 4
    w = torch.randn(nb, bw, bw, generator=gen, dtype=torch.float64)
    b = torch.randn(nb, bw, generator=gen, dtype=torch.float64)
    x = torch.randn(2, 5, nb * bw, generator=gen, dtype=torch.float64)
    dense = torch.block_diag(*[w[k] for k in range(nb)])
    want = x @ dense.T + b.reshape(-1)
    torch.testing.assert_close(orc.block_diagonal_gate(x, w, b), want)


def test_bounded_sqrt_value_and_derivative():
    x = torch.tensor([0.0, 1e-9, 2.5e-7, 1e-4, 0.25, 1.0], dtype=torch.float64, requires_grad=True)
    y = orc.BoundedSqrt.apply(x)
    torch.testing.assert_close(y.detach(), x.detach().sqrt())
    (g,) = torch.autograd.grad(y.sum(), x)
    assert g[0].item() == pytest.approx(1000.0)
    assert g[1].item() == pytest.approx(1000.0)
    assert g[2].item() == pytest.approx(1000.0)
    for k in (3, 4, 5):
        assert g[k].item() == pytest.approx(0.5 / x[k].item() ** 0.5)


def test_gate_math_invariants():
    case = orc.make_case(2, 12, 16, 4, seed=6)
    p = [case[k].double() for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]
    gates = orc.gate_math(*p)
    torch.testing.assert_close(gates.a ** 2 + gates.g ** 2, torch.ones_like(gates.a))
    sig = torch.sigmoid(p[5])
    torch.testing.assert_close(gates.a, sig.pow(8.0 * gates.r))
    torch.testing.assert_close(gates.z, gates.g * gates.i * p[0])
    assert (gates.r > 0).all() and (gates.r < 1).all()


def test_gate_math_stays_accurate_near_unit_decay():
    # sigma(Lambda)^8 ~ 0.99999: 1 - a^2 must come from expm1, not from cancellation.
    x = torch.zeros(1, 1, 4)
    w = torch.zeros(1, 4, 4)
    b = torch.zeros(1, 4)
    lam = torch.logit(torch.full((4,), 0.99999, dtype=torch.float64).pow(1 / 8)).float()
    g32 = orc.gate_math(x, w, b, w, b, lam).g
    g64 = orc.gate_math(x.double(), w.double(), b.double(), w.double(), b.double(), lam.double()).g
    assert ((g32.double() - g64).abs() / g64).max() < 1e-5


def test_masks_reset_and_padding_semantics():
    case = orc.make_case(2, 10, 8, 2, seed=7)
    p = [case[k].double() for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]
    reset = torch.zeros(2, 10, dtype=torch.bool)
    reset[:, 4] = True
    y, _ = orc.rglru_forward(*p, reset_mask=reset)
    changed = [t.clone() for t in p]
    changed[0][:, :4] += 5.0
    y2, _ = orc.rglru_forward(*changed, reset_mask=reset)
    torch.testing.assert_close(y[:, 4:], y2[:, 4:])          # history before the reset is discarded
    assert (y[:, :4] - y2[:, :4]).abs().max() > 1e-3
    gates = orc.gate_math(*p, reset_mask=reset)
    torch.testing.assert_close(gates.z[:, 4], gates.i[:, 4] * p[0][:, 4])   # g == 1 at reset

    active = torch.ones(2, 10, dtype=torch.bool)
    active[1, 6:8] = False
    y3, h3 = orc.rglru_forward(*p, active_mask=active)
    torch.testing.assert_close(y3[1, 6], y3[1, 5])           # padding leaves the state unchanged
    torch.testing.assert_close(y3[1, 7], y3[1, 5])
    torch.testing.assert_close(h3, y3[:, -1])


def test_final_state_dtype_rule():
    case = orc.make_case(2, 5, 8, 2, seed=8)
    p = [case[k].bfloat16() for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]
    y, h = orc.rglru_forward(*p)
    assert y.dtype == torch.bfloat16 and h.dtype == torch.float32 and h.shape == (2, 8)


# ---------------------------------------------------------------- backward

def test_explicit_backward_matches_autograd_fp64():
    case = orc.make_case(2, 13, 24, 3, seed=9, h0_std=0.5)
    p = [case[k].double() for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]
    p[2] = p[2] + 0.2
    reset = torch.zeros(2, 13, dtype=torch.bool)
    reset[:, 6] = True
    active = torch.ones(2, 13, dtype=torch.bool)
    active[0, -2:] = False
    dh = torch.randn(2, 24, dtype=torch.float64)
    kw = dict(h0=case["h0"].double(), reset_mask=reset, active_mask=active, dh_last=dh)
    _, _, auto = orc.rglru_autograd(*p, case["dy"].double(), **kw)
    hand = orc.rglru_backward_explicit(*p, case["dy"].double(), **kw)
    for name, grad in auto.items():
        torch.testing.assert_close(hand[name], grad, atol=1e-11, rtol=1e-10)


def test_gradcheck_tiny():
    case = orc.make_case(1, 4, 4, 2, seed=10)
    leaves = [case[k].double().requires_grad_(True) for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]

    def fn(*args):
        return orc.rglru_forward(*args)[0]

    assert torch.autograd.gradcheck(fn, leaves, eps=1e-6, atol=1e-6)


# ---------------------------------------------------------------- golden vectors from the reference

@pytest.mark.parametrize("name", ["rglru_plain_b2_t16_w32", "rglru_masks_b2_t16_w32", "rglru_odd_b3_t37_w65"])
def test_oracle_matches_reference_golden_vectors(golden_dir, name):
    d = _load(golden_dir, name)
    kw = dict(h0=d.get("h0"), reset_mask=d["reset"], active_mask=d["active"], dh_last=d.get("dh"))
    p = [d[k] for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")]
    y, h_last, grads = orc.rglru_autograd(*p, d["dy"], **kw)
    torch.testing.assert_close(y, d["y"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(h_last, d["h_last"], atol=1e-6, rtol=1e-6)
    for key in ("x", "w_a", "b_a", "w_x", "b_x", "lam"):
        torch.testing.assert_close(grads[key], d["g_" + key], atol=2e-5, rtol=2e-5)
    if "g_h0" in d:
        torch.testing.assert_close(grads["h0"], d["g_h0"], atol=1e-5, rtol=1e-5)
    # the hand-written backward, evaluated in fp64, agrees with the recorded fp32 gradients
    p64 = [t.double() for t in p]
    kw64 = {k: (v.double() if v is not None and v.is_floating_point() else v) for k, v in kw.items()}
    hand = orc.rglru_backward_explicit(*p64, d["dy"].double(), **kw64)
    for key in ("x", "w_a", "b_a", "w_x", "b_x", "lam"):
        ref = d["g_" + key].double()
        assert (hand[key] - ref).abs().max() <= 2e-5 * max(1.0, ref.abs().max().item())


def test_oracle_matches_reference_saturated_gate(golden_dir):
    d = _load(golden_dir, "rglru_saturated_b2_t8_w16")
    W = 16
    w_a = torch.zeros(4, 4, 4)
    b_a = torch.full((4, 4), -100.0)
    lam = torch.full((W,), 20.0)
    x = d["x"].clone().requires_grad_(True)
    lam_leaf = lam.clone().requires_grad_(True)
    ba_leaf = b_a.clone().requires_grad_(True)
    y, _ = orc.rglru_forward(x, w_a, ba_leaf, d["w_x"], d["b_x"], lam_leaf)
    y.square().mean().backward()
    torch.testing.assert_close(y.detach(), d["y"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(x.grad, d["g_x"], atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(lam_leaf.grad, d["g_lam"], atol=1e-9, rtol=1e-4)
    assert torch.isfinite(x.grad).all() and torch.isfinite(lam_leaf.grad).all()


def test_oracle_block_matches_reference_golden(golden_dir):
    d = _load(golden_dir, "block_b2_t9_d8_w12")
    out, cache = orc.recurrent_block_forward(d["x"], d)
    torch.testing.assert_close(out, d["full"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(cache[0], d["rnn_state"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(cache[1], d["conv_state"], atol=1e-6, rtol=1e-6)
    assert torch.equal(cache[2], d["segment_position"])
    pieces, state, start = [], None, 0
    for stop in list(d["splits"].tolist()) + [d["x"].shape[1]]:
        piece, state = orc.recurrent_block_forward(d["x"][:, start:stop], d, cache=state)
        pieces.append(piece)
        start = stop
    torch.testing.assert_close(torch.cat(pieces, dim=1), d["chunked"], atol=1e-6, rtol=1e-6)


def test_selftest_inputs_are_the_documented_closed_forms():
    a, z, h0, up = orc.selftest_inputs()
    assert a.shape == (1, 7, 257) and h0.shape == (1, 257)
    assert a[0, 0, 0].item() == pytest.approx(0.9)
    assert z[0, 0, 0].item() == pytest.approx(0.1)
    assert a[0, 1, 0].item() == pytest.approx(0.9 + 0.05 * np.sin(257 / 97.0), abs=1e-6)
    assert up[0, 6, 256].item() == pytest.approx(np.cos((7 * 257 - 1) / 71.0), abs=1e-5)
    assert 0.85 - 1e-6 <= a.min() and a.max() <= 0.95 + 1e-6


def test_initialisers_follow_reference_ranges():
    gen = torch.Generator().manual_seed(0)
    lam = orc.lambda_init(4096, gen)
    a8 = torch.sigmoid(lam.double()).pow(8)
    assert a8.min() >= 0.9 - 1e-6 and a8.max() <= 0.999 + 1e-6
    w, b = orc.gate_init(16, 4, gen)
    assert abs(w.std().item() - 0.5) < 0.08 and (b == 0).all()


# ----------------------------------------------------------------------------------------------
# causal depthwise convolution of the caller (griffin/griffin.py:474-487)
# ----------------------------------------------------------------------------------------------
def _conv_case(B=2, T=13, W=6, K=4, seed=21):
    g = torch.Generator().manual_seed(seed)
    px = torch.randn(B, T, W, generator=g, dtype=torch.float64)
    w = torch.randn(W, K, generator=g, dtype=torch.float64)
    b = torch.randn(W, generator=g, dtype=torch.float64)
    state = torch.randn(B, K - 1, W, generator=g, dtype=torch.float64)
    return px, w, b, state


def test_oracle_conv_equals_library_conv1d_on_one_document():
    """Positions 3, 4, ... (every tap live): the conv is F.conv1d over cat(state, input), depthwise."""
    px, w, b, state = _conv_case()
    B, T, W = px.shape
    K = w.shape[1]
    seg = torch.arange(K - 1, K - 1 + T).repeat(B, 1)
    out, new_state = orc.causal_conv(px, w, b, state, seg)
    padded = torch.cat([state, px], dim=1).transpose(1, 2)
    want = torch.nn.functional.conv1d(padded, w[:, None, :], b, groups=W).transpose(1, 2)
    torch.testing.assert_close(out, want, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(new_state, px[:, T - (K - 1):])


def test_oracle_conv_fresh_document_ignores_history_and_state():
    """Positions 0, 1, ...: taps reaching before the document start are dropped, so the carried state
    has no influence and the result is conv1d with zero left padding; a document that starts inside
    the sequence sees nothing from before its first token."""
    px, w, b, state = _conv_case()
    B, T, W = px.shape
    K = w.shape[1]
    seg = torch.arange(T).repeat(B, 1)
    out, _ = orc.causal_conv(px, w, b, state, seg)
    zero_padded = torch.nn.functional.pad(px.transpose(1, 2), (K - 1, 0))
    want = torch.nn.functional.conv1d(zero_padded, w[:, None, :], b, groups=W).transpose(1, 2)
    torch.testing.assert_close(out, want, atol=1e-12, rtol=1e-12)
    start = 5
    seg2 = seg.clone()
    seg2[:, start:] -= start
    out2, _ = orc.causal_conv(px, w, b, state, seg2)
    alone, _ = orc.causal_conv(px[:, start:], w, b, torch.zeros_like(state), seg[:, : T - start])
    torch.testing.assert_close(out2[:, start:], alone, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(out2[:, :start], out[:, :start], atol=1e-12, rtol=1e-12)


def test_oracle_conv_brute_force_and_split_invariance():
    px, w, b, state = _conv_case(B=1, T=7, W=3, K=3, seed=5)
    seg = torch.tensor([[4, 5, 0, 1, 2, 3, 0]])
    out, new_state = orc.causal_conv(px, w, b, state, seg)
    padded = torch.cat([state, px], dim=1)
    K = 3
    for t in range(7):
        for c in range(3):
            want = b[c].item()
            for lag in range(K):
                if seg[0, t] >= lag:
                    want += w[c, K - 1 - lag].item() * padded[0, K - 1 + t - lag, c].item()
            assert out[0, t, c].item() == pytest.approx(want, abs=1e-12)
    first, mid_state = orc.causal_conv(px[:, :4], w, b, state, seg[:, :4])
    second, end_state = orc.causal_conv(px[:, 4:], w, b, mid_state, seg[:, 4:])
    torch.testing.assert_close(torch.cat([first, second], dim=1), out, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(end_state, new_state)


def test_oracle_gelu_gate_is_the_library_tanh_gelu():
    v = torch.linspace(-12.0, 12.0, 4001, dtype=torch.float64)
    torch.testing.assert_close(orc.gelu_tanh(v), torch.nn.functional.gelu(v, approximate="tanh"), atol=1e-14, rtol=1e-13)
    assert orc.gelu_tanh(torch.tensor(0.0)).item() == 0.0
    assert orc.gelu_tanh(torch.tensor(30.0, dtype=torch.float64)).item() == pytest.approx(30.0, rel=1e-12)
    assert abs(orc.gelu_tanh(torch.tensor(-30.0, dtype=torch.float64)).item()) < 1e-12
    # close to, but not the same as, the exact GeLU x * Phi(x): the approximation error peaks near 5e-4
    exact = torch.nn.functional.gelu(v)
    gap = (orc.gelu_tanh(v) - exact).abs().max().item()
    assert 1e-4 < gap < 1e-3
    h = torch.linspace(-2.0, 3.0, 4001, dtype=torch.float64)
    torch.testing.assert_close(orc.gelu_gate(h, v), h * torch.nn.functional.gelu(v, approximate="tanh"), atol=1e-14, rtol=1e-13)


def test_oracle_padded_conv_reduces_to_dense_conv_and_skips_padding():
    """With every token active and documents that start at position 0 the padded walk is the dense
    convolution; inserting inactive tokens anywhere changes nothing for the active ones (they see the
    same previous active inputs) and yields zeros at the inserted places; brute force on one row."""
    px, w, b, state = _conv_case(B=2, T=11, W=5, K=4, seed=8)
    B, T, W = px.shape
    seg = torch.arange(3, 3 + T).repeat(B, 1)
    seg[1, 6:] -= 9                                           # row 1 starts a new document at t = 6
    ones = torch.ones(B, T, dtype=torch.bool)
    dense, dense_state = orc.causal_conv(px, w, b, state, seg)
    walk, walk_state = orc.causal_conv_padded(px, w, b, state, seg, ones)
    torch.testing.assert_close(walk, dense, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(walk_state[0], dense_state[0])
    # row 1 restarted: rows of the state that predate the document are cleared, not carried
    assert torch.equal(walk_state[1], px[1, T - 3:])
    # pad: insert inactive tokens (random content) after t = 2 and t = 7
    g = torch.Generator().manual_seed(1)
    keep = [0, 1, 2, None, None, 3, 4, 5, 6, 7, None, 8, 9, 10]
    px2 = torch.stack([px[:, k] if k is not None else torch.randn(B, W, generator=g, dtype=px.dtype) for k in keep], dim=1)
    seg2 = torch.stack([seg[:, k] if k is not None else torch.zeros(B, dtype=torch.long) for k in keep], dim=1)
    act2 = torch.tensor([k is not None for k in keep]).repeat(B, 1)
    walk2, state2 = orc.causal_conv_padded(px2, w, b, state, seg2, act2)
    live_cols = [i for i, k in enumerate(keep) if k is not None]
    torch.testing.assert_close(walk2[:, live_cols], walk, atol=1e-12, rtol=1e-12)
    assert torch.count_nonzero(walk2[:, [i for i, k in enumerate(keep) if k is None]]) == 0
    torch.testing.assert_close(state2, walk_state)
    # all tokens inactive: zeros out, state untouched
    none, same = orc.causal_conv_padded(px, w, b, state, seg, torch.zeros(B, T, dtype=torch.bool))
    assert torch.count_nonzero(none) == 0 and torch.equal(same, state)


def test_oracle_rmsnorm_closed_forms():
    """Unit scale: every row leaves with mean square 1 (up to eps); a constant row c becomes sign(c)
    (1 + g); scaling the input by a positive factor changes nothing; matches the library's rms_norm."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 7, 12, generator=g, dtype=torch.float64)
    scale = torch.randn(12, generator=g, dtype=torch.float64) * 0.3
    y = orc.rmsnorm(x, torch.zeros(12, dtype=torch.float64))
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5, 7, dtype=torch.float64), atol=1e-5, rtol=0)
    const = torch.full((3, 12), -2.5, dtype=torch.float64)
    torch.testing.assert_close(orc.rmsnorm(const, scale), -(1.0 + scale).expand(3, 12), atol=1e-6, rtol=0)
    torch.testing.assert_close(orc.rmsnorm(3.0 * x, scale, eps=0.0), orc.rmsnorm(x, scale, eps=0.0), atol=1e-12, rtol=1e-12)
    want = torch.nn.functional.rms_norm(x, (12,), weight=1.0 + scale, eps=1e-6)
    torch.testing.assert_close(orc.rmsnorm(x, scale), want, atol=1e-12, rtol=1e-12)
