"""GPU parity of the causal depthwise convolution kernels (C ABI: rglru_hip_conv_fwd / _bwd) against the
oracle's restatement of griffin/griffin.py:474-487 and autograd through it."""

import pytest
import torch

from oracle import rglru_oracle as orc
from tests.helpers import rel_err

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5     # norm-wise relative, fp32 storage
BF16_TOL = 2e-2     # bf16 storage, fp32 arithmetic, against the fp32 oracle on the bf16-rounded inputs


def _say(*args):
    print(*args, flush=True)


def _positions(B, T, kind, seed):
    """Token positions: one document continued from earlier calls, fresh documents, or several
    documents packed into each row."""
    if kind == "continued":
        return torch.arange(5, 5 + T).repeat(B, 1)
    if kind == "fresh":
        return torch.arange(T).repeat(B, 1)
    g = torch.Generator().manual_seed(seed)
    pos = torch.empty(B, T, dtype=torch.long)
    for b in range(B):
        p = int(torch.randint(0, 4, (1,), generator=g))
        for t in range(T):
            if t > 0 and float(torch.rand(1, generator=g)) < 0.15:
                p = 0
            pos[b, t] = p
            p += 1
    return pos


def _case(B, T, W, K, seed, with_state, with_bias):
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, T, W, generator=g)
    w = torch.randn(W, K, generator=g) * (1.0 / K) ** 0.5
    b = torch.randn(W, generator=g) * 0.1 if with_bias else None
    state = torch.randn(B, K - 1, W, generator=g) if with_state else None
    dout = torch.randn(B, T, W, generator=g)
    return u, w, b, state, dout


def _oracle(u, w, b, state, dout, pos, dtype):
    def prep(t):
        return None if t is None else t.to(dtype).to(torch.float32).requires_grad_(True)
    u_, w_, b_, s_ = prep(u), prep(w), prep(b), prep(state)
    B, T, W = u.shape
    K = w.shape[1]
    out, new_state = orc.causal_conv(u_, w_, torch.zeros(W) if b_ is None else b_,
                                     torch.zeros(B, K - 1, W) if s_ is None else s_, pos)
    leaves = [t for t in (u_, w_, b_, s_) if t is not None]
    grads = torch.autograd.grad(out, leaves, dout.to(dtype).to(torch.float32))
    names = [n for n, t in zip(("u", "w", "b", "state"), (u_, w_, b_, s_)) if t is not None]
    return out.detach(), new_state.detach(), dict(zip(names, grads))


def _hip(u, w, b, state, dout, pos, dtype):
    from griffin_amd.hip_block_ops import hip_causal_conv

    def prep(t):
        return None if t is None else t.to(dtype).cuda().requires_grad_(True)
    u_, b_, s_ = prep(u), prep(b), prep(state)
    w_ = w.to(dtype)[:, None, :].contiguous().cuda().requires_grad_(True)
    out, new_state = hip_causal_conv(u_, s_, w_, b_, pos.cuda())
    leaves = [t for t in (u_, w_, b_, s_) if t is not None]
    grads = list(torch.autograd.grad(out, leaves, dout.to(dtype).cuda()))
    torch.cuda.synchronize()
    names = [n for n, t in zip(("u", "w", "b", "state"), (u_, w_, b_, s_)) if t is not None]
    grads[1] = grads[1][:, 0, :]
    return out.detach(), new_state.detach(), dict(zip(names, grads))


CASES = [
    # B, T, W, K, positions, carried state, bias
    (2, 50, 64, 4, "packed", True, True),      # vector path, several documents per row
    (2, 37, 24, 4, "packed", True, True),      # fp32 rows of 96 bytes (vector path), bf16 rows of 48 (vector path)
    (3, 33, 13, 4, "packed", True, True),      # odd width: one element per thread
    (1, 2, 64, 4, "continued", True, True),    # shorter than the kernel: the new state mixes old state and input
    (2, 100, 128, 3, "fresh", False, True),    # three taps, no carried state
    (2, 40, 32, 2, "continued", True, False),  # two taps, no bias
    (2, 19, 16, 1, "packed", False, True),     # a single tap: a per-channel scale and shift
    (4, 300, 256, 4, "packed", True, True),    # several runs per sequence, halo across run boundaries
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", CASES)
def test_conv_matches_oracle(cfg, dtype):
    B, T, W, K, kind, with_state, with_bias = cfg
    _say("conv case", cfg, dtype)
    u, w, b, state, dout = _case(B, T, W, K, seed=3, with_state=with_state, with_bias=with_bias)
    pos = _positions(B, T, kind, seed=4)
    want_out, want_state, want_g = _oracle(u, w, b, state, dout, pos, dtype)
    got_out, got_state, got_g = _hip(u, w, b, state, dout, pos, dtype)
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    errs = {"out": rel_err(got_out.float(), want_out)}
    for name in want_g:
        errs["d" + name] = rel_err(got_g[name].float(), want_g[name])
    _say("  rel errors:", {k: "%.2e" % v for k, v in errs.items()})
    for name, err in errs.items():
        assert err < tol, (name, err)
    # the carried state is a copy of input rows: exact in the storage type
    assert torch.equal(got_state.float().cpu(), want_state.to(dtype).float())


def test_conv_split_equals_one_pass_at_training_shape():
    """B8 T2048 W1024 bf16: the sequence convolved in three pieces with the carried state equals one
    pass bit for bit (each output depends on the same K rows either way), and the input gradient is
    linear in the upstream gradient."""
    from griffin_amd.hip_block_ops import hip_causal_conv

    g = torch.Generator().manual_seed(9)
    B, T, W, K = 8, 2048, 1024, 4
    u = torch.randn(B, T, W, generator=g).bfloat16().cuda()
    w = (torch.randn(W, 1, K, generator=g) * 0.5).bfloat16().cuda()
    b = (torch.randn(W, generator=g) * 0.1).bfloat16().cuda()
    pos = torch.arange(T).repeat(B, 1).cuda()
    pos[3, 700:] -= 700
    whole, last = hip_causal_conv(u, None, w, b, pos)
    pieces, state, start = [], None, 0
    for stop in (5, 1031, T):
        piece, state = hip_causal_conv(u[:, start:stop].contiguous(), state, w, b, pos[:, start:stop].contiguous())
        pieces.append(piece)
        start = stop
    assert torch.equal(torch.cat(pieces, dim=1), whole)
    assert torch.equal(state, last)
    uu = u.clone().requires_grad_(True)
    out, _ = hip_causal_conv(uu, None, w, b, pos)
    d1 = torch.randn(B, T, W, generator=g).bfloat16().cuda()
    g1, = torch.autograd.grad(out, uu, d1, retain_graph=True)
    g2, = torch.autograd.grad(out, uu, 2 * d1)
    torch.cuda.synchronize()
    assert rel_err(g2.float(), 2 * g1.float()) < 1e-2


def test_conv_argument_errors():
    from griffin_amd.hip_block_ops import hip_causal_conv

    u = torch.randn(2, 8, 16, device="cuda")
    w = torch.randn(16, 1, 4, device="cuda")
    pos = torch.arange(8, device="cuda").repeat(2, 1)
    with pytest.raises(RuntimeError):
        hip_causal_conv(u.cpu(), None, w.cpu(), None, pos.cpu())
    with pytest.raises(ValueError):
        hip_causal_conv(u, None, torch.randn(16, 1, 9, device="cuda"), None, pos)      # kernel size beyond the maximum
    with pytest.raises(ValueError):
        hip_causal_conv(u, torch.zeros(2, 2, 16, device="cuda"), w, None, pos)         # state of the wrong length
    with pytest.raises(ValueError):
        hip_causal_conv(u, None, w, None, pos[:, :4])
    with pytest.raises(TypeError):
        hip_causal_conv(u.double(), None, w.double(), None, pos)


# ----------------------------------------------------------------------------------------------
# output gate h * gelu_tanh(v) (C ABI: rglru_hip_gelu_gate_fwd / _bwd)
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64), (3, 7, 13), (1, 1, 1), (4, 300, 256), (5, 1023)])
def test_gelu_gate_matches_oracle(shape, dtype):
    from griffin_amd.hip_block_ops import hip_gelu_gate

    _say("gelu gate case", shape, dtype)
    g = torch.Generator().manual_seed(11)
    h = torch.randn(*shape, generator=g) * 1.5
    v = torch.randn(*shape, generator=g) * 3.0          # covers the saturated tails of tanh
    dout = torch.randn(*shape, generator=g)
    hr = h.to(dtype).float().requires_grad_(True)
    vr = v.to(dtype).float().requires_grad_(True)
    want = orc.gelu_gate(hr, vr)
    want_dh, want_dv = torch.autograd.grad(want, (hr, vr), dout.to(dtype).float())
    hh = h.to(dtype).cuda().requires_grad_(True)
    vh = v.to(dtype).cuda().requires_grad_(True)
    got = hip_gelu_gate(hh, vh)
    got_dh, got_dv = torch.autograd.grad(got, (hh, vh), dout.to(dtype).cuda())
    torch.cuda.synchronize()
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    errs = {"out": rel_err(got.float(), want), "dh": rel_err(got_dh.float(), want_dh), "dv": rel_err(got_dv.float(), want_dv)}
    _say("  rel errors:", {k: "%.2e" % e for k, e in errs.items()})
    for name, err in errs.items():
        assert err < tol, (name, err)


def test_gelu_gate_special_values_at_training_shape():
    """B8 T2048 W1024 bf16: exact zeros where either factor is zero, the identity far in the positive
    tail, zero far in the negative tail, and linearity in h."""
    from griffin_amd.hip_block_ops import hip_gelu_gate

    g = torch.Generator().manual_seed(12)
    shape = (8, 2048, 1024)
    h = torch.randn(*shape, generator=g).bfloat16().cuda()
    v = (torch.randn(*shape, generator=g) * 2).bfloat16().cuda()
    assert torch.count_nonzero(hip_gelu_gate(h, torch.zeros_like(v))) == 0
    assert torch.count_nonzero(hip_gelu_gate(torch.zeros_like(h), v)) == 0
    big = torch.full_like(v, 40.0)
    assert torch.equal(hip_gelu_gate(h, big), (h.float() * 40.0).bfloat16())
    assert torch.count_nonzero(hip_gelu_gate(h, -big)) == 0
    out1 = hip_gelu_gate(h, v).float()
    out2 = hip_gelu_gate(2 * h, v).float()
    assert rel_err(out2, 2 * out1) < 1e-2


def test_gelu_gate_argument_errors():
    from griffin_amd.hip_block_ops import hip_gelu_gate

    a = torch.randn(4, 8, device="cuda")
    with pytest.raises(RuntimeError):
        hip_gelu_gate(a.cpu(), a.cpu())
    with pytest.raises(ValueError):
        hip_gelu_gate(a, a[:, :4])
    with pytest.raises(TypeError):
        hip_gelu_gate(a, a.bfloat16())
    with pytest.raises(TypeError):
        hip_gelu_gate(a.double(), a.double())


# ----------------------------------------------------------------------------------------------
# convolution over right-padded batches (C ABI: rglru_hip_conv_padded_fwd)
# ----------------------------------------------------------------------------------------------
def _padded_inputs(B, T, W, K, seed, pattern):
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, T, W, generator=g)
    w = torch.randn(W, K, generator=g) * (1.0 / K) ** 0.5
    b = torch.randn(W, generator=g) * 0.1
    state = torch.randn(B, K - 1, W, generator=g)
    if pattern == "right":                                   # rows of different lengths, padded on the right
        lengths = torch.randint(0, T + 1, (B,), generator=g)
        lengths[0] = T
        if B > 1:
            lengths[1] = 0                                   # an empty row: state must pass through
        active = torch.arange(T)[None, :] < lengths[:, None]
    elif pattern == "mixed":                                 # right-padded rows and rows with holes side by side:
        lengths = torch.randint(0, T + 1, (B,), generator=g)  # the two kinds go to different kernels of one call
        active = torch.arange(T)[None, :] < lengths[:, None]
        active[::2] = torch.rand((B + 1) // 2, T, generator=g) > 0.3
    else:                                                    # holes anywhere
        active = torch.rand(B, T, generator=g) > 0.3
    pos = _positions(B, T, "packed", seed + 1)
    return u, w, b, state, pos, active


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", [(3, 50, 64, 4, "right"), (4, 200, 24, 4, "holes"), (2, 130, 13, 3, "holes"),
                                 (3, 65, 128, 2, "right"), (2, 7, 16, 1, "holes"), (5, 300, 64, 4, "mixed"),
                                 (4, 2100, 256, 4, "right")])
def test_padded_conv_matches_oracle(cfg, dtype):
    from griffin_amd.hip_block_ops import hip_causal_conv_padded

    B, T, W, K, pattern = cfg
    _say("padded conv case", cfg, dtype)
    u, w, b, state, pos, active = _padded_inputs(B, T, W, K, seed=13, pattern=pattern)
    up = lambda t: t.to(dtype).float()
    want, want_state = orc.causal_conv_padded(up(u), up(w), up(b), up(state), pos, active)
    got, got_state = hip_causal_conv_padded(u.to(dtype).cuda(), state.to(dtype).cuda(),
                                            w.to(dtype)[:, None, :].contiguous().cuda(), b.to(dtype).cuda(),
                                            pos.cuda(), active.cuda())
    torch.cuda.synchronize()
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    err = rel_err(got.float(), want)
    _say("  rel error:", "%.2e" % err)
    assert err < tol
    assert torch.count_nonzero(got[~active.cuda()]) == 0
    # the carried window is made of copies of input or state rows (or zeros): exact in the storage type
    assert torch.equal(got_state.float().cpu(), want_state.to(dtype).float())


def test_padded_conv_all_active_equals_dense_kernel_at_training_shape():
    """B8 T2048 W1024 bf16, every token active, documents starting at position 0: the padded kernel
    and the dense kernel walk the same K rows per output and agree bit for bit."""
    from griffin_amd.hip_block_ops import hip_causal_conv, hip_causal_conv_padded

    g = torch.Generator().manual_seed(17)
    B, T, W, K = 8, 2048, 1024, 4
    u = torch.randn(B, T, W, generator=g).bfloat16().cuda()
    w = (torch.randn(W, 1, K, generator=g) * 0.5).bfloat16().cuda()
    b = (torch.randn(W, generator=g) * 0.1).bfloat16().cuda()
    pos = torch.arange(T).repeat(B, 1).cuda()
    pos[5, 1000:] -= 1000
    active = torch.ones(B, T, dtype=torch.bool, device="cuda")
    dense, _ = hip_causal_conv(u, None, w, b, pos)
    padded, _ = hip_causal_conv_padded(u, None, w, b, pos, active)
    assert torch.equal(dense, padded)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", [(3, 50, 64, 4, "right"), (4, 200, 24, 4, "holes"), (2, 130, 13, 3, "holes"),
                                 (3, 65, 128, 2, "right"), (2, 7, 16, 1, "holes"), (2, 300, 1024, 4, "holes"),
                                 (5, 300, 64, 4, "mixed"), (4, 700, 256, 3, "right")])
def test_padded_conv_gradients_match_oracle_autograd(cfg, dtype):
    """Reverse mode of the padded convolution (C ABI: rglru_hip_conv_padded_bwd) against autograd through
    the oracle's token-by-token loop: gradients at the input, the carried state, the taps and the bias."""
    from griffin_amd.hip_block_ops import hip_causal_conv_padded

    B, T, W, K, pattern = cfg
    _say("padded conv gradient case", cfg, dtype)
    u, w, b, state, pos, active = _padded_inputs(B, T, W, K, seed=29, pattern=pattern)
    dout = torch.randn(B, T, W, generator=torch.Generator().manual_seed(31))
    up = lambda t: t.to(dtype).float()
    ref = [up(t).clone().requires_grad_(True) for t in (u, w, b, state)]
    want, _ = orc.causal_conv_padded(ref[0], ref[1], ref[2], ref[3], pos, active)
    want.backward(up(dout))
    dev = [u.to(dtype).cuda().requires_grad_(True), w.to(dtype)[:, None, :].contiguous().cuda().requires_grad_(True),
           b.to(dtype).cuda().requires_grad_(True), state.to(dtype).cuda().requires_grad_(True)]
    got, _ = hip_causal_conv_padded(dev[0], dev[3], dev[1], dev[2], pos.cuda(), active.cuda())
    got.backward(dout.to(dtype).cuda())
    torch.cuda.synchronize()
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    names = ("input", "taps", "bias", "state")
    for name, r, d in zip(names, ref, dev):
        if K == 1 and name == "state":
            continue
        grad = d.grad.float().cpu().reshape(r.grad.shape)
        err = rel_err(grad, r.grad)
        _say("  d%s rel error: %.2e" % (name, err))
        assert err < tol, name
    # padding receives no gradient at all
    assert torch.count_nonzero(dev[0].grad[~active.cuda()]) == 0


# ----------------------------------------------------------------------------------------------
# RMSNorm in front of the block (C ABI: rglru_hip_rmsnorm_fwd / _bwd)
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64), (3, 7, 13), (1, 1, 768), (4, 33, 1024), (2, 5, 2560), (300, 24),
                                   (70, 4096), (9, 5000), (33, 8192)])
def test_rmsnorm_matches_oracle(shape, dtype):
    from griffin_amd.hip_block_ops import hip_rmsnorm

    from griffin_amd.hip_block_ops import rmsnorm_max_width

    _say("rmsnorm case", shape, dtype)
    if shape[-1] > rmsnorm_max_width(dtype):
        pytest.skip("wider than one wave holds in this storage type: the module uses the portable operators there")
    gen = torch.Generator().manual_seed(21)
    x = torch.randn(*shape, generator=gen) * 1.7 + 0.3
    scale = torch.randn(shape[-1], generator=gen) * 0.2
    dy = torch.randn(*shape, generator=gen)
    xr = x.to(dtype).float().requires_grad_(True)
    sr = scale.to(dtype).float().requires_grad_(True)
    want = orc.rmsnorm(xr, sr)
    want_dx, want_dg = torch.autograd.grad(want, (xr, sr), dy.to(dtype).float())
    xh = x.to(dtype).cuda().requires_grad_(True)
    sh = scale.to(dtype).cuda().requires_grad_(True)
    got = hip_rmsnorm(xh, sh)
    got_dx, got_dg = torch.autograd.grad(got, (xh, sh), dy.to(dtype).cuda())
    torch.cuda.synchronize()
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    errs = {"y": rel_err(got.float(), want), "dx": rel_err(got_dx.float(), want_dx), "dg": rel_err(got_dg.float(), want_dg)}
    _say("  rel errors:", {k: "%.2e" % e for k, e in errs.items()})
    for name, err in errs.items():
        assert err < tol, (name, err)


def test_rmsnorm_module_and_properties_at_training_shape():
    """B8 T2048 D768 bf16 through the module: rows leave with mean square (1 + g)^2-weighted ~ 1 for a
    zero scale, a positive rescaling of the input changes nothing (eps aside), and the module's state
    dict keeps the reference's single parameter name."""
    from griffin_amd import RMSNorm

    norm = RMSNorm(768).cuda().bfloat16()
    assert list(norm.state_dict()) == ["g"]
    gen = torch.Generator().manual_seed(22)
    x = (torch.randn(8, 2048, 768, generator=gen) * 3).bfloat16().cuda()
    y = norm(x)
    ms = y.float().pow(2).mean(-1)
    assert (ms - 1.0).abs().max().item() < 2e-2
    y4 = norm(4 * x)                                          # a power of two: exact in bf16
    assert rel_err(y4.float(), y.float()) < 1e-2
    with pytest.raises(ValueError):
        from griffin_amd.hip_block_ops import hip_rmsnorm
        hip_rmsnorm(x, torch.zeros(5, device="cuda", dtype=torch.bfloat16))


# ----------------------------------------------------------------------------------------------
# sum of the partial weight gradients of a split contraction (C ABI: rglru_hip_sum_sets)
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(8, 2048, 768), (16, 768, 1024), (3, 7, 13), (1, 64, 64), (9, 1, 5), (2, 1000001)])
def test_sum_sets_matches_a_float64_sum(shape, dtype):
    from griffin_amd.hip_block_ops import _sum_sets

    _say("sum of sets", shape, dtype)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(41)).to(dtype)
    want = x.double().sum(0)
    got = _sum_sets(x.cuda())
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == want.shape
    # fp32 accumulation, one rounding to the storage type
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    assert rel_err(got.double(), want) < tol
    # a view that is not contiguous takes the generic reduction and still agrees
    strided = x.cuda().transpose(0, 1) if x.dim() == 3 else None
    if strided is not None:
        assert rel_err(_sum_sets(strided).double(), x.double().transpose(0, 1).sum(0)) < tol


def test_sum_sets_rejects_bad_arguments():
    from griffin_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(64, device="cuda")
    assert lib.rglru_hip_sum_sets(buf.data_ptr(), buf.data_ptr(), 0, 8, 0, None) != 0
    assert lib.rglru_hip_sum_sets(None, buf.data_ptr(), 2, 8, 0, None) != 0
    assert lib.rglru_hip_sum_sets(buf.data_ptr(), buf.data_ptr(), 2, 8, 7, None) != 0


# ----------------------------------------------------------------------------------------------
# bias gradient of the block's Linear layers (C ABI: rglru_hip_colsum)
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64, 96), (3, 7, 13, 5), (1, 1, 768, 1024), (8, 2048, 768, 1024), (2, 129, 24, 1030)])
def test_hip_linear_matches_torch_linear(shape, dtype):
    """Output and all three gradients of hip_linear against torch.nn.functional.linear in fp64 on the same
    (rounded) operands; the bias gradient is the column sum the library computes."""
    from griffin_amd.hip_block_ops import hip_linear

    B, T, D, W = shape
    _say("linear case", shape, dtype)
    gen = torch.Generator().manual_seed(33)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    w = (torch.randn(W, D, generator=gen) / D ** 0.5).to(dtype)
    b = (torch.randn(W, generator=gen) * 0.1).to(dtype)
    dy = torch.randn(B, T, W, generator=gen).to(dtype)
    ref = [t.double().requires_grad_(True) for t in (x, w, b)]
    torch.nn.functional.linear(*ref).backward(dy.double())
    dev = [t.cuda().requires_grad_(True) for t in (x, w, b)]
    out = hip_linear(*dev)
    out.backward(dy.cuda())
    torch.cuda.synchronize()
    tol = 2e-5 if dtype == torch.float32 else BF16_TOL
    want = torch.nn.functional.linear(x.double(), w.double(), b.double())
    assert rel_err(out.double().cpu(), want) < tol
    for name, r, d in zip(("x", "weight", "bias"), ref, dev):
        err = rel_err(d.grad.double().cpu(), r.grad)
        _say("  d%s rel error: %.2e" % (name, err))
        assert err < tol, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64, 96), (3, 7, 13, 5), (8, 2048, 768, 1024)])
@pytest.mark.parametrize("used", ["both", "first", "second"])
def test_hip_linear_pair_matches_two_linear_layers(shape, dtype, used):
    """The block's two input projections as one autograd node (griffin/griffin.py:462-464): outputs and all
    five gradients against two torch.nn.functional.linear calls in fp64, also when only one of the two
    outputs takes part in the loss."""
    from griffin_amd.hip_block_ops import hip_linear_pair

    B, T, D, W = shape
    _say("linear pair case", shape, dtype, used)
    gen = torch.Generator().manual_seed(34)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    ws = [(torch.randn(W, D, generator=gen) / D ** 0.5).to(dtype) for _ in range(2)]
    bs = [(torch.randn(W, generator=gen) * 0.1).to(dtype) for _ in range(2)]
    dys = [torch.randn(B, T, W, generator=gen).to(dtype) for _ in range(2)]
    take = [used in ("both", "first"), used in ("both", "second")]
    ref = [t.double().requires_grad_(True) for t in (x, ws[0], bs[0], ws[1], bs[1])]
    outs = (torch.nn.functional.linear(ref[0], ref[1], ref[2]), torch.nn.functional.linear(ref[0], ref[3], ref[4]))
    sum((o * d.double()).sum() for o, d, t in zip(outs, dys, take) if t).backward()
    dev = [t.cuda().requires_grad_(True) for t in (x, ws[0], bs[0], ws[1], bs[1])]
    got = hip_linear_pair(*dev)
    sum((o.float() * d.cuda().float()).sum() for o, d, t in zip(got, dys, take) if t).backward()
    torch.cuda.synchronize()
    tol = 2e-5 if dtype == torch.float32 else BF16_TOL
    for o, w in zip(got, outs):
        assert rel_err(o.double().cpu(), w.detach()) < tol
    for name, r, d in zip(("x", "w1", "b1", "w2", "b2"), ref, dev):
        if r.grad is None:
            assert d.grad is None, name
            continue
        err = rel_err(d.grad.double().cpu(), r.grad)
        _say("  d%s rel error: %.2e" % (name, err))
        assert err < tol, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64, 3), (3, 37, 13, 4), (1, 1, 8, 2), (8, 2048, 1024, 4)])
def test_strided_gradient_outputs_equal_the_contiguous_ones(shape, dtype):
    """rglru_hip_conv_bwd with du_stride and rglru_hip_gelu_gate_bwd with dv_stride (C ABI): du and dv written as the
    column halves of one [B, T, 2 W + pad] matrix are bit for bit what the contiguous calls write, nothing else of
    that matrix is touched, and the other outputs do not change."""
    from griffin_amd import _lib
    from griffin_amd.hip_block_ops import _DTYPE_CODES, _dtype_code, _ptr, _stream_ptr

    B, T, W, K = shape
    _say("strided gradient outputs case", shape, dtype)
    lib = _lib.load()
    g = torch.Generator().manual_seed(35)
    rnd = lambda *s: torch.randn(*s, generator=g).to(dtype).cuda()
    u, dout, h, v, dgate = rnd(B, T, W), rnd(B, T, W), rnd(B, T, W), rnd(B, T, W) * 2, rnd(B, T, W)
    taps = (torch.randn(W, K, generator=g) * 0.4).to(dtype).cuda()
    pos = torch.arange(T).repeat(B, 1).cuda()
    pos[:, T // 2:] -= T // 2                                 # a document start in the middle of every row
    code, stream = _dtype_code(dtype), _stream_ptr(u.device)
    pad = 8 if W % 8 == 0 else 3                              # rows of whole 16-byte vectors where W allows the vector kernels
    ld = 2 * W + pad

    def conv_bwd(du):
        scratch = torch.empty(lib.rglru_hip_conv_scratch_bytes(B, T, W, K), dtype=torch.uint8, device="cuda")
        dtaps = torch.empty(W, K, dtype=dtype, device="cuda")
        dbias = torch.empty(W, dtype=dtype, device="cuda")
        _lib.check(lib.rglru_hip_conv_bwd(_ptr(u), None, _ptr(taps), _ptr(pos), _ptr(dout), _ptr(scratch), _ptr(du), du.stride(1),
                                          None, _ptr(dtaps), _ptr(dbias), B, T, W, K, code, _DTYPE_CODES[dtype], _DTYPE_CODES[dtype],
                                          stream), "rglru_hip_conv_bwd")
        return dtaps, dbias

    def gate_bwd(dv):
        dh = torch.empty_like(h)
        _lib.check(lib.rglru_hip_gelu_gate_bwd(_ptr(dgate), _ptr(h), _ptr(v), _ptr(dh), _ptr(dv), h.numel(), W, dv.stride(1),
                                               code, stream), "rglru_hip_gelu_gate_bwd")
        return dh

    du_c, dv_c = torch.empty_like(u), torch.empty_like(v)
    want_conv, want_dh = conv_bwd(du_c), gate_bwd(dv_c)
    both = torch.full((B, T, ld), 7.0, dtype=dtype, device="cuda")
    got_conv, got_dh = conv_bwd(both[..., :W]), gate_bwd(both[..., W:2 * W])
    torch.cuda.synchronize()
    assert torch.equal(both[..., :W], du_c)
    assert torch.equal(both[..., W:2 * W], dv_c)
    assert torch.all(both[..., 2 * W:] == 7.0)
    assert torch.equal(got_dh, want_dh)
    for a, b in zip(got_conv, want_conv):
        assert torch.equal(a, b)
    # a stride below the width is an error, not a memory fault
    with pytest.raises(ValueError):
        _lib.check(lib.rglru_hip_gelu_gate_bwd(_ptr(dgate), _ptr(h), _ptr(v), _ptr(torch.empty_like(h)), _ptr(dv_c), h.numel(), W, W - 1,
                                               code, stream), "rglru_hip_gelu_gate_bwd")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 64, 96), (3, 7, 13, 5), (8, 2048, 768, 1024)])
def test_hip_linear_pair_with_stacked_gradients(shape, dtype):
    """The pair's backward when its two incoming gradients are the column halves of one matrix (what the
    one-launch block forward's backward hands it): one GEMM for dx, one for both weight gradients, one column
    sum -- against two torch.nn.functional.linear calls in fp64."""
    from griffin_amd.hip_block_ops import _stacked_halves, hip_linear_pair

    B, T, D, W = shape
    _say("linear pair, stacked gradients, case", shape, dtype)
    gen = torch.Generator().manual_seed(36)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    ws = [(torch.randn(W, D, generator=gen) / D ** 0.5).to(dtype) for _ in range(2)]
    bs = [(torch.randn(W, generator=gen) * 0.1).to(dtype) for _ in range(2)]
    both = torch.randn(B, T, 2 * W, generator=gen).to(dtype)
    ref = [t.double().requires_grad_(True) for t in (x, ws[0], bs[0], ws[1], bs[1])]
    outs = (torch.nn.functional.linear(ref[0], ref[1], ref[2]), torch.nn.functional.linear(ref[0], ref[3], ref[4]))
    torch.autograd.backward(outs, [both[..., :W].double(), both[..., W:].double()])
    dev = [t.cuda().requires_grad_(True) for t in (x, ws[0], bs[0], ws[1], bs[1])]
    got = hip_linear_pair(*dev)
    both_d = both.cuda()
    halves = [both_d[..., :W], both_d[..., W:]]
    assert _stacked_halves(*halves) is not None
    torch.autograd.backward(got, halves)
    torch.cuda.synchronize()
    tol = 2e-5 if dtype == torch.float32 else BF16_TOL
    for name, r, d in zip(("x", "w1", "b1", "w2", "b2"), ref, dev):
        err = rel_err(d.grad.double().cpu(), r.grad)
        _say("  d%s rel error: %.2e" % (name, err))
        assert err < tol, name


# ----------------------------------------------------------------------------------------------
# convolution + RG-LRU + output gate in one forward launch (rglru_hip_block_fwd), griffin/griffin.py:464-520
# ----------------------------------------------------------------------------------------------
def _block_case(B, T, W, nb, K, kind, carried, strided, seed):
    """Operands of the block between its projections, bf16 on the GPU."""
    torch.manual_seed(seed)
    bw = W // nb
    bf = torch.bfloat16

    def rnd(*shape, scale=1.0):
        return (scale * torch.randn(*shape)).to(bf).cuda()

    p = {"w_a": rnd(nb, bw, bw, scale=bw ** -0.5), "b_a": rnd(nb, bw), "w_x": rnd(nb, bw, bw, scale=bw ** -0.5),
         "b_x": rnd(nb, bw), "weight": rnd(W, 1, K, scale=0.4), "bias": rnd(W, scale=0.1)}
    # decays of 0.9 .. 0.999 per token at an open gate, as the reference initialises them: the state then
    # carries across many tiles, so a wrong carry between tiles shows
    p["lam"] = torch.logit(torch.empty(W).uniform_(0.9, 0.999).pow(1.0 / 8.0)).to(bf).cuda()
    if strided:                                       # the two projections as halves of one wider buffer
        both = rnd(B, T, 2 * W + 16)
        p["u"], p["v"] = both[..., :W], both[..., W + 16:]
    else:
        p["u"], p["v"] = rnd(B, T, W), rnd(B, T, W)
    p["conv_state"] = rnd(B, K - 1, W) if (carried and K > 1) else None
    p["h0"] = torch.randn(B, W).cuda() if carried else None
    p["pos"] = _positions(B, T, kind, seed).cuda()
    return p


def _three_kernels(p):
    """The same computation as three launches through the autograd wrappers of the separate kernels."""
    from griffin_amd.hip_block_ops import hip_causal_conv, hip_gelu_gate
    from griffin_amd.hip_scan import hip_rglru

    x, new_conv = hip_causal_conv(p["u"], p["conv_state"], p["weight"], p["bias"], p["pos"])
    y, h_last = hip_rglru(x, p["w_a"], p["b_a"], p["w_x"], p["b_x"], p["lam"], 8.0, p["h0"], p["pos"] == 0, None)
    return hip_gelu_gate(y, p["v"].contiguous()), h_last, new_conv


BLOCK_FWD_CASES = [
    # B, T, W, nb, K, positions, carried state, strided rows
    (2, 128, 256, 2, 4, "fresh", False, False),
    (3, 200, 256, 2, 4, "packed", True, False),
    (3, 67, 128, 2, 4, "continued", True, True),
    (2, 1, 128, 4, 4, "continued", True, False),
    (2, 2, 128, 4, 3, "packed", True, False),
    (5, 130, 192, 3, 2, "packed", True, True),
    (2, 64, 96, 3, 4, "packed", False, False),
    (4, 333, 64, 1, 1, "packed", True, False),
    (8, 2048, 1024, 8, 4, "fresh", False, False),
    (8, 2048, 1024, 16, 4, "packed", True, True),
]


@pytest.mark.parametrize("case", BLOCK_FWD_CASES)
def test_block_forward_matches_the_three_kernels(case):
    """One launch against conv_fwd + fwd + gelu_gate (each checked against the oracle above and in
    test_hip_gpu.py): the convolved rows and the carried rows are bit-identical, y and the gated output
    agree to the rounding of a carry composed in another order (see test_hip_gpu.py on reproducibility)."""
    from griffin_amd.hip_block_ops import hip_block_forward

    B, T, W, nb, K, kind, carried, strided = case
    p = _block_case(B, T, W, nb, K, kind, carried, strided, seed=B + T)
    _say("block forward", case)
    from griffin_amd.hip_scan import FIRST_TOKEN_RESET

    with torch.no_grad():
        want_gated, want_h, want_conv = _three_kernels(p)
        got_gated, got_h, got_conv = hip_block_forward(
            p["u"], p["v"], p["conv_state"], p["weight"], p["bias"], p["pos"],
            FIRST_TOKEN_RESET if (kind == "fresh" and not carried) else None,   # positions 0 .. T-1: no flag tensor
            p["w_a"], p["b_a"], p["w_x"], p["b_x"], p["lam"], p["h0"], 8.0)
    torch.cuda.synchronize()
    if K > 1:
        assert torch.equal(got_conv, want_conv)
    # one bf16 rounding step at the largest value is 2^-8 of it
    assert rel_err(got_gated.float().cpu(), want_gated.float().cpu()) < 5e-3
    assert rel_err(got_h.cpu(), want_h.cpu()) < 1e-5
    # a changed bit here and there, not a systematic difference
    differing = (got_gated != want_gated).float().mean().item()
    assert differing < 1e-3, differing


@pytest.mark.parametrize("case", BLOCK_FWD_CASES)
def test_block_forward_gradients_match_the_three_kernels(case):
    """Autograd through the one-launch forward (its backward runs gate, scan and convolution reverse kernels
    on the x and y the forward kept) against autograd through the three separate operators."""
    from griffin_amd.hip_block_ops import hip_block_flags, hip_block_forward
    from griffin_amd.hip_scan import FIRST_TOKEN_RESET

    B, T, W, nb, K, kind, carried, strided = case
    p = _block_case(B, T, W, nb, K, kind, carried, strided, seed=B + T)
    names = [n for n in ("u", "v", "conv_state", "weight", "bias", "w_a", "b_a", "w_x", "b_x", "lam", "h0") if p[n] is not None]
    dg = torch.randn(B, T, W).to(torch.bfloat16).cuda()
    dh = torch.randn(B, W).cuda()
    dc = torch.randn(B, K - 1, W).to(torch.bfloat16).cuda()   # a later call's gradient at the carried rows
    _say("block forward gradients", case)

    def grads(fused):
        q = dict(p)
        for n in names:
            q[n] = p[n].detach().clone().requires_grad_(True)
        if fused:
            gated, h_last, carried_rows = hip_block_forward(
                q["u"], q["v"], q["conv_state"], q["weight"], q["bias"], q["pos"],
                FIRST_TOKEN_RESET if (kind == "fresh" and not carried) else hip_block_flags(q["pos"]) if B % 2 else None,
                q["w_a"], q["b_a"], q["w_x"], q["b_x"], q["lam"], q["h0"], 8.0)
        else:
            gated, h_last, carried_rows = _three_kernels(q)
        outs, ups = [gated, h_last], [dg, dh]
        if K > 1:
            outs.append(carried_rows)
            ups.append(dc)
        return torch.autograd.grad(outs, [q[n] for n in names], ups)

    want, got = grads(False), grads(True)
    torch.cuda.synchronize()
    for n, a, b in zip(names, got, want):
        assert a.shape == b.shape and a.dtype == b.dtype, n
        assert rel_err(a.float().cpu(), b.float().cpu()) < 5e-3, n


def test_block_forward_random_shapes():
    """Forty seeded draws of batch, length, width, gate blocks, taps, position pattern, carried state and row
    strides: outputs and, for every second draw, gradients against the three separate operators."""
    import random

    from griffin_amd.hip_block_ops import hip_block_forward
    from griffin_amd.hip_scan import FIRST_TOKEN_RESET

    rng = random.Random(20)
    for trial in range(40):
        bw, nb = rng.choice([32, 64, 128]), rng.choice([1, 2, 3, 5, 8])
        B, T = rng.choice([1, 2, 3, 7]), rng.choice([1, 2, 3, 5, 31, 64, 65, 127, 128, 200, 257, 500])
        K, kind = rng.choice([1, 2, 3, 4]), rng.choice(["fresh", "continued", "packed"])
        carried, strided, with_grads = rng.random() < 0.5, rng.random() < 0.4, trial % 2 == 1
        _say("block forward draw", trial, (B, T, bw * nb, nb, K, kind, carried, strided, with_grads))
        p = _block_case(B, T, bw * nb, nb, K, kind, carried, strided, seed=trial)
        names = [n for n in ("u", "v", "weight", "bias", "w_a", "b_a", "w_x", "b_x", "lam") if p[n] is not None]
        marker = FIRST_TOKEN_RESET if (kind == "fresh" and not carried) else None

        def run(fused):
            q = dict(p)
            for n in names:
                q[n] = p[n].detach().clone().requires_grad_(with_grads)
            if fused:
                outs = hip_block_forward(q["u"], q["v"], q["conv_state"], q["weight"], q["bias"], q["pos"], marker,
                                         q["w_a"], q["b_a"], q["w_x"], q["b_x"], q["lam"], q["h0"], 8.0)
            else:
                outs = _three_kernels(q)
            got = [o.detach() for o in outs]
            if with_grads:
                ups = [torch.full_like(outs[0], 0.5), torch.ones_like(outs[1])]
                got += list(torch.autograd.grad(list(outs[:2]), [q[n] for n in names], ups))
            return got

        with torch.set_grad_enabled(with_grads):
            want, got = run(False), run(True)
        torch.cuda.synchronize()
        if K > 1:
            assert torch.equal(got[2], want[2]), trial
        for i, (a, b) in enumerate(zip(got, want)):
            assert a.shape == b.shape, (trial, i)
            if a.numel():                                    # one tap carries no rows
                assert rel_err(a.float().cpu(), b.float().cpu()) < 1e-2, (trial, i)


def test_block_forward_argument_errors():
    from griffin_amd import _lib
    from griffin_amd.hip_block_ops import hip_block_forward_covers

    assert hip_block_forward_covers(1024, 8, 4, torch.bfloat16)
    assert not hip_block_forward_covers(1024, 8, 4, torch.float32)      # 16-bit storage only
    assert not hip_block_forward_covers(2560, 8, 4, torch.bfloat16)     # blocks of 320 channels: three launches
    assert not hip_block_forward_covers(1024, 8, 5, torch.bfloat16)
    lib = _lib.load()
    buf = torch.zeros(1 << 16, device="cuda", dtype=torch.bfloat16)
    p = buf.data_ptr()
    args = [p, 0, p, 0, None, p, None, 4, 1, p, None, None, None, None, p, None, None, p, 2, 16, 128, 2, 1, None]
    bad_stride = list(args); bad_stride[1] = 64
    assert lib.rglru_hip_block_fwd(*bad_stride) != 0 and b"stride" in lib.rglru_hip_last_error()
    unaligned = list(args); unaligned[0] = p + 2
    assert lib.rglru_hip_block_fwd(*unaligned) != 0 and b"aligned" in lib.rglru_hip_last_error()
    wide = list(args); wide[20] = 640
    assert lib.rglru_hip_block_fwd(*wide) != 0
