"""GPU tests of the module boundary and of the benchmark configurations (scan_mode="hip")."""

import copy

import pytest
import torch

from oracle import rglru_oracle as orc
from tests.helpers import PARAMS, hip_run, oracle_run, rel_err

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
BF16_TOL = 2e-2


def _say(*args):
    print(*args, flush=True)


def _module_from_case(case, nb, mode, dtype=torch.float32, device="cuda"):
    from griffin_amd import RG_LRU

    W = case["x"].shape[-1]
    module = RG_LRU(W, gate_blocks=nb, scan_mode=mode)
    module.load_state_dict({"recurrence_gate.weight": case["w_a"], "recurrence_gate.bias": case["b_a"],
                            "input_gate.weight": case["w_x"], "input_gate.bias": case["b_x"], "Lambda": case["lam"]})
    return module.to(device=device, dtype=dtype)


def test_full_module_hip_matches_sequential_backend():
    """Analogue of the reference's tests/test_rglru.py:170-204 (reset at t=17, 4 padded tokens)."""
    from griffin_amd import RG_LRU

    torch.manual_seed(0)
    sequential = RG_LRU(rnn_width=32, gate_blocks=4, scan_mode="sequential")
    hip = copy.deepcopy(sequential).cuda()
    hip.scan_mode = "hip"
    xs = torch.randn(2, 29, 32, requires_grad=True)
    xh = xs.detach().clone().cuda().requires_grad_(True)
    reset = torch.zeros(2, 29, dtype=torch.bool)
    reset[:, 17] = True
    active = torch.ones(2, 29, dtype=torch.bool)
    active[1, -4:] = False
    ys = sequential(xs, reset_mask=reset, active_mask=active)
    yh = hip(xh, reset_mask=reset.cuda(), active_mask=active.cuda())
    ys.square().mean().backward()
    yh.square().mean().backward()
    torch.testing.assert_close(yh.cpu(), ys, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(xh.grad.cpu(), xs.grad, atol=3e-5, rtol=3e-5)
    for ph, ps in zip(hip.parameters(), sequential.parameters()):
        torch.testing.assert_close(ph.grad.cpu(), ps.grad, atol=3e-5, rtol=3e-5)


def test_auto_mode_uses_validated_hip_path():
    from griffin_amd import RG_LRU, hip_scan_is_usable

    assert hip_scan_is_usable(torch.device("cuda"))
    assert hip_scan_is_usable("cuda:0")
    torch.manual_seed(1)
    auto = RG_LRU(rnn_width=64, gate_blocks=2, scan_mode="auto").cuda()
    seq = copy.deepcopy(auto)
    seq.scan_mode = "sequential"
    x = torch.randn(2, 70, 64, device="cuda")
    with torch.no_grad():
        ya, sa = auto(x, return_state=True)
        ys, ss = seq(x, return_state=True)
    assert sa.dtype == torch.float32 and sa.shape == (2, 64)
    torch.testing.assert_close(ya, ys, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(sa, ss, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(ya[:, -1], sa)
    # dtypes the kernels do not cover fall back to the portable scan instead of failing
    y16 = auto.half()(x.half())
    assert y16.dtype == torch.float16 and torch.isfinite(y16).all()


def test_explicit_hip_rejects_unsupported_dtype_and_shapes():
    from griffin_amd import RG_LRU

    module = RG_LRU(rnn_width=16, gate_blocks=2, scan_mode="hip").cuda()
    with pytest.raises(TypeError):
        module.double()(torch.randn(1, 4, 16, device="cuda", dtype=torch.float64))
    wide = RG_LRU(rnn_width=1026, gate_blocks=1, scan_mode="hip").cuda()
    with pytest.raises(ValueError, match="512"):
        wide(torch.randn(1, 4, 1026, device="cuda"))


def test_saturated_gate_stays_finite_in_bf16():
    """Analogue of tests/test_rglru.py:61-75 on the HIP path."""
    from griffin_amd import RG_LRU

    module = RG_LRU(rnn_width=16, gate_blocks=4, scan_mode="hip").cuda().to(torch.bfloat16)
    with torch.no_grad():
        module.recurrence_gate.weight.zero_()
        module.recurrence_gate.bias.fill_(-100)
        module.Lambda.fill_(20)
    x = torch.randn(2, 8, 16, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    y = module(x)
    y.float().square().mean().backward()
    assert torch.isfinite(y).all() and torch.isfinite(x.grad).all() and torch.isfinite(module.Lambda.grad).all()


def test_chunked_calls_with_carried_state_equal_one_call():
    case = orc.make_case(2, 200, 128, 2, seed=4, bias_std=0.3)
    module = _module_from_case(case, 2, "hip")
    x = case["x"].cuda()
    with torch.no_grad():
        whole, h_whole = module(x, return_state=True)
        first, h = module(x[:, :70].contiguous(), return_state=True)
        second, h = module(x[:, 70:133].contiguous(), h, return_state=True)
        third, h = module(x[:, 133:].contiguous(), h, return_state=True)
    torch.testing.assert_close(torch.cat([first, second, third], dim=1), whole, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(h, h_whole, atol=1e-6, rtol=1e-6)


def test_causality_on_the_hip_path():
    case = orc.make_case(2, 100, 64, 2, seed=5, bias_std=0.3)
    module = _module_from_case(case, 2, "hip")
    x = case["x"].cuda()
    changed = x.clone()
    changed[:, 40] += 10.0
    with torch.no_grad():
        a, b = module(x), module(changed)
    assert torch.equal(a[:, :40], b[:, :40])
    assert (a[:, 40:] - b[:, 40:]).abs().max() > 1e-3


def test_reset_isolates_documents_on_the_hip_path():
    case = orc.make_case(2, 96, 64, 2, seed=6, bias_std=0.3)
    module = _module_from_case(case, 2, "hip")
    x = case["x"].cuda()
    reset = torch.zeros(2, 96, dtype=torch.bool, device="cuda")
    reset[:, 50] = True
    changed = x.clone()
    changed[:, :50] += 3.0
    with torch.no_grad():
        a = module(x, reset_mask=reset)
        b = module(changed, reset_mask=reset)
    assert torch.equal(a[:, 50:], b[:, 50:])


# ------------------------------------------------------------------ benchmark configurations
def test_config1_reference_runnable_case_fp32():
    """B2 T256 W256, 8 blocks, fp32, h0 = 0: forward and every gradient within 1e-5."""
    case = orc.make_case(2, 256, 256, 8, seed=0)
    y, h_last, grads = hip_run(case, torch.float32)
    ry, rh, rgrads = oracle_run(case, torch.float32)
    _, _, g64 = oracle_run(case, torch.float64)
    errs = {"y": rel_err(y, ry), "h_last": rel_err(h_last, rh)}
    for name in grads:
        errs[name] = min(rel_err(grads[name], rgrads[name]), rel_err(grads[name], g64[name]))
    _say("config 1:", {k: "%.2e" % v for k, v in errs.items()})
    assert max(errs.values()) < FP32_TOL


def test_config2_training_shape_bf16():
    """B8 T2048 W1024, 8 blocks, bf16 storage / fp32 state, against the fp32 oracle."""
    case = orc.make_case(8, 2048, 1024, 8, seed=0)
    _say("config 2: running the CPU oracle (sequential scan, 2048 steps) ...")
    ry, rh, rgrads = oracle_run(case, torch.bfloat16)
    _say("config 2: oracle done, running the GPU path")
    y, h_last, grads = hip_run(case, torch.bfloat16)
    errs = {"y": rel_err(y.float(), ry), "h_last": rel_err(h_last, rh)}
    for name in grads:
        errs[name] = rel_err(grads[name].float(), rgrads[name])
    _say("config 2:", {k: "%.2e" % v for k, v in errs.items()})
    assert max(errs.values()) < BF16_TOL
    # What 16-bit weight gradients cost beyond their own final rounding: with bf16 parameters the 32 per-workgroup
    # partial sums of dW cross memory as bf16 (the reference accumulates in fp32 and rounds once).  The same step
    # with the same rounded values held in fp32 parameters keeps the partials and the result in fp32; rounding
    # that result to bf16 is what a single final rounding gives.
    from griffin_amd import hip_rglru

    leaves = [case[k].bfloat16().float().cuda().requires_grad_(True) for k in PARAMS]
    leaves[0] = case["x"].bfloat16().cuda().requires_grad_(True)
    y32, _ = hip_rglru(*leaves, 8.0)
    g32 = dict(zip(PARAMS, torch.autograd.grad(y32, leaves, case["dy"].bfloat16().cuda())))
    torch.cuda.synchronize()
    for name in ("w_a", "w_x"):
        once = g32[name].bfloat16().float()
        extra = rel_err(grads[name].float(), once)
        exact = rel_err(g32[name], rgrads[name])
        final = rel_err(once, rgrads[name])
        _say(f"config 2 d{name}: fp32 partials vs oracle {exact:.2e}, rounded once {final:.2e}, bf16 partials vs oracle "
             f"{errs[name]:.2e}, bf16 partials vs rounded once {extra:.2e}")
        # measured: 2.9e-4 with fp32 partials and an fp32 result; 2.0e-3 / 2.5e-3 once that result is rounded to
        # bf16; 2.0e-3 / 2.8e-3 with bf16 partials -- the final rounding dominates, the partials add < 1e-3
        assert exact < 2e-3 and errs[name] - final < 1e-3 and extra < 8e-3, name


def test_config3_long_context_slow_decay_bf16():
    """B1 W2560 (320-wide blocks), sigma(Lambda)^8 in [0.99, 0.9999].  The oracle is run on the
    first 4096 tokens; the full 32768-token length is covered by size-independent properties:
    splitting the sequence with carried state reproduces the one-call result, and the final
    state equals the last output."""
    from griffin_amd import hip_rglru

    W, nb = 2560, 8
    case = orc.make_case(1, 4096, W, nb, seed=3, lo=0.99, hi=0.9999)
    _say("config 3: oracle on 4096 tokens ...")
    ry, rh, rgrads = oracle_run(case, torch.bfloat16)
    y, h_last, grads = hip_run(case, torch.bfloat16)
    errs = {"y": rel_err(y.float(), ry), "h_last": rel_err(h_last, rh)}
    for name in grads:
        errs[name] = rel_err(grads[name].float(), rgrads[name])
    _say("config 3 (T=4096):", {k: "%.2e" % v for k, v in errs.items()})
    assert max(errs.values()) < BF16_TOL

    T = 32768
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(1, T, W, generator=gen).bfloat16().cuda()
    params = [case[k].bfloat16().cuda() for k in PARAMS[1:]]
    with torch.no_grad():
        whole, h_whole = hip_rglru(x, *params)
        h = None
        pieces = []
        for lo, hi in ((0, 10000), (10000, 10016), (10016, 25001), (25001, T)):
            piece, h = hip_rglru(x[:, lo:hi].contiguous(), *params, 8.0, h)
            pieces.append(piece)
    torch.cuda.synchronize()
    split = torch.cat(pieces, dim=1)
    assert rel_err(split.float(), whole.float()) < 1e-2        # pieces round h to bf16 only in the output
    assert rel_err(h, h_whole) < 1e-5
    assert rel_err(whole[:, -1].float(), h_whole) < 1e-2
    assert torch.isfinite(whole).all()
    # full-length backward: finite, and linear in the upstream gradient
    xg = x.clone().requires_grad_(True)
    pg = [t.clone().requires_grad_(True) for t in params]
    yg, _ = hip_rglru(xg, *pg)
    dy = torch.randn(1, T, W, generator=gen).bfloat16().cuda()
    g1 = torch.autograd.grad(yg, [xg] + pg, dy, retain_graph=True)
    g2 = torch.autograd.grad(yg, [xg] + pg, (2 * dy.float()).bfloat16())
    for a, b in zip(g1, g2):
        assert torch.isfinite(a).all()
        assert rel_err(b.float(), 2 * a.float()) < 2e-2


def test_config4_prefill_then_512_decode_steps():
    """B256 W1024: a 2048-token prefill scan, then 512 single-token steps with carried fp32 state;
    state parity against the sequential oracle after steps 1, 64 and 512."""
    from griffin_amd import PreparedParams, hip_rglru, hip_rglru_step

    B, W, nb, prefill, steps = 256, 1024, 8, 2048, 512
    gen = torch.Generator().manual_seed(11)
    bw = W // nb
    w_a, b_a = orc.gate_init(nb, bw, gen)
    w_x, b_x = orc.gate_init(nb, bw, gen)
    lam = orc.lambda_init(W, gen)
    dt = torch.bfloat16
    p_gpu = [t.to(dt).cuda() for t in (w_a, b_a, w_x, b_x, lam)]
    p_ref = [t.to(dt).float() for t in (w_a, b_a, w_x, b_x, lam)]
    # the oracle follows 4 of the 256 sequences through prefill + decode (CPU time); the rest of
    # the batch is checked for finiteness and for agreement between step and scan kernels
    xp = torch.randn(B, prefill, W, generator=gen).to(dt)
    xd = torch.randn(B, steps, W, generator=gen).to(dt)
    with torch.no_grad():
        _, state = hip_rglru(xp.cuda(), *p_gpu)
        state = state.contiguous()
        prep = PreparedParams(*p_gpu, 8.0, dt)
        xd_gpu = xd.cuda()
        marks = {}
        ys = []
        for t in range(steps):
            ys.append(hip_rglru_step(xd_gpu[:, t].contiguous(), prep, state))
            if t + 1 in (1, 64, 512):
                marks[t + 1] = state.clone()
        # the same 512 tokens through the scan kernel, from the same prefill state
        _, state_p = hip_rglru(xp.cuda(), *p_gpu)
        y_scan, state_scan = hip_rglru(xd_gpu, *p_gpu, 8.0, state_p)
    torch.cuda.synchronize()
    assert rel_err(state, state_scan) < 1e-5
    assert rel_err(torch.stack(ys, dim=1).float(), y_scan.float()) < 1e-2
    rows = [0, 1, 100, 255]
    xr = torch.cat([xp[rows], xd[rows]], dim=1).float()
    a_z = orc.gate_math(xr, *p_ref)
    h = orc.sequential_scan(a_z.a, a_z.z, torch.zeros(len(rows), W))
    for t, got in marks.items():
        err = rel_err(got[rows], h[:, prefill + t - 1])
        _say(f"config 4: state error after {t} decode steps: {err:.2e}")
        assert err < BF16_TOL


def test_module_decode_uses_step_kernel_and_tracks_parameter_updates():
    """T == 1 without gradients goes through the single-step kernel on a cached parameter image; the
    image must follow in-place parameter updates.  Reference behaviour: griffin/griffin.py:279-284."""
    case = orc.make_case(4, 6, 256, 2, seed=13, h0_std=0.5, bias_std=0.3)
    ref = _module_from_case(case, 2, "sequential", device="cpu")
    hip = _module_from_case(case, 2, "hip")
    x = case["x"]
    reset = torch.zeros(4, 6, dtype=torch.bool)
    reset[2, 3] = True
    active = torch.ones(4, 6, dtype=torch.bool)
    active[1, 4:] = False

    def decode(module, device):
        state = case["h0"].to(device)
        outs = []
        with torch.no_grad():
            for t in range(6):
                y, state = module(x[:, t:t + 1].to(device), state, reset_mask=reset[:, t:t + 1].to(device),
                                  active_mask=active[:, t:t + 1].to(device), return_state=True)
                outs.append(y)
        return torch.cat(outs, dim=1).cpu(), state.cpu()

    y_ref, h_ref = decode(ref, "cpu")
    y_hip, h_hip = decode(hip, "cuda")
    assert hip._prep_key is not None                          # the step path ran
    assert rel_err(y_hip, y_ref) < FP32_TOL and rel_err(h_hip, h_ref) < FP32_TOL
    # an optimiser-style in-place update must invalidate the cached image
    with torch.no_grad():
        for module in (ref, hip):
            module.Lambda.add_(0.25)
            module.input_gate.bias.add_(0.1)
    y_ref2, h_ref2 = decode(ref, "cpu")
    y_hip2, h_hip2 = decode(hip, "cuda")
    assert rel_err(y_ref2, y_ref) > 1e-3                      # the update matters
    assert rel_err(y_hip2, y_ref2) < FP32_TOL and rel_err(h_hip2, h_ref2) < FP32_TOL
    # with gradients enabled the same call takes the differentiable path
    xg = x[:, :1].cuda().requires_grad_(True)
    yg = hip(xg)
    yg.sum().backward()
    assert xg.grad is not None


def test_config5_recurrent_block_with_hip_scan():
    """d_model 768 -> width 1024 block: the HIP scan slotted into the block unchanged, forward and
    backward against the same block on the CPU with the sequential scan (fp32, reduced length),
    then the bf16 training shape B8 T2048 for finiteness and cache semantics."""
    from griffin_amd import RMSNorm, RecurrentBlock

    torch.manual_seed(5)
    cpu_block = RecurrentBlock(768, 1024, gate_blocks=8, scan_mode="sequential")
    cpu_norm = RMSNorm(768)                                  # the RMSNorm in front of the block
    with torch.no_grad():
        cpu_norm.g.copy_(0.1 * torch.randn(768))
    hip_block = copy.deepcopy(cpu_block).cuda()
    hip_norm = copy.deepcopy(cpu_norm).cuda()
    hip_block.scan_mode = None
    hip_block.rg_lru.scan_mode = "hip"
    x = torch.randn(2, 160, 768)
    xc = x.clone().requires_grad_(True)
    xh = x.clone().cuda().requires_grad_(True)
    up = torch.randn(2, 160, 768)
    yc = cpu_block(cpu_norm(xc))
    yh = hip_block(hip_norm(xh))
    yc.backward(up)
    yh.backward(up.cuda())
    assert rel_err(yh, yc) < 1e-4
    assert rel_err(xh.grad, xc.grad) < 1e-4
    assert rel_err(hip_norm.g.grad, cpu_norm.g.grad) < 2e-4
    for (name, ph), (_, pc) in zip(hip_block.named_parameters(), cpu_block.named_parameters()):
        assert rel_err(ph.grad, pc.grad) < 2e-4, name

    block16 = copy.deepcopy(hip_block).to(torch.bfloat16)
    xb = torch.randn(8, 2048, 768, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    out, cache = block16(xb, return_cache=True)
    out.float().square().mean().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(xb.grad).all()
    assert cache.rnn_state.dtype == torch.float32 and cache.rnn_state.shape == (8, 1024)
    assert cache.segment_position.tolist() == [2047] * 8
    with torch.no_grad():
        nxt, _ = block16(xb[:, :1].detach(), cache, return_cache=True)
    assert torch.isfinite(nxt).all()


def test_recurrent_block_right_padded_batch_trains_on_hip_kernels():
    """A right-padded batch with a packed second document (griffin/griffin.py:488-510): output, cache and
    every gradient of the block on the HIP kernels against the same block on the CPU, whose padded
    convolution is the token-by-token loop."""
    from griffin_amd import RecurrentBlock

    torch.manual_seed(9)
    cpu_block = RecurrentBlock(96, 128, gate_blocks=4, scan_mode="sequential")
    hip_block = copy.deepcopy(cpu_block).cuda()
    hip_block.scan_mode = None
    hip_block.rg_lru.scan_mode = "hip"
    B, T = 3, 90
    x = torch.randn(B, T, 96)
    active = torch.arange(T)[None, :] < torch.tensor([T, 41, 0])[:, None]
    pos = torch.arange(T).repeat(B, 1)
    pos[0, 50:] -= 50                                        # a second document in the full row
    xc = x.clone().requires_grad_(True)
    xh = x.clone().cuda().requires_grad_(True)
    up = torch.randn(B, T, 96)
    yc, cache_c = cpu_block(xc, segment_pos=pos, active_mask=active, return_cache=True)
    yh, cache_h = hip_block(xh, segment_pos=pos.cuda(), active_mask=active.cuda(), return_cache=True)
    yc.backward(up)
    yh.backward(up.cuda())
    assert rel_err(yh, yc) < 1e-4
    assert rel_err(cache_h.conv_state, cache_c.conv_state) < 1e-6
    assert rel_err(cache_h.rnn_state, cache_c.rnn_state) < 1e-4
    assert rel_err(xh.grad, xc.grad) < 1e-4
    assert torch.count_nonzero(xh.grad[~active.cuda()]) == 0
    for (name, ph), (_, pc) in zip(hip_block.named_parameters(), cpu_block.named_parameters()):
        assert rel_err(ph.grad, pc.grad) < 2e-4, name


def test_config5_recurrent_block_bf16_matches_fp32_oracle():
    """Config 5 at its stated storage type: RMSNorm(768) + RecurrentBlock(768, 1024), 8 gate blocks, bf16
    parameters and activations on the HIP kernels, T = 2048, against the oracle's block
    (griffin/griffin.py:68-80, 439-529) in fp32 on the same bf16-rounded parameters and inputs, forward
    and every gradient.  Two sequences instead of eight keep the CPU side to a few seconds; nothing in
    the block couples sequences."""
    from griffin_amd import RMSNorm, RecurrentBlock

    torch.manual_seed(9)
    B, T, D, W = 2, 2048, 768, 1024
    block = RecurrentBlock(D, W, gate_blocks=8, scan_mode="hip").to(torch.bfloat16)
    norm = RMSNorm(D)
    with torch.no_grad():
        norm.g.copy_(0.1 * torch.randn(D))
        block.rg_lru.recurrence_gate.bias.copy_(0.3 * torch.randn(8, W // 8))
        block.rg_lru.input_gate.bias.copy_(0.3 * torch.randn(8, W // 8))
    norm = norm.to(torch.bfloat16)
    x = torch.randn(B, T, D).to(torch.bfloat16)
    up = torch.randn(B, T, D).to(torch.bfloat16)

    # oracle, fp32, on the rounded values
    p = {k: v.clone().requires_grad_(True) for k, v in _block_params(block).items()}
    g = norm.g.detach().float().clone().requires_grad_(True)
    xr = x.float().requires_grad_(True)
    want, _ = orc.recurrent_block_forward(orc.rmsnorm(xr, g), p)
    names = list(p)
    want_grads = torch.autograd.grad(want, [xr, g] + [p[k] for k in names], up.float())

    hip_block, hip_norm = block.cuda(), norm.cuda()
    xh = x.cuda().requires_grad_(True)
    got = hip_block(hip_norm(xh))
    got.backward(up.cuda())
    torch.cuda.synchronize()
    mine = _block_params_grads(hip_block)
    errs = {"out": rel_err(got.float(), want), "x": rel_err(xh.grad.float(), want_grads[0]),
            "norm.g": rel_err(hip_norm.g.grad.float(), want_grads[1])}
    for name, ref in zip(names, want_grads[2:]):
        errs[name] = rel_err(mine[name], ref)
    _say("config 5 bf16 rel errors:", {k: "%.2e" % v for k, v in errs.items()})
    for name, err in errs.items():
        assert err < BF16_TOL, (name, err)


@pytest.mark.parametrize("cfg", [(2, 300, 96, 128, 4, 4), (3, 200, 64, 192, 3, 3), (2, 129, 48, 64, 2, 2),
                                 (2, 260, 96, 256, 2, 4)])
def test_one_launch_block_forward_against_the_oracle_directly(cfg):
    """The block's one-launch forward (convolution prologue, RG-LRU, output gate; bf16) against the oracle's
    block in fp32 on the same rounded parameters, forward and every gradient, at gate blocks of 32 (four to a
    unit), 64 (two to a unit) and 128 channels and with fewer than four taps: cfg = (B, T, D, W, blocks, taps)."""
    from griffin_amd import RecurrentBlock, hip_block_ops

    B, T, D, W, nb, K = cfg
    torch.manual_seed(21 + W)
    block = RecurrentBlock(D, W, conv_kernel_size=K, gate_blocks=nb, scan_mode="hip").to(torch.bfloat16)
    assert hip_block_ops.hip_block_forward_covers(W, nb, K, torch.bfloat16)
    with torch.no_grad():
        block.rg_lru.recurrence_gate.bias.copy_(0.3 * torch.randn(nb, W // nb))
        block.rg_lru.input_gate.bias.copy_(0.3 * torch.randn(nb, W // nb))
        block.temporal_conv.bias.copy_(0.1 * torch.randn(W))
    x = torch.randn(B, T, D).to(torch.bfloat16)
    up = torch.randn(B, T, D).to(torch.bfloat16)
    p = {k: v.clone().requires_grad_(True) for k, v in _block_params(block).items()}
    xr = x.float().requires_grad_(True)
    want, _ = orc.recurrent_block_forward(xr, p)
    names = list(p)
    want_grads = torch.autograd.grad(want, [xr] + [p[k] for k in names], up.float())

    hip_block = block.cuda()
    calls = []
    real = hip_block_ops.hip_block_forward

    def spy(*args, **kwargs):
        calls.append(1)
        return real(*args, **kwargs)

    hip_block_ops.hip_block_forward = spy
    try:
        xh = x.cuda().requires_grad_(True)
        got = hip_block(xh)
        got.backward(up.cuda())
        torch.cuda.synchronize()
    finally:
        hip_block_ops.hip_block_forward = real
    assert calls, "the one-launch forward did not run"
    mine = _block_params_grads(hip_block)
    errs = {"out": rel_err(got.float(), want), "x": rel_err(xh.grad.float(), want_grads[0])}
    for name, ref in zip(names, want_grads[1:]):
        errs[name] = rel_err(mine[name], ref)
    _say("one-launch block forward", cfg, {k: "%.2e" % v for k, v in errs.items()})
    for name, err in errs.items():
        assert err < BF16_TOL, (name, err)


# ------------------------------------------------------------------ failure handling
def test_bounded_wait_gives_up_instead_of_hanging():
    """With the poll budget forced to one, waves that do not find their carry at once record the
    failure and still run to the end of the kernel; a give-up is visible in the results themselves (the
    carry it could not get is NaN, and with it the chunk's outputs and its carry out) and never a
    silently wrong number; the next call with the normal budget is exact."""
    import ctypes

    from griffin_amd import _lib, hip_rglru_scan

    lib = _lib.load()
    B, T, W = 2, 4096, 256
    a = torch.full((B, T, W), 0.9, device="cuda")
    z = torch.ones(B, T, W, device="cuda")
    h0 = torch.zeros(B, W, device="cuda")
    out = torch.empty_like(a)
    ws = torch.empty(lib.rglru_hip_scan_workspace_bytes(B, T, W), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    previous = lib.rglru_hip_set_spin_limit(1)
    try:
        rc = lib.rglru_hip_scan_fwd(a.data_ptr(), z.data_ptr(), h0.data_ptr(), out.data_ptr(), ws.data_ptr(),
                                    B, T, W, stream)
        torch.cuda.synchronize()                               # returns: no wave is left spinning
    finally:
        lib.rglru_hip_set_spin_limit(previous)
    assert rc == 0
    status = ctypes.c_int(-1)
    assert lib.rglru_hip_workspace_status(ws.data_ptr(), B, T, W, 1, 1, stream, ctypes.byref(status)) == 0
    _say("failure word after a one-poll budget:", status.value)
    assert status.value in (0, 1)
    want = 10.0 * (1.0 - 0.9 ** torch.arange(1, T + 1, dtype=torch.float64))
    bad = torch.isnan(out)
    if status.value == 1:
        assert bad.any(), "a wave gave up but no result was poisoned"
    else:
        assert not bad.any()
    # whatever is not NaN is right: no silently wrong values
    finite = ~bad[0, :, 0]
    assert rel_err(out[0, :, 0][finite], want[finite.cpu()]) < 1e-5
    good = hip_rglru_scan(a, z, h0)
    assert rel_err(good[0, :, 0], want) < 1e-5


# ----------------------------------------------------------------------------------------------
# single-token decode of the recurrent block (rglru_hip_decode_prepare + rglru_hip_step_gated)
# ----------------------------------------------------------------------------------------------
def _block_params(block):
    """Parameters of a RecurrentBlock in the oracle's naming, fp32 on the CPU."""
    sd = {k: v.detach().float().cpu() for k, v in block.state_dict().items()}
    return {"lx_w": sd["linear_x.weight"], "lx_b": sd["linear_x.bias"], "ly_w": sd["linear_y.weight"],
            "ly_b": sd["linear_y.bias"], "conv_w": sd["temporal_conv.weight"][:, 0, :], "conv_b": sd["temporal_conv.bias"],
            "w_a": sd["rg_lru.recurrence_gate.weight"], "b_a": sd["rg_lru.recurrence_gate.bias"],
            "w_x": sd["rg_lru.input_gate.weight"], "b_x": sd["rg_lru.input_gate.bias"], "lam": sd["rg_lru.Lambda"],
            "lo_w": sd["linear_out.weight"], "lo_b": sd["linear_out.bias"]}


def _block_params_grads(block):
    """Gradients of a RecurrentBlock's parameters in the oracle's naming, fp32 on the CPU."""
    gd = {k: v.grad.detach().float().cpu() for k, v in block.named_parameters()}
    return {"lx_w": gd["linear_x.weight"], "lx_b": gd["linear_x.bias"], "ly_w": gd["linear_y.weight"],
            "ly_b": gd["linear_y.bias"], "conv_w": gd["temporal_conv.weight"][:, 0, :], "conv_b": gd["temporal_conv.bias"],
            "w_a": gd["rg_lru.recurrence_gate.weight"], "b_a": gd["rg_lru.recurrence_gate.bias"],
            "w_x": gd["rg_lru.input_gate.weight"], "b_x": gd["rg_lru.input_gate.bias"], "lam": gd["rg_lru.Lambda"],
            "lo_w": gd["linear_out.weight"], "lo_b": gd["linear_out.bias"]}


@pytest.mark.parametrize("dtype,tol", [(torch.float32, FP32_TOL), (torch.bfloat16, BF16_TOL)])
def test_block_decode_matches_oracle(dtype, tol):
    """Prefill of 9 tokens, then 7 single-token steps with the carried cache, against the oracle's
    block run the same way (analogue of the reference's tests/test_recurrentblock.py chunk test)."""
    from griffin_amd import RecurrentBlock

    torch.manual_seed(3)
    block = RecurrentBlock(24, 64, gate_blocks=2, scan_mode="hip")
    with torch.no_grad():
        for prm in block.parameters():
            prm.copy_(prm.to(dtype).float())            # parameters exactly representable in the storage type
        block.temporal_conv.bias.copy_((0.1 * torch.randn(64)).to(dtype).float())
    params = _block_params(block)
    block = block.cuda().to(dtype).eval()
    x = torch.randn(3, 16, 24).to(dtype).float()
    want, cache_o = [], None
    with torch.no_grad():
        piece, cache_o = orc.recurrent_block_forward(x[:, :9], params, cache=cache_o)
        want.append(piece)
        for t in range(9, 16):
            piece, cache_o = orc.recurrent_block_forward(x[:, t:t + 1], params, cache=cache_o)
            want.append(piece)
        xg = x.to(dtype).cuda()
        got, cache = [], None
        piece, cache = block(xg[:, :9], return_cache=True)
        got.append(piece)
        for t in range(9, 16):
            piece, cache = block(xg[:, t:t + 1], cache=cache, return_cache=True)
            got.append(piece)
    torch.cuda.synchronize()
    want, got = torch.cat(want, dim=1), torch.cat(got, dim=1)
    errs = {"out": rel_err(got.float(), want), "rnn_state": rel_err(cache.rnn_state, cache_o[0]),
            "conv_state": rel_err(cache.conv_state.float(), cache_o[1])}
    _say("block decode", dtype, {k: "%.2e" % v for k, v in errs.items()})
    for name, err in errs.items():
        assert err < tol, (name, err)
    assert torch.equal(cache.segment_position.cpu(), cache_o[2])
    assert cache.rnn_state.dtype == torch.float32


def test_block_decode_with_padding_and_restart_matches_portable_block():
    """Rows that pause (inactive tokens) and a row that starts a new document mid-stream: the decode
    kernels against the same block on the CPU with the sequential scan (whose padded path follows
    griffin/griffin.py:488-510)."""
    from griffin_amd import RecurrentBlock

    torch.manual_seed(4)
    cpu_block = RecurrentBlock(16, 32, gate_blocks=2, scan_mode="sequential").eval()
    hip_block = copy.deepcopy(cpu_block).cuda()
    hip_block.rg_lru.scan_mode = "hip"
    B, steps = 4, 10
    x = torch.randn(B, steps, 16)
    active = torch.ones(B, steps, dtype=torch.bool)
    active[1, 3:5] = False
    active[2, 7] = False
    active[3, :] = True
    positions = torch.arange(steps).repeat(B, 1)
    positions[0, 6:] -= 6                                    # row 0 starts a new document at step 6
    with torch.no_grad():
        cache_c = cache_h = None
        for t in range(steps):
            # explicit positions on some steps, positions derived from the cache on the others
            explicit = positions[:, t:t + 1] if (t >= 6 or t < 3) else None
            mask = active[:, t:t + 1]
            oc, cache_c = cpu_block(x[:, t:t + 1], cache=cache_c, segment_pos=explicit, active_mask=mask, return_cache=True)
            oh, cache_h = hip_block(x[:, t:t + 1].cuda(), cache=cache_h,
                                    segment_pos=None if explicit is None else explicit.cuda(),
                                    active_mask=mask.cuda(), return_cache=True)
            torch.testing.assert_close(oh.cpu(), oc, atol=2e-5, rtol=2e-5)
            torch.testing.assert_close(cache_h.rnn_state.cpu(), cache_c.rnn_state, atol=2e-5, rtol=2e-5)
            torch.testing.assert_close(cache_h.conv_state.cpu(), cache_c.conv_state, atol=1e-6, rtol=1e-6)
            assert torch.equal(cache_h.segment_position.cpu(), cache_c.segment_position), t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", [(5, 64, 2, 0), (256, 1024, 8, 0), (3, 40, 1, 3), (7, 320, 1, 8)])
def test_block_decode_step_takes_strided_rows(cfg, dtype):
    """The decode kernels read their two projections as rows of a wider buffer (row strides through the
    C ABI): results are bit-identical to the same call on contiguous copies, on the vector path
    (16-byte-aligned strides) and on the element path (the padded buffers)."""
    from griffin_amd import RG_LRU
    from griffin_amd.hip_block_ops import hip_block_decode_step

    B, W, nb, pad = cfg
    torch.manual_seed(B + W)
    rg = RG_LRU(W, gate_blocks=nb, scan_mode="hip").cuda().to(dtype)
    prep = rg._prepared(dtype, torch.device("cuda", 0))
    both = torch.randn(B, 2 * W + pad, device="cuda").to(dtype)
    u, v = both[:, :W], both[:, W + pad:]
    assert not u.is_contiguous() and not v.is_contiguous()
    taps = (0.3 * torch.randn(W, 1, 4, device="cuda")).to(dtype)
    bias = (0.1 * torch.randn(W, device="cuda")).to(dtype)
    conv_state = torch.randn(B, 3, W, device="cuda").to(dtype)
    prev_pos = torch.randint(-1, 5, (B,), device="cuda")
    active = (torch.rand(B, device="cuda") < 0.8).to(torch.uint8)
    h = torch.randn(B, W, device="cuda")
    _say("strided decode rows", cfg, dtype)
    got = hip_block_decode_step(u, v, conv_state, taps, bias, prev_pos, None, active, prep, h)
    want = hip_block_decode_step(u.contiguous(), v.contiguous(), conv_state, taps, bias, prev_pos, None, active,
                                 prep, h)
    torch.cuda.synchronize()
    for name, a, b in zip(("gated", "rnn_state", "conv_state", "position"), got, want):
        assert torch.equal(a, b), name
    assert got[0].is_contiguous() and got[0].shape == (B, W)


def test_decode_row_stride_below_width_is_rejected():
    """Row strides smaller than the width are argument errors (checked on the host, nothing is launched)."""
    from griffin_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(4096, device="cuda")
    p = buf.data_ptr()
    rc = lib.rglru_hip_decode_prepare(p, 16, None, p, None, None, None, None, p, p, p, p, 2, 32, 4, 0, 0, None)
    assert rc != 0 and b"stride" in lib.rglru_hip_last_error()


def test_block_under_autocast_with_fp32_master_parameters():
    """Mixed-precision training as a trainer sets it up: fp32 parameters, `torch.autocast(bfloat16)` around the
    forward.  The block on the HIP kernels returns bf16, every parameter gets an fp32 gradient, and all of it agrees
    with the fp32 block on the CPU to bf16 accuracy; a forward on a side stream and one on a non-contiguous input
    agree with it too."""
    from griffin_amd import RecurrentBlock

    torch.manual_seed(0)
    B, T, D, W = 2, 300, 96, 256
    ref = RecurrentBlock(D, W, gate_blocks=4, scan_mode="sequential")
    hip = copy.deepcopy(ref).cuda()
    hip.scan_mode = None
    hip.rg_lru.scan_mode = "hip"
    x = torch.randn(B, T, D)
    up = torch.randn(B, T, D)
    xc = x.clone().requires_grad_(True)
    xh = x.clone().cuda().requires_grad_(True)
    yc = ref(xc)
    yc.backward(up)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        yh = hip(xh)
    assert yh.dtype == torch.bfloat16
    yh.float().backward(up.cuda())
    torch.cuda.synchronize()
    assert rel_err(yh.float(), yc) < BF16_TOL and rel_err(xh.grad, xc.grad) < BF16_TOL
    for (name, ph), (_, pc) in zip(hip.named_parameters(), ref.named_parameters()):
        assert ph.grad.dtype == torch.float32, name
        assert rel_err(ph.grad, pc.grad) < BF16_TOL, name
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            y_side = hip(xh.detach())
        side.synchronize()
        assert rel_err(y_side, yc) < 1e-5
        strided = x.transpose(0, 1).contiguous().transpose(0, 1).cuda()
        assert not strided.is_contiguous()
        assert rel_err(hip(strided), yc) < 1e-5


# ----------------------------------------------------------------------------------------------
# random sweeps of the block: the HIP kernels against the same block on the CPU, driven the same way
# ----------------------------------------------------------------------------------------------
def _random_block_pair(rng, dtype, widths, dims):
    """A RecurrentBlock with random geometry on the CPU (fp32 values rounded to `dtype`) and its copy on the HIP path."""
    from griffin_amd import RecurrentBlock

    bw = rng.choice(widths)
    nb = rng.choice([1, 2, 4, 8])
    if bw * nb > 1280:
        nb = max(1, 1280 // bw)
    W, D, K = bw * nb, rng.choice(dims), rng.choice([4, 4, 4, 2, 3])
    ref = RecurrentBlock(D, W, gate_blocks=nb, conv_kernel_size=K, scan_mode="sequential")
    with torch.no_grad():
        ref.rg_lru.recurrence_gate.bias.copy_(0.3 * torch.randn_like(ref.rg_lru.recurrence_gate.bias))
        ref.rg_lru.input_gate.bias.copy_(0.3 * torch.randn_like(ref.rg_lru.input_gate.bias))
    ref = ref.to(dtype).float()
    hip = copy.deepcopy(ref).to(dtype).cuda()
    hip.scan_mode = None
    hip.rg_lru.scan_mode = "hip"
    return ref, hip, (D, W, nb, K)


def test_random_blocks_train_like_the_cpu_block():
    """Forty random blocks (fixed seed): storage type, gate block width and count, model width, convolution size,
    batch, length; plain, packed documents, right padding, both, or two calls chained through the cache.  Output,
    cache and every gradient against the block on the CPU with the sequential scan."""
    import random

    rng = random.Random(11)
    failures = []
    for index in range(40):
        torch.manual_seed(1100 + index)
        dtype = rng.choice([torch.float32, torch.bfloat16, torch.bfloat16])
        ref, hip, (D, W, nb, K) = _random_block_pair(rng, dtype, [8, 16, 24, 32, 64, 96, 128, 160, 320], [32, 48, 96, 256, 768])
        B = rng.choice([1, 2, 3, 8])
        T = rng.choice([1, 2, 3, 4, 5, 17, 32, 33, 64, 100, 255, 256, 600, 1024])
        if B * T * W > 1500000:
            T = max(1, 1500000 // (B * W))
        kind = rng.choice(["plain", "packed", "padded", "both", "chunked"])
        _say("random block", index, str(dtype), (B, T, D, W, nb, K), kind)
        x = torch.randn(B, T, D).to(dtype).float()
        up = torch.randn(B, T, D).to(dtype).float()
        kw = {}
        if kind in ("packed", "both"):
            pos = torch.arange(T).repeat(B, 1)
            for b in range(B):
                if T > 2 and rng.random() < 0.7:
                    cut = rng.randrange(1, T)
                    pos[b, cut:] -= cut
            kw["segment_pos"] = pos
        if kind in ("padded", "both"):
            lens = torch.tensor([rng.choice([T, T, max(0, T - 1), T // 2, 0]) for _ in range(B)])
            kw["active_mask"] = torch.arange(T)[None, :] < lens[:, None]
        xc = x.clone().requires_grad_(True)
        xh = x.to(dtype).cuda().requires_grad_(True)
        if kind == "chunked" and T >= 2:
            cut = rng.randrange(1, T)
            y1, cache_c = ref(xc[:, :cut], return_cache=True)
            y2, cache_c = ref(xc[:, cut:], cache_c, return_cache=True)
            yc = torch.cat([y1, y2], 1)
            z1, cache_h = hip(xh[:, :cut], return_cache=True)
            z2, cache_h = hip(xh[:, cut:], cache_h, return_cache=True)
            yh = torch.cat([z1, z2], 1)
        else:
            yc, cache_c = ref(xc, return_cache=True, **kw)
            yh, cache_h = hip(xh, return_cache=True, **{k: v.cuda() for k, v in kw.items()})
        yc.backward(up)
        yh.backward(up.to(dtype).cuda())
        torch.cuda.synchronize()
        errs = {"y": rel_err(yh.float(), yc), "dx": rel_err(xh.grad.float(), xc.grad),
                "rnn_state": rel_err(cache_h.rnn_state.float(), cache_c.rnn_state),
                "conv_state": rel_err(cache_h.conv_state.float(), cache_c.conv_state),
                "position": 0.0 if torch.equal(cache_h.segment_position.cpu(), cache_c.segment_position) else 1.0}
        for (name, ph), (_, pc) in zip(hip.named_parameters(), ref.named_parameters()):
            errs[name] = rel_err(ph.grad.float(), pc.grad)
        tol = 2e-4 if dtype == torch.float32 else BF16_TOL
        if not max(errs.values()) < tol:
            failures.append((index, kind, {k: "%.2e" % v for k, v in errs.items() if not v < tol}))
    assert not failures, failures


def test_random_prefill_and_decode_like_the_cpu_block():
    """Forty random prefill + single-token decode runs (fixed seed) with document restarts and rows that stop,
    against the CPU block called with the same slices.  The same call pattern matters: the reference's all-active
    convolution keeps a finished document's rows in the cache (griffin/griffin.py:487) and its padded one uses the
    whole window (:496-500), so step-by-step calls and one pass over the sequence differ there by design."""
    import random

    rng = random.Random(12)
    failures = []
    for index in range(40):
        torch.manual_seed(1200 + index)
        dtype = rng.choice([torch.float32, torch.bfloat16, torch.bfloat16])
        ref, hip, (D, W, nb, K) = _random_block_pair(rng, dtype, [8, 16, 24, 32, 40, 64, 96, 128, 160, 320, 384], [32, 48, 96, 256])
        ref, hip = ref.eval(), hip.eval()
        B = rng.choice([1, 2, 3, 16, 17, 64, 100, 256])
        T0, S = rng.choice([0, 1, 2, 3, 5, 40]), rng.choice([1, 2, 5, 12])
        T = T0 + S
        kind = rng.choice(["plain", "restart", "padded", "both"])
        _say("random decode", index, str(dtype), (B, T0, S, D, W, nb, K), kind)
        x = torch.randn(B, T, D).to(dtype).float()
        kw = {}
        active = torch.ones(B, T, dtype=torch.bool)
        if kind in ("restart", "both"):
            pos = torch.arange(T).repeat(B, 1)
            for b in range(B):
                if T > 1 and rng.random() < 0.5:
                    cut = rng.randrange(max(T0, 1) if T0 < T else T - 1, T)
                    pos[b, cut:] -= cut
            kw["segment_pos"] = pos
        if kind in ("padded", "both"):
            for b in range(B):
                if rng.random() < 0.4:
                    active[b, rng.randrange(T0, T + 1):] = False
            kw["active_mask"] = active
        cuts = ([(0, T0)] if T0 else []) + [(t, t + 1) for t in range(T0, T)]
        with torch.no_grad():
            cache_c = cache_h = None
            outs_c, outs_h = [], []
            xh = x.to(dtype).cuda()
            for lo, hi in cuts:
                yc, cache_c = ref(x[:, lo:hi], cache_c, return_cache=True, **{k: v[:, lo:hi] for k, v in kw.items()})
                yh, cache_h = hip(xh[:, lo:hi], cache_h, return_cache=True, **{k: v[:, lo:hi].cuda() for k, v in kw.items()})
                outs_c.append(yc)
                outs_h.append(yh)
        torch.cuda.synchronize()
        live = active[..., None]
        errs = {"y": rel_err(torch.cat(outs_h, 1).float().cpu() * live, torch.cat(outs_c, 1) * live),
                "rnn_state": rel_err(cache_h.rnn_state.float(), cache_c.rnn_state),
                "conv_state": rel_err(cache_h.conv_state.float(), cache_c.conv_state),
                "position": 0.0 if torch.equal(cache_h.segment_position.cpu(), cache_c.segment_position) else 1.0}
        tol = 2e-4 if dtype == torch.float32 else BF16_TOL
        if not max(errs.values()) < tol:
            failures.append((index, kind, {k: "%.2e" % v for k, v in errs.items() if not v < tol}))
    assert not failures, failures
