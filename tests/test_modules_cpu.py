"""Host-side mirror of the reference's module interface, exercised on the CPU.

Each test is the analogue of one of the reference's own behavioural tests (tests/test_rglru.py,
tests/test_recurrentblock.py), plus checks against the golden vectors recorded from the reference."""

import copy
import os

import numpy as np
import pytest
import torch

from griffin_amd import BlockDiagonalLinear, RG_LRU, RecurrentBlock, hip_scan_is_usable
from griffin_amd import hip_rglru, hip_rglru_scan
from oracle import rglru_oracle as orc


def _load(golden_dir, name):
    data = np.load(os.path.join(golden_dir, name + ".npz"))
    return {k: torch.from_numpy(data[k]) for k in data.files}


def test_earlier_token_changes_later_hidden_state():          # reference tests/test_rglru.py:19-32
    torch.manual_seed(0)
    module = RG_LRU(rnn_width=6).eval()
    x = torch.randn(2, 5, 6)
    changed = x.clone()
    changed[:, 0, :] += 3.0
    with torch.no_grad():
        diff = (module(x)[:, 1:] - module(changed)[:, 1:]).abs().max()
    assert diff > 1e-6


def test_returns_final_state():                               # tests/test_rglru.py:35-46
    torch.manual_seed(0)
    module = RG_LRU(rnn_width=6).eval()
    x = torch.randn(2, 5, 6)
    with torch.no_grad():
        output, final_state = module(x, return_state=True)
    assert output.shape == x.shape and final_state.shape == (2, 6)
    torch.testing.assert_close(output[:, -1, :], final_state)


def test_block_diagonal_lecun_gates():                        # tests/test_rglru.py:49-58
    torch.manual_seed(0)
    module = RG_LRU(rnn_width=64, gate_blocks=16)
    assert isinstance(module.recurrence_gate, BlockDiagonalLinear)
    assert module.recurrence_gate.weight.shape == (16, 4, 4)
    assert abs(module.recurrence_gate.weight.std().item() - 0.5) < 0.08
    assert RG_LRU(rnn_width=257, gate_blocks=16).recurrence_gate.weight.shape == (1, 257, 257)
    assert set(dict(module.named_parameters())) == {
        "Lambda", "recurrence_gate.weight", "recurrence_gate.bias", "input_gate.weight", "input_gate.bias"}
    a8 = torch.sigmoid(module.Lambda.detach().double()).pow(8)
    assert a8.min() >= 0.9 - 1e-6 and a8.max() <= 0.999 + 1e-6


def test_bounded_sqrt_gradients_in_bfloat16():                # tests/test_rglru.py:61-75
    module = RG_LRU(rnn_width=16, gate_blocks=4).to(torch.bfloat16)
    with torch.no_grad():
        module.recurrence_gate.weight.zero_()
        module.recurrence_gate.bias.fill_(-100)
        module.Lambda.fill_(20)
    x = torch.randn(2, 8, 16, dtype=torch.bfloat16, requires_grad=True)
    output = module(x)
    output.float().square().mean().backward()
    assert torch.isfinite(output).all() and torch.isfinite(x.grad).all()
    assert torch.isfinite(module.Lambda.grad).all()


def test_associative_matches_sequential():                    # tests/test_rglru.py:78-109
    torch.manual_seed(0)
    sequential = RG_LRU(rnn_width=8, gate_blocks=4, scan_mode="sequential")
    associative = copy.deepcopy(sequential)
    associative.scan_mode = "associative"
    xs = torch.randn(2, 11, 8, requires_grad=True)
    xa = xs.detach().clone().requires_grad_(True)
    reset = torch.zeros(2, 11, dtype=torch.bool)
    reset[:, 6] = True
    ys = sequential(xs, reset_mask=reset)
    ya = associative(xa, reset_mask=reset)
    ys.square().mean().backward()
    ya.square().mean().backward()
    torch.testing.assert_close(ys, ya, atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(xs.grad, xa.grad, atol=2e-6, rtol=2e-6)
    for ps, pa in zip(sequential.parameters(), associative.parameters()):
        torch.testing.assert_close(ps.grad, pa.grad, atol=2e-6, rtol=2e-6)


@pytest.mark.parametrize("mode", ["hip", "fused"])
def test_explicit_hip_rejects_cpu_tensors(mode):              # tests/test_rglru.py:112-119
    module = RG_LRU(rnn_width=8, gate_blocks=4, scan_mode=mode)
    with pytest.raises(RuntimeError, match="CUDA"):
        module(torch.randn(2, 7, 8))


def test_operators_reject_cpu_tensors():
    with pytest.raises(RuntimeError, match="CUDA"):
        hip_rglru_scan(torch.rand(1, 3, 4), torch.rand(1, 3, 4), torch.rand(1, 4))
    with pytest.raises(RuntimeError, match="CUDA"):
        hip_rglru(torch.rand(1, 3, 4), torch.rand(1, 4, 4), torch.rand(1, 4), torch.rand(1, 4, 4), torch.rand(1, 4),
                  torch.rand(4))


def test_auto_validation_rejects_non_gpu_device():            # tests/test_rglru.py:122-124
    assert not hip_scan_is_usable(torch.device("cpu"))
    assert not hip_scan_is_usable("cpu")


def test_argument_validation_matches_reference_error_types():  # griffin/griffin.py:171-172, 200-235
    with pytest.raises(ValueError):
        RG_LRU(rnn_width=8, scan_mode="warp")
    module = RG_LRU(rnn_width=8, gate_blocks=4, scan_mode="sequential")
    with pytest.raises(ValueError):
        module(torch.randn(2, 8))
    with pytest.raises(ValueError):
        module(torch.randn(2, 3, 7))
    with pytest.raises(ValueError):
        module(torch.randn(2, 3, 8), reset_mask=torch.zeros(2, 4, dtype=torch.bool))
    with pytest.raises(ValueError):
        module(torch.randn(2, 3, 8), active_mask=torch.ones(3, 3, dtype=torch.bool))
    with pytest.raises(ValueError):
        module(torch.randn(2, 3, 8), torch.zeros(2, 7))
    module.scan_mode = "nonsense"                              # the mode is read on every call
    with pytest.raises(ValueError):
        module(torch.randn(2, 3, 8))


def test_masks_accept_non_bool_tensors():                     # griffin/griffin.py:214, 223
    torch.manual_seed(1)
    module = RG_LRU(rnn_width=8, gate_blocks=2, scan_mode="sequential").eval()
    x = torch.randn(2, 6, 8)
    reset = torch.zeros(2, 6, dtype=torch.bool)
    reset[:, 3] = True
    active = torch.ones(2, 6, dtype=torch.bool)
    active[1, 4:] = False
    with torch.no_grad():
        want = module(x, reset_mask=reset, active_mask=active)
        got = module(x, reset_mask=reset.long(), active_mask=active.float())
    torch.testing.assert_close(got, want)


@pytest.mark.parametrize("name", ["rglru_plain_b2_t16_w32", "rglru_masks_b2_t16_w32", "rglru_odd_b3_t37_w65"])
@pytest.mark.parametrize("mode", ["sequential", "associative"])
def test_module_matches_reference_golden_vectors(golden_dir, name, mode):
    d = _load(golden_dir, name)
    nb, bw, _ = d["w_a"].shape
    module = RG_LRU(rnn_width=nb * bw, gate_blocks=nb, scan_mode=mode)
    module.load_state_dict({"recurrence_gate.weight": d["w_a"], "recurrence_gate.bias": d["b_a"],
                            "input_gate.weight": d["w_x"], "input_gate.bias": d["b_x"], "Lambda": d["lam"]})
    x = d["x"].clone().requires_grad_(True)
    h0 = d["h0"].clone().requires_grad_(True) if "h0" in d else None
    y, h_last = module(x, h0, reset_mask=d["reset"], active_mask=d["active"], return_state=True)
    loss = (y * d["dy"]).sum()
    if "dh" in d:
        loss = loss + (h_last * d["dh"]).sum()
    loss.backward()
    torch.testing.assert_close(y, d["y"], atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(h_last, d["h_last"], atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(x.grad, d["g_x"], atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(module.Lambda.grad, d["g_lam"], atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(module.recurrence_gate.weight.grad, d["g_w_a"], atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(module.input_gate.bias.grad, d["g_b_x"], atol=2e-5, rtol=2e-5)


# ------------------------------------------------------------------ recurrent block (caller)
def test_recurrent_block_preserves_shape():                   # tests/test_recurrentblock.py:8-15
    block = RecurrentBlock(input_dim=10, rnn_width=13)
    assert block(torch.randn(2, 7, 10)).shape == (2, 7, 10)


def test_future_token_does_not_change_past_outputs():         # tests/test_recurrentblock.py:18-30
    torch.manual_seed(0)
    block = RecurrentBlock(input_dim=6, rnn_width=6).eval()
    x = torch.randn(2, 8, 6)
    changed = x.clone()
    changed[:, 4, :] += 10.0
    with torch.no_grad():
        torch.testing.assert_close(block(x)[:, :4], block(changed)[:, :4])


def test_cached_chunks_match_full_sequence():                 # tests/test_recurrentblock.py:33-50
    torch.manual_seed(0)
    block = RecurrentBlock(input_dim=8, rnn_width=12).eval()
    x = torch.randn(2, 9, 8)
    with torch.no_grad():
        full = block(x)
        first, cache = block(x[:, :3], return_cache=True)
        second, cache = block(x[:, 3:7], cache, return_cache=True)
        third, _ = block(x[:, 7:], cache, return_cache=True)
    torch.testing.assert_close(full, torch.cat([first, second, third], dim=1), atol=1e-6, rtol=1e-6)


def test_recurrent_block_matches_reference_golden(golden_dir):
    d = _load(golden_dir, "block_b2_t9_d8_w12")
    block = RecurrentBlock(8, 12, gate_blocks=16, scan_mode="sequential").eval()
    block.load_state_dict({
        "linear_x.weight": d["lx_w"], "linear_x.bias": d["lx_b"], "linear_y.weight": d["ly_w"],
        "linear_y.bias": d["ly_b"], "linear_out.weight": d["lo_w"], "linear_out.bias": d["lo_b"],
        "temporal_conv.weight": d["conv_w"][:, None, :], "temporal_conv.bias": d["conv_b"],
        "rg_lru.recurrence_gate.weight": d["w_a"], "rg_lru.recurrence_gate.bias": d["b_a"],
        "rg_lru.input_gate.weight": d["w_x"], "rg_lru.input_gate.bias": d["b_x"], "rg_lru.Lambda": d["lam"]})
    with torch.no_grad():
        full, cache = block(d["x"], return_cache=True)
        pieces, state, start = [], None, 0
        for stop in d["splits"].tolist() + [d["x"].shape[1]]:
            piece, state = block(d["x"][:, start:stop], state, return_cache=True)
            pieces.append(piece)
            start = stop
    torch.testing.assert_close(full, d["full"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(torch.cat(pieces, dim=1), d["chunked"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(cache.rnn_state, d["rnn_state"], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(cache.conv_state, d["conv_state"], atol=1e-6, rtol=1e-6)
    assert torch.equal(cache.segment_position, d["segment_position"])


def test_right_padded_batch_matches_unpadded_rows():
    """Padding must neither advance the state nor enter the convolution history."""
    torch.manual_seed(2)
    block = RecurrentBlock(input_dim=8, rnn_width=12, scan_mode="sequential").eval()
    x = torch.randn(2, 9, 8)
    active = torch.ones(2, 9, dtype=torch.bool)
    active[1, 6:] = False
    with torch.no_grad():
        padded, cache = block(x, active_mask=active, return_cache=True)
        short, short_cache = block(x[1:, :6], return_cache=True)
    torch.testing.assert_close(padded[1:, :6], short, atol=1e-6, rtol=1e-6)
    assert (padded[1, 6:] == 0).all()
    torch.testing.assert_close(cache.rnn_state[1:], short_cache.rnn_state, atol=1e-6, rtol=1e-6)
    assert cache.segment_position.tolist() == [8, 5]


def test_portable_module_agrees_with_oracle():
    case = orc.make_case(2, 20, 24, 3, seed=4, h0_std=0.5)
    module = RG_LRU(24, gate_blocks=3, scan_mode="sequential")
    module.load_state_dict({"recurrence_gate.weight": case["w_a"], "recurrence_gate.bias": case["b_a"],
                            "input_gate.weight": case["w_x"], "input_gate.bias": case["b_x"], "Lambda": case["lam"]})
    with torch.no_grad():
        y, h = module(case["x"], case["h0"], return_state=True)
    ry, rh = orc.rglru_forward(*[case[k] for k in ("x", "w_a", "b_a", "w_x", "b_x", "lam")], h0=case["h0"])
    torch.testing.assert_close(y, ry, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(h, rh, atol=1e-6, rtol=1e-6)


def test_default_positions_are_built_once_and_match_the_general_rule():
    """A call without cache, explicit positions or padding resolves to positions 0 .. T-1; the tensors are
    shared between calls (griffin/griffin.py:309-338 for previous position -1 and every token active)."""
    from griffin_amd import modules

    x = torch.zeros(3, 7, 4)
    first = modules._resolve_segment_positions(x, None)
    again = modules._resolve_segment_positions(x, None)
    assert first is again
    general = modules._resolve_segment_positions(x, None, torch.full((3,), -1), None)
    assert torch.equal(first, general)
    assert torch.equal(modules._default_positions(3, 7, x.device)[1], general == 0)


def test_packed_flags_follow_in_place_updates_of_the_mask():
    """pack_flags remembers the bytes of a reset mask only while the mask is not written to."""
    from griffin_amd.hip_scan import pack_flags

    mask = torch.zeros(2, 5, dtype=torch.bool)
    mask[0, 0] = True
    a = pack_flags(mask, None)
    assert pack_flags(mask, None) is a and a.tolist() == [[1, 0, 0, 0, 0], [0, 0, 0, 0, 0]]
    mask[1, 3] = True                                        # bumps the tensor's version counter
    b = pack_flags(mask, None)
    assert b is not a and b.tolist() == [[1, 0, 0, 0, 0], [0, 0, 0, 1, 0]]
    both = pack_flags(mask, torch.ones(2, 5, dtype=torch.bool))
    assert both.tolist() == b.tolist()


def test_stacked_decode_projection_follows_the_two_linear_layers():
    """The one-GEMM form of linear_x / linear_y used by single-token decode (griffin/griffin.py:462-464)
    returns what the two layers return, and is rebuilt when a weight or bias is written to."""
    from griffin_amd import RecurrentBlock

    torch.manual_seed(0)
    block = RecurrentBlock(12, 16, gate_blocks=2, scan_mode="sequential")
    token = torch.randn(5, 12)
    with torch.no_grad():
        px, py = block._decode_projections(token)
        assert px.shape == py.shape == (5, 16) and px.stride(0) == 32
        assert torch.allclose(px, block.linear_x(token), atol=1e-6)
        assert torch.allclose(py, block.linear_y(token), atol=1e-6)
        held = block._stacked_projection
        block._decode_projections(token)
        assert block._stacked_projection is held
        block.linear_y.bias.add_(1.0)
        block.linear_x.weight.mul_(2.0)
        px, py = block._decode_projections(token)
        assert block._stacked_projection is not held
        assert torch.allclose(px, block.linear_x(token), atol=1e-6)
        assert torch.allclose(py, block.linear_y(token), atol=1e-6)
    assert "_stacked_projection" not in block.state_dict()


def test_inference_mode_pass_then_training_step_at_the_same_shape():
    """An evaluation pass under inference_mode followed by a training step at the same (batch, length): the
    default positions and the packed flags remembered from the first must be usable by the second (an
    inference tensor cannot be saved for backward).  The reference builds them on every call."""
    from griffin_amd import modules
    from griffin_amd.hip_scan import _PACKED_FLAGS, pack_flags

    modules._DEFAULT_POSITIONS.clear()
    _PACKED_FLAGS.clear()
    torch.manual_seed(0)
    block = RecurrentBlock(12, 16, gate_blocks=2, scan_mode="sequential")
    x = torch.randn(2, 9, 12)
    with torch.inference_mode():
        block(x)
        pos, first = modules._default_positions(2, 9, x.device)
        packed = pack_flags(first, None)
    assert not pos.is_inference() and not first.is_inference() and not packed.is_inference()
    assert pack_flags(first, None) is packed
    leaf = x.clone().requires_grad_(True)
    block(leaf).sum().backward()
    assert torch.isfinite(leaf.grad).all() and leaf.grad.abs().max() > 0

    class Keep(torch.autograd.Function):                      # what the HIP operators do with the flag bytes
        @staticmethod
        def forward(ctx, t, flags):
            ctx.save_for_backward(flags)
            return t * 2.0

        @staticmethod
        def backward(ctx, g):
            return g * 2.0, None

    Keep.apply(leaf, packed).sum().backward()


def test_caches_are_dropped_by_invalidate_and_module_state_changes():
    """Writes through ``.data`` bump no version counter; ``invalidate_caches`` (and ``to``, ``train``/``eval``,
    ``load_state_dict``) drop the stacked decode projection and the RG-LRU's parameter image."""
    torch.manual_seed(0)
    block = RecurrentBlock(12, 16, gate_blocks=2, scan_mode="sequential")
    token = torch.randn(5, 12)
    with torch.no_grad():
        block._decode_projections(token)
        block.rg_lru._prep, block.rg_lru._prep_key = object(), ("stale",)
        held = block._stacked_projection
        block.linear_x.weight.data.mul_(3.0)                   # invisible to the (data_ptr, version) key
        block._decode_projections(token)
        assert block._stacked_projection is held
        block.invalidate_caches()
        assert block._stacked_projection is None and block.rg_lru._prep is None and block.rg_lru._prep_key is None
        px, _ = block._decode_projections(token)
        assert torch.allclose(px, block.linear_x(token), atol=1e-6)
        for change in (lambda: block.eval(), lambda: block.train(), lambda: block.double(),
                       lambda: block.load_state_dict(copy.deepcopy(block.state_dict()))):
            block._decode_projections(token.to(block.linear_x.weight.dtype))
            block.rg_lru._prep, block.rg_lru._prep_key = object(), ("stale",)
            assert block._stacked_projection is not None
            change()
            assert block._stacked_projection is None and block.rg_lru._prep is None


def test_stacked_halves_are_recognised_only_when_they_are_one_matrix():
    """hip_block_ops._stacked_halves: the two gradients the block's backward writes side by side are found again
    as one [rows, 2 W] matrix; anything else (separate tensors, swapped halves, a gap, other strides) is not."""
    from griffin_amd.hip_block_ops import _stacked_halves

    both = torch.arange(2 * 3 * 8, dtype=torch.float32).view(2, 3, 8)
    left, right = both[..., :4], both[..., 4:]
    got = _stacked_halves(left, right)
    assert got is not None and got.shape == (6, 8) and torch.equal(got, both.view(6, 8))
    assert got.data_ptr() == both.data_ptr()
    assert _stacked_halves(right, left) is None
    assert _stacked_halves(left, None) is None
    assert _stacked_halves(left.contiguous(), right.contiguous()) is None
    assert _stacked_halves(left, right.clone()) is None
    wide = torch.zeros(2, 3, 10)
    assert _stacked_halves(wide[..., :4], wide[..., 4:8]) is None          # rows are 10 apart, not 8
    assert _stacked_halves(both[:, ::2, :4], both[:, ::2, 4:]) is None    # every other row
    one_row = torch.zeros(1, 1, 8)
    assert _stacked_halves(one_row[..., :4], one_row[..., 4:]).shape == (1, 8)
    offset = torch.zeros(5 + 2 * 3 * 8)[5:].view(2, 3, 8)                 # a storage offset carries over
    got = _stacked_halves(offset[..., :4], offset[..., 4:])
    assert got is not None and got.storage_offset() == 5
