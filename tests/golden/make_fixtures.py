"""Write small golden vectors for the RG-LRU path from the reference implementation.

Run once, in the build container, where the reference checkout is mounted at /root/reference:

    python tests/golden/make_fixtures.py

The reference is only imported here; the resulting ``*.npz`` files (inputs, parameters, masks and
the reference's outputs and gradients, a few KB each) are what the tests read.  Composite behaviour
(reset + padding + carried state + gradients in one call, and the recurrent block with its cache)
is the part that no closed form pins, so that is what is recorded.
"""

import os
import sys

import numpy as np
import torch

REFERENCE = os.environ.get("GRIFFIN_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def _np(t):
    return t.detach().cpu().numpy()


def rglru_case(name, B, T, W, blocks, seed, with_reset, with_padding, with_h0, with_dh):
    from griffin import RG_LRU

    torch.manual_seed(seed)
    mod = RG_LRU(rnn_width=W, gate_blocks=blocks, scan_mode="sequential")
    with torch.no_grad():  # non-zero biases so their gradients are exercised
        mod.recurrence_gate.bias.normal_(0.0, 0.3)
        mod.input_gate.bias.normal_(0.0, 0.3)
    x = torch.randn(B, T, W, requires_grad=True)
    reset = torch.zeros(B, T, dtype=torch.bool)
    active = torch.ones(B, T, dtype=torch.bool)
    if with_reset:
        reset[:, T // 2] = True
        reset[0, 0] = True
    if with_padding:
        active[B - 1, T - 3:] = False
    h0 = (0.5 * torch.randn(B, W)).requires_grad_(True) if with_h0 else None
    dy = torch.randn(B, T, W)
    dh = torch.randn(B, W) if with_dh else None
    y, h_last = mod(x, h0, reset_mask=reset, active_mask=active, return_state=True)
    loss = (y * dy).sum()
    if dh is not None:
        loss = loss + (h_last * dh).sum()
    loss.backward()
    out = {
        "x": _np(x), "w_a": _np(mod.recurrence_gate.weight), "b_a": _np(mod.recurrence_gate.bias),
        "w_x": _np(mod.input_gate.weight), "b_x": _np(mod.input_gate.bias), "lam": _np(mod.Lambda),
        "reset": _np(reset), "active": _np(active), "dy": _np(dy),
        "y": _np(y), "h_last": _np(h_last),
        "g_x": _np(x.grad), "g_w_a": _np(mod.recurrence_gate.weight.grad),
        "g_b_a": _np(mod.recurrence_gate.bias.grad), "g_w_x": _np(mod.input_gate.weight.grad),
        "g_b_x": _np(mod.input_gate.bias.grad), "g_lam": _np(mod.Lambda.grad),
    }
    if h0 is not None:
        out["h0"] = _np(h0)
        out["g_h0"] = _np(h0.grad)
    if dh is not None:
        out["dh"] = _np(dh)
    np.savez(os.path.join(HERE, name + ".npz"), **out)
    print("wrote", name, {k: v.shape for k, v in out.items() if k in ("x", "w_a")})


def saturated_case(name):
    """The reference's bounded-sqrt case (tests/test_rglru.py:61-75) evaluated in fp32."""
    from griffin import RG_LRU

    torch.manual_seed(3)
    mod = RG_LRU(rnn_width=16, gate_blocks=4, scan_mode="sequential")
    with torch.no_grad():
        mod.recurrence_gate.weight.zero_()
        mod.recurrence_gate.bias.fill_(-100)
        mod.Lambda.fill_(20)
    x = torch.randn(2, 8, 16, requires_grad=True)
    y = mod(x)
    y.square().mean().backward()
    np.savez(os.path.join(HERE, name + ".npz"), x=_np(x), w_x=_np(mod.input_gate.weight),
             b_x=_np(mod.input_gate.bias), y=_np(y), g_x=_np(x.grad), g_lam=_np(mod.Lambda.grad),
             g_b_a=_np(mod.recurrence_gate.bias.grad))
    print("wrote", name)


def block_case(name, B, T, D, W, blocks, seed, splits):
    from griffin import RecurrentBlock

    torch.manual_seed(seed)
    blk = RecurrentBlock(input_dim=D, rnn_width=W, gate_blocks=blocks, scan_mode="sequential").eval()
    with torch.no_grad():
        blk.temporal_conv.bias.normal_(0.0, 0.1)
        blk.linear_x.bias.normal_(0.0, 0.1)
    x = torch.randn(B, T, D)
    with torch.no_grad():
        full, cache = blk(x, return_cache=True)
        pieces, state, start = [], None, 0
        for stop in splits + [T]:
            piece, state = blk(x[:, start:stop], state, return_cache=True)
            pieces.append(piece)
            start = stop
    out = {
        "x": _np(x), "full": _np(full), "chunked": _np(torch.cat(pieces, dim=1)),
        "rnn_state": _np(cache.rnn_state), "conv_state": _np(cache.conv_state),
        "segment_position": _np(cache.segment_position),
        "lx_w": _np(blk.linear_x.weight), "lx_b": _np(blk.linear_x.bias),
        "ly_w": _np(blk.linear_y.weight), "ly_b": _np(blk.linear_y.bias),
        "lo_w": _np(blk.linear_out.weight), "lo_b": _np(blk.linear_out.bias),
        "conv_w": _np(blk.temporal_conv.weight[:, 0, :]), "conv_b": _np(blk.temporal_conv.bias),
        "w_a": _np(blk.rg_lru.recurrence_gate.weight), "b_a": _np(blk.rg_lru.recurrence_gate.bias),
        "w_x": _np(blk.rg_lru.input_gate.weight), "b_x": _np(blk.rg_lru.input_gate.bias),
        "lam": _np(blk.rg_lru.Lambda), "splits": np.array(splits),
    }
    np.savez(os.path.join(HERE, name + ".npz"), **out)
    print("wrote", name)


def main():
    sys.path.insert(0, REFERENCE)
    rglru_case("rglru_plain_b2_t16_w32", 2, 16, 32, 4, seed=11, with_reset=False, with_padding=False,
               with_h0=False, with_dh=False)
    rglru_case("rglru_masks_b2_t16_w32", 2, 16, 32, 4, seed=12, with_reset=True, with_padding=True,
               with_h0=True, with_dh=True)
    rglru_case("rglru_odd_b3_t37_w65", 3, 37, 65, 16, seed=13, with_reset=True, with_padding=True,
               with_h0=True, with_dh=False)
    saturated_case("rglru_saturated_b2_t8_w16")
    block_case("block_b2_t9_d8_w12", 2, 9, 8, 12, 16, seed=14, splits=[3, 7])


if __name__ == "__main__":
    main()
