"""Times both kernel pairs of the bf16 fast path -- tiles with a look-back between workgroups, and one workgroup per
(sequence, 32-channel slab) chain -- over a grid of shapes and compares the faster one with what the library picks
(rglru_hip_backward_path, i.e. the time models in fwd_chain_pays, rglru_fused.h).

    python -m griffin_amd.selection_sweep [--quick]

One line per shape: forward + reverse-scan kernel time of each pair in microseconds (library event hook, median of
five), the faster pair, the library's choice, and a mark where the choice is slower by more than 5 %.  The tiled
figure includes the 6 us parameter launch that the chain forward does itself.  The constants in fwd_chain_pays are a
fit to this output on an MI355X; on a part with another number of compute units or another memory system, refit.
"""

from __future__ import annotations

import sys

import torch

from . import _lib, hip_rglru, set_chain_forward
from .hip_scan import kernel_path

PREPARE_US = 6.0


def shapes(quick: bool):
    widths = ((1024, 8),) if quick else ((512, 4), (1024, 8), (1024, 16), (2048, 16), (4096, 32), (2048, 64))
    batches = (1, 8, 16, 64) if quick else (1, 2, 4, 6, 8, 9, 12, 16, 24, 32, 64)
    for W, nb in widths:
        for B in batches:
            for T in (128, 256, 512, 1024, 2048, 8192):
                if 2 * 256 * 512 <= B * T * W <= 8 * 8192 * 1024 * 2:
                    yield B, T, W, nb
    if not quick:
        yield from ((256, 2048, 1024, 8), (64, 2048, 1024, 8), (32, 8192, 1024, 8), (128, 512, 1024, 8))


def time_pair(lib, B, T, W, nb, mode):
    """(forward, reverse scan) kernel microseconds with the kernel pair forced to `mode` (1 tiled, 2 chain)."""
    gen = torch.Generator().manual_seed(0)
    bw, dt = W // nb, torch.bfloat16
    x = torch.randn(B, T, W, generator=gen).to(dt).cuda().requires_grad_(True)
    dy = torch.randn(B, T, W, generator=gen).to(dt).cuda()
    params = [(torch.randn(nb, bw, bw, generator=gen) / bw ** 0.5).to(dt).cuda().requires_grad_(True), torch.zeros(nb, bw, dtype=dt, device="cuda", requires_grad=True),
              (torch.randn(nb, bw, bw, generator=gen) / bw ** 0.5).to(dt).cuda().requires_grad_(True), torch.zeros(nb, bw, dtype=dt, device="cuda", requires_grad=True),
              torch.logit(torch.rand(W, generator=gen) * 0.09 + 0.9).to(dt).cuda().requires_grad_(True)]

    def step():
        return torch.autograd.grad(hip_rglru(x, *params, 8.0)[0], [x] + params, dy)

    was = set_chain_forward(mode)
    try:
        for _ in range(2):
            step()
        lib.rglru_hip_set_timing(1)
        fwd, rev = [], []
        for _ in range(5):
            step()
            step()
            fwd.append(lib.rglru_hip_kernel_ms(0) * 1e3)
            rev.append(lib.rglru_hip_kernel_ms(1) * 1e3)
        lib.rglru_hip_set_timing(0)
    finally:
        set_chain_forward(was)
    return sorted(fwd)[2], sorted(rev)[2]


def main(argv):
    lib = _lib.load()
    wrong = total = 0
    for B, T, W, nb in shapes("--quick" in argv):
        tiled = time_pair(lib, B, T, W, nb, 1)
        chain = time_pair(lib, B, T, W, nb, 2)
        t_tiled, t_chain = sum(tiled) + PREPARE_US, sum(chain)
        picked_chain = kernel_path(B, T, W, nb, torch.bfloat16) == _lib.PATH_FAST_CHAIN
        t_picked, t_other = (t_chain, t_tiled) if picked_chain else (t_tiled, t_chain)
        slow = t_picked > 1.05 * t_other
        wrong += slow
        total += 1
        print("B%-3d T%-5d W%-5d bw%-4d chains %5d  tiled %6.1f + %6.1f (+%.0f)  chain %6.1f + %6.1f  faster: %s  picked: %s%s" % (
            B, T, W, W // nb, B * W // 32, tiled[0], tiled[1], PREPARE_US, chain[0], chain[1],
            "chain" if t_chain < t_tiled else "tiled", "chain" if picked_chain else "tiled", "   <-- slower by more than 5 %" if slow else ""), flush=True)
    print("shapes %d, picks slower by more than 5 %%: %d" % (total, wrong))


if __name__ == "__main__":
    main(sys.argv[1:])
