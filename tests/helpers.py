"""Shared helpers of the GPU parity tests: oracle runs and norm-wise error measures."""

import torch

from oracle import rglru_oracle as orc

PARAMS = ("x", "w_a", "b_a", "w_x", "b_x", "lam")


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max |got - want| / max(|want|): the norm-wise relative error used for every tolerance."""
    want = want.detach().double().cpu()
    got = got.detach().double().cpu()
    scale = want.abs().max().item()
    return (got - want).abs().max().item() / (scale if scale > 0 else 1.0)


def oracle_run(case, dtype=torch.float32, reset=None, active=None, dh_last=None, c=8.0):
    """Oracle forward + autograd backward on the CPU.  For bf16 cases the oracle gets the
    bf16-rounded tensors upcast to fp32, so that only compute error is measured."""
    def prep(t):
        return t.to(dtype).to(torch.float32) if dtype != torch.float64 else t.double()
    p = [prep(case[k]) for k in PARAMS]
    h0 = None if case.get("h0") is None else case["h0"].float()
    dy = prep(case["dy"])
    y, h_last, grads = orc.rglru_autograd(*p, dy, c=c, h0=h0, reset_mask=reset, active_mask=active,
                                          dh_last=dh_last)
    return y, h_last, grads


def hip_run(case, dtype=torch.float32, reset=None, active=None, dh_last=None, c=8.0, device="cuda"):
    """Same computation through the HIP operator (C ABI) on the GPU."""
    from griffin_amd import hip_rglru

    leaves = [case[k].to(dtype).to(device).requires_grad_(True) for k in PARAMS]
    h0 = None if case.get("h0") is None else case["h0"].float().to(device).requires_grad_(True)
    rm = None if reset is None else reset.to(device)
    am = None if active is None else active.to(device)
    y, h_last = hip_rglru(*leaves, c, h0, rm, am)
    outs, gouts = [y], [case["dy"].to(dtype).to(device)]
    if dh_last is not None:
        outs.append(h_last)
        gouts.append(dh_last.to(device))
    wrt = leaves + ([h0] if h0 is not None else [])
    grads = torch.autograd.grad(outs, wrt, gouts)
    torch.cuda.synchronize()
    names = list(PARAMS) + (["h0"] if h0 is not None else [])
    return y.detach(), h_last.detach(), dict(zip(names, grads))
