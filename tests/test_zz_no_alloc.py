"""The forward entry point that allocates nothing (rglru_hip_fwd_static) against rglru_hip_fwd.

Both are called through the C ABI on the same inputs; the static variant takes its workspace from a
device array inside the library.  Two calls in a row, the second on a smaller input, so that stale
contents of the shared array from the first call would show."""

import pytest
import torch

from oracle import rglru_oracle as orc
from tests.helpers import rel_err

pytestmark = pytest.mark.gpu


def _forward_pair(lib, _lib, dtype, B, T, W, nb, seed, with_flags):
    code = _lib.RGLRU_BF16 if dtype == torch.bfloat16 else _lib.RGLRU_F32
    case = orc.make_case(B, T, W, nb, seed=seed, h0_std=0.5, bias_std=0.3)
    dev = torch.device("cuda", 0)
    x = case["x"].to(dtype).to(dev)
    params = [case[k].to(dtype).to(dev).contiguous() for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
    h0 = case["h0"].float().to(dev)
    flags = None
    if with_flags:
        flags = torch.zeros(B, T, dtype=torch.uint8, device=dev)
        flags[:, T // 3] = _lib.FLAG_RESET
        flags[B - 1, T - 3:] = _lib.FLAG_INACTIVE
    stream = torch.cuda.current_stream().cuda_stream
    prep = torch.empty(lib.rglru_hip_prep_bytes(W, nb, code), dtype=torch.uint8, device=dev)
    _lib.check(lib.rglru_hip_prepare(*(t.data_ptr() for t in params), 8.0, W, nb, code, code, prep.data_ptr(), stream),
               "prepare")
    ws = torch.empty(lib.rglru_hip_workspace_bytes(B, T, W, nb), dtype=torch.uint8, device=dev)
    y_ref, y_new = torch.empty_like(x), torch.empty_like(x)
    hl_ref = torch.empty(B, W, device=dev)
    hl_new = torch.empty(B, W, device=dev)
    fl = None if flags is None else flags.data_ptr()
    _lib.check(lib.rglru_hip_fwd(x.data_ptr(), prep.data_ptr(), h0.data_ptr(), fl, y_ref.data_ptr(), hl_ref.data_ptr(),
                                 ws.data_ptr(), B, T, W, nb, code, stream), "fwd")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    _lib.check(lib.rglru_hip_fwd_static(x.data_ptr(), prep.data_ptr(), h0.data_ptr(), fl, y_new.data_ptr(),
                                        hl_new.data_ptr(), B, T, W, nb, code, stream), "fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return y_ref, hl_ref, y_new, hl_new


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 1e-2), (torch.float32, 1e-6)])
def test_static_forward_matches_workspace_forward(dtype, tol):
    from griffin_amd import _lib

    lib = _lib.load()
    assert lib.rglru_hip_static_workspace_bytes() == 16 << 20
    # first a call that fills most of the built-in workspace, then a smaller one right behind it
    for shape, seed, with_flags in (((8, 2048, 1024, 8), 1, False), ((2, 200, 256, 2), 2, True)):
        B, T, W, nb = shape
        assert lib.rglru_hip_workspace_bytes(B, T, W, nb) <= lib.rglru_hip_static_workspace_bytes()
        print("static forward", dtype, shape, flush=True)
        y_ref, hl_ref, y_new, hl_new = _forward_pair(lib, _lib, dtype, B, T, W, nb, seed, with_flags)
        assert torch.isfinite(y_new.float()).all()
        # the two runs differ at most by the rounding of a different carry composition order
        assert rel_err(y_new.float(), y_ref.float()) < tol
        assert rel_err(hl_new, hl_ref) < tol


def test_static_forward_rejects_what_does_not_fit():
    from griffin_amd import _lib

    lib = _lib.load()
    B, T, W, nb = 64, 4096, 1024, 8
    assert lib.rglru_hip_workspace_bytes(B, T, W, nb) > lib.rglru_hip_static_workspace_bytes()
    fake = 256                                                  # never dereferenced: rejected on the host
    rc = lib.rglru_hip_fwd_static(fake, fake, None, None, fake, None, B, T, W, nb, _lib.RGLRU_BF16, None)
    assert rc == 2
    assert b"built-in" in lib.rglru_hip_last_error()
