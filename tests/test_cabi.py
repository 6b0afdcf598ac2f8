"""The C-ABI library: it loads, exports every symbol the header declares, and validates arguments
on the host before touching a GPU (no kernel is launched here)."""

import ctypes
import os
import re

import pytest

from griffin_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rglru_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rglru_hip_[a-z_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from griffin_amd import build

        build.build()
    return _lib.load()


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(_lib.EXPORTED_SYMBOLS)


def test_build_compiles_every_kernel_source():
    """Every .hip file under griffin_amd/csrc is part of the library (a new translation unit that the build
    list misses would compile nowhere and its entry points would be undefined at load time)."""
    from griffin_amd import build

    present = sorted(f for f in os.listdir(build.CSRC) if f.endswith(".hip"))
    assert sorted(build.SOURCES) == present


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(raw, name), name
    assert lib.rglru_hip_abi_version() == _lib.ABI_VERSION
    assert lib.rglru_hip_max_block_width() == 512


def test_size_queries(lib):
    assert lib.rglru_hip_prep_bytes(1024, 8, _lib.RGLRU_BF16) > 2 * 8 * 128 * 128 * 2
    assert lib.rglru_hip_prep_bytes(1024, 8, _lib.RGLRU_F32) > lib.rglru_hip_prep_bytes(1024, 8, _lib.RGLRU_BF16)
    assert lib.rglru_hip_prep_bytes(1024, 7, _lib.RGLRU_F32) == 0          # width not divisible
    assert lib.rglru_hip_prep_bytes(4096, 2, _lib.RGLRU_F32) == 0          # block wider than 512
    small = lib.rglru_hip_workspace_bytes(2, 64, 256, 8)
    large = lib.rglru_hip_workspace_bytes(2, 4096, 256, 8)
    assert 0 < small < large
    assert lib.rglru_hip_workspace_bytes(0, 64, 256, 8) == 0
    assert lib.rglru_hip_scan_workspace_bytes(2, 100, 65) > 0
    assert lib.rglru_hip_scan_workspace_bytes(2, 0, 65) == 0


def test_argument_errors_are_reported_without_a_gpu(lib):
    # null pointers and bad shapes are rejected on the host, with a message
    assert lib.rglru_hip_scan_fwd(None, None, None, None, None, 1, 1, 1, None) == 1
    assert b"null" in lib.rglru_hip_last_error()
    assert lib.rglru_hip_fwd(None, None, None, None, None, None, None, 2, 8, 1024, 7, _lib.RGLRU_BF16, None) == 1
    assert b"divisible" in lib.rglru_hip_last_error()
    assert lib.rglru_hip_fwd(None, None, None, None, None, None, None, 2, 8, 4096, 2, _lib.RGLRU_BF16, None) == 2
    assert b"512" in lib.rglru_hip_last_error()
    assert lib.rglru_hip_step(None, None, None, None, None, 4, 64, 2, 7, None) == 1
    assert b"dtype" in lib.rglru_hip_last_error()
    with pytest.raises(ValueError):
        _lib.check(1, "probe")
    with pytest.raises(RuntimeError):
        _lib.check(3, "probe")


def test_oversized_sequences_are_rejected_on_the_host(lib):
    """Per-sequence slices of the workspace are addressed with 32-bit offsets: a sequence whose
    checkpoints (4 W bytes per 16 tokens) reach 2 GiB is refused before anything is launched."""
    fake = ctypes.c_void_p(256)            # never dereferenced: the size checks come first
    args = lambda T, W: (fake, fake, None, None, fake, None, fake, 1, T, W, W // 128, _lib.RGLRU_BF16, None)
    assert lib.rglru_hip_fwd(*args(1 << 23, 1024)) == 2          # T W = 2^33
    assert b"per-sequence" in lib.rglru_hip_last_error()
    assert lib.rglru_hip_fwd(*args(1 << 24, 512)) == 2
    assert lib.rglru_hip_fwd(fake, fake, None, None, fake, None, fake, 1 << 20, 2048, 1024, 8, _lib.RGLRU_BF16, None) == 2


def test_spin_limit_hook_round_trips(lib):
    previous = lib.rglru_hip_set_spin_limit(1234)
    assert lib.rglru_hip_set_spin_limit(previous) == 1234


def test_reproducible_switch_round_trips(lib):
    previous = lib.rglru_hip_set_reproducible(1)
    assert lib.rglru_hip_set_reproducible(previous) == 1
    assert lib.rglru_hip_set_reproducible(previous) == previous


def test_chain_forward_switch_round_trips(lib):
    previous = lib.rglru_hip_set_chain_forward(2)
    assert lib.rglru_hip_set_chain_forward(7) == 2          # out of range selects the default
    assert lib.rglru_hip_set_chain_forward(previous) == 0


def test_block_forward_queries_and_errors_without_a_gpu(lib):
    """Where the one-launch block forward applies, and its host-side argument checks (nothing is launched)."""
    assert lib.rglru_hip_block_fwd_path(1024, 8, 4, _lib.RGLRU_BF16) == 1      # blocks of 128 channels
    assert lib.rglru_hip_block_fwd_path(1024, 16, 4, _lib.RGLRU_BF16) == 1     # 64
    assert lib.rglru_hip_block_fwd_path(1024, 32, 1, _lib.RGLRU_BF16) == 1     # 32, a single tap
    assert lib.rglru_hip_block_fwd_path(2560, 8, 4, _lib.RGLRU_BF16) == 0      # 320: three launches
    assert lib.rglru_hip_block_fwd_path(1024, 8, 4, _lib.RGLRU_F32) == 0
    assert lib.rglru_hip_block_fwd_path(1024, 8, 5, _lib.RGLRU_BF16) == 0
    fake = ctypes.c_void_p(256)            # never dereferenced: the checks come first
    # (u, u_stride, v, v_stride, conv_state, taps, conv_bias, K, vec_dtype, prep, h0, flags, x_conv, y, gated,
    #  new_conv_state, h_last, ws, B, T, W, nb, dtype, stream)
    base = [fake, 0, fake, 0, None, fake, None, 4, _lib.RGLRU_BF16, fake, None, None, None, None, fake, None, None, fake,
            2, 16, 128, 2, _lib.RGLRU_BF16, None]
    wide = list(base); wide[20], wide[21] = 640, 2
    assert lib.rglru_hip_block_fwd(*wide) == 2
    assert b"block_fwd" in lib.rglru_hip_last_error()
    no_gate = list(base); no_gate[2] = None
    assert lib.rglru_hip_block_fwd(*no_gate) == 1
    short = list(base); short[1] = 64
    assert lib.rglru_hip_block_fwd(*short) == 1
    assert b"stride" in lib.rglru_hip_last_error()
    odd = list(base); odd[0] = ctypes.c_void_p(258)
    assert lib.rglru_hip_block_fwd(*odd) == 2
    assert b"aligned" in lib.rglru_hip_last_error()
    assert lib.rglru_hip_block_flags(None, None, 4, None) == 1
    # the sentinel for "every row starts a document" is not a flag array of the decode steps
    assert lib.rglru_hip_step(fake, fake, fake, ctypes.c_void_p(1), fake, 4, 64, 2, _lib.RGLRU_BF16, None) == 1
    assert b"FIRST_RESET" in lib.rglru_hip_last_error()
