"""The C-ABI library loads, exports every symbol the header declares, and
rejects bad arguments with an error code and message before touching a GPU."""
import ctypes
import os
import re

import pytest

from daisy_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "daisy_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(daisy_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 8
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/daisy_hip.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes prototype in daisy_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names


def test_abi_version():
    assert _lib.load().daisy_abi_version() == _lib.ABI_VERSION


def test_workspace_queries_need_no_gpu():
    lib = _lib.load()
    assert lib.daisy_decode_workspace_bytes(64, 16, 128, 4096, 1) == 0
    assert lib.daisy_decode_workspace_bytes(1, 2, 128, 4096, 4) == 1 * 2 * 4 * 130 * 4
    assert lib.daisy_decode_workspace_bytes(0, 2, 128, 4096, 4) == 0
    assert lib.daisy_kda_workspace_bytes(4, 8192, 16, 128, 128, 64) > 0


def test_split_count_the_library_picks():
    """nsplit = 0 lets the library choose; the workspace size shows the choice (B * H * splits * (D + 2) floats).
    About 512 rows per workgroup, at most about 1024 workgroups, and shorter splits (down to 128 rows) when a few
    (batch, head) pairs would otherwise leave most compute units idle."""
    lib = _lib.load()

    def splits(B, H, n_rows, D=128):
        nbytes = lib.daisy_decode_workspace_bytes(B, H, D, n_rows, 0)
        return 1 if nbytes == 0 else nbytes // (B * H * (D + 2) * 4)

    assert splits(64, 16, 4096) == 1          # BASELINE config 4: one workgroup per (batch, head) already fills the chip
    assert splits(16, 8, 4096) == 8           # 512 rows each
    assert splits(1, 12, 8192) == 16          # the generator's batch of one (model_specs/daisy_milli.yml): 512 rows each
    assert splits(1, 12, 1024) == 8           # few pairs, short ring: 128 rows each
    assert splits(1, 6, 8192) == 32
    assert splits(4, 12, 300) == 2
    assert splits(1, 1, 100) == 1
    for B, H, n in ((1, 1, 10 ** 6), (3, 5, 70000)):
        assert 1 <= splits(B, H, n) <= 64


def _err():
    return _lib.load().daisy_last_error().decode()


def test_prefill_argument_errors():
    lib = _lib.load()
    s3 = (ctypes.c_int64 * 3)(8, 8, 8)
    rc = lib.daisy_prefill_fwd(None, s3, None, s3, None, s3, None, None, None, None, s3, None, None,
                               1, 8, 1, 64, 4, 0.12, 0, None)
    assert rc == -1 and "non-NULL" in _err()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    rc = lib.daisy_prefill_fwd(p, s3, p, s3, p, s3, None, None, None, p, s3, None, None, 1, 8, 1, 7, 4, 0.12, 0, None)
    assert rc == -2 and "head_dim" in _err()
    rc = lib.daisy_prefill_fwd(p, s3, p, s3, p, s3, p, None, None, p, s3, None, None, 1, 8, 1, 64, 4, 0.12, 0, None)
    assert rc == -1 and "cos and sin" in _err()
    rc = lib.daisy_prefill_fwd(p, s3, p, s3, p, s3, None, None, None, p, s3, None, None, 0, 8, 1, 64, 4, 0.12, 0, None)
    assert rc == -1 and "positive" in _err()
    # Rotation tables without a buffer for the rotated keys: refused (head dims of the matrix-core kernel),
    # as are flag bits (none is defined).
    big = ctypes.create_string_buffer(4096)
    a = (ctypes.addressof(big) + 15) & ~15
    for D in (64, 128):
        rc = lib.daisy_prefill_fwd(a, s3, a, s3, a, s3, a, a, None, a, s3, None, None, 1, 8, 1, D, 4, 0.12, 0, None)
        assert rc == -1 and "k_out" in _err()
    rc = lib.daisy_prefill_fwd(a, s3, a, s3, a, s3, None, None, None, a, s3, None, None, 1, 8, 1, 64, 4, 0.12, 1, None)
    assert rc == -1 and "flags" in _err()


def test_decode_argument_errors():
    lib = _lib.load()
    s2 = (ctypes.c_int64 * 2)(128, 128)
    s3 = (ctypes.c_int64 * 3)(128, 128, 128)
    buf = ctypes.create_string_buffer(1024)
    p = (ctypes.addressof(buf) + 15) & ~15

    def call(D=128, n_rows=4, new_idx=0, kc=p, ws=None, ws_bytes=0, nsplit=1):
        return lib.daisy_decode_fwd(p, s2, p, s2, p, s2, kc, s3, kc, s3, None, None, p, s2, 1, 1, D,
                                    n_rows, new_idx, 0, 0.12, nsplit, ws, ws_bytes, None)
    assert call(D=33) == -2 and "head_dim" in _err()
    assert call(D=258) == -2 and "head_dim" in _err()
    assert call(new_idx=4) == -1 and "new_idx" in _err()
    assert call(n_rows=0) == -1
    assert call(kc=None) == -1 and "cache pointers" in _err()
    assert call(n_rows=1024, nsplit=4) == -3 and "workspace" in _err()


def test_kda_argument_errors():
    lib = _lib.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    for Dk, Dv in ((136, 128), (60, 128), (128, 20), (0, 128)):      # Dk: a multiple of 8 up to 128; Dv: a multiple of 8
        rc = lib.daisy_kda_chunk_fwd(p, p, p, p, 0, p, None, p, None, 1, 64, 1, Dk, Dv, 64, 0.1, 1, 1e-6, None, 0, None)
        assert rc == -2 and "Dk" in _err(), (Dk, Dv)
        assert lib.daisy_kda_workspace_bytes(1, 64, 1, Dk, Dv, 64) == 0
        rc = lib.daisy_kda_recurrent_fwd(p, p, p, p, 0, p, None, p, None, 1, 1, 1, Dk, Dv, 0.1, 1, 1e-6, None)
        assert rc == -2 and "Dk" in _err(), (Dk, Dv)
    # narrower and wider heads share the workspace of the 128 x 128 layout (value columns go through it in passes)
    assert lib.daisy_kda_workspace_bytes(1, 64, 1, 64, 64, 64) == lib.daisy_kda_workspace_bytes(1, 64, 1, 128, 256, 64) > 0
    rc = lib.daisy_kda_chunk_fwd(p, p, p, p, 0, p, None, p, None, 1, 64, 1, 64, 256, 64, 0.1, 1, 1e-6, None, 0, None)
    assert rc == -3 and "workspace" in _err()
    rc = lib.daisy_kda_chunk_fwd(None, p, p, p, 0, p, None, p, None, 1, 64, 1, 128, 128, 64, 0.1, 1, 1e-6, None, 0, None)
    assert rc == -1
    rc = lib.daisy_kda_chunk_fwd(p, p, p, p, 0, p, None, p, None, 1, 64, 1, 128, 128, 64, 0.1, 1, 1e-6, None, 0, None)
    assert rc == -3 and "workspace" in _err()
    rc = lib.daisy_kda_gate_fwd(None, p, None, p, 4, 2, 8, 0, 1.0, 20.0, None)
    assert rc == -1


def test_cpu_tensors_are_refused():
    import torch
    from daisy_amd import CausalSelfAttention
    os.environ["DISABLE_O_ZERO_INIT"] = "1"
    attn = CausalSelfAttention(dim=128, num_heads=2, head_dim=64, max_seq_len=64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        attn(torch.randn(1, 8, 128), None)
