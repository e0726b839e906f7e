"""The C-ABI shared library: builds for gfx950 without a GPU, loads, exports every symbol declared in
include/lvar_sparse_attn.h, and validates arguments before touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lvar_sparse_attn.h")


@pytest.fixture(scope="module")
def lib():
    from lvar_amd import _lib
    from lvar_amd.build import LIB_PATH, build_library
    if not os.path.exists(LIB_PATH):
        build_library()
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lvar_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    from lvar_amd import _lib
    names = declared_symbols()
    assert set(names) == set(_lib.EXPORTED_SYMBOLS), names
    for n in names:
        assert getattr(lib, n) is not None


def test_version_and_arch(lib):
    assert lib.lvar_version() >= 100
    assert lib.lvar_target_arch() == b"gfx950"
    assert lib.lvar_status_string(0) == b"ok"
    assert b"invalid" in lib.lvar_status_string(-1) and b"unsupported" in lib.lvar_status_string(-2)


def test_argument_validation_without_device(lib):
    """Bad arguments are rejected on the host before any HIP call is made."""
    from lvar_amd._lib import LvarTensor
    null = LvarTensor(None, 0, 0, 0)
    fake = LvarTensor(0x1000, 128 * 16 * 128, 16 * 128, 128)          # aligned, never dereferenced
    odd = LvarTensor(0x1008, 128 * 16 * 128, 16 * 128, 128)           # misaligned base
    one = ctypes.c_void_p(0x2000)
    assert lib.lvar_dense_attn_fwd(null, fake, fake, fake, one, one, None, 1, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(odd, fake, fake, fake, one, one, None, 1, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, fake, fake, one, one, None, 0, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, fake, fake, one, one, None, 1, 1, 16, 16, 128, -1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, null, null, None, None, None, 1, 1, 16, 16, 128, 1.0, None) == -1   # no outputs at all
    assert lib.lvar_colsum_fwd(fake, fake, one, one, None, 1, 1, 16, 16, 128, 100, 1.0, None) == -1           # group not a multiple of 32
    assert lib.lvar_colsum_fwd(fake, fake, None, one, None, 1, 1, 16, 16, 128, 192, 1.0, None) == -1
    assert lib.lvar_csp_attn_fwd(fake, fake, fake, null, fake, None, None, one, one, 1, 16, 100, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -1
    assert lib.lvar_csp_attn_fwd(fake, fake, fake, null, fake, None, None, None, one, 1, 16, 192, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -1
    assert lib.lvar_block_sparse_attn_fwd(fake, fake, fake, fake, None, None, one, 0, 0, one, 0, 0, 4, 4, 64, 64, 1, 1, 16, 16, 128, 1.0, None) == -2
    assert lib.lvar_block_sparse_attn_fwd(fake, fake, fake, fake, None, None, None, 0, 0, one, 0, 0, 4, 4, 128, 64, 1, 1, 16, 16, 128, 1.0, None) == -1


def test_python_wrappers_fail_loudly_without_gpu():
    import torch
    from lvar_amd import sparse_attn_ops as ops
    q = torch.zeros(1, 1, 64, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.dense_attn(q, q, q)
    with pytest.raises(TypeError):
        ops.dense_attn(q.float(), q.float(), q.float())
    with pytest.raises(AssertionError):
        ops.csp_attn(q, q, q, None, torch.zeros(1, 1, 1, 3, dtype=torch.int32), torch.zeros(1, 1, 1, dtype=torch.int32), q, 1)


def test_missing_library_is_an_import_error(monkeypatch):
    from lvar_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("LVAR_AMD_LIB", "/nonexistent/liblvar.so")
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _lib.load()
