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
    assert lib.lvar_dense_attn_fwd(null, fake, fake, fake, one, one, None, 1, 1, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(odd, fake, fake, fake, one, one, None, 1, 1, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, fake, fake, one, one, None, 0, 1, 1, 16, 16, 128, 1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, fake, fake, one, one, None, 1, 1, 1, 16, 16, 128, -1.0, None) == -1
    assert lib.lvar_dense_attn_fwd(fake, fake, null, null, None, None, None, 1, 1, 1, 16, 16, 128, 1.0, None) == -1   # no outputs at all
    assert lib.lvar_dense_attn_fwd(fake, fake, fake, fake, one, one, None, 1, 6, 4, 16, 16, 128, 1.0, None) == -1   # 6 query heads over 4 K/V heads
    assert lib.lvar_colsum_fwd(fake, fake, one, one, None, 1, 6, 0, 16, 16, 128, 192, 1.0, None) == -1
    assert lib.lvar_colsum_fwd(fake, fake, one, one, None, 1, 1, 1, 16, 16, 128, 100, 1.0, None) == -1           # group not a multiple of 32
    assert lib.lvar_colsum_fwd(fake, fake, None, one, None, 1, 1, 1, 16, 16, 128, 192, 1.0, None) == -1
    assert lib.lvar_csp_attn_fwd(fake, fake, fake, null, fake, None, None, one, one, 1, 16, 100, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -2   # groups of 100 rows: no workgroup shape
    assert lib.lvar_csp_attn_fwd(fake, fake, fake, null, fake, None, None, one, one, 1, 16, 0, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -1
    assert lib.lvar_dense_attn_rcp_fwd(fake, fake, fake, fake, None, 1, 1, 1, 16, 16, 128, 1.0, None) == -1                # no place for the row constant
    assert lib.lvar_csp_attn_fwd(fake, fake, fake, null, fake, None, None, None, one, 1, 16, 192, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -1
    assert lib.lvar_block_sparse_attn_fwd(fake, fake, fake, fake, None, None, one, 0, 0, one, 0, 0, 4, 4, 96, 64, 1, 1, 16, 16, 128, 1.0, None) == -2    # 96-row query blocks
    assert lib.lvar_block_sparse_attn_fwd(fake, fake, fake, fake, None, None, one, 0, 0, one, 0, 0, 4, 4, 128, 32, 1, 1, 16, 16, 128, 1.0, None) == -2   # 32-key blocks
    wide = LvarTensor(0x1000, 1 << 30, 1 << 26, 1 << 23)                # row stride of 2^23 elements: beyond the 24-bit gather addressing
    assert lib.lvar_csp_attn_fwd(fake, wide, fake, null, fake, None, None, one, one, 1, 16, 192, 1, 1, 16, 16, 128, 1.0, 1.0, None) == -2
    assert lib.lvar_block_sparse_attn_fwd(fake, fake, fake, fake, None, None, None, 0, 0, one, 0, 0, 4, 4, 128, 64, 1, 1, 16, 16, 128, 1.0, None) == -1


def test_list_build_and_upsample_argument_validation(lib):
    from lvar_amd._lib import LvarTensor
    null = LvarTensor(None, 0, 0, 0)
    fake = LvarTensor(0x1000, 128 * 16 * 128, 16 * 128, 128)
    one = ctypes.c_void_p(0x2000)
    assert lib.lvar_topk_token_lists(None, 100, one, 100, one, 4, 100, 10, 0, None) == -1            # no scores
    assert lib.lvar_topk_token_lists(one, 100, one, 100, one, 4, 100, 101, 0, None) == -1            # k > Lk
    assert lib.lvar_topk_token_lists(one, 99, one, 100, one, 4, 100, 10, 0, None) == -1              # row stride < Lk
    assert lib.lvar_topk_token_lists(one, 100, one, 5, one, 4, 100, 10, 0, None) == -1               # output row shorter than k
    assert lib.lvar_topk_token_lists(one, 100, one, 100, one, 4, 100, 10, 101, None) == -1           # zero fill beyond the row
    assert lib.lvar_topk_token_lists(one, 100, one, 100, one, 0, 100, 10, 0, None) == 0              # no rows: nothing to launch
    assert lib.lvar_remap_concat_lists(one, 100, 100, None, 0, 8, one, 200, one, 2, 3, 4, 64, 500, 0, None) == -1   # local run without a table
    assert lib.lvar_remap_concat_lists(one, 100, 100, one, 8, 8, one, 70, one, 2, 3, 4, 64, 500, 0, None) == -1     # 64 + 8 > output row
    assert lib.lvar_remap_concat_lists(one, 100, 100, None, 0, 0, one, 64, one, 2, 0, 4, 64, 500, 0, None) == -1    # no source groups
    assert lib.lvar_mask_to_lists(one, 10, one, 10, one, 3, 10, 0, None) == -1                    # multiple_of must be positive
    assert lib.lvar_mask_to_lists(one, 10, one, 9, one, 3, 10, 1, None) == -1                     # output row shorter than n
    assert lib.lvar_mask_to_lists(one, 10, one, 10, one, 0, 10, 1, None) == 0
    # fused upsample: Lq must be dst_side^2 and the cache must exist
    args = (one, one, 1, 16, 192, 1, 1, 16, 16, 128, 1.0, 1.0, None)
    assert lib.lvar_csp_attn_upsample_fwd(fake, fake, fake, fake, 2, 5, fake, None, None, *args) == -1         # 25 != 16
    assert lib.lvar_csp_attn_upsample_fwd(fake, fake, fake, null, 2, 4, fake, None, None, *args) == -1


def test_header_is_plain_c(tmp_path):
    """The public header must be usable from C (the reference's other bindings are C/C++)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    src = tmp_path / "use.c"
    src.write_text('#include "lvar_sparse_attn.h"\nint main(void) { lvar_tensor_t t = {0, 0, 0, 0}; (void)t; return lvar_version() ? 0 : 1; }\n')
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.dirname(HEADER), "-c", str(src),
                        "-o", str(tmp_path / "use.o")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


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


def test_torch_binding_loads_and_declines_cpu_tensors(lib):
    """The compiled fast path of dense_attn is optional: when it is built it must load, bind to the C-ABI
    library and hand anything but plain device tensors back to the general path (None)."""
    import os
    import torch
    from lvar_amd import _lib
    path = os.path.join(os.path.dirname(_lib.__file__), "_lvar_torch.so")
    if not os.path.exists(path):
        pytest.skip("torch binding not built")
    mod = _lib.torch_binding()
    assert mod is not None and hasattr(mod, "fast_dense_attn") and hasattr(mod, "bind")
    x = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16)
    assert mod.fast_dense_attn(x, x, x, None) is None            # CPU tensors: not its case, and no GPU call is made
