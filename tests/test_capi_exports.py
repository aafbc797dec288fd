"""The C-ABI library loads on a host without a GPU and exports every symbol that
include/nzhip.h declares (no compute calls are made here)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nzhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nzhip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("nzhip_gemm", "nzhip_tensorcore_gemm", "nzhip_im2col", "nzhip_col2im", "nzhip_conv2d_forward",
                 "nzhip_add_broadcast", "nzhip_relu", "nzhip_malloc", "nzhip_free_async", "nzhip_sync_ptr"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from neuzephyr_amd import capi
    lib = capi.load()
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing
    assert sorted(capi.EXPORTS) == declared_symbols()
    assert lib.nzhip_version() >= 100


def test_python_plumbing_never_touches_the_oracle():
    for name in ("capi.py", "__init__.py", "build.py"):
        src = open(os.path.join(ROOT, "neuzephyr_amd", name)).read()
        assert "import oracle" not in src and "from oracle" not in src and "nz_oracle" not in src
