"""CPU: the C-ABI library loads and exports every symbol declared in include/momoe_hip.h;
host-side argument validation works without a GPU (no compute calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "momoe-impl_amd", "momoe_amd", "libmomoe_hip.so")
HEADER = os.path.join(ROOT, "include", "momoe_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(momoe_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import subprocess, sys
        subprocess.check_call([sys.executable, os.path.join(ROOT, "momoe-impl_amd", "build.py")])
    import torch  # noqa: F401  the HIP runtime the library binds to
    return ctypes.CDLL(LIB)


def test_every_declared_symbol_is_exported(lib):
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n


def test_binding_table_matches_header():
    from momoe_amd import _hip
    assert sorted(_hip.EXPORTED_SYMBOLS) == _declared()
    assert _hip.abi_version() == 3
    assert _hip.status_string(0) == "ok" and "unsupported" in _hip.status_string(2)


def test_size_queries_and_argument_validation(lib):
    lib.momoe_tile_table_ints.restype = ctypes.c_int64
    lib.momoe_index_workspace_bytes.restype = ctypes.c_int64
    i64 = ctypes.c_int64
    assert lib.momoe_tile_table_ints(i64(8192), i64(128), i64(8), 128) == 4 + 4 * (512 + 128)
    assert lib.momoe_index_workspace_bytes(i64(8192), i64(128)) >= (128 * 32 + 8 * 8192) * 4
    # null pointers / bad sizes are rejected on the host before anything is launched
    z = ctypes.c_void_p(0)
    assert lib.momoe_combine(z, z, z, i64(1), i64(8), i64(1), i64(1), z) == 1
    assert lib.momoe_wgrad(z, i64(8), z, z, i64(8), z, z, z, i64(1), i64(1), i64(8), i64(8), i64(1),
                           z, i64(0), z) == 1
    lib.momoe_wgrad_workspace_bytes.restype = ctypes.c_int64
    # at most 8 partial tiles of 256 KiB per workgroup (256), fewer when there are few rows
    assert lib.momoe_wgrad_workspace_bytes(i64(128), i64(2048), i64(2048), i64(65536)) == 2048 * 262144
    assert lib.momoe_wgrad_workspace_bytes(i64(2), i64(64), i64(64), i64(9000)) == 4 * 262144
    assert lib.momoe_wgrad_workspace_bytes(i64(2), i64(64), i64(64), i64(100)) == 0


def test_host_modules_refuse_cpu_tensors():
    import torch
    import momoe_amd
    layer = momoe_amd.MoMoE(32, 32, 2, 1, Wl1_ND2H=torch.zeros(2, 32, 64), Wl2_NHD=torch.zeros(2, 32, 32))
    with pytest.raises(RuntimeError):
        layer(torch.zeros(1, 4, 32), torch.ones(2, 4, dtype=torch.int32), torch.ones(2, 4))
    with pytest.raises(AssertionError):
        momoe_amd.MoMoE(32, 32, 2, 1, save_percent=101, Wl1_ND2H=torch.zeros(2, 32, 64),
                        Wl2_NHD=torch.zeros(2, 32, 32))
