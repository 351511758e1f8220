"""The C ABI without a GPU: the built library loads, exports every function include/maya_moe.h declares, and its
host-only entry points (sizes, support tables, layouts) answer like the CPU checker's."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "maya_moe.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef struct.*?\}\s*\w+;", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(maya_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def maya():
    from maya_amd import lib
    if not os.path.exists(lib.LIB_PATH):
        from maya_amd import build
        build.build()
    return lib


def test_every_declared_function_is_exported(maya):
    names = declared_functions()
    assert len(names) >= 28
    L = C.CDLL(maya.LIB_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    from maya_amd import exl3, prefill
    assert set(maya.EXPORTS + exl3.EXPORTS + prefill.EXPORTS) == set(names)


def test_sizes_and_support_tables(maya, oracle):
    L = maya.load()
    for t, bytes_, vals in ((maya.Q8_0, 34, 32), (maya.Q4_K, 144, 256), (maya.IQ2_S, 82, 256), (maya.IQ1_S, 50, 256),
                            (maya.IQ1_M, 56, 256), (maya.IQ2_XXS, 66, 256)):
        assert L.maya_moe_supported(t) == 1
        assert L.maya_moe_block_bytes(t) == bytes_ and L.maya_moe_block_values(t) == vals
        assert maya.row_bytes(t, 4096) == oracle.row_bytes(t, 4096) == 4096 // vals * bytes_
    assert L.maya_moe_supported(2) == 0 and maya.row_bytes(maya.IQ2_S, 100) == 0
    l, n = maya.layout(maya.IQ2_S, maya.IQ2_S, 4096, 2048)
    assert n == 3 * 2048 * 4096 // 256 * 82 and l.up_off == 2048 * 16 * 82 and l.down_off == 2 * l.up_off
    with pytest.raises(maya.MayaError):
        maya.layout(maya.IQ2_S, maya.IQ2_S, 4000, 2048)


def test_exl3_host_entry_points(maya):
    from maya_amd import exl3
    # exl3::k2_supported: even K2 2..16 with every codebook, odd 3 / 5 / 7 with mul1 only
    for k2 in range(0, 20):
        for cb in range(0, 4):
            want = (cb in (0, 1, 2) and k2 in (2, 4, 6, 8, 10, 12, 14, 16)) or (cb == 2 and k2 in (3, 5, 7))
            assert exl3.supported(k2, cb) == want, (k2, cb)
    assert exl3.trellis_bytes(4096, 2048, 6) == 4096 * 2048 * 6 // 16
    l, n = exl3.make_layout(4096, 2048, 6, 2)
    assert exl3.load().maya_exl3_workspace_bytes(C.byref(l), 4, 8) > 4 * 8 * (4096 + 2048) * 4
    assert exl3.load().maya_exl3_workspace_bytes(C.byref(l), 0, 8) == 0
