"""The C-ABI library builds, loads and exports every symbol include/plow_moe.h declares (no GPU
needed: nothing is executed on a device here)."""
import ctypes as C
import os
import re

from plow_amd import abi, lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "plow_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(plow_moe_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(lib.LIB_PATH):
        from plow_amd import build
        build.build(verbose=False)
    so = C.CDLL(lib.LIB_PATH)
    names = declared()
    assert sorted(names) == sorted(lib.EXPORTS)
    for n in names:
        assert hasattr(so, n), n
    so.plow_moe_abi.restype = C.c_uint32
    assert so.plow_moe_abi() == 1


def test_descriptor_layout():
    assert C.sizeof(abi.PlowDevInst) == 64
    assert abi.PlowDevInst.t.offset == 16 and abi.PlowDevInst.i.offset == 32
    assert C.sizeof(abi.PlowMoeRoute) == 8
    d = abi.inst(abi.OP_MOE_ALIGN_PF, t=[3, None, 5], i=[1, 2, 3], f=[2.5])
    assert d.t[1] == abi.TENSOR_NONE and d.t[7] == abi.TENSOR_NONE and d.fj[0].f == 2.5
    assert abi.max_rows(64, 9, 257) == 64 * 9 + 257 * 63
