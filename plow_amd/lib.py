"""Loader of the operator's C-ABI library and a thin object wrapper over it.

The wrapper mirrors how plow's runtime drives a native MoE route: load the object, check its ABI
marker, then hand it op descriptors and a tensor-handle table (crates/plowrt/src/exec/gpu/moe_lt.rs:
697-814, :1134-1322). There is no fallback: if the library is missing the import-time error says how
to build it, and every call goes to the HIP kernels.
"""
import ctypes as C
import os

from . import abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libplow_moe_gfx950.so")

EXPORTS = ["plow_moe_abi", "plow_moe_create", "plow_moe_destroy", "plow_moe_last_error",
           "plow_moe_exec", "plow_moe_exec_many", "plow_moe_pf", "plow_moe_dec",
           "plow_moe_set_min_rows", "plow_moe_check", "plow_moe_exec_noalloc", "plow_moe_reserve_staging"]

_lib = None


class MoeError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"plow_moe error {code}: {text}")
        self.code = code


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built; run `python -m plow_amd.build` "
                          "(or __graft_entry__.build()). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    P, I = C.POINTER, C.POINTER(abi.PlowDevInst)
    lib.plow_moe_abi.restype = C.c_uint32
    lib.plow_moe_create.argtypes = [P(C.c_void_p), C.c_int]
    lib.plow_moe_destroy.argtypes = [C.c_void_p]
    lib.plow_moe_destroy.restype = None
    lib.plow_moe_last_error.argtypes = [C.c_void_p]
    lib.plow_moe_last_error.restype = C.c_char_p
    lib.plow_moe_exec.argtypes = [C.c_void_p, I, P(C.c_void_p), C.c_void_p]
    lib.plow_moe_exec_many.argtypes = [C.c_void_p, I, C.c_uint32, P(C.c_void_p), C.c_void_p]
    lib.plow_moe_check.argtypes = [C.c_void_p, I, P(C.c_void_p)]
    for name in ("plow_moe_pf", "plow_moe_dec"):
        getattr(lib, name).argtypes = [C.c_void_p, I, C.c_uint32, P(C.c_void_p), C.c_uint32, C.c_void_p]
    lib.plow_moe_set_min_rows.argtypes = [C.c_void_p, C.c_int, C.c_int]
    lib.plow_moe_exec_noalloc.argtypes = [I, P(C.c_void_p), C.c_void_p, C.c_char_p, C.c_size_t]
    lib.plow_moe_exec_noalloc.restype = C.c_int
    lib.plow_moe_reserve_staging.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t]
    _lib = lib
    return lib


class Moe:
    """One operator context on one GPU."""

    def __init__(self, device=0):
        self.lib = load()
        if self.lib.plow_moe_abi() != 1:
            raise ImportError("libplow_moe_gfx950.so: unexpected ABI marker")
        h = C.c_void_p()
        rc = self.lib.plow_moe_create(C.byref(h), device)
        if rc:
            raise MoeError(rc, "plow_moe_create failed (is this an MI355X / gfx950?)")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.lib.plow_moe_destroy(self.h)
            self.h = None

    __del__ = close

    def _ck(self, rc, allow=()):
        if rc and rc not in allow:
            raise MoeError(rc, self.lib.plow_moe_last_error(self.h).decode())
        return rc

    def exec(self, inst, table, stream=None):
        return self._ck(self.lib.plow_moe_exec(self.h, C.byref(inst), table, stream))

    def exec_many(self, insts, table, stream=None):
        arr = insts if not isinstance(insts, (list, tuple)) else abi.inst_array(insts)
        return self._ck(self.lib.plow_moe_exec_many(self.h, arr, len(arr), table, stream))

    def check(self, inst, table):
        """0 if the op would run, else the negative refusal code (no exception)."""
        return self.lib.plow_moe_check(self.h, C.byref(inst), table)

    def last_error(self):
        return self.lib.plow_moe_last_error(self.h).decode()

    def pf(self, insts, table, rows, stream=None):
        arr = abi.inst_array(insts)
        return self._ck(self.lib.plow_moe_pf(self.h, arr, len(arr), table, rows, stream), allow=(abi.ROLLBACK,))

    def dec(self, insts, table, rows, stream=None):
        arr = abi.inst_array(insts)
        return self._ck(self.lib.plow_moe_dec(self.h, arr, len(arr), table, rows, stream), allow=(abi.ROLLBACK,))

    def reserve_staging(self, token_rows, hidden):
        """Room for the fp4 x fp4 arm's quantized token rows (allocates: set-up time only)."""
        return self._ck(self.lib.plow_moe_reserve_staging(self.h, token_rows, hidden))

    def set_min_rows(self, variant, min_rows):
        return self._ck(self.lib.plow_moe_set_min_rows(self.h, variant, min_rows))
