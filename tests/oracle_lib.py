"""ctypes access to the CPU oracle (oracle/liboracle.so) and, where it was built, to plow's own CPU
kernel library (oracle/_ref/libplow_ref.so). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

from plow_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")


def load_oracle():
    so = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
    lib = C.CDLL(so)
    lib.plow_oracle_exec.argtypes = [C.POINTER(abi.PlowDevInst), C.POINTER(C.c_void_p), C.c_uint32]
    lib.plow_oracle_exec.restype = C.c_int
    lib.plow_oracle_exec_many.argtypes = [C.POINTER(abi.PlowDevInst), C.c_uint32,
                                          C.POINTER(C.c_void_p), C.c_uint32]
    lib.plow_oracle_exec_many.restype = C.c_int
    lib.plow_oracle_pin_workers.argtypes = [C.c_int]
    lib.plow_oracle_pin_workers.restype = None
    lib.plow_oracle_f2bf.argtypes = [C.c_float]
    lib.plow_oracle_f2bf.restype = C.c_uint16
    lib.plow_oracle_bf2f.argtypes = [C.c_uint16]
    lib.plow_oracle_bf2f.restype = C.c_float
    lib.plow_oracle_f32_to_e4m3.argtypes = [C.c_float]
    lib.plow_oracle_f32_to_e4m3.restype = C.c_uint8
    lib.plow_oracle_e4m3_to_f32.argtypes = [C.c_uint8]
    lib.plow_oracle_e4m3_to_f32.restype = C.c_float
    lib.plow_oracle_e2m1.argtypes = [C.c_uint8]
    lib.plow_oracle_e2m1.restype = C.c_float
    lib.plow_oracle_e8m0.argtypes = [C.c_uint8]
    lib.plow_oracle_e8m0.restype = C.c_float
    lib.plow_oracle_f2bf_n.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    lib.plow_oracle_e4m3_encode_n.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    lib.plow_oracle_split_e4m3_n.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.plow_oracle_mx_act_quant.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.plow_oracle_mx_act_e8m0.argtypes = [C.c_float]
    lib.plow_oracle_mx_act_e8m0.restype = C.c_uint8
    lib.plow_oracle_mx_act_fp4.argtypes = [C.c_float]
    lib.plow_oracle_mx_act_fp4.restype = C.c_uint8
    return lib


def load_ref():
    so = os.path.join(ORACLE_DIR, "_ref", "libplow_ref.so")
    if not os.path.exists(so):
        return None
    lib = C.CDLL(so)
    lib.plow_ref_init.argtypes = [C.c_int]
    lib.plow_ref_init.restype = C.c_int
    lib.plow_ref_exec.argtypes = [C.POINTER(abi.PlowDevInst), C.POINTER(C.c_void_p), C.c_uint32]
    lib.plow_ref_exec.restype = C.c_int
    lib.plow_ref_has.argtypes = [C.c_uint16]
    lib.plow_ref_has.restype = C.c_int
    lib.plow_ref_init(0)  # scalar golden tier: the bit-level reference
    return lib


def table_of(arrays):
    """void*[] over numpy arrays (None = NULL). Keeps nothing alive: hold the arrays yourself."""
    t = (C.c_void_p * len(arrays))()
    for n, a in enumerate(arrays):
        t[n] = None if a is None else a.ctypes.data
    return t


def run(lib_fn, inst, tensors, *extra):
    rc = lib_fn(C.byref(inst), tensors, *extra)
    assert rc == 0, f"op {inst.op} failed rc={rc}"


def f2bf(a):
    """float32 array -> bf16 bits (uint16), round to nearest even; NaN keeps a payload bit."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7F800000) == 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    t = ((u >> 16) | np.where(u & 0xFFFF, 0x40, 0)).astype(np.uint16)
    return np.where(nan, t, r)


def bf2f(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


ROUTE_DT = np.dtype([("eid", np.uint32), ("gate", np.float32)])
