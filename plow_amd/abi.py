"""ctypes mirror of include/plow_moe.h: the 64-byte op descriptor, opcodes and enums.

The descriptor is byte-identical to plow's ``PlowDevInst`` (runtime/common/dev_isa.h:1607-1613;
Rust mirror ``DevInst64`` in crates/packet/src/dev.rs): ``u16 op, u16 blocks, PlowFJ fj[3],
u16 t[8], u32 i[8]`` with ``t`` at byte 16.
"""
import ctypes as C

TENSOR_NONE = 0xFFFF
EXPERT_UNUSED = 0xFFFFFFFF
MPF_BM = 64
ROUTE_MAX_TOPK = 16

# opcodes (runtime/common/dev_isa.h)
OP_RMSNORM = 1
OP_GEMM = 8
OP_GEMM_GLU = 20
OP_QUANT_FP8 = 32
OP_MOE_COMBINE = 43
OP_MOE_GROUP_GLU_FP8_BLK = 48
OP_MOE_GROUP_DOWN_FP8_BLK = 49
OP_MOE_ROUTER_TOPK = 56
OP_MOE_EXPERT_GLU_GEMMA_FP8 = 65
OP_MOE_EXPERT_DOWN_GEMMA_FP8 = 66
OP_MOE_GROUP_GLU_GEMMA_PF = 75
OP_MOE_GROUP_DOWN_GEMMA_PF = 76
OP_MOE_GROUP_GLU_GEMMA_PF_W8A8 = 81
OP_MOE_GROUP_DOWN_GEMMA_PF_W8A8 = 82
OP_MOE_ROUTER_TOPK_PF = 83
OP_MOE_ALIGN_PF = 84
OP_MOE_GROUP_GLU_PF = 85
OP_MOE_GROUP_DOWN_PF = 86
OP_MOE_COMBINE_PF = 87
OP_MOE_GLU_MX = 150
OP_MOE_DOWN_MX = 151
OP_MOE_GLU_MX_PF = 152
OP_MOE_DOWN_MX_PF = 153
OP_GEMM_F32 = 180
OP_QUANT_FP8_BLOCK128 = 184
OP_MOE_GLU_FP8_BLOCK128 = 188
OP_MOE_QUANT_FP8_BLOCK128 = 189
OP_MOE_DOWN_FP8_BLOCK128 = 190

ENC_BF16, ENC_FP8BLK, ENC_MXFP4 = 0, 1, 2
ARM_A16, ARM_W8A8, ARM_W8A8_P16, ARM_W8A8_SPLIT, ARM_W8A8_SPLIT_P16, ARM_W8A8_XQ, ARM_W4A16 = 0, 2, 3, 4, 5, 6, 8
ARM_A4W4, ARM_A4W4_P16 = 0, 1     # enc 2: fp4 on both operands (the reference's default for mxfp4); DOWN with a bf16 part
ROUTER_RAW_MARK = 0x52545241       # op 180 i7: the score carries its top-k (one launch)
ACT_GELU_TANH, ACT_SILU = 0, 1
ROUTE_SIGMOID, ROUTE_NORM_TOPK, ROUTE_BIAS, ROUTE_F32_LOGIT, ROUTE_HASH, ROUTE_SQRT_SOFTPLUS = 1, 2, 4, 8, 16, 32

E_OK, E_INVAL, E_UNSUPPORTED, E_DEVICE, E_NOMEM, ROLLBACK = 0, -22, -95, -5, -12, 1


class PlowFJ(C.Union):
    _fields_ = [("f", C.c_float), ("u", C.c_uint32)]


class PlowDevInst(C.Structure):
    _fields_ = [
        ("op", C.c_uint16),
        ("blocks", C.c_uint16),
        ("fj", PlowFJ * 3),
        ("t", C.c_uint16 * 8),
        ("i", C.c_uint32 * 8),
    ]


assert C.sizeof(PlowDevInst) == 64 and PlowDevInst.t.offset == 16


class PlowMoeRoute(C.Structure):
    _fields_ = [("eid", C.c_uint32), ("gate", C.c_float)]


def max_rows(T, k, n_exp):
    """Capacity of the gathered arrays (runtime/amd/op_moe.h:2252-2255)."""
    return T * k + n_exp * (MPF_BM - 1)


def inst(op, t=(), i=(), f=(), blocks=1, slots=0):
    """Build one descriptor. ``t``: up to 8 handles (None = absent); ``i``: up to 8 ints;
    ``f``: up to 3 floats placed in fj[n].f; ``slots``: the routed slots (T * k) of the batch in
    fj[2].u, this library's row-count statement on the grouped expert ops (0 = not stated)."""
    d = PlowDevInst()
    d.op, d.blocks = op, blocks
    for n in range(8):
        h = t[n] if n < len(t) else None
        d.t[n] = TENSOR_NONE if h is None else int(h)
    for n, v in enumerate(i):
        d.i[n] = int(v) & 0xFFFFFFFF
    for n, v in enumerate(f):
        d.fj[n].f = float(v)
    if slots:
        d.fj[2].u = int(slots)
    return d


def inst_array(insts):
    arr = (PlowDevInst * len(insts))()
    for n, d in enumerate(insts):
        C.memmove(C.byref(arr, n * 64), C.byref(d), 64)
    return arr
