"""Small deterministic cases shared by the golden-vector writer and the tests.

Each builder returns (inst, arrays, outs): the descriptor in THIS library's op numbering, the list of
numpy arrays behind the handle table (index = handle) and the handles of the outputs.
"""
import numpy as np

import oracle_lib as ol
from plow_amd import abi


def rng_of(seed):
    return np.random.default_rng(seed)


ROUTE_CASES = [
    # name, E, k, T, flags, ties (0 none, 1 integer-snapped logits, 2 all equal), bias
    ("dsv3_sigmoid_bias_f32", 256, 8, 64, 1 | 2 | 4 | 8, 0, True),
    ("c1_softmax_f32", 64, 6, 16, 8, 0, False),
    ("qwen_softmax_norm_f32", 128, 8, 33, 2 | 8, 0, False),
    ("ragged_sigmoid_bf16", 33, 4, 7, 1 | 2, 0, False),
    ("gptoss_softmax_bf16", 32, 4, 5, 0, 0, False),
    ("ties_snapped", 64, 8, 12, 1 | 2 | 8, 1, False),
    ("ties_all_equal", 48, 6, 3, 8, 2, False),
    ("k_over_16", 64, 20, 4, 1 | 8, 0, False),
    ("kimi_384", 384, 8, 9, 1 | 2 | 4 | 8, 0, True),
]


def route_inputs(name, E, k, T, flags, ties, with_bias, seed=1234):
    r = rng_of(seed + sum(map(ord, name)))
    lg = (r.standard_normal((T, E)) * 2.0).astype(np.float32)
    if ties == 1:
        lg = np.trunc(lg).astype(np.float32)
    if ties == 2:
        lg[:] = 0.5
    logit = lg if flags & 8 else ol.f2bf(lg)
    bias = (r.standard_normal(E) * 0.05).astype(np.float32) if with_bias else None
    return logit, bias


def route_inst(E, k, T, flags, with_bias, route_scale=2.5, n_group=0, topk_group=0, tail=0,
               logit_scale=0.0):
    return abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1, None, 3 if with_bias else None],
                    i=[0, E, k, flags, T, tail, n_group, topk_group], f=[route_scale, logit_scale])


def align_inst(T, E, k):
    return abi.inst(abi.OP_MOE_ALIGN_PF, t=[0, 1, 2, 3, 4], i=[T, E, k])


def align_arrays(table, T, E, k):
    R = abi.max_rows(T, k, E)
    return [np.zeros(3 * E + 1, np.int32), table, np.full(R, 7, np.uint32), np.full(R, 7, np.uint32),
            np.full(R, 7.0, np.float32)]


def randn_bf16(r, shape, std):
    return ol.f2bf((r.standard_normal(shape) * std).astype(np.float32))


def e4m3_bytes(r, shape):
    """Random e4m3 payload bytes without the two NaN codes."""
    b = r.integers(0, 256, size=shape, dtype=np.uint8)
    b[(b & 0x7F) == 0x7F] = 0x3A
    return b
