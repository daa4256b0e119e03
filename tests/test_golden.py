"""The in-repo oracle replayed against golden vectors written by plow's own CPU kernels
(tests/golden/make_golden.py, scalar golden tier). Bit-exact everywhere: tables, meta, row maps,
f32 logits / partials and bf16 outputs."""
import os

import numpy as np
import pytest

import cases
import oracle_lib as ol
from plow_amd import abi

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "plow_cpu_golden.npz"))


def run(oracle, inst, arrays, nthreads=1):
    ol.run(oracle.plow_oracle_exec, inst, ol.table_of(arrays), nthreads)


def as_route(a):
    return np.ascontiguousarray(a).view(ol.ROUTE_DT).reshape(-1)


@pytest.mark.parametrize("case", cases.ROUTE_CASES, ids=[c[0] for c in cases.ROUTE_CASES])
@pytest.mark.parametrize("nthreads", [1, 3])
def test_route_and_align(oracle, case, nthreads):
    name, E, k, T, flags, ties, wb = case
    logit = G[f"route/{name}/logit"]
    bias = G[f"route/{name}/bias"] if wb else None
    table = np.zeros(T * k, dtype=ol.ROUTE_DT)
    run(oracle, cases.route_inst(E, k, T, flags, wb), [table, logit, None, bias], nthreads)
    assert np.array_equal(table.view(np.uint32).reshape(-1, 2), G[f"route/{name}/table"])
    arrs = cases.align_arrays(table, T, E, k)
    run(oracle, cases.align_inst(T, E, k), arrs, nthreads)
    assert np.array_equal(arrs[0], G[f"route/{name}/meta"])
    rows = int(arrs[0][3 * E]) * abi.MPF_BM
    assert np.array_equal(arrs[2][:rows], G[f"route/{name}/row_token"])
    assert np.array_equal(arrs[3][:rows], G[f"route/{name}/row_partidx"])
    assert np.array_equal(arrs[4][:rows].view(np.uint32), G[f"route/{name}/row_gate"].view(np.uint32))
    assert np.all(arrs[2][rows:] == 7)  # nothing written past the padded extent


def test_router_score(oracle):
    x, w, want = G["score/x"], G["score/w"], G["score/out"]
    M, K = x.shape
    N = w.shape[0]
    for nt in (1, 4):
        o = np.zeros((M, N), np.float32)
        run(oracle, abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[M, N, K]), [o, x, w], nt)
        assert np.array_equal(o.view(np.uint32), want.view(np.uint32))


def test_combine(oracle):
    part, res, sh = G["combine/part"], G["combine/res"], G["combine/shared"]
    T, H = res.shape
    k = part.shape[0] // T
    o = np.zeros((T, H), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, 2, 3], i=[H, k, T]), [o, res, sh, part], 3)
    assert np.array_equal(o, G["combine/out"])
    o = np.zeros((T, H), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, None, None, 3], i=[H, k, T]), [o, None, None, part])
    assert np.array_equal(o, G["combine/out_plain"])
    # the decode op 43 is the same expression at T = 1
    o1 = np.zeros((1, H), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_COMBINE, t=[0, 1, 2, 3], i=[H, k]), [o1, res[:1], sh[:1], part[:k]])
    assert np.array_equal(o1[0], G["combine/out"][0])


@pytest.mark.parametrize("act", [0, 1])
def test_bf16_grouped_experts(oracle, act):
    """Reference ops 75/76 (fused gate_up table) == ops 85/86 at enc 0 over a {gate, up, down} table."""
    logit, x = G["bf16grp/logit"], G["bf16grp/x"]
    gu, dn = np.ascontiguousarray(G["bf16grp/gate_up"]), np.ascontiguousarray(G["bf16grp/down"])
    E, I2, H = gu.shape
    I, T, k = I2 // 2, x.shape[0], 2
    table = np.zeros(T * k, dtype=ol.ROUTE_DT)
    run(oracle, cases.route_inst(E, k, T, 8, False, route_scale=1.0), [table, logit, None, None])
    al = cases.align_arrays(table, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    wtab = np.array([[gu[e].ctypes.data, gu[e].ctypes.data + I * H * 2, dn[e].ctypes.data]
                     for e in range(E)], dtype=np.uint64)
    R = al[2].shape[0]
    fu = np.zeros((R, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, None, 4, 5], i=[I, H, E, 0, 0, act, 0, 0]),
        [fu, x, wtab, None, al[0], al[2]], 3)
    assert np.array_equal(fu, G[f"bf16grp/fu_act{act}"])
    part = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, None, 4, None, 6, 7], i=[H, I, E, 0]),
        [part, fu, wtab, None, al[0], None, al[3], al[4]], 3)
    assert np.array_equal(part.view(np.uint32), G[f"bf16grp/part_act{act}"].view(np.uint32))


@pytest.mark.parametrize("act", [0, 1])
def test_bf16_grouped_experts_fused_table(oracle, act):
    """Reference ops 75 / 76 under their own numbers, over the fused table ewt[E][2]."""
    logit, x = G["bf16grp/logit"], G["bf16grp/x"]
    gu, dn = np.ascontiguousarray(G["bf16grp/gate_up"]), np.ascontiguousarray(G["bf16grp/down"])
    E, I2, H = gu.shape
    I, T, k = I2 // 2, x.shape[0], 2
    table = np.zeros(T * k, dtype=ol.ROUTE_DT)
    run(oracle, cases.route_inst(E, k, T, 8, False, route_scale=1.0), [table, logit, None, None])
    al = cases.align_arrays(table, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    ewt = np.array([[gu[e].ctypes.data, dn[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    fu = np.zeros((al[2].shape[0], I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_GEMMA_PF, t=[0, 1, 2, 3, 4], i=[I, H, E, 0, 0, act]), [fu, x, ewt, al[0], al[2]], 3)
    assert np.array_equal(fu, G[f"bf16grp/fu_act{act}"])
    part = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_GEMMA_PF, t=[0, 1, 2, 3, 4, 5], i=[H, I, E]), [part, fu, ewt, al[0], al[3], al[4]], 3)
    assert np.array_equal(part.view(np.uint32), G[f"bf16grp/part_act{act}"].view(np.uint32))


def test_mxfp4_decode_experts(oracle):
    """Reference flat ops 150/151 == ops 48/49 at enc 2 over per-expert pointers into the flat tensor."""
    Wgu, Sgu = np.ascontiguousarray(G["mxdec/Wgu"]), np.ascontiguousarray(G["mxdec/Sgu"])
    Wd, Sd = np.ascontiguousarray(G["mxdec/Wd"]), np.ascontiguousarray(G["mxdec/Sd"])
    x, tab = G["mxdec/x"], as_route(G["mxdec/table"])
    E, I2, K2 = Wgu.shape
    I, K, B, k = I2 // 2, K2 * 2, x.shape[0], 2
    wtab = np.array([[Wgu[e].ctypes.data, Wgu[e].ctypes.data + I * (K // 2), Wd[e].ctypes.data]
                     for e in range(E)], dtype=np.uint64)
    stab = np.array([[Sgu[e].ctypes.data, Sgu[e].ctypes.data + I * (K // 32), Sd[e].ctypes.data]
                     for e in range(E)], dtype=np.uint64)
    fu = np.zeros((B * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[0, 1, 2, 3, 4], i=[B * k, I, K, E, k, 1, 2]),
        [fu, x, tab, wtab, stab], 2)
    assert np.array_equal(fu, G["mxdec/fu"])
    part = np.full((B * k, K), 9.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_FP8_BLK, t=[0, 1, 2, 3, 4], i=[B * k, K, I, E, 0, 0, 2]),
        [part, fu, tab, wtab, stab], 2)
    assert np.array_equal(part.view(np.uint32), G["mxdec/part"].view(np.uint32))


def test_flat_mxfp4_ops(oracle):
    """Reference ops 150 - 153 under their own numbers: blocked and interleaved gate / up rows, per-expert
    biases, and the gathered-row twins after op 84."""
    Wgu, Sgu = np.ascontiguousarray(G["mxdec/Wgu"]), np.ascontiguousarray(G["mxdec/Sgu"])
    Wd, Sd = np.ascontiguousarray(G["mxdec/Wd"]), np.ascontiguousarray(G["mxdec/Sd"])
    x, tab = G["mxdec/x"], as_route(G["mxdec/table"])
    E, I2, K2 = Wgu.shape
    I, K, B, k = I2 // 2, K2 * 2, x.shape[0], 2
    fu = np.zeros((B * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[k, I, K, E, 1, 1, B]), [fu, x, tab, Wgu, Sgu], 2)
    assert np.array_equal(fu, G["mxdec/fu"])
    part = np.full((B * k, K), 9.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_DOWN_MX, t=[0, 1, 2, 3, 4], i=[k, K, I, E, 0, 0, B]), [part, fu, tab, Wd, Sd], 2)
    assert np.array_equal(part.view(np.uint32), G["mxdec/part"].view(np.uint32))
    bgu, bd = G["mxflat/bias_gu"], G["mxflat/bias_d"]
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 0, 0, B]), [fu, x, tab, Wgu, Sgu, bgu], 3)
    assert np.array_equal(fu, G["mxflat/fu_l0_bias_gelu"])
    part[:] = 9.0
    run(oracle, abi.inst(abi.OP_MOE_DOWN_MX, t=[0, 1, 2, 3, 4, 5], i=[k, K, I, E, 0, 0, B]), [part, fu, tab, Wd, Sd, bd], 3)
    assert np.array_equal(part.view(np.uint32), G["mxflat/part_bias"].view(np.uint32))
    al = cases.align_arrays(tab, B, E, k)
    run(oracle, cases.align_inst(B, E, k), al, 1)
    fug = np.zeros_like(G["mxflat/pf_fu"])
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX_PF, t=[0, 1, 2, 3, 4, 5], i=[I, K, E, 1, 0, 1]), [fug, x, Wgu, Sgu, al[0], al[2]], 3)
    assert np.array_equal(fug, G["mxflat/pf_fu"])
    partg = np.full((B * k, K), 9.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_DOWN_MX_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[K, I, E]),
        [partg, fug, Wd, Sd, al[0], None, al[3], al[4]], 3)
    assert np.array_equal(partg.view(np.uint32), G["mxflat/pf_part"].view(np.uint32))


def test_flat_mxfp4_pair_activations(oracle):
    """Activations that transform the up branch too (2 situ, 3 swiglu_oai) with their immediates in
    fj[0] / fj[1], against plow's CPU kernels on ops 150 and 152; a clamp activation (4, plow's AMD path
    only) against the silu path it reduces to."""
    Wgu, Sgu = np.ascontiguousarray(G["mxdec/Wgu"]), np.ascontiguousarray(G["mxdec/Sgu"])
    x, tab, bgu = G["mxdec/x"], as_route(G["mxdec/table"]), G["mxflat/bias_gu"]
    E, I2, K2 = Wgu.shape
    I, K, B, k = I2 // 2, K2 * 2, x.shape[0], 2
    for act, f in ((2, (2.0, 1.5)), (3, (1.702, 7.0)), (2, (3.0, 0.0))):
        fu = np.zeros((B * k, I), np.uint16)
        run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 1, act, B], f=f),
            [fu, x, tab, Wgu, Sgu, bgu], 2)
        assert np.array_equal(fu, G[f"mxflat/fu_act{act}_{f[0]}_{f[1]}"]), (act, f)
    al = cases.align_arrays(tab, B, E, k)
    run(oracle, cases.align_inst(B, E, k), al, 1)
    fug = np.zeros_like(G["mxflat/pf_fu_act3"])
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX_PF, t=[0, 1, 2, 3, 4, 5, 6], i=[I, K, E, 0, 0, 3], f=(1.702, 7.0)),
        [fug, x, Wgu, Sgu, al[0], al[2], bgu], 3)
    assert np.array_equal(fug, G["mxflat/pf_fu_act3"])
    # swiglu_oai with a limit <= 0 poisons
    fu = np.zeros((B * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 1, 3, B], f=(1.702, 0.0)),
        [fu, x, tab, Wgu, Sgu, bgu], 2)
    live = as_route(G["mxdec/table"])["eid"] < E
    assert np.all((fu[live] & 0x7FFF) > 0x7F80)
    # the clamp activation with a limit beyond every value is silu(g) * u
    fa, fb = np.zeros((B * k, I), np.uint16), np.zeros((B * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 1, 4, B], f=(0.0, 1e30)),
        [fa, x, tab, Wgu, Sgu, bgu], 2)
    run(oracle, abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 1, 1, B]), [fb, x, tab, Wgu, Sgu, bgu], 2)
    assert np.array_equal(fa, fb)


def test_per_channel_fp8_decode_experts(oracle):
    gu8, d8 = np.ascontiguousarray(G["pcdec/gu8"]), np.ascontiguousarray(G["pcdec/d8"])
    sgu, sd = np.ascontiguousarray(G["pcdec/sgu"]), np.ascontiguousarray(G["pcdec/sd"])
    x, tab = G["pcdec/x"], as_route(G["pcdec/table"])
    E, I2, H = gu8.shape
    I, B, k = I2 // 2, x.shape[0], 2
    ewt = np.array([[gu8[e].ctypes.data, d8[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    est = np.array([[sgu[e].ctypes.data, sd[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    ewt[4] = 0
    fu = np.zeros((B * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_EXPERT_GLU_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[k, I, H, E, 0, B, 0]),
        [fu, x, tab, ewt, est], 2)
    assert np.array_equal(fu, G["pcdec/fu"])
    part = np.full((B * k, H), 9.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_EXPERT_DOWN_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[k, H, I, E, 0, B]),
        [part, fu, tab, ewt, est], 2)
    assert np.array_equal(part.view(np.uint32), G["pcdec/part"].view(np.uint32))


def test_per_row_quant(oracle):
    x = G["quant32/x"]
    M, K = x.shape
    xq, sc = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[M, K]), [xq, x, sc], 2)
    assert np.array_equal(xq, G["quant32/xq"])
    assert np.array_equal(sc.view(np.uint32), G["quant32/scale"].view(np.uint32))


@pytest.mark.parametrize("key", ["quant32w/1", "quant32w/15", "quant32w/17", "quant32w/257", "quant32n"])
def test_per_row_quant_edges(oracle, key):
    """Widths off the vector width, signed-zero rows, and rows with NaN / infinities."""
    x = G[key + "/x"].copy()
    M, K = x.shape
    xq, sc = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[M, K]), [xq, x, sc], 3)
    assert np.array_equal(xq, G[key + "/xq"])
    assert np.array_equal(sc.view(np.uint32), G[key + "/scale"].view(np.uint32))


@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("K", [17, 1024])
def test_per_row_quant_fused_gate_up(oracle, act, K):
    """Reference op 32 with gate / up bound: x = bf16(act(gate) * up) is produced, then quantized."""
    key = f"quant32f/{act}/{K}"
    gate, up = G[key + "/gate"], G[key + "/up"]
    M = gate.shape[0]
    x, xq, sc = np.zeros((M, K), np.uint16), np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2, 3, 4], i=[M, K, act]), [xq, x, sc, gate, up], 2)
    assert np.array_equal(x, G[key + "/x"])
    assert np.array_equal(xq, G[key + "/xq"])
    assert np.array_equal(sc.view(np.uint32), G[key + "/scale"].view(np.uint32))


def test_dense_shared_expert(oracle):
    x, wg, wu, wd = G["dense/x"], G["dense/wg"], G["dense/wu"], G["dense/wd"]
    M, K = x.shape
    N = wg.shape[0]
    fu = np.zeros((M, N), np.uint16)
    run(oracle, abi.inst(abi.OP_GEMM_GLU, t=[0, 1, 2, None, None, 5], i=[M, N, K, 0, 0, 1]),
        [fu, x, wg, None, None, wu], 2)
    assert np.array_equal(fu, G["dense/fu"])
    y = np.zeros((M, K), np.uint16)
    run(oracle, abi.inst(abi.OP_GEMM, t=[0, 1, 2], i=[M, K, N]), [y, fu, wd], 2)
    assert np.array_equal(y, G["dense/y"])


def test_rmsnorm_and_its_per_row_quantizer(oracle):
    """Op 1 against plow's CPU kernel (runtime/cpu/dev/golden/norm.c:15-43): gamma with an output row
    offset, weightless, and with the per-row quantizer of the rounded row."""
    x, gam = G["rmsnorm/x"], G["rmsnorm/gamma"]
    rows, feat = x.shape
    o1 = np.zeros((rows + 2, feat), np.uint16)
    run(oracle, abi.inst(abi.OP_RMSNORM, t=[0, 1, 2], i=[rows, feat, 2], f=[1e-6]), [o1, x, gam], 2)
    assert np.array_equal(o1, G["rmsnorm/out_row2"]) and not o1[:2].any()
    o2 = np.zeros((rows, feat), np.uint16)
    run(oracle, abi.inst(abi.OP_RMSNORM, t=[0, 1], i=[rows, feat, 0], f=[1e-5]), [o2, x], 1)
    assert np.array_equal(o2, G["rmsnorm/out_plain"])
    o3, q3, s3 = np.zeros((rows, feat), np.uint16), np.zeros((rows, feat), np.uint8), np.zeros(rows, np.float32)
    run(oracle, abi.inst(abi.OP_RMSNORM, t=[0, 1, 2, 3, 4], i=[rows, feat, 0], f=[1e-6]), [o3, x, gam, q3, s3], 3)
    assert np.array_equal(o3, G["rmsnorm/out_q"]) and np.array_equal(q3, G["rmsnorm/xq"])
    assert np.array_equal(s3.view(np.uint32), G["rmsnorm/scale"].view(np.uint32))
    # the 1x128 form (AMD only): by definition the 1x128 quantizer op over the rounded row
    o4, q4, s4 = np.zeros((rows, feat), np.uint16), np.zeros((rows, feat), np.uint8), np.zeros((feat // 128, rows), np.float32)
    run(oracle, abi.inst(abi.OP_RMSNORM, t=[0, 1, 2, 3, 4], i=[rows, feat, 0, 0, 128], f=[1e-6]), [o4, x, gam, q4, s4], 2)
    q5, s5 = np.zeros((rows, feat), np.uint8), np.zeros((feat // 128, rows), np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[rows, feat]), [q5, o4, s5], 1)
    assert np.array_equal(o4, o3) and np.array_equal(q4, q5) and np.array_equal(s4.view(np.uint32), s5.view(np.uint32))
