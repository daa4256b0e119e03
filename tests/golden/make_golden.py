"""Writes the golden vectors under tests/golden/ by running plow's OWN CPU kernels, compiled from the
mounted plow tree into oracle/_ref/libplow_ref.so (scalar golden tier).

Run where the plow tree is mounted:   make -C oracle ref && python tests/golden/make_golden.py
The fixtures hold inputs and expected outputs only; tests/test_golden.py replays them through the
in-repo oracle on any machine. Reference op numbers used: 83/84/87 routing, 180 router score,
75/76 bf16 grouped experts, 150-153 flat mxfp4 experts, 65/66 per-channel fp8 decode
experts, 32 per-row activation quant, 20/8 dense GLU / GEMM, 1 RMSNorm.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import cases  # noqa: E402
import oracle_lib as ol  # noqa: E402
from plow_amd import abi  # noqa: E402


def main():
    ref = ol.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libplow_ref.so is not built (make -C oracle ref)")
    out = {}

    def run(inst, arrays, nblk=1):
        ol.run(ref.plow_ref_exec, inst, ol.table_of(arrays), nblk)

    # --- routing: 83 -> 84 ---------------------------------------------------------------------
    for name, E, k, T, flags, ties, wb in cases.ROUTE_CASES:
        logit, bias = cases.route_inputs(name, E, k, T, flags, ties, wb)
        table = np.zeros(T * k, dtype=ol.ROUTE_DT)
        run(cases.route_inst(E, k, T, flags, wb), [table, logit, None, bias], nblk=3)
        arrs = cases.align_arrays(table, T, E, k)
        run(cases.align_inst(T, E, k), arrs)
        rows = int(arrs[0][3 * E]) * abi.MPF_BM
        out[f"route/{name}/logit"] = logit
        if wb:
            out[f"route/{name}/bias"] = bias
        out[f"route/{name}/table"] = table.view(np.uint32).reshape(-1, 2)
        out[f"route/{name}/meta"] = arrs[0]
        out[f"route/{name}/row_token"] = arrs[2][:rows]
        out[f"route/{name}/row_partidx"] = arrs[3][:rows]
        out[f"route/{name}/row_gate"] = arrs[4][:rows]

    r = cases.rng_of(77)
    # --- router score 180 ------------------------------------------------------------------------
    M, N, K = 6, 40, 768
    x, w = cases.randn_bf16(r, (M, K), 1.0), cases.randn_bf16(r, (N, K), 0.02)
    o = np.zeros((M, N), np.float32)
    run(abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[M, N, K]), [o, x, w], nblk=2)
    out.update({"score/x": x, "score/w": w, "score/out": o})

    # --- combine 87 ------------------------------------------------------------------------------
    H, k, T = 160, 5, 6
    part = r.standard_normal((T * k, H)).astype(np.float32)
    res, sh = cases.randn_bf16(r, (T, H), 1.0), cases.randn_bf16(r, (T, H), 1.0)
    o = np.zeros((T, H), np.uint16)
    run(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, 2, 3], i=[H, k, T]), [o, res, sh, part], nblk=4)
    o2 = np.zeros((T, H), np.uint16)
    run(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, None, None, 3], i=[H, k, T]), [o2, None, None, part])
    out.update({"combine/part": part, "combine/res": res, "combine/shared": sh, "combine/out": o,
                "combine/out_plain": o2})

    # --- bf16 grouped experts: reference ops 75 / 76 over a fused gate_up table -------------------
    E, k, T, H, I = 6, 2, 10, 128, 96
    logit, _ = cases.route_inputs("bf16_group", E, k, T, 8, 0, False)
    table = np.zeros(T * k, dtype=ol.ROUTE_DT)
    run(cases.route_inst(E, k, T, 8, False, route_scale=1.0), [table, logit, None, None])
    al = cases.align_arrays(table, T, E, k)
    run(cases.align_inst(T, E, k), al)
    gu = [cases.randn_bf16(r, (2 * I, H), 0.05) for _ in range(E)]
    dn = [cases.randn_bf16(r, (H, I), 0.05) for _ in range(E)]
    ewt = np.array([[g.ctypes.data, d.ctypes.data] for g, d in zip(gu, dn)], dtype=np.uint64)
    x = cases.randn_bf16(r, (T, H), 1.0)
    R = al[2].shape[0]
    for act in (0, 1):
        fu = np.zeros((R, I), np.uint16)
        run(abi.inst(75, t=[0, 1, 2, 3, 4], i=[I, H, E, 0, 0, act]), [fu, x, ewt, al[0], al[2]], nblk=3)
        part = np.zeros((T * k, H), np.float32)
        run(abi.inst(76, t=[0, 1, 2, 3, 4, 5], i=[H, I, E]), [part, fu, ewt, al[0], al[3], al[4]], nblk=3)
        out[f"bf16grp/fu_act{act}"] = fu
        out[f"bf16grp/part_act{act}"] = part
    out.update({"bf16grp/logit": logit, "bf16grp/x": x, "bf16grp/gate_up": np.stack(gu),
                "bf16grp/down": np.stack(dn)})

    # --- flat mxfp4 decode experts: reference ops 150 / 151 (layout 1 = gate rows then up rows) ---
    E, k, B, K, I = 4, 2, 3, 128, 64
    Wgu = r.integers(0, 256, size=(E, 2 * I, K // 2), dtype=np.uint8)
    Sgu = r.integers(118, 130, size=(E, 2 * I, K // 32), dtype=np.uint8)
    Wd = r.integers(0, 256, size=(E, K, I // 2), dtype=np.uint8)
    Sd = r.integers(118, 130, size=(E, K, I // 32), dtype=np.uint8)
    x = cases.randn_bf16(r, (B, K), 1.0)
    tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
    tab["eid"] = [0, 3, 2, 1, 3, abi.EXPERT_UNUSED]
    tab["gate"] = r.random(B * k).astype(np.float32)
    fu = np.zeros((B * k, I), np.uint16)
    run(abi.inst(150, t=[0, 1, 2, 3, 4], i=[k, I, K, E, 1, 1, B]), [fu, x, tab, Wgu, Sgu], nblk=2)
    part = np.full((B * k, K), 9.0, np.float32)
    run(abi.inst(151, t=[0, 1, 2, 3, 4], i=[k, K, I, E, 0, 0, B]), [part, fu, tab, Wd, Sd], nblk=2)
    out.update({"mxdec/Wgu": Wgu, "mxdec/Sgu": Sgu, "mxdec/Wd": Wd, "mxdec/Sd": Sd, "mxdec/x": x,
                "mxdec/table": tab.view(np.uint32).reshape(-1, 2), "mxdec/fu": fu, "mxdec/part": part})

    # --- per-channel fp8 decode experts: reference ops 65 / 66 (gelu_tanh, fused gate_up) ---------
    E, k, B, H, I = 5, 2, 3, 128, 64
    gu8 = [cases.e4m3_bytes(r, (2 * I, H)) for _ in range(E)]
    d8 = [cases.e4m3_bytes(r, (H, I)) for _ in range(E)]
    sgu = [(r.random(2 * I) * 0.01 + 1e-3).astype(np.float32) for _ in range(E)]
    sd = [(r.random(H) * 0.01 + 1e-3).astype(np.float32) for _ in range(E)]
    ewt = np.array([[a.ctypes.data, b.ctypes.data] for a, b in zip(gu8, d8)], dtype=np.uint64)
    est = np.array([[a.ctypes.data, b.ctypes.data] for a, b in zip(sgu, sd)], dtype=np.uint64)
    ewt[4] = 0  # a non-resident expert: GLU writes nothing, DOWN writes zeros
    x = cases.randn_bf16(r, (B, H), 1.0)
    tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
    tab["eid"] = [1, 0, 4, 2, abi.EXPERT_UNUSED, 3]
    tab["gate"] = r.random(B * k).astype(np.float32)
    fu = np.zeros((B * k, I), np.uint16)
    run(abi.inst(65, t=[0, 1, 2, 3, 4], i=[k, I, H, E, 0, B]), [fu, x, tab, ewt, est], nblk=2)
    part = np.full((B * k, H), 9.0, np.float32)
    run(abi.inst(66, t=[0, 1, 2, 3, 4], i=[k, H, I, E, 0, B]), [part, fu, tab, ewt, est], nblk=2)
    out.update({"pcdec/gu8": np.stack(gu8), "pcdec/d8": np.stack(d8), "pcdec/sgu": np.stack(sgu),
                "pcdec/sd": np.stack(sd), "pcdec/x": x, "pcdec/table": tab.view(np.uint32).reshape(-1, 2),
                "pcdec/fu": fu, "pcdec/part": part})

    # --- per-row activation quant: reference op 32 ------------------------------------------------
    M, K = 7, 384
    x = cases.randn_bf16(r, (M, K), 3.0)
    x[3] = 0  # an all-zero row hits the 1e-12 scale floor
    xq, sc = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    run(abi.inst(32, t=[0, 1, 2], i=[M, K]), [xq, x.copy(), sc], nblk=2)
    out.update({"quant32/x": x, "quant32/xq": xq, "quant32/scale": sc})

    # --- dense shared expert: reference ops 20 (GLU, silu) and 8 ----------------------------------
    M, N, K = 5, 48, 128
    x = cases.randn_bf16(r, (M, K), 1.0)
    wg, wu = cases.randn_bf16(r, (N, K), 0.05), cases.randn_bf16(r, (N, K), 0.05)
    wd = cases.randn_bf16(r, (K, N), 0.05)
    fu = np.zeros((M, N), np.uint16)
    run(abi.inst(20, t=[0, 1, 2, None, None, 5], i=[M, N, K, 0, 0, 1]), [fu, x, wg, None, None, wu], nblk=2)
    y = np.zeros((M, K), np.uint16)
    run(abi.inst(8, t=[0, 1, 2], i=[M, K, N]), [y, fu, wd], nblk=2)
    out.update({"dense/x": x, "dense/wg": wg, "dense/wu": wu, "dense/wd": wd, "dense/fu": fu, "dense/y": y})

    # --- op 32 edges (drawn last so that the vectors above keep their values): widths that are not a
    # multiple of the vector width, rows with NaN / infinities, and the fused gate/up arm ----------
    for K in (1, 15, 17, 257):
        M = 3
        x = cases.randn_bf16(r, (M, K), 2.0)
        x[1] = 0x8000 * (np.arange(K) & 1)      # signed zeros only: the 1e-12 scale floor
        x[2, 0] = ol.f2bf(np.float32(448.0))
        xq, sc = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
        run(abi.inst(32, t=[0, 1, 2], i=[M, K]), [xq, x.copy(), sc], nblk=2)
        out.update({f"quant32w/{K}/x": x, f"quant32w/{K}/xq": xq, f"quant32w/{K}/scale": sc})
    M, K = 4, 40
    x = cases.randn_bf16(r, (M, K), 2.0)
    x[0, 3], x[0, 17] = 0x7FC0, 0xFFC1          # NaN of either sign among finite values
    x[1, 5] = 0x7F80                            # +inf
    x[2, 8], x[2, 9], x[2, 30] = 0xFF80, 0x7FC0, 0x7F80
    xq, sc = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    run(abi.inst(32, t=[0, 1, 2], i=[M, K]), [xq, x.copy(), sc])
    out.update({"quant32n/x": x, "quant32n/xq": xq, "quant32n/scale": sc})
    for act in (0, 1):
        for K in (17, 1024):
            M = 5
            gate, up = cases.randn_bf16(r, (M, K), 3.0), cases.randn_bf16(r, (M, K), 1.5)
            x, xq, sc = np.zeros((M, K), np.uint16), np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
            run(abi.inst(32, t=[0, 1, 2, 3, 4], i=[M, K, act]), [xq, x, sc, gate, up], nblk=2)
            out.update({f"quant32f/{act}/{K}/gate": gate, f"quant32f/{act}/{K}/up": up, f"quant32f/{act}/{K}/x": x,
                        f"quant32f/{act}/{K}/xq": xq, f"quant32f/{act}/{K}/scale": sc})

    # --- flat mxfp4 ops again (drawn last): interleaved layout with per-expert biases (150 / 151), and
    # the gathered-row twins 152 / 153 after 84, on the mxdec weights above ----------------------------
    Wgu, Sgu, Wd, Sd = out["mxdec/Wgu"], out["mxdec/Sgu"], out["mxdec/Wd"], out["mxdec/Sd"]
    E, I, K = Wgu.shape[0], Wgu.shape[1] // 2, Wgu.shape[2] * 2
    k, B = 2, 3
    x = out["mxdec/x"]
    tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
    tab["eid"], tab["gate"] = out["mxdec/table"][:, 0], out["mxdec/table"][:, 1].view(np.float32)
    bgu, bd = cases.randn_bf16(r, (E, 2 * I), 0.5), cases.randn_bf16(r, (E, K), 0.5)
    fu = np.zeros((B * k, I), np.uint16)
    run(abi.inst(150, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 0, 0, B]), [fu, x, tab, Wgu, Sgu, bgu], nblk=2)
    part = np.full((B * k, K), 9.0, np.float32)
    run(abi.inst(151, t=[0, 1, 2, 3, 4, 5], i=[k, K, I, E, 0, 0, B]), [part, fu, tab, Wd, Sd, bd], nblk=2)
    out.update({"mxflat/bias_gu": bgu, "mxflat/bias_d": bd, "mxflat/fu_l0_bias_gelu": fu, "mxflat/part_bias": part})
    al = cases.align_arrays(tab, B, E, k)
    run(cases.align_inst(B, E, k), al)
    rows = int(al[0][3 * E]) * abi.MPF_BM
    fug = np.zeros((rows, I), np.uint16)
    run(abi.inst(152, t=[0, 1, 2, 3, 4, 5], i=[I, K, E, 1, 0, 1]), [fug, x, Wgu, Sgu, al[0], al[2]], nblk=3)
    partg = np.full((B * k, K), 9.0, np.float32)
    run(abi.inst(153, t=[0, 1, 2, 3, 4, None, 6, 7], i=[K, I, E]), [partg, fug, Wd, Sd, al[0], None, al[3], al[4]], nblk=3)
    out.update({"mxflat/pf_fu": fug, "mxflat/pf_part": partg})

    # --- pair-form activations on the flat mxfp4 GLU ops (drawn after everything above): 2 situ
    # (beta, linear beta) and 3 swiglu_oai (alpha, limit) with biases, decode (150) and gathered rows (152)
    for act, f in ((2, (2.0, 1.5)), (3, (1.702, 7.0)), (2, (3.0, 0.0))):
        fu = np.zeros((B * k, I), np.uint16)
        run(abi.inst(150, t=[0, 1, 2, 3, 4, 5], i=[k, I, K, E, 1, act, B], f=f), [fu, x, tab, Wgu, Sgu, bgu], nblk=2)
        out[f"mxflat/fu_act{act}_{f[0]}_{f[1]}"] = fu
    fug = np.zeros((rows, I), np.uint16)
    run(abi.inst(152, t=[0, 1, 2, 3, 4, 5, 6], i=[I, K, E, 0, 0, 3], f=(1.702, 7.0)), [fug, x, Wgu, Sgu, al[0], al[2], bgu], nblk=3)
    out["mxflat/pf_fu_act3"] = fug

    # --- RMSNorm op 1 (its own generator, after everything above): plain with gamma and a row offset,
    # weightless, and with the per-row quantizer fused
    rn = cases.rng_of(1001)
    rows, feat = 5, 384
    xn, gam = cases.randn_bf16(rn, (rows, feat), 1.5), cases.randn_bf16(rn, (feat,), 1.0)
    o1 = np.zeros((rows + 2, feat), np.uint16)
    run(abi.inst(1, t=[0, 1, 2], i=[rows, feat, 2], f=[1e-6]), [o1, xn, gam], nblk=2)
    o2 = np.zeros((rows, feat), np.uint16)
    run(abi.inst(1, t=[0, 1], i=[rows, feat, 0], f=[1e-5]), [o2, xn], nblk=1)
    o3, q3, s3 = np.zeros((rows, feat), np.uint16), np.zeros((rows, feat), np.uint8), np.zeros(rows, np.float32)
    run(abi.inst(1, t=[0, 1, 2, 3, 4], i=[rows, feat, 0], f=[1e-6]), [o3, xn, gam, q3, s3], nblk=3)
    out.update({"rmsnorm/x": xn, "rmsnorm/gamma": gam, "rmsnorm/out_row2": o1, "rmsnorm/out_plain": o2,
                "rmsnorm/out_q": o3, "rmsnorm/xq": q3, "rmsnorm/scale": s3})

    path = os.path.join(HERE, "plow_cpu_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
