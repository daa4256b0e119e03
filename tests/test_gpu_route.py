"""Routing on the GPU (ops 180, 83, 84, 87, 184, 32) against golden vectors from plow's CPU kernels
and against the oracle: everything bit-exact."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from gpu_harness import dev_table, from_dev, to_dev
from plow_amd import abi

pytestmark = pytest.mark.gpu

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "plow_cpu_golden.npz"))


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def gpu_route(moe, logit, bias, E, k, T, flags, **kw):
    tail = kw.get("tail", 0)
    table = torch.zeros((T * (k + tail), 2), dtype=torch.int32, device="cuda")
    arrs = [table, to_dev(logit), None, to_dev(bias)]
    moe.exec(cases.route_inst(E, k, T, flags, bias is not None, **kw), dev_table(arrs))
    torch.cuda.synchronize()
    return from_dev(table, ol.ROUTE_DT)


def gpu_align(moe, table, T, E, k):
    R = abi.max_rows(T, k, E)
    arrs = [torch.zeros(3 * E + 1, dtype=torch.int32, device="cuda"), to_dev(table),
            torch.full((R,), 7, dtype=torch.int32, device="cuda"),
            torch.full((R,), 7, dtype=torch.int32, device="cuda"),
            torch.full((R,), 7.0, dtype=torch.float32, device="cuda")]
    moe.exec(cases.align_inst(T, E, k), dev_table(arrs))
    torch.cuda.synchronize()
    return (arrs[0].cpu().numpy(), arrs[2].cpu().numpy().view(np.uint32),
            arrs[3].cpu().numpy().view(np.uint32), arrs[4].cpu().numpy())


@pytest.mark.parametrize("case", cases.ROUTE_CASES, ids=[c[0] for c in cases.ROUTE_CASES])
def test_route_and_align_match_plow_cpu_golden(moe, case):
    name, E, k, T, flags, ties, wb = case
    print(f"[case] route {name}", flush=True)
    logit = G[f"route/{name}/logit"]
    bias = G[f"route/{name}/bias"] if wb else None
    if flags & 4 and not wb:
        flags &= ~4
    table = gpu_route(moe, logit, bias, E, k, T, flags)
    assert np.array_equal(table.view(np.uint32).reshape(-1, 2), G[f"route/{name}/table"])
    meta, rt, rp, rg = gpu_align(moe, table, T, E, k)
    assert np.array_equal(meta, G[f"route/{name}/meta"])
    rows = int(meta[3 * E]) * abi.MPF_BM
    assert np.array_equal(rt[:rows], G[f"route/{name}/row_token"])
    assert np.array_equal(rp[:rows], G[f"route/{name}/row_partidx"])
    assert np.array_equal(rg[:rows].view(np.uint32), G[f"route/{name}/row_gate"].view(np.uint32))
    assert np.all(rt[rows:] == 7)


@pytest.mark.parametrize("E,k,T,flags,ng,tg,tail", [
    (256, 8, 4096, 1 | 2 | 4 | 8, 8, 4, 1),      # DeepSeek-V3 prefill routing
    (256, 8, 64, 1 | 2 | 4 | 8, 8, 4, 1),
    (384, 8, 128, 1 | 2 | 4 | 8, 0, 0, 1),       # Kimi-K2
    (128, 8, 2048, 2 | 8, 0, 0, 0),              # Qwen3, softmax + renorm
    (64, 6, 16, 8, 0, 0, 0),
    (1000, 16, 5, 1 | 8, 20, 7, 0),
    (96, 20, 3, 8, 0, 0, 1),                     # k above 16: sentinel slots
    (256, 6, 700, 32 | 2 | 4 | 8, 0, 0, 1),      # sqrt-softplus scores (DeepSeek-V4 routing), bias + renorm
    (384, 8, 33, 32 | 1 | 8, 8, 3, 0),           # the same with bit 0 also set (sqrt-softplus wins) and groups
])
def test_route_and_align_match_oracle(moe, oracle, E, k, T, flags, ng, tg, tail):
    print(f"[case] route-oracle E={E} k={k} T={T} flags={flags} groups={ng}/{tg}", flush=True)
    r = cases.rng_of(E * 7 + T)
    logit = (r.standard_normal((T, E)) * 1.5).astype(np.float32)
    if T >= 64:  # engineered near-ties: duplicate a few logits inside rows
        logit[::3, 5] = logit[::3, 9]
        logit[::5, E - 1] = logit[::5, 0]
    bias = (r.standard_normal(E) * 0.05).astype(np.float32) if flags & 4 else None
    kw = dict(n_group=ng, topk_group=tg, tail=tail, route_scale=2.5)
    got = gpu_route(moe, logit, bias, E, k, T, flags, **kw)
    want = np.zeros(T * (k + tail), dtype=ol.ROUTE_DT)
    ol.run(oracle.plow_oracle_exec, cases.route_inst(E, k, T, flags, bias is not None, **kw),
           ol.table_of([want, logit, None, bias]), 8)
    assert np.array_equal(got["eid"], want["eid"])
    assert np.array_equal(got["gate"].view(np.uint32), want["gate"].view(np.uint32))
    ka, Ea = k + tail, E + tail
    dev = gpu_align(moe, got, T, Ea, ka)
    al = cases.align_arrays(want, T, Ea, ka)
    ol.run(oracle.plow_oracle_exec, cases.align_inst(T, Ea, ka), ol.table_of(al), 1)
    rows = int(al[0][3 * Ea]) * abi.MPF_BM
    assert np.array_equal(dev[0], al[0])
    assert np.array_equal(dev[1][:rows], al[2][:rows]) and np.array_equal(dev[2][:rows], al[3][:rows])
    assert np.array_equal(dev[3][:rows].view(np.uint32), al[4][:rows].view(np.uint32))


@pytest.mark.parametrize("T,E,k", [(32768, 257, 9), (50000, 64, 8), (2049, 1056, 1), (116508, 9, 9)])
def test_align_of_long_tables(moe, oracle, T, E, k):
    """The align alone on tables of 2^18 slots and more (the multi-workgroup form with hundreds of slot chunks),
    with a skewed expert popularity, unused slots and one expert that nobody picks."""
    print(f"[case] align-long T={T} E={E} k={k}", flush=True)
    r = cases.rng_of(T + E)
    table = np.zeros(T * k, dtype=ol.ROUTE_DT)
    pop = 1.0 / (1.0 + np.arange(E)) ** 0.7
    pop[E // 2] = 0.0
    table["eid"] = r.choice(E, size=T * k, p=pop / pop.sum()).astype(np.uint32)
    table["eid"][r.integers(0, T * k, size=T * k // 50)] = 0xFFFFFFFF
    table["gate"] = r.random(T * k, dtype=np.float32)
    dev = gpu_align(moe, table, T, E, k)
    al = cases.align_arrays(table, T, E, k)
    ol.run(oracle.plow_oracle_exec, cases.align_inst(T, E, k), ol.table_of(al), 1)
    rows = int(al[0][3 * E]) * abi.MPF_BM
    assert np.array_equal(dev[0], al[0])
    assert np.array_equal(dev[1][:rows], al[2][:rows]) and np.array_equal(dev[2][:rows], al[3][:rows])
    assert np.array_equal(dev[3][:rows].view(np.uint32), al[4][:rows].view(np.uint32))
    assert np.all(dev[1][rows:] == 7)


@pytest.mark.parametrize("flags", [1 | 8, 1 | 2 | 8, 2 | 8, 8, 32 | 8, 32 | 2 | 8],
                         ids=["sigmoid", "sigmoid-renorm", "softmax-renorm", "softmax", "sqrtsoftplus", "sqrtsoftplus-renorm"])
def test_route_on_logits_at_the_ends_of_the_exponential(moe, oracle, flags):
    """Logits that drive the score transform's exponential through its special inputs: overflow and underflow
    thresholds (88.72, -103.97) and their neighbours, the |x| >= 88 test, infinities (sigmoid only: a softmax
    row with +inf has no defined scores), zeros of both signs, denormals. The oracle calls the C library."""
    print(f"[case] route-extreme flags={flags}", flush=True)
    E, k, T = 160, 8, 96
    r = cases.rng_of(flags + 77)
    edge = np.array([88.0, 88.5, 88.72, 88.7228, 88.73, 89.0, 100.0, 103.9, 103.97, 103.9721, 104.0, 126.0, 150.0,
                     87.9999, 1e-45, 1e-38, 1e-20, 0.0, 3e38], np.float32)
    for v in list(edge[:13]):
        edge = np.append(edge, [np.nextafter(v, np.float32(0)), np.nextafter(v, np.float32(1e9))])
    edge = np.concatenate([edge, -edge]).astype(np.float32)
    sigmoid = bool(flags & (1 | 32))                     # the per-expert transforms (sqrt-softplus: the same ends)
    if sigmoid:
        edge = np.concatenate([edge, np.array([np.inf, -np.inf], np.float32)])
    logit = (r.standard_normal((T, E)) * 2.0).astype(np.float32)
    for t in range(T):
        n = 1 + t % 12                                   # a few special values a row, at moving places
        pos = r.choice(E, n, replace=False)
        vals = edge[(np.arange(n) * 7 + t * 5) % len(edge)]
        if not sigmoid:                                  # softmax subtracts the row maximum: keep x - max finite and
            vals = -np.abs(vals)                         # let it reach the underflow side instead
        logit[t, pos] = vals
    kw = dict(n_group=0, topk_group=0, tail=0, route_scale=1.0)
    got = gpu_route(moe, logit, None, E, k, T, flags, **kw)
    want = np.zeros(T * k, dtype=ol.ROUTE_DT)
    ol.run(oracle.plow_oracle_exec, cases.route_inst(E, k, T, flags, False, **kw),
           ol.table_of([want, logit, None, None]), 8)
    assert np.array_equal(got["eid"], want["eid"])
    assert np.array_equal(got["gate"].view(np.uint32), want["gate"].view(np.uint32))


# K a multiple of 64 and 2^17 outputs or more: the matrix-unit form (64 tokens x 32 experts per workgroup, a ring of
# four 64-k chunks): 4, 2, 1, 16, 3, 5, 7 and 112 chunks, ragged in tokens and in experts
# Few outputs and K a multiple of 256: one token x 64 experts per consumer wave, 1 / 2 / 4 tokens per
# workgroup (ragged in tokens and experts: (3, 100), (15, 130), (17, 100)); (6, 40, 768) etc. on the 8 x 8 tiles
@pytest.mark.parametrize("M,N,K", [(3, 100, 512), (2, 64, 256), (5, 64, 1280), (15, 130, 1024), (16, 64, 2048),
                                   (17, 100, 512), (1, 128, 4096), (8, 128, 4096),
                                   (6, 40, 768), (64, 256, 7168), (1, 384, 7168), (700, 1000, 264),
                                   (700, 1000, 256), (520, 520, 128), (1030, 300, 64), (1500, 288, 1024),
                                   (413, 331, 192), (1024, 1024, 128), (2048, 512, 192),
                                   (2048, 1024, 192), (4096, 512, 320), (520, 260, 448), (512, 256, 7168),
                                   (16, 8192, 256), (8200, 16, 128), (70, 1900, 64)])  # fewer rows than a block holds
def test_router_score_bit_exact(moe, oracle, M, N, K):
    print(f"[case] score {M}x{N}x{K}", flush=True)
    if (M, N, K) == (6, 40, 768):
        x, w, want = G["score/x"], G["score/w"], G["score/out"]
    else:
        r = cases.rng_of(M + N)
        x, w = cases.randn_bf16(r, (M, K), 1.0), cases.randn_bf16(r, (N, K), 0.02)
        want = np.zeros((M, N), np.float32)
        ol.run(oracle.plow_oracle_exec, abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[M, N, K]),
               ol.table_of([want, x, w]), 8)
    out = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    moe.exec(abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[M, N, K]), dev_table([out, to_dev(x), to_dev(w)]))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_combine_bit_exact(moe, oracle):
    part, res, sh = G["combine/part"], G["combine/res"], G["combine/shared"]
    T, H = res.shape
    k = part.shape[0] // T
    out = torch.zeros((T, H), dtype=torch.int16, device="cuda")
    moe.exec(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, 2, 3], i=[H, k, T]),
             dev_table([out, to_dev(res), to_dev(sh), to_dev(part)]))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), G["combine/out"])
    out.zero_()
    moe.exec(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, None, None, 3], i=[H, k, T]),
             dev_table([out, None, None, to_dev(part)]))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), G["combine/out_plain"])
    # a larger ragged case incl. the row-band form (i3 = first row) against the oracle
    r = cases.rng_of(5)
    T, H, k = 37, 7168, 9
    part = r.standard_normal((T * k, H)).astype(np.float32)
    res = cases.randn_bf16(r, (T, H), 1.0)
    want = np.zeros((T, H), np.uint16)
    ol.run(oracle.plow_oracle_exec, abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, None, 3], i=[H, k, T]),
           ol.table_of([want, res, None, part]), 8)
    out = torch.zeros((T, H), dtype=torch.int16, device="cuda")
    tbl = dev_table([out, to_dev(res), None, to_dev(part)])
    moe.exec(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, None, 3], i=[H, k, 20, 0]), tbl)
    moe.exec(abi.inst(abi.OP_MOE_COMBINE_PF, t=[0, 1, None, 3], i=[H, k, 17, 20]), tbl)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want)


def test_quant_ops_bit_exact(moe, oracle):
    r = cases.rng_of(9)
    # 1x128: random rows, an all-zero group, and rows whose group amax is exactly 448 so that the
    # scale is 1 and the hardware conversion is exercised on every e4m3 rounding boundary
    grid = np.array([oracle.plow_oracle_e4m3_to_f32(c) for c in range(127)], np.float32)
    mids = ((grid[:-1].astype(np.float64) + grid[1:]) / 2).astype(np.float32)
    vals = np.concatenate([grid, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(999))])
    vals = ol.bf2f(ol.f2bf(vals))  # the op's input is bf16
    M, K = 16, 1024
    x = ol.bf2f(cases.randn_bf16(r, (M, K), 2.0))
    x[3, 256:384] = 0
    both_signs = np.concatenate([vals, -vals])
    blk = np.resize(both_signs, (8 * 8, 127))    # 64 groups of 127 crafted values + one 448
    assert blk.size >= both_signs.size
    for n in range(blk.shape[0]):
        row, grp = 6 + n // 8, n % 8
        x[row, grp * 128:grp * 128 + 127] = blk[n]
        x[row, grp * 128 + 127] = 448.0
    xb = ol.f2bf(x)
    want_q, want_s = np.zeros((M, K), np.uint8), np.zeros((K // 128, M + 3), np.float32)
    inst = abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[M, K, M + 3])
    ol.run(oracle.plow_oracle_exec, inst, ol.table_of([want_q, xb, want_s]), 4)
    q = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros((K // 128, M + 3), dtype=torch.float32, device="cuda")
    moe.exec(inst, dev_table([q, to_dev(xb), s]))
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), want_q)
    # per-row
    x2 = G["quant32/x"]
    M2, K2 = x2.shape
    q2 = torch.zeros((M2, K2), dtype=torch.uint8, device="cuda")
    s2 = torch.zeros(M2, dtype=torch.float32, device="cuda")
    moe.exec(abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[M2, K2]), dev_table([q2, to_dev(x2), s2]))
    torch.cuda.synchronize()
    assert np.array_equal(q2.cpu().numpy(), G["quant32/xq"])
    assert np.array_equal(s2.cpu().numpy().view(np.uint32), G["quant32/scale"].view(np.uint32))


def test_refusals(moe):
    """Typed refusal before launch, with a message; nothing is enqueued."""
    t = dev_table([torch.zeros(8, device="cuda")] * 8)
    assert moe.check(abi.inst(999, t=[0]), t) == abi.E_UNSUPPORTED
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1, None, 3], i=[0, 64, 4, 1, 2]), t) == abi.E_INVAL
    assert "bias" in moe.last_error()
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 64, 8, 1, 2, 0, 8, 1]), t) == 0
    # hash selection (flag bit 4) has no table operand on this op; bits above 5 name nothing
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 64, 8, 1 | 16, 2]), t) == abi.E_INVAL
    assert "hash" in moe.last_error()
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 64, 8, 64, 2]), t) == abi.E_INVAL
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 64, 8, 32 | 8, 2]), t) == 0
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 60, 8, 1, 2, 0, 8, 4]), t) == abi.E_INVAL
    assert moe.check(abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1], i=[0, 64, 8, 1, 2, 0, 32, 2]), t) == abi.E_INVAL
    assert moe.check(abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5], i=[256, 256, 4, 2, 0, 1, 0, 5]), t) == abi.E_UNSUPPORTED
    assert moe.check(abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[4, 100]), t) == abi.E_INVAL
    with pytest.raises(Exception):
        moe.exec(abi.inst(abi.OP_MOE_ALIGN_PF, t=[0, 1, 2, 3], i=[4, 8, 2]), t)


@pytest.mark.parametrize("rows,feat,gamma", [(5, 384, True), (64, 7168, True), (3, 16384, False), (7, 8, True), (300, 2048, True)])
def test_rmsnorm_with_fused_quantizers(moe, oracle, rows, feat, gamma):
    """Op 1, the step before the path (plow runtime/cpu/dev/golden/norm.c:15-43, runtime/amd/op_norm.h:
    486-551). The sum of squares is a tree here and an index-order loop in the oracle (as in plow's GPU
    and CPU kernels): the normalized row may differ in the last bf16 bit now and then, no more. The fused
    quantizers must produce exactly what the separate quantizer ops produce from the row this kernel
    wrote: per row (as op 32) and per 1x128 group (as op 184)."""
    print(f"[case] rmsnorm rows={rows} feat={feat} gamma={gamma}", flush=True)
    r = cases.rng_of(rows + feat)
    x = cases.randn_bf16(r, (rows, feat), 1.5)
    g = cases.randn_bf16(r, (feat,), 1.0) if gamma else None
    want = np.zeros((rows, feat), np.uint16)
    ol.run(oracle.plow_oracle_exec, abi.inst(abi.OP_RMSNORM, t=[0, 1, 2 if gamma else None], i=[rows, feat], f=[1e-6]),
           ol.table_of([want, x, g]), 4)
    dx, dg = to_dev(x), (to_dev(g) if gamma else None)
    for mode in (0, 1, 2):
        if mode == 2 and feat % 128:
            continue
        out = torch.zeros((rows, feat), dtype=torch.int16, device="cuda")
        xq = torch.zeros((rows, feat), dtype=torch.uint8, device="cuda")
        sc = torch.zeros((feat // 128, rows) if mode == 2 else (rows,), dtype=torch.float32, device="cuda")
        t = [0, 1, 2 if gamma else None] + ([3, 4] if mode else [])
        moe.exec(abi.inst(abi.OP_RMSNORM, t=t, i=[rows, feat, 0, 0, 128 if mode == 2 else 0], f=[1e-6]),
                 dev_table([out, dx, dg, xq, sc]))
        torch.cuda.synchronize()
        got = out.cpu().numpy().view(np.uint16)
        a, b = ol.bf2f(got), ol.bf2f(want)
        assert (got == want).mean() > 0.99
        assert np.all(np.abs(a - b) <= 2.0 ** -7 * np.abs(b) + 1e-30)          # one bf16 step at most
        if mode:
            q2 = np.zeros((rows, feat), np.uint8)
            s2 = np.zeros(tuple(sc.shape), np.float32)
            op = abi.OP_QUANT_FP8 if mode == 1 else abi.OP_QUANT_FP8_BLOCK128
            row_in = np.ascontiguousarray(got)          # held here: the table keeps nothing alive
            ol.run(oracle.plow_oracle_exec, abi.inst(op, t=[0, 1, 2], i=[rows, feat]), ol.table_of([q2, row_in, s2]), 2)
            assert np.array_equal(xq.cpu().numpy(), q2)
            assert np.array_equal(sc.cpu().numpy().view(np.uint32), s2.view(np.uint32))


@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 15, 16, 40])
@pytest.mark.parametrize("shape", ["dsv3", "qwen", "kimi"])
def test_router_score_that_carries_its_topk_equals_the_op_pair(moe, oracle, T, shape):
    """Op 180 with the router mark (plow's raw router segment): below 16 tokens one launch in which the
    score's workgroups count themselves off and the last arrival of a token group runs its top-k, two
    launches from there. Logits and table are the bytes of op 180 followed by op 83, on the device and in
    the oracle; also on a second run (the counters are back at zero), with the counters left zero."""
    from plow_amd import layer, synth
    kw = {"dsv3": dict(H=1024, E=256, I=256, k=8, scoring="sigmoid", norm_topk=True, bias=True, n_group=8, topk_group=4,
                       route_scale=2.5, n_shared=1, shared_mode="fold"),
          "qwen": dict(H=512, E=128, I=256, k=8, scoring="softmax", norm_topk=True),
          "kimi": dict(H=768, E=384, I=256, k=8, scoring="sigmoid", norm_topk=True, bias=True, route_scale=2.827,
                       n_shared=1, shared_mode="fold")}[shape]
    pair = layer.plan_layer(layer.MoeConfig(f"router-{shape}", T=T, enc="bf16", arm="a16", **kw))
    raw = layer.plan_layer(layer.MoeConfig(f"router-raw-{shape}", T=T, enc="bf16", arm="a16", router_raw=True, **kw))
    assert "topk" not in raw.names
    ref = synth.bind(pair, "cuda", seed=T)
    moe.exec_many([pair.insts[pair.index(l)] for l in ("score", "topk")], ref.table())
    torch.cuda.synchronize()
    dev = synth.bind(raw, "cuda", seed=T)
    host = synth.to_host(dev)
    for rep in range(2):
        dev.t["logit"].fill_(float("nan"))
        dev.t["table"].fill_(-1)
        moe.exec(raw.insts[raw.index("score")], dev.table())
        torch.cuda.synchronize()
        assert np.array_equal(dev.np("logit").view(np.uint32), ref.np("logit").view(np.uint32)), rep
        assert np.array_equal(dev.np("table"), ref.np("table")), rep
        assert not dev.np("router_ctr").any()
    ol.run(oracle.plow_oracle_exec, raw.insts[raw.index("score")], host.table(), 4)
    assert np.array_equal(host.np("logit").view(np.uint32), ref.np("logit").view(np.uint32))
    assert np.array_equal(host.np("table"), ref.np("table"))


def test_router_score_that_carries_its_topk_refusals(moe):
    from plow_amd import layer, synth
    plan = layer.plan_layer(layer.MoeConfig("router-raw", T=2, H=512, E=64, I=256, k=4, scoring="sigmoid", bias=True,
                                            enc="bf16", arm="a16", router_raw=True))
    dev = synth.bind(plan, "cuda", seed=1)
    good = plan.insts[plan.index("score")]
    assert moe.check(good, dev.table()) == 0

    def variant(**kw):
        c = abi.PlowDevInst()
        C.memmove(C.byref(c), C.byref(good), C.sizeof(c))
        for name, (idx, val) in kw.items():
            getattr(c, name)[idx] = val
        return c
    assert moe.check(variant(t=(5, abi.TENSOR_NONE)), dev.table()) == abi.E_INVAL          # no counters
    assert moe.check(variant(t=(3, abi.TENSOR_NONE)), dev.table()) == abi.E_INVAL          # no table
    assert moe.check(variant(t=(4, abi.TENSOR_NONE)), dev.table()) == abi.E_INVAL          # bias flag without a bias
    assert moe.check(variant(i=(4, good.i[4] & ~abi.ROUTE_F32_LOGIT)), dev.table()) == abi.E_INVAL
    assert moe.check(variant(i=(3, 0)), dev.table()) == abi.E_INVAL                          # k = 0
    assert moe.check(variant(i=(5, 2)), dev.table()) == abi.E_UNSUPPORTED                   # interpreter signal
