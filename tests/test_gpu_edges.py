"""Edge cases on the GPU, all bit-exact: empty and degenerate routing tables through align (op 84), the
largest expert count, every slot on one expert, and the per-row quantizer (op 32) at widths off the
vector width, on rows with NaN / infinities and with its fused gate/up arm, against vectors from plow's
own CPU kernel."""
import os

import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from gpu_harness import dev_table, to_dev
from plow_amd import abi

pytestmark = pytest.mark.gpu

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "plow_cpu_golden.npz"))
UNUSED = abi.EXPERT_UNUSED


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def table_of_eids(eids, seed):
    tab = np.zeros(len(eids), dtype=ol.ROUTE_DT)
    tab["eid"] = eids
    tab["gate"] = cases.rng_of(seed).random(len(eids)).astype(np.float32)
    return tab


def align_cases():
    r = cases.rng_of(31)
    out = []
    out.append(("empty", 0, 16, 4, np.zeros(0, np.uint32)))
    out.append(("all-sentinel", 40, 16, 4, np.full(160, UNUSED, np.uint32)))
    e = r.integers(0, 1056, 300 * 8).astype(np.uint32)
    e[r.choice(e.size, 50, replace=False)] = UNUSED
    e[7] = 1056                                        # first id past the table: not counted
    out.append(("E=1056", 300, 1056, 8, e))
    out.append(("one-expert", 20000, 8, 2, np.tile(np.array([3, 5], np.uint32), 20000)))
    # counts of exactly 64, 128, 0 and 1: no padding for the first two, a whole pad tile less one for the last
    e = np.concatenate([np.full(64, 0), np.full(128, 1), np.full(1, 3)]).astype(np.uint32)
    out.append(("tile-multiples", 193, 4, 1, r.permutation(e)))
    out.append(("one-slot", 1, 1, 1, np.zeros(1, np.uint32)))
    return out


@pytest.mark.parametrize("case", align_cases(), ids=lambda c: c[0])
def test_align_edges(moe, oracle, case):
    name, T, E, k, eids = case
    print(f"[case] align {name} T={T} E={E} k={k}", flush=True)
    tab = table_of_eids(eids, 3)
    want = cases.align_arrays(tab if T else np.zeros(1, dtype=ol.ROUTE_DT), T, E, k)
    ol.run(oracle.plow_oracle_exec, cases.align_inst(T, E, k), ol.table_of(want), 1)
    R = abi.max_rows(T, k, E)
    dev = [torch.full((3 * E + 1,), -5, dtype=torch.int32, device="cuda"), to_dev(want[1]),
           torch.full((R,), 7, dtype=torch.int32, device="cuda"),
           torch.full((R,), 7, dtype=torch.int32, device="cuda"),
           torch.full((R,), 7.0, dtype=torch.float32, device="cuda")]
    moe.exec(cases.align_inst(T, E, k), dev_table(dev))
    torch.cuda.synchronize()
    meta = dev[0].cpu().numpy()
    assert np.array_equal(meta, want[0])
    rows = int(meta[3 * E]) * abi.MPF_BM
    live = int((eids < E).sum())
    assert int(meta[E:2 * E].sum()) == live and rows <= R
    assert np.array_equal(dev[1 + 1].cpu().numpy().view(np.uint32)[:rows], want[2][:rows])
    assert np.array_equal(dev[1 + 2].cpu().numpy().view(np.uint32)[:rows], want[3][:rows])
    assert np.array_equal(dev[1 + 3].cpu().numpy().view(np.uint32)[:rows], want[4][:rows].view(np.uint32))
    assert np.all(dev[2].cpu().numpy()[rows:] == 7)    # nothing written past the padded rows


def gpu_quant_row(moe, x, gate=None, up=None, act=0):
    M, K = x.shape
    q = torch.full((M, K), 0xA5, dtype=torch.uint8, device="cuda")
    s = torch.full((M,), -1.0, dtype=torch.float32, device="cuda")
    xd, gd, ud = to_dev(x), to_dev(gate), to_dev(up)
    t = [0, 1, 2] + ([3, 4] if gate is not None else [])
    moe.exec(abi.inst(abi.OP_QUANT_FP8, t=t, i=[M, K, act]), dev_table([q, xd, s, gd, ud]))
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy(), xd.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("key", ["quant32w/1", "quant32w/15", "quant32w/17", "quant32w/257", "quant32n"])
def test_per_row_quant_edges(moe, key):
    print(f"[case] op32 {key}", flush=True)
    q, s, _ = gpu_quant_row(moe, G[key + "/x"])
    assert np.array_equal(s.view(np.uint32), G[key + "/scale"].view(np.uint32))
    assert np.array_equal(q, G[key + "/xq"])


def test_per_row_quant_wide_and_nonfinite_vector_path(moe, oracle):
    """65544 columns (several strides of the row loop) with NaN / infinities, on the 8-wide path."""
    r = cases.rng_of(41)
    M, K = 4, 65544
    x = cases.randn_bf16(r, (M, K), 2.0)
    x[1, [5, 4099, 65543]] = [0x7FC0, 0xFFC0, 0x7F80]
    x[2, 70] = 0xFF80
    x[3] = 0
    want_q, want_s = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    xin = x.copy()                                      # the table holds addresses only: keep it alive
    ol.run(oracle.plow_oracle_exec, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[M, K]),
           ol.table_of([want_q, xin, want_s]), 4)
    q, s, _ = gpu_quant_row(moe, x)
    assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(q, want_q)


@pytest.mark.parametrize("K", [17, 1024])
def test_per_row_quant_fused_silu_bit_exact(moe, K):
    key = f"quant32f/1/{K}"
    print(f"[case] op32 fused {key}", flush=True)
    q, s, x = gpu_quant_row(moe, np.zeros_like(G[key + "/x"]), G[key + "/gate"], G[key + "/up"], act=1)
    assert np.array_equal(x, G[key + "/x"])
    assert np.array_equal(s.view(np.uint32), G[key + "/scale"].view(np.uint32))
    assert np.array_equal(q, G[key + "/xq"])


@pytest.mark.parametrize("K", [17, 1024])
def test_per_row_quant_fused_gelu(moe, oracle, K):
    """gelu_tanh goes through the device's tanhf: the produced row is held to the reference's own bound
    (1 % of the row's range, plow runtime/tests/cpu_dev_avx512_gemm_test.c:305-316) and the codes must be
    exactly the quantization of the row the device produced."""
    key = f"quant32f/0/{K}"
    q, s, x = gpu_quant_row(moe, np.zeros_like(G[key + "/x"]), G[key + "/gate"], G[key + "/up"], act=0)
    xr, xg = ol.bf2f(G[key + "/x"]), ol.bf2f(x)
    hi = np.abs(xr).max(axis=1, keepdims=True)
    assert np.all(np.abs(xg - xr) <= 0.01 * hi)
    assert np.all(np.abs(s - G[key + "/scale"]) <= 0.01 * G[key + "/scale"])
    M = x.shape[0]
    want_q, want_s = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    xin = x.copy()
    ol.run(oracle.plow_oracle_exec, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[M, K]),
           ol.table_of([want_q, xin, want_s]), 2)
    assert np.array_equal(q, want_q) and np.array_equal(s.view(np.uint32), want_s.view(np.uint32))


def test_per_row_quant_refusals_and_poison(moe):
    x = cases.randn_bf16(cases.rng_of(2), (2, 16), 1.0)
    t = dev_table([torch.zeros(32, dtype=torch.uint8, device="cuda"), to_dev(x),
                   torch.zeros(2, device="cuda"), to_dev(x), None])
    assert moe.check(abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2, 3], i=[2, 16, 1]), t) == abi.E_INVAL   # gate without up
    assert moe.check(abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[2, 0]), t) == abi.E_INVAL
    # a pair-form activation is not a gate-only one: the reference poisons, so the row and its codes are NaN
    q, s, xo = gpu_quant_row(moe, np.zeros_like(x), x, x, act=2)
    assert np.all((xo & 0x7F80) == 0x7F80) and np.all((xo & 0x7F) != 0)
    assert np.all((q & 0x7F) == 0x7F)


@pytest.mark.parametrize("arm,enc,T", [("w8a8", "fp8blk", 24), ("a16", "mxfp4", 5), ("w8a8", "fp8blk", 600), ("a4w4", "mxfp4", 300),
                                       ("a16", "bf16", 9), ("a16", "bf16", 200), ("a16dec", "mxfp4", 3), ("a16dec", "fp8blk", 40)])
def test_layer_chain_replays_from_a_hip_graph(moe, arm, enc, T):
    """The op chain of a layer allocates nothing and clears nothing through the runtime, so a caller may
    capture it: captured once, replayed four times with new activations and other work in between, every
    replay must equal the eager result bit for bit. The bf16 cases carry two dense shared experts (ops 20 / 8):
    at a few tokens those run on the context's second stream, forked off and joined back inside the captured run,
    as K slices with their partial sums in the staging; at 200 tokens on the tiled kernel in their place. The a16dec
    cases run the table-driven decode experts (ops 48 / 49): at 3 tokens the matrix-vector form reads its rows from
    the routing table the captured top-k writes, at 40 the slots are sorted into the context's workspace."""
    from plow_amd import layer, synth
    print(f"[case] graph replay arm={arm} enc={enc} T={T}", flush=True)
    shared = dict(n_shared=2, shared_mode="dense") if enc == "bf16" else dict(n_shared=1, shared_mode="fold")
    cfg = layer.MoeConfig("graph", H=512, E=16, I=512 if arm == "a4w4" else 256, k=4, T=T, scoring="sigmoid", norm_topk=True,
                          bias=True, enc=enc, arm=arm, **shared)
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=11)
    insts, table = abi.inst_array(plan.insts), dev.table()
    moe.exec_many(insts, table, torch.cuda.current_stream().cuda_stream)   # first calls set kernel attributes
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        moe.exec_many(insts, table, side.cuda_stream)
        graph.capture_end()
    torch.cuda.synchronize()
    xs = [synth.randn_bf16((cfg.T, cfg.H), 1.0, dev.device, 500 + n) for n in range(4)]
    for n, x in enumerate(xs):
        dev.t["x"].copy_(x)
        dev.t["out"].zero_()
        moe.exec_many(insts, table, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want_out, want_table = dev.t["out"].clone(), dev.t["table"].clone()
        dev.t["out"].zero_()
        dev.t["table"].zero_()
        scratch = torch.randn(1 << 16, device="cuda").sum()       # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dev.t["table"], want_table), f"replay {n}: routing differs"
        assert torch.equal(dev.t["out"], want_out), f"replay {n}: output differs"
        assert bool(torch.isfinite(scratch))


def test_dense_ops_on_the_second_stream_keep_the_order_of_the_run(moe):
    """A run's dense ops of a few rows are launched on the context's second stream beside the ops before them that
    share no operand with them. Two runs of [RMSNorm, dense GLU, dense GEMM]: one where the GLU reads the row the
    norm writes (it must wait for it) and one where the norm works on tensors of its own (the dense ops may run
    beside it); both must give the bytes of the same ops issued one at a time."""
    M, N, K = 24, 256, 512
    r = cases.rng_of(77)
    x, other = to_dev(cases.randn_bf16(r, (M, K), 1.0)), to_dev(cases.randn_bf16(r, (M, K), 1.0))
    wg, wu, wd = (to_dev(cases.randn_bf16(r, s, 0.05)) for s in ((N, K), (N, K), (K, N)))
    st = torch.cuda.current_stream().cuda_stream
    for norm_in, norm_out in ((0, 1), (8, 9)):   # handles: 0 x, 1 xn, 2 wg, 3 wu, 4 fu, 5 wd, 6 y, 8 other, 9 other_n
        ops = [abi.inst(abi.OP_RMSNORM, t=[norm_out, norm_in, None], i=[M, K], f=[1e-6]),
               abi.inst(abi.OP_GEMM_GLU, t=[4, 1, 2, None, None, 3], i=[M, N, K, 0, 0, 1]),
               abi.inst(abi.OP_GEMM, t=[6, 4, 5], i=[M, K, N, 0, 0, 0])]
        res = []
        for many in (False, True):
            xn = torch.zeros((M, K), dtype=torch.int16, device="cuda") if norm_out == 1 else x.clone()
            fu = torch.zeros((M, N), dtype=torch.int16, device="cuda")
            y = torch.zeros((M, K), dtype=torch.int16, device="cuda")
            on = torch.zeros((M, K), dtype=torch.int16, device="cuda")
            tab = dev_table([x, xn, wg, wu, fu, wd, y, None, other, on])
            if many:
                moe.exec_many(abi.inst_array(ops), tab, st)
            else:
                for op in ops:
                    moe.exec(op, tab, st)
            torch.cuda.synchronize()
            res.append((fu.clone(), y.clone(), on.clone(), xn.clone()))
        for a, b in zip(*res):
            assert torch.equal(a, b)
        assert bool((res[1][1] != 0).any())
