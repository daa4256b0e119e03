"""plow_moe_exec_noalloc, the entry point that allocates nothing (its workspace is a static device array
inside the library), against plow_moe_exec on the same inputs: bit-identical, on two calls in a row, the
second with a smaller batch, for the ops that use the workspace - slot-major decode experts 65 / 66 inside
whole layers, 48 / 49 on bf16 and block-fp8 weights, flat mxfp4 150 / 151 and their gathered-row twins
152 / 153, the align op beyond 4096 slots (its one-workgroup form) - with the device's free memory
unchanged across the calls; and its refusal of a batch beyond its limit."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def noalloc_fn():
    from plow_amd import abi
    from plow_amd.lib import load
    lib = load()
    fn = lib.plow_moe_exec_noalloc
    fn.argtypes = [C.POINTER(abi.PlowDevInst), C.POINTER(C.c_void_p), C.c_void_p, C.c_char_p, C.c_size_t]
    fn.restype = C.c_int
    return fn


def run_noalloc(fn, plan, dev):
    import torch
    err = C.create_string_buffer(256)
    table = dev.table()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for d in plan.insts:
        rc = fn(C.byref(d), table, None, err, 256)
        assert rc == 0, (d.op, rc, err.value.decode())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the entry point that allocates nothing changed the device's free memory"


def call_noalloc(fn, insts, table):
    """The ops one by one through the entry point; the device's free memory must not move."""
    import torch
    err = C.create_string_buffer(256)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for d in insts:
        assert fn(C.byref(d), table, None, err, 256) == 0, (d.op, err.value.decode())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the entry point that allocates nothing changed the device's free memory"


def layer_cfg(kind, T):
    from plow_amd import layer
    if kind == "fp8pc":     # ops 65 / 66: per-channel fp8 weights, slot-major
        return layer.MoeConfig("na-pc", H=512, E=16, I=256, k=4, T=T, scoring="softmax", norm_topk=True,
                               enc="fp8pc", arm="a16")
    raise KeyError(kind)


@pytest.mark.parametrize("kind", ["fp8pc"])
def test_noalloc_matches_exec_on_two_calls_second_smaller(kind):
    import torch
    from plow_amd import layer, synth
    from plow_amd.lib import Moe
    fn = noalloc_fn()
    assert fn(None, None, None, None, 0) == 0           # set-up only
    moe = Moe(0)
    for T in (37, 5):                                    # the second call is the smaller one
        print(f"[case] noalloc {kind} T={T}", flush=True)
        cfg = layer_cfg(kind, T)
        plan = layer.plan_layer(cfg)
        ref = synth.bind(plan, "cuda", seed=T)
        moe.exec_many(plan.insts, ref.table())
        torch.cuda.synchronize()
        got = synth.bind(plan, "cuda", seed=T)
        run_noalloc(fn, plan, got)
        for name in ("table", "meta", "fu", "part", "out"):
            assert ref.np(name).tobytes() == got.np(name).tobytes(), (T, name)
        assert np.isfinite(ref.t["out"].float().cpu().numpy()).all()
    moe.close()


def test_noalloc_flat_mxfp4_decode_ops():
    """Ops 150 / 151 over flat [E][rows][K/2] tensors: the workspace also holds the per-expert pointer
    tables the kernels read."""
    import torch
    import oracle_lib as ol
    from gpu_harness import dev_table, to_dev
    from plow_amd import abi
    from plow_amd.lib import Moe
    fn = noalloc_fn()
    moe = Moe(0)
    E, I, K, k = 6, 256, 512, 3
    r = np.random.default_rng(5)
    W1 = to_dev(r.integers(0, 256, size=(E, 2 * I, K // 2), dtype=np.uint8))
    S1 = to_dev(r.integers(118, 126, size=(E, 2 * I, K // 32), dtype=np.uint8))
    W2 = to_dev(r.integers(0, 256, size=(E, K, I // 2), dtype=np.uint8))
    S2 = to_dev(r.integers(118, 126, size=(E, K, I // 32), dtype=np.uint8))
    for B in (9, 2):
        print(f"[case] noalloc flat mxfp4 B={B}", flush=True)
        tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
        for b in range(B):
            tab["eid"][b * k:(b + 1) * k] = r.choice(E, size=k, replace=False)
        tab["gate"] = r.random(B * k).astype(np.float32)
        x = to_dev(ol.f2bf(r.standard_normal((B, K)).astype(np.float32)))
        outs = []
        for use_noalloc in (False, True):
            fu = torch.zeros((B * k, I), dtype=torch.int16, device="cuda")
            part = torch.full((B * k, K), 7.0, dtype=torch.float32, device="cuda")
            t = [fu, x, to_dev(tab), W1, S1, None, part, W2, S2]
            glu = abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[k, I, K, E, 1, abi.ACT_SILU, B])
            down = abi.inst(abi.OP_MOE_DOWN_MX, t=[6, 0, 2, 7, 8], i=[k, K, I, E, 0, 0, B])
            table = dev_table(t)
            if use_noalloc:
                err = C.create_string_buffer(256)
                for d in (glu, down):
                    assert fn(C.byref(d), table, None, err, 256) == 0, err.value.decode()
            else:
                moe.exec_many([glu, down], table)
            torch.cuda.synchronize()
            outs.append((fu.cpu().numpy(), part.cpu().numpy()))
        assert np.array_equal(outs[0][0], outs[1][0])
        assert np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32))
        assert np.isfinite(outs[1][1]).all() and np.abs(outs[1][1]).max() > 0
    moe.close()


@pytest.mark.parametrize("enc", ["bf16", "fp8blk"])
def test_noalloc_slot_major_decode_ops(enc):
    """Ops 48 / 49 (table-driven decode experts, sorted by expert inside the workspace) on bf16 and block-fp8
    weights, incl. a sentinel slot: the same bytes as through a context, on two calls, the second smaller."""
    import torch
    import oracle_lib as ol
    from gpu_harness import dev_table, to_dev
    from plow_amd import abi
    from plow_amd.lib import Moe
    fn = noalloc_fn()
    moe = Moe(0)
    E, I, H, k = 6, 128, 256, 3
    r = np.random.default_rng(17)
    code = abi.ENC_BF16 if enc == "bf16" else abi.ENC_FP8BLK

    def weights(N, K):
        if enc == "bf16":
            return to_dev(ol.f2bf((r.standard_normal((N, K)) * 0.05).astype(np.float32))), None
        b = r.integers(0, 256, (N, K), dtype=np.uint8)
        b[(b & 0x7F) == 0x7F] = 0x30                                   # no NaN codes
        return to_dev(b), to_dev((r.random(((N + 127) // 128, K // 128)) * 0.02 + 1e-3).astype(np.float32))
    mats = [[weights(I, H), weights(I, H), weights(H, I)] for _ in range(E)]
    wtab = to_dev(np.array([[m[j][0].data_ptr() for j in range(3)] for m in mats], dtype=np.uint64))
    stab = None if enc == "bf16" else to_dev(np.array([[m[j][1].data_ptr() for j in range(3)] for m in mats], dtype=np.uint64))
    for B in (11, 3):
        print(f"[case] noalloc ops 48 / 49 enc={enc} B={B}", flush=True)
        tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
        tab["eid"] = r.integers(0, E, B * k)
        tab["eid"][1] = abi.EXPERT_UNUSED
        tab["gate"] = (r.random(B * k) + 0.1).astype(np.float32)
        x, tabd = to_dev(ol.f2bf(r.standard_normal((B, H)).astype(np.float32))), to_dev(tab)
        sh = 4 if stab is not None else None
        glu = abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[0, 1, 2, 3, sh], i=[B * k, I, H, E, k, 1, code])
        down = abi.inst(abi.OP_MOE_GROUP_DOWN_FP8_BLK, t=[5, 0, 2, 3, sh], i=[B * k, H, I, E, 0, 0, code])
        outs = []
        for use_noalloc in (False, True):
            fu = torch.full((B * k, I), 0x1234, dtype=torch.int16, device="cuda")
            part = torch.full((B * k, H), 9.0, dtype=torch.float32, device="cuda")
            table = dev_table([fu, x, tabd, wtab, stab, part])
            if use_noalloc:
                call_noalloc(fn, (glu, down), table)
            else:
                moe.exec_many([glu, down], table)
            torch.cuda.synchronize()
            outs.append((fu.cpu().numpy(), part.cpu().numpy()))
        assert np.array_equal(outs[0][0], outs[1][0])
        assert np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32))
        assert np.isfinite(outs[1][1]).all() and np.abs(outs[1][1]).max() > 0
    moe.close()


def test_noalloc_gathered_flat_mxfp4_ops_and_a_long_align():
    """Ops 152 / 153 (flat mxfp4 tensors on gathered rows; their pointer tables are built in the workspace)
    behind op 84, and op 84 alone at 6000 slots, beyond the 4096 the workspace's chunk histograms cover: the
    one-workgroup align serves it. All bytes equal to the context path."""
    import torch
    import oracle_lib as ol
    from gpu_harness import dev_table, to_dev
    from plow_amd import abi
    from plow_amd.lib import Moe
    fn = noalloc_fn()
    moe = Moe(0)
    E, I, K, k = 5, 128, 512, 2
    r = np.random.default_rng(23)
    Wgu = to_dev(r.integers(0, 256, (E, 2 * I, K // 2), dtype=np.uint8))
    Sgu = to_dev(r.integers(120, 128, (E, 2 * I, K // 32), dtype=np.uint8))
    Wd = to_dev(r.integers(0, 256, (E, K, I // 2), dtype=np.uint8))
    Sd = to_dev(r.integers(120, 128, (E, K, I // 32), dtype=np.uint8))
    for B in (40, 7):
        print(f"[case] noalloc ops 84 + 152 / 153 B={B}", flush=True)
        tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
        for b in range(B):
            tab["eid"][b * k:(b + 1) * k] = r.choice(E, size=k, replace=False)
        tab["gate"] = (r.random(B * k) + 0.1).astype(np.float32)
        x, tabd = to_dev(ol.f2bf(r.standard_normal((B, K)).astype(np.float32))), to_dev(tab)
        R = abi.max_rows(B, k, E)
        align = abi.inst(abi.OP_MOE_ALIGN_PF, t=[0, 1, 2, 3, 4], i=[B, E, k])
        glu = abi.inst(abi.OP_MOE_GLU_MX_PF, t=[5, 6, 7, 8, 0, 2, None], i=[I, K, E, 1, 0, abi.ACT_SILU])
        down = abi.inst(abi.OP_MOE_DOWN_MX_PF, t=[9, 5, 10, 11, 0, None, 3, 4], i=[K, I, E])
        outs = []
        for use_noalloc in (False, True):
            meta = torch.zeros(3 * E + 1, dtype=torch.int32, device="cuda")
            rt, rp = (torch.full((R,), -1, dtype=torch.int32, device="cuda") for _ in range(2))
            rg = torch.zeros(R, dtype=torch.float32, device="cuda")
            fu = torch.full((R, I), 0x1234, dtype=torch.int16, device="cuda")
            part = torch.full((B * k, K), 9.0, dtype=torch.float32, device="cuda")
            table = dev_table([meta, tabd, rt, rp, rg, fu, x, Wgu, Sgu, part, Wd, Sd])
            if use_noalloc:
                call_noalloc(fn, (align, glu, down), table)
            else:
                for d in (align, glu, down):
                    moe.exec(d, table)
            torch.cuda.synchronize()
            outs.append([t.cpu().numpy() for t in (meta, rt, rp, fu, part)])
        for a, b in zip(*outs):
            assert a.tobytes() == b.tobytes()
        assert np.isfinite(outs[1][4]).all() and np.abs(outs[1][4]).max() > 0
    # op 84 alone, 1500 tokens x 4 slots = 6000 slots over 37 experts
    T, E2, k2 = 1500, 37, 4
    tab = np.zeros(T * k2, dtype=ol.ROUTE_DT)
    tab["eid"] = r.integers(0, E2, T * k2)
    tab["gate"] = r.random(T * k2).astype(np.float32)
    tabd, R = to_dev(tab), abi.max_rows(T, k2, E2)
    align = abi.inst(abi.OP_MOE_ALIGN_PF, t=[0, 1, 2, 3, 4], i=[T, E2, k2])
    outs = []
    for use_noalloc in (False, True):
        meta = torch.zeros(3 * E2 + 1, dtype=torch.int32, device="cuda")
        rt, rp = (torch.full((R,), -1, dtype=torch.int32, device="cuda") for _ in range(2))
        rg = torch.zeros(R, dtype=torch.float32, device="cuda")
        table = dev_table([meta, tabd, rt, rp, rg])
        if use_noalloc:
            call_noalloc(fn, (align,), table)
        else:
            moe.exec(align, table)
        torch.cuda.synchronize()
        outs.append([t.cpu().numpy() for t in (meta, rt, rp, rg)])
    rows = int(outs[0][0][3 * E2]) * abi.MPF_BM
    assert rows >= T * k2
    assert np.array_equal(outs[0][0], outs[1][0])
    for a, b in zip(outs[0][1:], outs[1][1:]):
        assert a[:rows].tobytes() == b[:rows].tobytes()
    moe.close()


def test_noalloc_refuses_a_batch_beyond_its_workspace():
    import torch
    from plow_amd import abi
    fn = noalloc_fn()
    dummy = torch.zeros(64, dtype=torch.int32, device="cuda")
    table = (C.c_void_p * 5)(*[dummy.data_ptr()] * 5)
    # op 65 with k * B = 4097 slots: one over the limit; refused before anything is launched
    d = abi.inst(abi.OP_MOE_EXPERT_GLU_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[1, 256, 512, 8, 0, 4097, 1])
    err = C.create_string_buffer(256)
    assert fn(C.byref(d), table, None, err, 256) == abi.E_INVAL
    assert b"exceed the workspace" in err.value and b"4096" in err.value
    d = abi.inst(abi.OP_MOE_EXPERT_GLU_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[1, 256, 512, 2000, 0, 4, 1])
    assert fn(C.byref(d), table, None, err, 256) == abi.E_INVAL
    torch.cuda.synchronize()
