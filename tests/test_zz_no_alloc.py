"""plow_moe_exec_noalloc, the entry point that allocates nothing (its workspace is a static device array
inside the library), against plow_moe_exec on the same inputs: bit-identical, on two calls in a row, the
second with a smaller batch, for the ops that use the workspace (slot-major decode experts 65 / 66 and
48 / 49, flat mxfp4 150 / 151) inside whole layers; and its refusal of a batch beyond its limit."""
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
    for d in plan.insts:
        rc = fn(C.byref(d), dev.table(), None, err, 256)
        assert rc == 0, (d.op, rc, err.value.decode())
    torch.cuda.synchronize()


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
