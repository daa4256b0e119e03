"""Runs one layer plan on the HIP operator and on the CPU oracle over the same bytes."""
import ctypes as C
import os

import numpy as np
import torch

import oracle_lib as ol
from plow_amd import abi, synth
from plow_amd.layer import MoeConfig, plan_layer

NTHREADS = min(16, os.cpu_count() or 1)

# Output tolerance of the benchmark definition: bf16 output, f32 accumulation.
MAX_ABS_FRAC = 2e-2     # max |out - ref| <= 2e-2 * max |ref|
MEAN_REL = 5e-3         # mean |out - ref| / mean |ref| <= 5e-3


def run_device(moe, plan, dev, labels=None):
    insts = plan.insts if labels is None else [plan.insts[plan.index(l)] for l in labels]
    print(f"[gpu] {plan.cfg.name} T={plan.cfg.T} ops={[i.op for i in insts]}", flush=True)
    moe.exec_many(insts, dev.table())
    torch.cuda.synchronize()


def run_oracle(oracle, plan, host, labels=None, nthreads=NTHREADS):
    insts = plan.insts if labels is None else [plan.insts[plan.index(l)] for l in labels]
    arr = abi.inst_array(insts)
    rc = oracle.plow_oracle_exec_many(arr, len(arr), host.table(), nthreads)
    assert rc == 0, rc


def both(moe, oracle, cfg: MoeConfig, seed=0, **bind_kw):
    plan = plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=seed, **bind_kw)
    host = synth.to_host(dev)
    run_device(moe, plan, dev)
    run_oracle(oracle, plan, host)
    return plan, dev, host


def assert_routing_equal(plan, dev, host):
    """Routing indices, gates, counts, offsets and the row permutation: bit-exact."""
    cfg = plan.cfg
    td, th = dev.np("table"), host.np("table")
    assert np.array_equal(td["eid"], th["eid"]), "selected experts differ"
    assert np.array_equal(td["gate"].view(np.uint32), th["gate"].view(np.uint32)), "gates differ"
    md, mh = dev.np("meta"), host.np("meta")
    assert np.array_equal(md, mh), "meta (rowoff | cnt | tilep) differs"
    rows = int(mh[3 * cfg.E_all]) * abi.MPF_BM
    for name in ("row_token", "row_partidx"):
        assert np.array_equal(dev.np(name)[:rows], host.np(name)[:rows]), name
    assert np.array_equal(dev.np("row_gate")[:rows].view(np.uint32), host.np("row_gate")[:rows].view(np.uint32))
    return rows


def assert_output_close(out_dev_bits, out_ref_bits, what="out"):
    a, b = ol.bf2f(out_dev_bits).astype(np.float64), ol.bf2f(out_ref_bits).astype(np.float64)
    assert np.all(np.isfinite(a)), f"{what}: non-finite values"
    err = np.abs(a - b)
    mx, mean_rel = err.max() / np.abs(b).max(), err.mean() / np.abs(b).mean()
    print(f"[parity] {what}: max_abs/max|ref| = {mx:.3e} (<= {MAX_ABS_FRAC}), "
          f"mean rel = {mean_rel:.3e} (<= {MEAN_REL})", flush=True)
    assert mx <= MAX_ABS_FRAC and mean_rel <= MEAN_REL, (what, mx, mean_rel)
    return mx, mean_rel


def dev_table(arrays):
    """void*[] over torch tensors (None = NULL)."""
    t = (C.c_void_p * len(arrays))()
    for n, a in enumerate(arrays):
        t[n] = None if a is None else a.data_ptr()
    return t


def to_dev(a):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).cuda()
    if a.dtype == ol.ROUTE_DT:
        return torch.from_numpy(a.view(np.int32).reshape(-1, 2)).cuda()
    return torch.from_numpy(a).cuda()


def from_dev(t, dtype):
    a = t.detach().cpu().contiguous().numpy()
    return a.view(dtype).reshape(-1) if dtype == ol.ROUTE_DT else a.view(dtype)
