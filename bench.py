"""Benchmark of the MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|...] [--tokens T]

A step is one pass of the whole layer chain (router score -> top-k -> align -> activation quant ->
grouped gate|up + SwiGLU -> grouped down -> combine) over one batch of synthetic input that is already
resident in HBM. Prints ONE JSON line.

With no --config the line carries both headline cells of the metric: at the top level the
DeepSeek-V3-shaped decode batch of 64 tokens (time per layer, tokens/s, the roofline of its dominant
kernel measured live with HIP events on the launch stream, the CPU baseline of the whole batch), and
under "prefill_4k" the same layer at 4096 tokens with a skewed router (its own time, roofline against
both HBM and the fp8 matrix peak, CPU baseline from a sample of its tokens). Both cells share one set
of expert weights. With --config only that cell is run and reported at the top level.
"""
import argparse
import hashlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0          # MI355X datasheet
FP8_PEAK_TFLOPS = 5000.0       # dense fp8 MFMA
FP4_PEAK_TFLOPS = 10100.0      # dense fp4 MFMA
BF16_PEAK_TFLOPS = 2500.0      # dense bf16 MFMA
CPU_THREADS_CAP = 16           # the GPU box's CPU share for one GPU


def expert_bytes(cfg):
    """Algorithmic bytes of ONE expert's three matrices (payload + scales)."""
    I, H = cfg.I, cfg.H
    if cfg.enc == "fp8blk":
        return 3 * I * H + 3 * ((I + 127) // 128) * ((H + 127) // 128) * 4
    if cfg.enc == "mxfp4":
        return 3 * I * H // 2 + 3 * I * H // 32
    if cfg.enc == "fp8pc":
        return 3 * I * H + (2 * I + H) * 4
    return 6 * I * H


def measured_traffic(cfg_name, tokens, op):
    """HBM bytes per launch of one op's kernel from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
    recorded in profiles/traffic.json, or None. A record counts only while the kernel source it was
    measured on is unchanged (sha256 of the source file, taken when the profile was made): a figure
    measured on another kernel is not a measurement of this one."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        recs = json.load(f)["records"]
    for r in recs:
        if (r["config"], r["tokens"], r["op"]) != (cfg_name, tokens, op):
            continue
        src = os.path.join(ROOT, r["source"])
        if not os.path.exists(src):
            return None
        with open(src, "rb") as f:
            if hashlib.sha256(f.read()).hexdigest() != r["source_sha256"]:
                return None
        return int(r["bytes_per_launch"])
    return None


def make_cfg(layer, a, name, tokens):
    cfg = layer.config(name, tokens or None)
    if name == "c5":
        # Zipf(1.2)-like expert popularity through a selection bias; the prefill pair (ops 81 / 82)
        # from 128 tokens on, the decode ops (65 / 66 semantics, bf16 activations) below
        cfg.bias = True
        cfg.arm = "w8a8" if cfg.T >= 128 else "a16"
        # the decode arm's ops 65 / 66 sort the slots themselves: plow's chain for them has no op 84
        cfg.emit_align = False
    if name == "c4" and not a.arm and cfg.T * cfg.k_all <= 128:
        # a few tokens: plow's decode experts (ops 48 / 49, table driven, slot-major rows; no op 84 in their chain),
        # the same arithmetic as arm 8 of the grouped ops the larger batches run
        cfg.arm, cfg.emit_align = "a16dec", False
    if a.arm == "w8a8det":      # the deterministic fused down -> combine on the block-fp8 W8A8 arm
        cfg.arm, cfg.det_combine = "w8a8", True
    elif a.arm:
        cfg.arm = a.arm
    if a.part_bf16:             # plow's bf16-partial arms (op 86 i7 = 3 / 1 / 5, op 87 i7 = 1): half the bytes of the part round trip
        cfg.part_bf16 = True
    # --raw-router: below 16 tokens the decode router as one op, the score carrying its top-k, as plow emits it
    # (crates/devgen/src/mla.rs:3294-3312); the same bytes, and measured level with the two ops per layer
    if cfg.T < 16 and not cfg.det_combine and a.raw_router:
        cfg.router_raw = True
    return cfg


def run_cell(a, name, tokens, steps, warmup, share=None, cpu_mode="full"):
    """Time one configuration; returns (record, bound tensors). ``share``: a binding of the same layer at
    another batch size whose expert weights are reused. ``cpu_mode``: "full" times the CPU port on the
    whole batch, "sample" on a bounded sample of its tokens, None skips it."""
    import numpy as np
    import torch
    from plow_amd import abi, layer, synth
    from plow_amd.lib import Moe

    cfg = make_cfg(layer, a, name, tokens)
    plan = layer.plan_layer(cfg)
    hot = 3.0 if name == "c3" else 0.0
    # c6: popularity falling off like rank^-0.5, as in plow's bench of this shape
    zipf = a.zipf if a.zipf >= 0.0 else {"c5": 1.2, "c6": 0.5}.get(name, 0.0)
    dev = synth.bind(plan, "cuda", seed=0, hot_expert=hot, zipf=zipf, share=share)
    moe = Moe(0)
    stream = torch.cuda.current_stream().cuda_stream
    insts = abi.inst_array(plan.insts)
    table = dev.table()

    def step():
        moe.exec_many(insts, table, stream)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps

    # per-op durations, HIP events on the launch stream
    per_op = {n: [] for n in plan.names}
    for _ in range(max(5, min(steps, 20))):
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(len(plan.insts) + 1)]
        evs[0].record()
        for n, d in enumerate(plan.insts):
            moe.exec(d, table, stream)
            evs[n + 1].record()
        torch.cuda.synchronize()
        for n, nm in enumerate(plan.names):
            per_op[nm].append(evs[n].elapsed_time(evs[n + 1]) * 1e3)
    op_us = {n: statistics.mean(v) for n, v in per_op.items()}

    if "align" in plan.names:
        cnt = dev.np("meta")[cfg.E_all:2 * cfg.E_all]
    else:                                            # no op 84 in the chain: rows per expert from the routing table
        eid = dev.np("table")["eid"]
        cnt = np.bincount(eid[eid < cfg.E_all], minlength=cfg.E_all)
    hit = int((cnt > 0).sum())                       # experts whose weights must stream (incl. shared)
    rows = int(cnt.sum())
    eb = expert_bytes(cfg)
    H, T = cfg.H, cfg.T
    layer_bytes = hit * eb + cfg.E * H * 2 + (cfg.E * 4 if cfg.bias else 0) + 2 * T * H * 2
    dom = max(("glu", "down"), key=lambda n: op_us[n])
    frac_w = 2.0 / 3.0 if dom == "glu" else 1.0 / 3.0
    # bytes of an element of the intermediate the DOWN reads: e4m3 + a scale per 128, e2m1 + a byte per 32, bf16
    mid = {"w8a8": 1.0 + 4.0 / 128.0, "w8a8q": 1.0 + 4.0 / 128.0, "a4w4": 0.5 + 1.0 / 32.0}.get(cfg.arm, 2.0)
    act_in = T * H * (1 if cfg.arm == "w8a8" else 2) if dom == "glu" else rows * cfg.I * mid
    # the matrix unit's peak in the type the arm multiplies in
    mfma_peak = (FP4_PEAK_TFLOPS if cfg.arm == "a4w4" else
                 FP8_PEAK_TFLOPS if cfg.arm.startswith("w8a8") else BF16_PEAK_TFLOPS)
    dom_bytes = hit * eb * frac_w + act_in
    dom_flops = 2.0 * rows * (2 if dom == "glu" else 1) * cfg.I * H
    achieved = dom_bytes / (op_us[dom] * 1e-6) / 1e9
    achieved_tf = dom_flops / (op_us[dom] * 1e-6) / 1e12
    flops = 2.0 * rows * 3 * cfg.I * H + 2.0 * T * cfg.E * H
    traffic = measured_traffic(cfg.name, T, dom)
    roof = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
            "traffic_over_algorithmic": round(traffic / dom_bytes, 3) if traffic else None,
            "bytes_per_launch": int(dom_bytes), "us_per_launch": round(op_us[dom], 2),
            # the time each roof allows this launch: the larger one is the roof that binds
            "roof_us": {"hbm": round(dom_bytes / (HBM_PEAK_GBS * 1e9) * 1e6, 1),
                        "mfma": round(dom_flops / (mfma_peak * 1e12) * 1e6, 1)},
            "mfma": {"achieved": round(achieved_tf, 1), "peak": mfma_peak, "unit": "TFLOP/s",
                     "frac": round(achieved_tf / mfma_peak, 4), "flops_per_launch": dom_flops}}
    rec = {
        "value": round(ms * 1e3, 2), "unit": "us/layer", "ms_per_step": round(ms, 4), "steps": steps, "warmup": warmup,
        "dtype": {"fp8blk": "fp8_e4m3", "mxfp4": "fp4_e2m1", "fp8pc": "fp8_e4m3", "bf16": "bf16"}[cfg.enc],
        "config": {"workload": f"{cfg.name}: H={cfg.H} E={cfg.E}+{cfg.n_shared} I={cfg.I} top{cfg.k} "
                               f"T={cfg.T} enc={cfg.enc} arm={cfg.arm} groups={cfg.n_group}/{cfg.topk_group}",
                   "tokens": T, "experts_hit": hit, "rows": rows,
                   "rows_per_expert": {"min": int(cnt[:cfg.E].min()), "median": float(np.median(cnt[:cfg.E])),
                                       "max": int(cnt[:cfg.E].max()), "mean": float(cnt[:cfg.E].mean()),
                                       "below_64": int((cnt[:cfg.E] < 64).sum()),
                                       "pad_frac": round(float(((cnt + 63) // 64 * 64).sum() / max(1, cnt.sum()) - 1.0), 4)}},
        "tokens_per_s": round(T / (ms * 1e-3), 1),
        "layer": {"algorithmic_bytes": int(layer_bytes), "hbm_frac": round(layer_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                  "flops": flops, "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / mfma_peak, 4)},
        "op_us": {n: round(v, 2) for n, v in op_us.items()},
        "roofline": roof,
    }
    if cpu_mode:
        rec["cpu_baseline"] = cpu_baseline(a, name, cfg, dev, cpu_mode)
    moe.close()
    return rec, dev


def cpu_baseline(a, name, cfg, dev, mode):
    """The in-repo CPU port of plow's path on this machine's host cores, the method of plow's own CPU
    bench (runtime/tests/cpu_dev_moe_gemma_test.c:109-155): worker threads with a barrier between ops,
    fresh inputs (and so fresh routing) for every repetition, median. "full": the whole batch;
    "sample": the first tokens of the batch, scaled to the batch by tokens (an extrapolation: the
    weight bytes a sample streams do not grow in proportion)."""
    import torch
    import oracle_lib as ol
    from plow_amd import abi, layer, synth
    oracle = ol.load_oracle()
    # worker threads: the CPUs this process may run on, capped at the box's share for one GPU; each worker pinned
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(CPU_THREADS_CAP, avail)
    oracle.plow_oracle_pin_workers(1)
    T = cfg.T
    Tc = T if mode == "full" else min(T, 32)
    ccfg = make_cfg(layer, a, name, Tc)
    cplan = layer.plan_layer(ccfg)
    chost = synth.Bound(cplan, "cpu")
    for nm, sp in cplan.specs.items():
        if sp.role in ("scratch", "out", "table"):
            chost.alloc(nm)
    full_host = synth.to_host(dev)
    for nm in ("Wr", "bias", "residual", "Ws_gate", "Ws_up", "Ws_down", "wtab", "stab", "ewt", "est"):
        if nm in full_host.t:
            chost.t[nm] = full_host.t[nm]
    if "residual" in chost.t:
        chost.t["residual"] = chost.t["residual"][:Tc].contiguous()
    chost.experts = full_host.experts
    cinsts = abi.inst_array(cplan.insts)
    times = []
    reps = 5 if mode == "sample" else 3 if a.steps < 10 else 5
    for rep in range(reps):
        # rep 0: the batch the GPU ran (its first Tc tokens); later reps: fresh activations, fresh routing
        chost.t["x"] = (full_host.t["x"][:Tc].contiguous() if rep == 0
                        else synth.randn_bf16((Tc, cfg.H), 1.0, torch.device("cpu"), 7000 + rep))
        chost._table = None
        t0 = time.perf_counter()
        rc = oracle.plow_oracle_exec_many(cinsts, len(cinsts), chost.table(), cores)
        times.append(time.perf_counter() - t0)
        assert rc == 0
    oracle.plow_oracle_pin_workers(0)
    cpu_us = statistics.median(times) * 1e6
    sample = (f"the whole batch of {T} tokens through the whole chain, {reps} repetitions with fresh activations "
              f"and routing each, median" if Tc == T else
              f"first {Tc} of {T} tokens through the whole chain, {reps} repetitions with fresh activations and "
              f"routing, median {cpu_us:.0f} us, scaled by {T}/{Tc} (extrapolated: a sample streams more weight bytes per token)")
    return {"value": round(cpu_us * T / Tc, 1), "unit": "us/layer", "cores": cores, "cores_available": os.cpu_count(),
            "cores_allowed": avail, "kind": "port",
            "tier": "scalar restatement of plow's golden CPU kernels (plow's AVX-512 / AMX tiers do not run the block-fp8 arm)",
            "pinned": True, "reps": reps, "rep_us": [round(t * 1e6, 1) for t in times], "sample": sample}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="", help="one configuration only (c1..c6); default: c2 with c3 under prefill_4k")
    ap.add_argument("--tokens", type=int, default=0)
    ap.add_argument("--arm", default="", help="override the configuration's arm (a16 | w8a8 | w8a8q | w8a8atomic | w8a8det | a4w4)")
    ap.add_argument("--zipf", type=float, default=-1.0, help="override the expert popularity exponent")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--part-bf16", action="store_true", help="bf16 partial rows between DOWN and combine (the reference's part16 arms) instead of f32")
    ap.add_argument("--raw-router", action="store_true", help="below 16 tokens: the score op carries its top-k (one launch)")
    ap.add_argument("--calib", action="store_true",
                    help="also run a plain 1 GiB device copy three times (a kernel of known traffic, "
                         "for scaling hardware counters read under rocprofv3 --pmc)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (all experts of a layer resident, no collectives); "
              f"--gpus {a.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import torch
    torch.cuda.set_device(0)
    both = not a.config
    name = a.config or "c2"
    rec, dev = run_cell(a, name, a.tokens, a.steps, a.warmup, cpu_mode=None if a.no_cpu else ("full" if name != "c3" else "sample"))
    out = {"metric": "moe_layer_us", "value": rec["value"], "unit": rec["unit"], "n_gpus": 1, "steps": a.steps,
           "warmup": a.warmup, "ms_per_step": rec["ms_per_step"], "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": rec["dtype"], "data": "synthetic"}
    out.update({k: v for k, v in rec.items() if k not in out})
    if both:
        # the other headline cell: the same layer (same expert weights) at 4096 tokens, skewed router
        psteps = max(3, min(a.steps, 10))
        prec, pdev = run_cell(a, "c3", 0, psteps, min(a.warmup, 2), share=dev, cpu_mode=None if a.no_cpu else "sample")
        out["prefill_4k"] = prec
        del pdev
    if a.calib:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    print(json.dumps(out))


if __name__ == "__main__":
    main()
