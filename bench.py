"""Benchmark of the MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|...] [--tokens T]

A step is one pass of the whole layer chain (router score -> top-k -> align -> activation quant ->
grouped gate|up + SwiGLU -> grouped down -> combine) over one batch of synthetic input that is already
resident in HBM. Prints ONE JSON line: layer time, tokens/s, the roofline of the dominant kernel
(measured live with HIP events on the launch stream) and a CPU baseline (the in-repo CPU port of
plow's path timed on this machine's host cores).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0          # MI355X datasheet
# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled
# by what the same counter reads for a 1 GiB copy): profiles/c2_decode_b64_pmc_fetch_write.txt.
# Keyed by (config, tokens, kernel); anything not measured reports null.
MEASURED_TRAFFIC = {("c2", 64, "glu"): 6511993344, ("c2", 64, "down"): 3263917773,
                    ("c3", 4096, "glu"): 11578979226, ("c3", 4096, "down"): 6576948429}
FP8_PEAK_TFLOPS = 5000.0       # dense fp8 MFMA


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c2")
    ap.add_argument("--tokens", type=int, default=0)
    ap.add_argument("--arm", default="", help="override the configuration's arm (a16 | w8a8)")
    ap.add_argument("--zipf", type=float, default=-1.0, help="override the expert popularity exponent")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib", action="store_true",
                    help="also run a plain 1 GiB device copy three times (a kernel of known traffic, "
                         "for scaling hardware counters read under rocprofv3 --pmc)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (all experts of a layer resident, no collectives); "
              f"--gpus {a.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from plow_amd import abi, layer, synth
    from plow_amd.lib import Moe

    torch.cuda.set_device(0)
    cfg = layer.config(a.config, a.tokens or None)
    if a.config == "c5":
        # Zipf(1.2)-like expert popularity through a selection bias; the prefill pair (ops 81 / 82)
        # from 128 tokens on, the decode ops (65 / 66 semantics, bf16 activations) below
        cfg.bias = True
        cfg.arm = "w8a8" if cfg.T >= 128 else "a16"
    if a.arm:
        cfg.arm = a.arm
    plan = layer.plan_layer(cfg)
    hot = 3.0 if a.config == "c3" else 0.0
    # c6: popularity falling off like rank^-0.5, as in plow's bench of this shape
    zipf = a.zipf if a.zipf >= 0.0 else {"c5": 1.2, "c6": 0.5}.get(a.config, 0.0)
    dev = synth.bind(plan, "cuda", seed=0, hot_expert=hot, zipf=zipf)
    moe = Moe(0)
    stream = torch.cuda.current_stream().cuda_stream
    insts = abi.inst_array(plan.insts)
    table = dev.table()

    def step():
        moe.exec_many(insts, table, stream)

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps

    # per-op durations, HIP events on the launch stream
    per_op = {n: [] for n in plan.names}
    for _ in range(max(5, min(a.steps, 20))):
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(len(plan.insts) + 1)]
        evs[0].record()
        for n, d in enumerate(plan.insts):
            moe.exec(d, table, stream)
            evs[n + 1].record()
        torch.cuda.synchronize()
        for n, name in enumerate(plan.names):
            per_op[name].append(evs[n].elapsed_time(evs[n + 1]) * 1e3)
    op_us = {n: statistics.mean(v) for n, v in per_op.items()}

    if a.calib:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    meta = dev.np("meta")
    cnt = meta[cfg.E_all:2 * cfg.E_all]
    hit = int((cnt > 0).sum())                       # experts whose weights must stream (incl. shared)
    eb = expert_bytes(cfg)
    H, T = cfg.H, cfg.T
    layer_bytes = hit * eb + cfg.E * H * 2 + (cfg.E * 4 if cfg.bias else 0) + 2 * T * H * 2
    dom = max(("glu", "down"), key=lambda n: op_us[n])
    frac_w = 2.0 / 3.0 if dom == "glu" else 1.0 / 3.0
    act_in = T * H * (1 if cfg.arm == "w8a8" else 2) if dom == "glu" else int(cnt.sum()) * cfg.I
    dom_bytes = hit * eb * frac_w + act_in
    achieved = dom_bytes / (op_us[dom] * 1e-6) / 1e9
    flops = 2.0 * int(cnt.sum()) * 3 * cfg.I * H + 2.0 * T * cfg.E * H

    out = {
        "metric": "moe_layer_us", "value": round(ms * 1e3, 2), "unit": "us/layer",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": {"fp8blk": "fp8_e4m3", "mxfp4": "fp4_e2m1", "fp8pc": "fp8_e4m3", "bf16": "bf16"}[cfg.enc],
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: H={cfg.H} E={cfg.E}+{cfg.n_shared} I={cfg.I} top{cfg.k} "
                               f"T={cfg.T} enc={cfg.enc} arm={cfg.arm} groups={cfg.n_group}/{cfg.topk_group}",
                   "tokens": T, "experts_hit": hit, "rows": int(cnt.sum()),
                   "rows_per_expert": {"min": int(cnt[:cfg.E].min()), "median": float(np.median(cnt[:cfg.E])),
                                       "max": int(cnt[:cfg.E].max()), "mean": float(cnt[:cfg.E].mean()),
                                       "below_64": int((cnt[:cfg.E] < 64).sum()),
                                       "pad_frac": round(float(((cnt + 63) // 64 * 64).sum() / max(1, cnt.sum()) - 1.0), 4)}},
        "tokens_per_s": round(T / (ms * 1e-3), 1),
        "layer": {"algorithmic_bytes": int(layer_bytes), "hbm_frac": round(layer_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                  "flops": flops, "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / FP8_PEAK_TFLOPS, 4)},
        "op_us": {n: round(v, 2) for n, v in op_us.items()},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((cfg.name, T, dom)),
                     "bytes_per_launch": int(dom_bytes), "us_per_launch": round(op_us[dom], 2)},
    }

    if not a.no_cpu:
        import oracle_lib as ol
        oracle = ol.load_oracle()
        cores = min(16, os.cpu_count() or 1)
        # bounded sample: the same layer on the first Tc tokens (every op of the chain, all experts those
        # tokens hit), scaled to the full batch by tokens
        Tc = min(T, 8 if cfg.T <= 256 else 16)
        ccfg = layer.config(a.config, Tc)
        cplan = layer.plan_layer(ccfg)
        chost = synth.Bound(cplan, "cpu")
        for name, sp in cplan.specs.items():
            if sp.role in ("scratch", "out", "table"):
                chost.alloc(name)
        full_host = synth.to_host(dev)
        for name in ("Wr", "bias", "residual", "Ws_gate", "Ws_up", "Ws_down"):
            if name in full_host.t:
                chost.t[name] = full_host.t[name]
        chost.t["x"] = full_host.t["x"][:Tc].contiguous()
        for name in ("wtab", "stab", "ewt", "est"):
            if name in full_host.t:
                chost.t[name] = full_host.t[name]
        chost.experts = full_host.experts
        cinsts = abi.inst_array(cplan.insts)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            rc = oracle.plow_oracle_exec_many(cinsts, len(cinsts), chost.table(), cores)
            times.append(time.perf_counter() - t0)
            assert rc == 0
        cpu_us = statistics.median(times) * 1e6
        out["cpu_baseline"] = {"value": round(cpu_us * T / Tc, 1), "unit": "us/layer", "cores": cores,
                               "kind": "port",
                               "sample": f"first {Tc} of {T} tokens through the whole chain, median of 3, "
                                         f"scaled by {T}/{Tc}; measured {cpu_us:.0f} us"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
