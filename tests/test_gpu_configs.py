"""The benchmark configurations at their real shapes: routing bit-exact, outputs within the
benchmark tolerance. Configurations too large for the oracle to replay whole (the prefill sizes) are
checked on routing for every token and, for a sample of aligned rows chosen from the expert segments
themselves, on the intermediate, the partials and the layer output: a token's results depend only on
its own activation row and the weights, so the oracle replays the sampled rows' tokens as a small
batch over the same weights (the method of plow's runtime/tests/moe_pf_w8a8_gfx950_test.hip:144-160,
:315-341: sampled routed rows, per-row relative L2 error, mean / p99 / max)."""
import dataclasses

import numpy as np
import pytest
import torch

import oracle_lib as ol
from gpu_harness import (assert_output_close, assert_routing_equal, both, run_device, run_oracle)
from plow_amd import abi, layer, synth

pytestmark = pytest.mark.gpu

# per-row relative L2 bars of the sampled comparison (device against oracle over the same bytes; the
# two differ in the f32 order inside one matrix instruction and in the hardware exponential of the
# tiled epilogue): fp8 / bf16 intermediate as plow's own GPU test holds it (3e-2,
# runtime/tests/moe_gemma_gfx950_test.c:1080-1203). A row whose largest intermediate value lands one
# bf16 step apart gets a slightly different quantization scale on the two sides, and with it a
# different rounding of many of its fp8 codes (measured: per-row relL2 up to 2.7e-2 on such rows, 5e-4
# on average); its partial inherits that, so the partials carry the intermediate's bar. The layer
# output sums k of them.
REL_L2_MID = 3e-2
REL_L2_PART = 3e-2
REL_L2_OUT = 2e-2


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def test_c1_small_bf16_layer(moe, oracle):
    cfg = layer.config("c1")
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    assert_output_close(dev.np("out"), host.np("out"), "c1 out")


@pytest.mark.parametrize("B", [1, 16, 128])
def test_c4_kimi_k2_mxfp4_decode(moe, oracle, B):
    cfg = layer.config("c4", B)
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"), f"c4 B={B} out")


@pytest.mark.parametrize("B", [1, 4, 14])
def test_c4_kimi_k2_mxfp4_decode_on_the_decode_expert_ops(moe, oracle, B):
    """The chain the benchmark runs at a few tokens: plow's table-driven decode experts (ops 48 / 49, slot-major
    rows) in place of the grouped ops, no op 84 among the ops timed (the plan here keeps it, for the row maps the
    routing check reads); up to 128 routed rows the matrix-vector form lists its rows from the routing table."""
    import dataclasses
    cfg = dataclasses.replace(layer.config("c4", B), arm="a16dec")
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert [i.op for i in plan.insts if i.op in (48, 49)] == [48, 49]
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"), f"c4 B={B} out (ops 48 / 49)")


def print_popularity(cnt, T, k, s=1.2):
    """The realised expert popularity (share of the tokens that chose the expert, experts sorted by it) next to
    what Zipf(s) gives: k experts drawn without replacement with weights rank^-s (10000 seeded draws by the
    Gumbel top-k construction). The configuration reaches its popularity through a selection bias added to the
    router's scores, not by sampling, so the two agree in shape (a hot head, a long thin tail), not in law."""
    E = len(cnt)
    r = np.random.default_rng(12)
    w = np.log(np.arange(1, E + 1, dtype=np.float64) ** -s)
    draws = np.argsort(-(w[None, :] + r.gumbel(size=(10000, E))), axis=1)[:, :k]
    want = np.bincount(draws.reshape(-1), minlength=E) / 10000.0
    got = np.sort(np.asarray(cnt, np.float64))[::-1] / T
    ranks = [n for n in (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128) if n <= E]
    print(f"[popularity] T={T} k={k}: share of tokens per expert by popularity rank, realised | Zipf({s})", flush=True)
    print("[popularity] " + "  ".join(f"r{n}: {got[n - 1]:.3f}|{want[n - 1]:.3f}" for n in ranks), flush=True)
    live = got > 0
    if live.sum() >= 8:
        lr = np.log(np.arange(1, E + 1))[live]
        slope = np.polyfit(lr[3:], np.log(got[live])[3:], 1)[0]
        slope_w = np.polyfit(np.log(np.arange(1, E + 1))[3:], np.log(np.maximum(want, 1e-9))[3:], 1)[0]
        print(f"[popularity] log-log slope beyond rank 3: realised {slope:.2f}, Zipf({s}) drawn without replacement {slope_w:.2f}; "
              f"experts hit {int(live.sum())}/{E}", flush=True)


def c5_config(T, arm):
    """Qwen3-shaped per-channel fp8 with the expert popularity the configuration asks for: a selection
    bias falling off like Zipf(1.2) over a seeded permutation of the experts."""
    cfg = layer.config("c5", T)
    cfg.arm = arm
    cfg.bias = True
    return cfg


@pytest.mark.parametrize("arm", ["a16", "w8a8"])
@pytest.mark.parametrize("T", [1, 8, 64])
def test_c5_qwen3_per_channel_fp8(moe, oracle, T, arm):
    print(f"[case] c5 T={T} arm={arm} zipf=1.2", flush=True)
    plan, dev, host = both(moe, oracle, c5_config(T, arm), seed=0, zipf=1.2)
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"), f"c5 T={T} {arm} out")


@pytest.mark.parametrize("T", [512, 2048])
def test_c5_qwen3_per_channel_fp8_prefill_sizes(moe, oracle, T):
    """The two sizes of the batch sweep at which the per-channel W8A8 pair (ops 32 / 81 / 32 / 82) runs
    the tiled kernels at H 4096, I 1536, E 128; the hottest expert holds (nearly) every token, i.e. up to
    sixteen 128-row tiles."""
    print(f"[case] c5 T={T} arm=w8a8 zipf=1.2", flush=True)
    cfg = c5_config(T, "w8a8")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, zipf=1.2)
    run_device(moe, plan, dev)
    cnt = check_prefill_sampled(oracle, cfg, plan, dev)
    print_popularity(cnt[:cfg.E], T, cfg.k)
    assert cnt.max() >= 0.9 * T          # Zipf(1.2): the most popular expert is chosen by (nearly) every token


def test_c5_qwen3_per_channel_fp8_bf16_activations_prefill(moe, oracle):
    """The same layer on ops 65 / 66 (bf16 activations, slot-major intermediate) at 512 tokens: from 16
    rows per expert on average these run the tiled kernels too (rows gathered by token, scattered by slot;
    DOWN reads the slot rows)."""
    T = 512
    print(f"[case] c5 T={T} arm=a16 zipf=1.2", flush=True)
    cfg = c5_config(T, "a16")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, zipf=1.2)
    run_device(moe, plan, dev)
    cnt = check_prefill_sampled(oracle, cfg, plan, dev)
    assert cnt.max() >= 0.9 * T


def test_c3_dsv3_prefill_4k(moe, oracle):
    print("[case] c3", flush=True)
    cfg = layer.config("c3")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, hot_expert=3.0)
    run_device(moe, plan, dev)
    cnt = check_prefill_sampled(oracle, cfg, plan, dev)
    assert cnt[:cfg.E].max() >= 2.0 * cnt[:cfg.E].mean()        # the skew the configuration asks for


def test_c4_kimi_k2_mxfp4_prefill_fp4_activations(moe, oracle):
    """The Kimi-K2 shape at prefill on the fp4 x fp4 arm (activations quantized to mxfp4 per 32 values), expert
    popularity falling off like 1 / rank so that the hottest expert spans more than one 128-row tile."""
    print("[case] c4 a4w4 T=2048", flush=True)
    cfg = layer.config("c4", 2048)
    cfg.arm = "a4w4"
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, zipf=1.0)
    run_device(moe, plan, dev)
    cnt = check_prefill_sampled(oracle, cfg, plan, dev)
    assert cnt[:cfg.E].max() > 128      # more than one row tile


@pytest.mark.parametrize("arm", ["w8a8", "a16"])
def test_c6_glm_tp8_slice_prefill_8k(moe, oracle, arm):
    """The shape of plow's own gfx950 prefill bench (288 experts, top-8, H 4096, I 256 per rank, 8192
    tokens), fp8 activations and bf16 activations, both on the tiled kernels."""
    print(f"[case] c6 arm={arm}", flush=True)
    cfg = layer.config("c6")
    cfg.arm = arm
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, zipf=0.5)
    run_device(moe, plan, dev)
    check_prefill_sampled(oracle, cfg, plan, dev)


def sample_aligned_rows(cfg, meta, n_target=320, seed=0):
    """Aligned rows that walk the places a tiled kernel can go wrong: first / middle / last row of every
    128-row tile of the hottest expert and of the folded shared expert, every row of the smallest
    segment (below 64 rows when there is one), first and last row of the first and last live expert,
    the row either side of every 64-row boundary of the hottest expert, and random live rows up to
    ``n_target``."""
    Ea = cfg.E_all
    rowoff, cnt = meta[:Ea].astype(np.int64), meta[Ea:2 * Ea].astype(np.int64)
    rows = []

    def tiles_of(e):
        c = int(cnt[e])
        for t0 in range(0, c, 128):
            last = min(t0 + 127, c - 1)
            rows.extend(int(rowoff[e]) + r for r in (t0, (t0 + last) // 2, last))
        for b in range(64, c, 64):
            rows.extend(int(rowoff[e]) + r for r in (b - 1, b))

    hot = int(np.argmax(cnt[:cfg.E]))
    tiles_of(hot)
    if cfg.tail:
        tiles_of(cfg.E)
    live = np.nonzero(cnt > 0)[0]
    small = live[np.argmin(cnt[live])]
    rows.extend(int(rowoff[small]) + r for r in range(min(int(cnt[small]), 64)))
    for e in (live[0], live[-1]):
        rows.extend([int(rowoff[e]), int(rowoff[e] + cnt[e] - 1)])
    r = np.random.default_rng(seed)
    all_live = np.concatenate([np.arange(rowoff[e], rowoff[e] + cnt[e]) for e in live])
    extra = max(0, n_target - len(set(rows)))
    rows.extend(int(v) for v in r.choice(all_live, size=min(extra, len(all_live)), replace=False))
    return np.array(sorted(set(rows)), dtype=np.int64), hot, int(small)


def rel_l2_rows(a, b):
    a, b = a.astype(np.float64), b.astype(np.float64)
    num = ((a - b) ** 2).sum(axis=1)
    den = np.maximum((b ** 2).sum(axis=1), 1e-30)
    return np.sqrt(num / den)


def report_rows(what, a, b, bar):
    assert np.all(np.isfinite(a)), f"{what}: non-finite values"
    rel = np.sort(rel_l2_rows(a, b))
    p99 = rel[int(0.99 * (len(rel) - 1))]
    print(f"[parity] {what}: rows={len(rel)} relL2 mean={rel.mean():.3e} p99={p99:.3e} max={rel[-1]:.3e} "
          f"maxabs={np.abs(a - b).max():.3e} (bar {bar})", flush=True)
    assert rel[-1] <= bar, (what, rel[-1])


def e4m3_to_f32(u8):
    return torch.from_numpy(np.ascontiguousarray(u8)).view(torch.float8_e4m3fn).float().numpy()


def mxfp4_to_f64(codes, scales):
    """mxfp4 rows [R][n / 2] (element 2i in the low nibble of byte i) with E8M0 rows [R][n / 32]"""
    ladder = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    c = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(codes.shape[0], -1)
    v = ladder[c & 7] * np.where(c & 8, -1.0, 1.0)
    return v * np.repeat(np.exp2(scales.astype(np.float64) - 127.0), 32, axis=1)


def check_prefill_sampled(oracle, cfg, plan, dev):
    w8a8 = cfg.arm == "w8a8"
    pc = cfg.enc == "fp8pc"
    quant = (("xq", "ascale") if pc else ("xq", "xs")) if w8a8 else ()
    # routing and activation quant for every token, on the CPU
    host = synth.Bound(plan, "cpu")
    for name in ("logit", "table", "meta", "row_token", "row_partidx", "row_gate") + quant:
        host.alloc(name)
    for name in ("x", "Wr", "bias"):
        if name in dev.t:
            host.t[name] = dev.t[name].cpu()
    run_oracle(oracle, plan, host, labels=["score", "topk", "align"] + (["quant_x"] if w8a8 else []))
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    for name in quant:
        assert np.array_equal(dev.np(name).view(np.uint8), host.np(name).view(np.uint8)), name
    meta = host.np("meta")
    cnt = meta[cfg.E_all:2 * cfg.E_all]
    print(f"[{cfg.name}] rows/expert min {cnt[:cfg.E].min()} median {np.median(cnt[:cfg.E])} max {cnt[:cfg.E].max()} "
          f"(x{cnt[:cfg.E].max() / cnt[:cfg.E].mean():.2f} mean), {int((cnt < 64).sum())} experts below 64 rows", flush=True)

    # the sample: aligned rows -> their tokens; the oracle replays those tokens as a small batch
    srows, hot, small = sample_aligned_rows(cfg, meta)
    row_token = host.np("row_token")
    pick = np.unique(row_token[srows]).astype(np.int64)
    assert row_token[srows].max() < cfg.T
    print(f"[{cfg.name}] sample: {len(srows)} aligned rows (hottest expert {hot}: {int(cnt[hot])} rows, smallest live "
          f"segment expert {small}: {int(cnt[small])} rows) over {len(pick)} tokens", flush=True)
    sub_cfg = dataclasses.replace(cfg, T=len(pick))
    sub = layer.plan_layer(sub_cfg)
    full_host = synth.to_host(dev)
    sh = synth.Bound(sub, "cpu")
    for name, sp in sub.specs.items():
        if sp.role in ("scratch", "out", "table"):
            sh.alloc(name)
    sh.t["x"] = full_host.t["x"][torch.from_numpy(pick)].contiguous()
    for name in ("Wr", "bias", "wtab", "stab", "ewt", "est"):
        if name in full_host.t:
            sh.t[name] = full_host.t[name]
    sh.experts = full_host.experts
    run_oracle(oracle, sub, sh)
    ka = cfg.k_all
    assert np.array_equal(sh.np("table")["eid"].reshape(len(pick), ka),
                          host.np("table")["eid"].reshape(cfg.T, ka)[pick])

    # every slot of every sampled token: aligned row on the device and in the replay
    def row_of_slot(partidx, n_rows, n_slots):
        inv = np.full(n_slots, -1, np.int64)
        r = np.arange(n_rows)
        ok = partidx[:n_rows] != abi.EXPERT_UNUSED
        inv[partidx[:n_rows][ok]] = r[ok]
        return inv
    inv_d = row_of_slot(host.np("row_partidx"), rows, cfg.T * ka)
    sub_rows = int(sh.np("meta")[3 * sub_cfg.E_all]) * abi.MPF_BM
    inv_s = row_of_slot(sh.np("row_partidx"), sub_rows, len(pick) * ka)
    slots_d = (pick[:, None] * ka + np.arange(ka)[None, :]).reshape(-1)
    slots_s = np.arange(len(pick) * ka)
    live = sh.np("table")["eid"] < cfg.E_all
    slots_d, slots_s = slots_d[live], slots_s[live]
    rd, rs = inv_d[slots_d], inv_s[slots_s]
    assert (rd >= 0).all() and (rs >= 0).all()
    assert set(srows.tolist()) <= set(rd.tolist())       # the chosen rows are among those compared
    rd_t = torch.from_numpy(rd).to(dev.device)

    def gather(name, idx_t):
        return dev.t[name][idx_t].cpu()

    if cfg.arm == "a4w4":
        fu_d = mxfp4_to_f64(gather("fu4", rd_t).numpy(), gather("fsc", rd_t).numpy())
        fu_s = mxfp4_to_f64(sh.np("fu4")[rs], sh.np("fsc")[rs])
        report_rows(f"{cfg.name} fu4*fsc (dequantized intermediate)", fu_d, fu_s, REL_L2_MID)
    elif w8a8 and not pc:
        fq_d = e4m3_to_f32(gather("fq", rd_t).numpy()) * np.repeat(gather("fs", rd_t).numpy(), 128, axis=1)
        fq_s = e4m3_to_f32(sh.np("fq")[rs]) * np.repeat(sh.np("fs")[rs], 128, axis=1)
        report_rows(f"{cfg.name} fq*fs (dequantized intermediate)", fq_d, fq_s, REL_L2_MID)
    else:
        # ops 65 / 66 (per-channel weights, bf16 activations) keep the intermediate by routing slot
        slot_major = pc and not w8a8
        fu_d = ol.bf2f(gather("fu", torch.from_numpy(slots_d).to(dev.device) if slot_major else rd_t)
                       .view(torch.int16).numpy().view(np.uint16))
        fu_s = ol.bf2f(sh.np("fu")[slots_s if slot_major else rs])
        report_rows(f"{cfg.name} fu (bf16 intermediate)", fu_d, fu_s, REL_L2_MID)
        if pc and w8a8:
            f8_d = e4m3_to_f32(gather("fu8", rd_t).numpy()) * gather("fscale", rd_t).numpy()[:, None]
            f8_s = e4m3_to_f32(sh.np("fu8")[rs]) * sh.np("fscale")[rs][:, None]
            report_rows(f"{cfg.name} fu8*fscale (requantized intermediate)", f8_d, f8_s, REL_L2_MID)
    part_d = gather("part", torch.from_numpy(slots_d).to(dev.device)).float().numpy()
    part_s = sh.t["part"][torch.from_numpy(slots_s)].float().numpy()
    report_rows(f"{cfg.name} part", part_d, part_s, REL_L2_PART)
    out_d = dev.np("out")[pick]
    report_rows(f"{cfg.name} out", ol.bf2f(out_d), ol.bf2f(sh.np("out")), REL_L2_OUT)
    assert_output_close(out_d, sh.np("out"), f"{cfg.name} sampled out")
    return cnt
