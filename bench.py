#!/usr/bin/env python3
"""Benchmark of the fused-MoE path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--headline-only] [--no-cpu-baseline]
                    [--calibrate-copy] [--no-sustained]

One "step" is one pass of the whole path (moe_sorting + gate/up GEMM with SiLU*up + down GEMM +
top-k combine) over one batch of synthetic, already-quantised inputs resident in HBM.  The headline
workload is the DeepSeek-V3-shaped fp8 layer at 8192 tokens (the configuration the target of the
metric is quoted on); the other benchmark configurations are reported under "workloads" in the
same JSON line.  Prints exactly one JSON line on stdout.

--calibrate-copy appends one plain device copy of 1 GiB (torch's copy kernel) after the timed
region: under `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` its reading gives the factor that
turns the counter into bytes for the GEMM kernels of the same run.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "fused-MoE TFLOP/s (prefill) + HBM GB/s (decode), % of MI355X roofline, 1 GPU"
HEADLINE = "cfg3_dsv3_fp8"
DOMINANT = "moe_gemm0_gate_up_silu"  # the kernel the roofline entry is about
# published MI355X peaks: dense MFMA TFLOP/s (TOP/s for int8) and HBM GB/s
PEAK_MFMA = {"bf16": 2500.0, "fp8": 5000.0, "int8": 5000.0}
PEAK_HBM = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def run_workload(cfg, steps, warmup, seed=0, fused_quant=0, hot_expert=False, weight_permute=0, min_warm_ms=0.0):
    """Times `steps` passes of the path (fused_quant 2: the int8 path re-quantises the intermediate activations
    per row and runs the down GEMM on int8 MFMAs).  The dominant kernel's duration comes from HIP events the
    library records on the launch stream inside the timed region, the other kernels' from an untimed
    pass just before it."""
    import torch

    import therock_amd as ta
    from therock_amd import _lib
    from therock_amd import inputs as mi

    dev = torch.device("cuda:0")
    inp = mi.make_inputs_torch(cfg, dev, seed)
    if hot_expert:  # expert 0 in every token's top-k: one expert with `tokens` rows among decode-sized ones
        ids = inp["topk_ids"].clone()
        ids[~(ids == 0).any(dim=1), cfg.topk - 1] = 0
        inp["topk_ids"] = ids.contiguous()
    if weight_permute:  # g and d as ck_tile's example hands them to its kernel (b_nr_kr_kw_nw_kv), read in place
        inp["g"], inp["d"] = ta.permute_weights(inp["g"]), ta.permute_weights(inp["d"])
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit, fused_quant=fused_quant,
                                 weight_permute=weight_permute)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, dev)
    args = ta.make_args(traits, buf, inp["a"], inp["g"], inp["d"], inp["topk_ids"], inp["topk_weight"],
                        a_scale=inp["a_scale"], g_scale=inp["g_scale"], d_scale=inp["d_scale"])
    for _ in range(warmup):
        assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    # (the workloads reported beside the headline one: decode-sized passes take well under a millisecond, and the
    # first 10 to 20 ms of passes after the host has been busy building inputs run up to 8 % slower - keep warming
    # up until that much GPU time has gone by)
    w0 = time.perf_counter()
    while (time.perf_counter() - w0) * 1e3 < min_warm_ms:
        for _ in range(10):
            ta.fused_moe(traits, args)
        torch.cuda.synchronize()
    # Per-kernel durations of every kernel: an untimed pass with an event pair around each launch.  Those
    # records sit between the launches and lengthen a pass by a few microseconds each, so the timed region
    # below keeps only the pair around the dominant kernel (the gate+up GEMM), which is what the roofline
    # entry is computed from.
    _lib.profile_start()
    for _ in range(max(3, min(steps, 10))):
        ta.fused_moe(traits, args)
    torch.cuda.synchronize()
    kern = _lib.profile_stop()
    _lib.profile_start(kinds=[DOMINANT])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ta.fused_moe(traits, args)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    dom = _lib.profile_stop()
    if DOMINANT in dom:
        kern[DOMINANT] = dom[DOMINANT]
    ms = (t1 - t0) * 1e3 / steps
    post_pad = int(buf.total[0])
    active = int(torch.unique(inp["topk_ids"]).numel())
    kavg = {k: v[0] / max(v[1], 1) for k, v in kern.items()}
    T, K, H, I = cfg.tokens, cfg.topk, cfg.hidden, cfg.inter
    flops0, flops1 = 4.0 * T * K * H * I, 2.0 * T * K * H * I
    byt = mi.decode_bytes(cfg, active, post_pad)
    gemm_ms = kavg.get("moe_gemm0_gate_up_silu", 0) + kavg.get("moe_gemm1_down", 0) + kavg.get("moe_combine", 0) + kavg.get("moe_prep", 0)
    res = {
        "workload": cfg.name, "dtype": cfg.dtype, "fused_quant": fused_quant, "tokens": T, "hidden": H, "inter": I, "experts": cfg.experts,
        "topk": K, "block_m": cfg.unit, "tile_rows": ta.fused_moe_tile_rows(traits, T, cfg.experts, K, H, I),
        "ms_per_step": ms, "tflops": cfg.flops / ms / 1e9,
        "tokens_per_s": T / ms * 1e3, "algorithmic_GB": byt / 1e9, "hbm_GBps": byt / ms / 1e6,
        "frac_mfma_peak": cfg.flops / ms / 1e9 / PEAK_MFMA[cfg.dtype], "frac_hbm_peak": byt / ms / 1e6 / PEAK_HBM,
        "gemm_only_ms": gemm_ms, "post_pad": post_pad, "active_experts": active,
        "kernel_avg_ms": {k: round(v, 5) for k, v in kavg.items()},
        "gemm0_tflops": flops0 / kavg["moe_gemm0_gate_up_silu"] / 1e9 if "moe_gemm0_gate_up_silu" in kavg else None,
        "gemm1_tflops": flops1 / kavg["moe_gemm1_down"] / 1e9 if "moe_gemm1_down" in kavg else None,
    }
    return res, inp, buf


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "moe_gemm_hbm_traffic.txt")


def measured_traffic(workload, gemm):
    """HBM bytes per launch of the gate+up (gemm 0) or down (gemm 1) GEMM as measured with rocprofv3 counters (a
    committed summary: lines of `workload gemm0_fetch gemm0_write gemm1_fetch gemm1_write`, bytes); None when there
    is no entry."""
    try:
        for ln in open(TRAFFIC_FILE):
            f = ln.split()
            if len(f) >= 5 and f[0] == workload:
                return float(f[1 + 2 * gemm]) + float(f[2 + 2 * gemm])
    except (OSError, ValueError):
        pass
    return None


def roofline_of(cfg, res, gemm=0):
    """Roofline entry of a workload's gate+up GEMM (gemm 0, the dominant kernel: 2/3 of the FLOPs) or down GEMM
    (gemm 1).  Algorithmic work per launch: gemm0 4*T*K*H*I FLOP, bytes = the active experts' gate/up weights and
    scales + the token matrix + Y written; gemm1 2*T*K*H*I FLOP, bytes = the active experts' down weights and scales
    + Y read + the per-slot partial rows written."""
    key = "moe_gemm0_gate_up_silu" if gemm == 0 else "moe_gemm1_down"
    kms = res["kernel_avg_ms"].get(key)
    if not kms:
        return None
    T, K, H, I = cfg.tokens, cfg.topk, cfg.hidden, cfg.inter
    traffic = measured_traffic(cfg.name, gemm)
    family = ("moe_gemm_big_kernel" if res["tile_rows"] > 128 else
              "moe_gemm_decode_kernel" if res["tile_rows"] == 32 and gemm == 0 else "moe_gemm_kernel")
    kname = family + (" (gemm0: gate+up, SiLU*up)" if gemm == 0 else " (gemm1: down)")
    b = {"bf16": 2, "fp8": 1, "int8": 1}[cfg.dtype]
    y_b = 1 if cfg.dtype == "fp8" else 2
    ae = res["active_experts"]
    if gemm == 0:
        flop = 4.0 * T * K * H * I
        byt = ae * 2 * I * H * b + ae * 2 * I * 4 + T * H * b + res["post_pad"] * I * y_b
    else:
        flop = 2.0 * T * K * H * I
        yq_b = 1 if res.get("fused_quant") else y_b  # re-quantised intermediate activations
        byt = ae * H * I * b + ae * H * 4 + res["post_pad"] * I * yq_b + res["post_pad"] * H * 2
    gbps = byt / kms / 1e6
    tflops = flop / kms / 1e9
    # prefill-sized workloads (tens of rows or more per expert) are graded against the MFMA peak, the
    # decode regime against HBM; the other fraction is reported beside it
    if T * K / cfg.experts >= 64:
        return {"kernel": kname, "bound": "mfma", "achieved": tflops, "peak": PEAK_MFMA[cfg.dtype], "unit": "TFLOP/s",
                "frac": tflops / PEAK_MFMA[cfg.dtype], "avg_launch_ms": kms, "traffic": traffic,
                "algorithmic_flop": flop, "algorithmic_bytes": byt, "hbm_GBps": gbps, "hbm_frac": gbps / PEAK_HBM}
    return {"kernel": kname, "bound": "hbm", "achieved": gbps, "peak": PEAK_HBM, "unit": "GB/s",
            "frac": gbps / PEAK_HBM, "avg_launch_ms": kms, "traffic": traffic, "algorithmic_bytes": byt,
            "algorithmic_flop": flop, "mfma_TFLOPs": tflops, "mfma_frac": tflops / PEAK_MFMA[cfg.dtype]}


def _smi_sample():
    """One reading of the package power (W) and the shader clock (MHz) from amd-smi; None where it cannot be had."""
    import subprocess

    try:
        out = subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    return parse_smi(out)


def parse_smi(text):
    """(socket power in W, clock of the first shader engine in MHz or None) from `amd-smi metric -p -c`; None without
    a power reading."""
    import re

    pw = re.search(r"SOCKET_POWER:\s*([0-9.]+)\s*W", text)
    ck = re.search(r"GFX_0:\s*\n\s*CLK:\s*([0-9.]+)\s*MHz", text)
    if not pw:
        return None
    return float(pw.group(1)), (float(ck.group(1)) if ck else None)


def _power_cap():
    import re
    import subprocess

    try:
        out = subprocess.run(["rocm-smi", "--showmaxpower"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r"Max Graphics Package Power \(W\):\s*([0-9.]+)", out)
    return float(m.group(1)) if m else None


def run_power_probe(cfg, samples=3):
    """Package power and shader clock while the headline path runs back to back.  Outside the timed region; None when
    amd-smi gives no reading."""
    import torch

    import therock_amd as ta
    from therock_amd import inputs as mi

    if _smi_sample() is None:
        return None
    dev = torch.device("cuda:0")
    inp = mi.make_inputs_torch(cfg, dev, 0)
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, dev)
    args = ta.make_args(traits, buf, inp["a"], inp["g"], inp["d"], inp["topk_ids"], inp["topk_weight"],
                        a_scale=inp["a_scale"], g_scale=inp["g_scale"], d_scale=inp["d_scale"])
    # The readings are taken by a child process that is started while the device is idle and then runs amd-smi a few
    # times on its own; this process meanwhile does nothing but queue passes.  (It must not start a process while it
    # is submitting work: a fork makes the pages of the submitting process copy-on-write, and a launch that writes
    # its kernel arguments into such a page while the child still exists moves the page away from under the GPU.)
    import subprocess

    torch.cuda.synchronize()
    script = f"sleep 1.5; for i in $(seq {samples}); do timeout -k 2 8 amd-smi metric -p -c; echo ====; sleep 0.3; done"
    try:
        child = subprocess.Popen(["bash", "-c", script], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
    except OSError:
        return None
    deadline = time.perf_counter() + 30.0
    while child.poll() is None and time.perf_counter() < deadline:
        for _ in range(8):
            ta.fused_moe(traits, args)
        torch.cuda.synchronize()
    torch.cuda.synchronize()
    if child.poll() is None:
        child.kill()
    try:
        out = child.communicate(timeout=15)[0]
    except subprocess.TimeoutExpired:
        return None
    watts, clocks = [], []
    for part in out.split("===="):
        r = parse_smi(part)
        if r:
            watts.append(r[0])
            if r[1]:
                clocks.append(r[1])
    if not watts:
        return None
    return {"socket_power_w": sum(watts) / len(watts), "power_cap_w": _power_cap(),
            "gfx_clock_mhz": sum(clocks) / len(clocks) if clocks else None, "samples": len(watts),
            "what": f"amd-smi while {cfg.name} passes run back to back"}


def run_sustained(dtype):
    """The matrix-core rate this device sustains for the workload's MFMA instruction on register operands, with no
    memory traffic at all: with operands that toggle like real data (the ceiling of any kernel on this box, set by
    the package's power limit) and with zeros (where the published peak is reached)."""
    from therock_amd import _lib

    rnd = _lib.mfma_sustained(dtype, 1600, False)
    zer = _lib.mfma_sustained(dtype, 600, True)
    return {"random_operands": rnd, "zero_operands": zer, "unit": "TFLOP/s",
            "what": "independent MFMAs on register operands, 2 waves per SIMD, no memory traffic; measured live"}


def run_router(cfg, steps, warmup):
    """Router front-end of the same workload (softmax or sigmoid over [tokens, experts] fp32 logits,
    top-k): an HBM-bound pass over the logits, reported beside the path it feeds."""
    import torch

    import therock_amd as ta
    from therock_amd import _lib

    g = torch.Generator(device="cuda").manual_seed(1)
    logits = torch.randn((cfg.tokens, cfg.experts), device="cuda", generator=g)
    act = "sigmoid" if cfg.router.startswith("sigmoid") else "softmax"
    for _ in range(warmup):
        ta.topk_softmax(logits, cfg.topk, activation=act, renormalize=True)
    torch.cuda.synchronize()
    _lib.profile_start()
    for _ in range(steps):
        ta.topk_softmax(logits, cfg.topk, activation=act, renormalize=True)
    torch.cuda.synchronize()
    k = _lib.profile_stop()["topk_softmax"]
    ms = k[0] / max(k[1], 1)
    byt = cfg.tokens * cfg.experts * 4 + cfg.tokens * cfg.topk * 8
    return {"kernel": "topk_softmax_kernel", "activation": act, "avg_launch_ms": ms, "bytes": byt,
            "GBps": byt / ms / 1e6 if ms > 0 else None}


def run_neighbours(cfg, inp, buf, steps):
    """The callers and data formats either side of the path, on the headline workload's shapes: per-token
    activation quantisation, MoE smooth-quant, the weight pre-shuffle (a slice of the experts), and the gate+up /
    down GEMMs as stand-alone launches on the sorted arrays the path has just produced.  Wall time per call from
    events on the launch stream; bytes are the algorithmic ones of each step."""
    import torch

    import therock_amd as ta

    T, H, I, E, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.topk
    qd = "fp8" if cfg.dtype == "fp8" else "int8"
    out = {}

    def timed(fn, n):
        for _ in range(3):  # (the first calls on freshly allocated outputs run up to 15 % slower)
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((T, H), device="cuda", generator=g).to(torch.bfloat16)
    ms = timed(lambda: ta.rowwise_quant(x, qd), steps)
    out["rowwise_quant"] = {"ms": ms, "GBps": T * H * 3 / ms / 1e6, "what": f"[{T}, {H}] bf16 -> {qd} + scale"}
    sm = torch.rand((E, H), device="cuda", generator=g) + 0.5
    ms = timed(lambda: ta.moe_smoothquant(x, sm, inp["topk_ids"], qd), max(3, steps // 2))
    out["moe_smoothquant"] = {"ms": ms, "GBps": (T * H * 2 + K * T * H) / ms / 1e6,
                              "what": f"[{T}, {H}] bf16 -> [{K}, {T}, {H}] {qd} + scales"}
    del sm
    ne = min(E, 32)
    w = inp["d"][:ne]
    ms = timed(lambda: ta.permute_weights(w), 3)
    out["permute_weights"] = {"ms": ms, "GBps": 2 * w.numel() * w.element_size() / ms / 1e6,
                              "what": f"{ne} experts of d [{H}, {I}] to ck_tile's pre-shuffled layout"}
    if cfg.dtype in ("bf16", "fp8"):
        y = torch.empty((T * K, I), dtype=torch.bfloat16, device="cuda")
        # the caller owns the workspace: allocated once, outside the timed calls
        ws0 = torch.empty((ta.moe_flatmm_get_workspace_size(ta.GEMM1_GATE_UP, inp["a"], inp["g"], y, buf.sorted_ids,
                                                            buf.sorted_eid, buf.total, T, K, cfg.unit),),
                          dtype=torch.uint8, device="cuda")
        ms = timed(lambda: ta.moe_flatmm(ta.GEMM1_GATE_UP, inp["a"], inp["g"], y, buf.sorted_ids, buf.sorted_eid, buf.total,
                                         T, K, cfg.unit, scale_m=inp["a_scale"], scale_n=inp["g_scale"], workspace=ws0),
                   max(3, steps // 2))
        out["flatmm_gate_up"] = {"ms": ms, "tflops": 4.0 * T * K * H * I / ms / 1e9, "what": "stand-alone gate+up GEMM, bf16 C"}
        if cfg.dtype == "fp8":
            yq, ys = ta.rowwise_quant(y, "fp8")
        else:
            yq, ys = y, None
        c = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
        del ws0
        ws1 = torch.empty((ta.moe_flatmm_get_workspace_size(ta.GEMM2, yq, inp["d"], c, buf.sorted_ids, buf.sorted_eid,
                                                            buf.total, T, K, cfg.unit),), dtype=torch.uint8, device="cuda")
        ms = timed(lambda: ta.moe_flatmm(ta.GEMM2, yq, inp["d"], c, buf.sorted_ids, buf.sorted_eid, buf.total, T, K, cfg.unit,
                                         sorted_weights=buf.sorted_w, scale_m=ys, scale_n=inp["d_scale"], workspace=ws1),
                   max(3, steps // 2))
        out["flatmm_down"] = {"ms": ms, "tflops": 2.0 * T * K * H * I / ms / 1e9,
                              "what": "stand-alone down GEMM + combine, added to bf16 C"}
    return out


def cpu_baseline(cfg, inp, max_rows=256, n_experts=3):
    """ck_tile's own host reference (oracle/_ref) timed on this machine's cores on a bounded
    sample of the workload: every row routed to each of a few experts (T'=rows, E'=1, K'=1 per expert), operands
    de-quantised to fp32 because the reference ignores scale tensors.  Falls back to the C
    restatement when oracle/_ref is not built."""
    import numpy as np
    import torch

    import oracle

    H, I = cfg.hidden, cfg.inter

    def deq(x, scale):
        x = x.float()
        return (x * scale[..., None]) if scale is not None else x

    def rows(x, idx):  # row gather that also works for 8-bit float storage
        return x.view(torch.uint8)[idx].view(x.dtype) if x.element_size() == 1 else x[idx]

    # the experts of the first token's first slots, one E'=1 problem each: 10 to 20 s of CPU work on the headline workload
    experts = []
    for e in inp["topk_ids"][0].tolist():
        if e not in experts:
            experts.append(int(e))
    experts = experts[:n_experts]
    use_ref = oracle.ck_ref() is not None
    flops, dt, n_rows = 0.0, 0.0, []
    for e0 in experts:
        t_idx, k_idx = torch.nonzero(inp["topk_ids"] == e0, as_tuple=True)
        t_idx, k_idx = t_idx[:max_rows], k_idx[:max_rows]
        n = int(t_idx.numel())
        a = deq(rows(inp["a"], t_idx), None if inp["a_scale"] is None else inp["a_scale"][t_idx]).cpu().numpy()
        g = deq(inp["g"][e0], None if inp["g_scale"] is None else inp["g_scale"][e0]).cpu().numpy()[None]
        d = deq(inp["d"][e0], None if inp["d_scale"] is None else inp["d_scale"][e0]).cpu().numpy()[None]
        ids = np.zeros((n, 1), dtype=np.int32)
        w = inp["topk_weight"][t_idx, k_idx].cpu().numpy().reshape(n, 1)
        t0 = time.perf_counter()
        if use_ref:
            s = oracle.ck_moe_sorting(ids, w, 1, cfg.unit)
            oracle.ck_fused_moe(a, g, d, *s, cfg.unit, n, 1, H, I, 1, f32_inputs=True)
        else:
            s = oracle.moe_sorting(ids, w, 1, cfg.unit)
            oracle.fused_moe(a, oracle.DT_F32, g, oracle.DT_F32, d, oracle.DT_F32, *s, cfg.unit, n, 1, H, I, 1)
        dt += time.perf_counter() - t0
        flops += 6.0 * n * H * I
        n_rows.append(n)
    sample = (f"the rows routed to experts {experts} of {cfg.name} ({n_rows} rows), each as a T'=rows, E'=1, K'=1 problem "
              f"(same H={H}, I={I}), de-quantised fp32 operands")
    if use_ref:
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference", "seconds": dt,
                "sample": sample + "; ck_tile::reference_moe_sorting + reference_fused_moe (GEMM phase is "
                "single-threaded by construction, the final top-k reduce uses all cores)"}
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
            "seconds": dt, "sample": sample + "; C restatement of the ck_tile reference (oracle/moe_oracle.c)"}


MAX_LINE_BYTES = 4096  # the one JSON line on stdout stays below this; everything else goes to stderr


def _r(x, n=4):
    return None if x is None else float(f"{x:.{n}g}")


def _roof_short(r):
    """The roofline fields a reader of the one-line result needs (the long form is printed on stderr)."""
    if not r:
        return None
    out = {"kernel": r["kernel"], "bound": r["bound"], "achieved": _r(r["achieved"], 5), "peak": r["peak"],
           "unit": r["unit"], "frac": _r(r["frac"]), "traffic": r.get("traffic"),
           "avg_launch_ms": _r(r["avg_launch_ms"], 5), "algorithmic_bytes": r.get("algorithmic_bytes"),
           "algorithmic_flop": r.get("algorithmic_flop")}
    if "sustained_peak" in r:  # the rate this device sustains for the same MFMA on register operands, measured live
        out["sustained_peak"] = _r(r["sustained_peak"], 5)
        out["frac_of_sustained"] = _r(r["frac_of_sustained"])
    return out


def _workload_short(r):
    """ms per pass, the rate the workload is graded on and its fraction of that peak."""
    if "error" in r:
        return {"error": r["error"][:80]}
    rows_per_expert = r["tokens"] * r["topk"] / r["experts"]
    if rows_per_expert >= 64:
        return {"ms": _r(r["ms_per_step"]), "rate": _r(r["tflops"]), "unit": "TFLOP/s", "frac": _r(r["frac_mfma_peak"], 3)}
    return {"ms": _r(r["ms_per_step"]), "rate": _r(r["hbm_GBps"]), "unit": "GB/s", "frac": _r(r["frac_hbm_peak"], 3)}


def build_line(cfg, steps, warmup, res, roof, roof1, cpu, router, neighbours, workloads, sustained=None, power=None):
    """The one JSON line of the result: headline fields, the two roofline entries, the CPU baseline and one short
    record per other workload.  Kept under MAX_LINE_BYTES: readers that keep only the tail of stdout must still
    see a whole line."""
    if cpu:
        cpu = {k: (_r(v, 5) if isinstance(v, float) else v) for k, v in cpu.items()}
        if len(cpu.get("sample", "")) > 300:
            cpu["sample"] = cpu["sample"][:297] + "..."
    line = {
        "metric": METRIC, "value": _r(res["tflops"], 6), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": _r(res["ms_per_step"], 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {"bf16": "bf16", "fp8": "fp8_e4m3", "int8": "int8"}[cfg.dtype],
        "data": "synthetic (seeded N(0,1) activations, N(0,0.02) weights, pre-quantised, resident in HBM)",
        "config": {"workload": f"{cfg.name}: tokens={cfg.tokens} hidden={cfg.hidden} inter={cfg.inter} "
                               f"experts={cfg.experts} topk={cfg.topk} block_m={cfg.unit} router={cfg.router}",
                   "path": "moe_sorting + gemm0(gate,up,SiLU*up) + gemm1(down) + combine, one stream"},
        "frac_of_mfma_peak": _r(res["frac_mfma_peak"]), "tokens_per_s": _r(res["tokens_per_s"], 6),
        "hbm_GBps": _r(res["hbm_GBps"], 5), "kernel_avg_ms": {k: _r(v, 4) for k, v in res["kernel_avg_ms"].items()},
        "roofline": _roof_short(roof), "roofline_gemm1": _roof_short(roof1), "cpu_baseline": cpu,
    }
    if sustained:
        line["mfma_sustained"] = {"random_operands": _r(sustained["random_operands"], 5),
                                  "zero_operands": _r(sustained["zero_operands"], 5), "unit": sustained["unit"],
                                  "frac_of_sustained": _r(res["tflops"] / sustained["random_operands"])}
    if power:
        line["power"] = {"socket_power_w": _r(power["socket_power_w"]), "power_cap_w": power.get("power_cap_w"),
                         "gfx_clock_mhz": _r(power.get("gfx_clock_mhz"))}
    if router and "avg_launch_ms" in router:
        line["router_ms"] = _r(router["avg_launch_ms"])
    if neighbours and "error" not in neighbours:
        line["neighbours_ms"] = {k: _r(v["ms"]) for k, v in neighbours.items()}
    line["workloads"] = {name: _workload_short(r) for name, r in workloads.items()}
    # never let the line outgrow what a tail of stdout holds: drop the optional parts, longest first
    for key in ("workloads", "neighbours_ms", "kernel_avg_ms"):
        if len(json.dumps(line, separators=(",", ":"))) < MAX_LINE_BYTES:
            break
        line.pop(key, None)
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=HEADLINE)
    ap.add_argument("--headline-only", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true")
    ap.add_argument("--no-sustained", action="store_true", help="skip the measurement of the sustained MFMA rate")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="the named workload, the kernels either side of the path and the router only (profiling runs)")
    # variations of the named workload, for profiling runs of what `extra_workloads` reports
    ap.add_argument("--tokens", type=int, default=0, help="token count instead of the workload's own")
    ap.add_argument("--fused-quant", type=int, default=0, choices=(0, 2),
                    help="int8 workloads: 2 = re-quantise the intermediate activations (down GEMM on int8 MFMAs)")
    ap.add_argument("--router", default="", help="routing instead of the workload's own (e.g. zipf)")
    ap.add_argument("--hot-expert", action="store_true", help="expert 0 in every token's top-k")
    ap.add_argument("--weight-permute", type=int, default=0, choices=(0, 1), help="1 = weights in ck_tile's pre-shuffled layout")
    ap.add_argument("--name", default="", help="name to report the varied workload under")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures one GPU only; run with --gpus 1 (the path is single-GPU: across "
                 "GPUs the experts would be sharded with the sort's local-expert mask, which is not built here)")
    import torch

    from therock_amd import inputs as mi

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    cfg = mi.CONFIGS[a.workload]
    if a.tokens or a.router or a.name:
        cfg = cfg.scaled(name=a.name or f"{cfg.name}_t{a.tokens or cfg.tokens}{'_' + a.router if a.router else ''}",
                         tokens=a.tokens or cfg.tokens, router=a.router or cfg.router)
    log(f"[bench] {cfg}")
    res, inp, buf = run_workload(cfg, a.steps, a.warmup, fused_quant=a.fused_quant, hot_expert=a.hot_expert,
                                 weight_permute=a.weight_permute)
    log(f"[bench] {cfg.name}: {res['ms_per_step']:.3f} ms/step, {res['tflops']:.1f} TFLOP/s, kernels {res['kernel_avg_ms']}")
    roof = roofline_of(cfg, res)
    if a.calibrate_copy:
        src = torch.arange(1 << 28, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        log(f"[bench] calibration copy: {src.numel() * 4} bytes read, {dst.numel() * 4} bytes written")
        del src, dst
    sustained = None
    if not a.no_sustained:
        try:
            sustained = run_sustained(cfg.dtype)
            log(f"[bench] sustained MFMA rate: {sustained}")
            for r in (roof,):
                if r and r["bound"] == "mfma":
                    r["sustained_peak"] = sustained["random_operands"]
                    r["frac_of_sustained"] = r["achieved"] / sustained["random_operands"]
        except Exception as e:
            log(f"[bench] sustained MFMA rate failed: {e!r}")
    power = None
    if not a.no_sustained:
        try:
            power = run_power_probe(cfg)
            log(f"[bench] power while the path runs: {power}")
            torch.cuda.empty_cache()
        except Exception as e:
            log(f"[bench] power probe failed: {e!r}")
    cpu = None
    if not a.no_cpu_baseline:
        try:
            cpu = cpu_baseline(cfg, inp)
            log(f"[bench] cpu baseline: {cpu}")
        except Exception as e:  # the baseline is a report, never a reason to lose the measurement
            log(f"[bench] cpu baseline failed: {e!r}")
    neighbours = None
    if not a.headline_only:  # (a profiled --headline-only run holds launches of the path and the router only)
        try:
            neighbours = run_neighbours(cfg, inp, buf, a.steps)
            log(f"[bench] neighbours: {neighbours}")
        except Exception as e:
            neighbours = {"error": repr(e)}
    del inp, buf
    torch.cuda.empty_cache()
    try:
        router = run_router(cfg, a.steps, a.warmup)
        log(f"[bench] router: {router}")
    except Exception as e:
        router = {"error": repr(e)}

    others = {}
    if not a.headline_only and not a.no_other_workloads:
        for name, c in mi.CONFIGS.items():
            if name == cfg.name:
                continue
            try:
                steps = max(5, a.steps // 2)
                r, i2, b2 = run_workload(c, steps, a.warmup, min_warm_ms=30.0)
                r["roofline"] = roofline_of(c, r)
                r["roofline_gemm1"] = roofline_of(c, r, 1)
                others[name] = r
                log(f"[bench] {name}: {r['ms_per_step']:.3f} ms/step, {r['tflops']:.1f} TFLOP/s, "
                    f"{r['hbm_GBps']:.0f} GB/s, kernels {r['kernel_avg_ms']}")
                del i2, b2
                torch.cuda.empty_cache()
            except Exception as e:
                log(f"[bench] {name} failed: {e!r}")
                others[name] = {"error": repr(e)}

    # Beyond the benchmark configurations: the int8 model at a prefill-sized token count, with the intermediate
    # activations kept in bf16 (fused_quant 0) or re-quantised to int8 so that the down GEMM runs on int8 MFMAs
    # (fused_quant 2), batches between decode and prefill (40 rows per expert), and decode-sized batches whose routing
    # is skewed (Zipf; one expert in every token's top-k).
    extra = {}
    if not a.headline_only and not a.no_other_workloads:
        i8 = mi.CONFIGS["cfg4_decode_int8_t256"]
        cases = {
            "cfg4_model_int8_t8192_fused_quant0": (i8.scaled(name="cfg4_model_int8_t8192_fused_quant0", tokens=8192), {}),
            "cfg4_model_int8_t8192_fused_quant2": (i8.scaled(name="cfg4_model_int8_t8192_fused_quant2", tokens=8192), {"fused_quant": 2}),
            # 40 rows per expert: the decode kernel with two token blocks per tile
            "cfg4_model_int8_t640": (i8.scaled(name="cfg4_model_int8_t640", tokens=640), {}),
            "cfg2_mixtral_bf16_t160": (mi.CONFIGS["cfg2_mixtral_bf16"].scaled(name="cfg2_mixtral_bf16_t160", tokens=160), {}),
            "cfg4_decode_int8_t256_zipf": (i8.scaled(name="cfg4_decode_int8_t256_zipf", router="zipf"), {}),
            # fp8: the sort sees ~40 active experts of ~70 rows and takes the 320-row tiles (the host's average says 8 rows)
            "cfg3_dsv3_fp8_t256_zipf": (mi.CONFIGS["cfg3_dsv3_fp8"].scaled(name="cfg3_dsv3_fp8_t256_zipf", tokens=256, router="zipf"), {}),
            "cfg4_decode_int8_t256_hot_expert": (i8.scaled(name="cfg4_decode_int8_t256_hot_expert"), {"hot_expert": True}),
            # the headline workload and the decode workload with weights in ck_tile's pre-shuffled layout
            "cfg3_dsv3_fp8_preshuffled": (mi.CONFIGS["cfg3_dsv3_fp8"].scaled(name="cfg3_dsv3_fp8_preshuffled"), {"weight_permute": 1}),
            "cfg4_decode_int8_t64_preshuffled": (mi.CONFIGS["cfg4_decode_int8_t64"].scaled(name="cfg4_decode_int8_t64_preshuffled"),
                                                 {"weight_permute": 1}),
        }
        for name, (c, kw) in cases.items():
            try:
                r, i2, b2 = run_workload(c, max(5, a.steps // 2), a.warmup, min_warm_ms=30.0, **kw)
                r["roofline"] = roofline_of(c, r)
                r["roofline_gemm1"] = roofline_of(c, r, 1)
                extra[name] = r
                log(f"[bench] {name}: {r['ms_per_step']:.3f} ms/step, {r['tflops']:.1f} TFLOP/s, "
                    f"{r['hbm_GBps']:.0f} GB/s, kernels {r['kernel_avg_ms']}")
                del i2, b2
                torch.cuda.empty_cache()
            except Exception as e:
                log(f"[bench] {name} failed: {e!r}")
                extra[name] = {"error": repr(e)}

    for group, items in (("workloads", others), ("extra_workloads", extra)):
        for name, r in items.items():  # the full per-workload records go to stderr, one JSON object per line
            log("[bench-detail] " + json.dumps({"group": group, "name": name, **r}))
    log("[bench-detail] " + json.dumps({"group": "headline", "name": cfg.name, **res, "router": router,
                                        "neighbours": neighbours}))
    roof1 = roofline_of(cfg, res, 1)
    if sustained and roof1 and roof1["bound"] == "mfma":
        roof1["sustained_peak"] = sustained["random_operands"]
        roof1["frac_of_sustained"] = roof1["achieved"] / sustained["random_operands"]
    line = build_line(cfg, a.steps, a.warmup, res, roof, roof1, cpu, router, neighbours, {**others, **extra}, sustained, power)
    print(json.dumps(line, separators=(",", ":")), flush=True)


if __name__ == "__main__":
    main()
