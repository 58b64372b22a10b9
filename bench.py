#!/usr/bin/env python3
"""Benchmark of the Mamba inference hot path on one MI355X.

A "step" is one selective-scan forward over the isolated-scan workload
(batch 8, T 2048, d_inner 1536, d_state 16, bf16 storage, SiLU gate fused),
inputs resident in HBM.  Prints ONE JSON line; `value` is algorithmic bytes per
launch / mean launch time (GB/s), the figure the HBM roofline fraction is taken from.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0
SCAN_PROFILE = os.path.join(ROOT, "profiles", "m1_scan_c2_bf16.md")


def profile_figures(profile, source, keys):
    """Figures a committed rocprofv3 summary states in machine-readable lines (`key: number`), together with the hash of
    the kernel source they were taken from (`kernels_sha16: X`).  Counter runs cannot share a process with the timed
    run, so these are read, not measured here; every figure is None when the kernel source has changed since."""
    import hashlib
    import re
    path = os.path.join(ROOT, "profiles", profile)
    try:
        text = open(path).read()
        sha = re.search(r"^kernels_sha16:\s*([0-9a-f]{16})", text, re.M).group(1)
    except (OSError, AttributeError):
        return {k: None for k in keys}, "no profile"
    now = hashlib.sha256(open(os.path.join(ROOT, "mamba_rs_amd", "csrc", source), "rb").read()).hexdigest()[:16]
    if now != sha:
        return {k: None for k in keys}, f"stale: profile taken from {source} {sha}, source is {now}"
    out = {}
    for k in keys:
        m = re.search(r"^" + re.escape(k) + r":\s*([0-9.eE+-]+)", text, re.M)
        out[k] = float(m.group(1)) if m else None
    return out, "profiles/" + profile


def profiled_scan_traffic():
    """HBM bytes per scan call (both kernels) from the FETCH_SIZE / WRITE_SIZE summary, and the instruction-issue time
    of the call from the instruction counters of the same file."""
    f, src = profile_figures("m1_scan_c2_bf16.md", "m1_scan.hip", ["traffic_bytes_per_call", "issue_bound_us_per_call"])
    n = f["traffic_bytes_per_call"]
    return (int(n) if n is not None else None), f["issue_bound_us_per_call"], src


def scan_algorithmic_bytes(batch, T, di, ds, s, gated=True):
    """delta,u read + y written (+ gate read) + B,C read + h read/write (f32) + a_neg + D."""
    act = batch * T * di * s
    return 3 * act + (act if gated else 0) + 2 * batch * T * ds * s + 2 * 4 * batch * di * ds + 4 * di * ds + 4 * di


def spin_steps(step, sync, seconds=0.15):
    """Untimed decode steps until the GPU has been under load for `seconds` (its clocks settle within about 50 ms of
    sustained work; eight steps of a small model are over before they move), as the kernel and prefill legs do."""
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        for _ in range(16):
            step()
        sync()


def loaded_libraries(names):
    """Paths of the shared libraries with these name prefixes that are mapped into this process."""
    found = set()
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                path = line.rsplit(" ", 1)[-1].strip()
                if any(os.path.basename(path).startswith(n) for n in names):
                    found.add(path)
    except OSError:
        pass
    return sorted(found)


def make_inputs(batch, T, di, ds, seed=42):
    import numpy as np
    from util import scan_inputs
    rng = np.random.default_rng(seed)
    return scan_inputs(rng, batch, T, di, ds, s4d=True)


def gpu_leg(args, inp, shape):
    import torch
    from mamba_rs_amd import ops
    batch, T, di, ds = shape
    dev = "cuda:0"
    bf = torch.bfloat16
    t = {k: torch.from_numpy(v).to(dev) for k, v in inp.items()}
    delta, u, z = t["delta"].to(bf), t["u"].to(bf), t["z"].to(bf)
    Bm, Cm = t["B"].to(bf), t["C"].to(bf)
    a_neg, D = t["a_neg"], t["D"]
    h = torch.zeros(batch, di, ds, device=dev)
    y = torch.empty_like(delta)
    ws_bytes = ops.ssm_scan_workspace_bytes(batch, T, di, ds)
    # the workspace is zeroed once here, so the op is told that its flag area is zero (MRS_SCAN_FLAGS_ZERO): the T-split
    # route then is one launch per call; every call leaves the flags zero again
    ws = torch.zeros(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    flags = ops.GATE_SILU | ops.A_S4D_REAL | ops.SCAN_FLAGS_ZERO

    def step():
        ops.ssm_scan_fwd(h, y, delta, u, Bm, Cm, a_neg, D, gate=z, flags=flags, workspace=ws)

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)            # 256 MiB read + 256 MiB written
        torch.cuda.synchronize()
    # The first calls after an idle period run with the GPU's clocks still ramping (measured: a fixed-work v_fmac kernel
    # takes 76 us per launch at first, 69 us after ~10 ms of load, 54 us at the top state).  `first_calls_ms` is the
    # contract's measurement taken right here, from idle (W warm-up calls, then K timed); then the op is run untimed for
    # --spinup-ms, and the W warm-ups + K timed calls of the headline figure follow on the machine as a serving loop sees it.
    def timed_block():
        for _ in range(args.warmup):
            h.zero_()
            step()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.steps):
            step()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.steps
    first_calls_ms = timed_block()
    if args.spinup_ms > 0:
        t_end = time.perf_counter() + args.spinup_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(50):
                step()
            torch.cuda.synchronize()
    for _ in range(args.warmup):
        h.zero_()
        step()
    torch.cuda.synchronize()
    # timed region: exactly K launches, HIP events on the launch stream (torch's current stream)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    per = []
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = start.elapsed_time(stop)
    # per-launch durations with one event pair each (a second pass, reported as the median)
    for _ in range(min(args.steps, 50)):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); step(); b.record()
        per.append((a, b))
    torch.cuda.synchronize()
    med_ms = sorted(x.elapsed_time(y_) for x, y_ in per)[len(per) // 2]
    assert torch.isfinite(y.float()).all().item()
    # side figures, each measured like the headline (the op runs untimed for a share of --spinup-ms first: the host-side
    # check above let the GPU idle, and the clocks drop within a millisecond of idling): the same call as two launches
    # (pass A, pass B), and the same call without the S4D-real shortcut -- what a trained checkpoint (a general A) gets,
    # on the route the library picks for it (two launches)
    def side_figure(fl):
        def call():
            ops.ssm_scan_fwd(h, y, delta, u, Bm, Cm, a_neg, D, gate=z, flags=fl, workspace=ws)
        t_end = time.perf_counter() + max(args.spinup_ms, 0.0) * 0.4e-3
        call()
        while time.perf_counter() < t_end:
            for _ in range(50):
                call()
            torch.cuda.synchronize()
        for _ in range(3):
            call()
        ta, tb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ta.record()
        for _ in range(20):
            call()
        tb.record()
        torch.cuda.synchronize()
        return ta.elapsed_time(tb) / 20
    two_ms = side_figure(ops.GATE_SILU | ops.A_S4D_REAL | ops.SCAN_TWO_LAUNCHES)
    gen_ms = side_figure(ops.GATE_SILU | ops.SCAN_FLAGS_ZERO)
    return dict(ms_per_step=ev_ms / args.steps, wall_ms_per_step=wall_ms / args.steps, median_launch_ms=med_ms,
                general_a_ms_per_step=gen_ms, two_launch_ms_per_step=two_ms, first_calls_ms=first_calls_ms)


def cpu_leg(inp, shape, nbytes, budget_s=12.0):
    """The oracle's restatement of the reference CPU scan (src/mamba_ssm/cpu/prefill.rs:241-315),
    all host cores, f32, same workload; repeated until ~budget_s of CPU time."""
    import numpy as np
    import orc
    batch, T, di, ds = shape
    h0 = np.zeros((batch, di, ds), np.float32)
    silu_z = inp["z"]
    args = (h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    orc.m1_scan_cpu(*args, gate=silu_z, gate_mode=2)  # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        orc.m1_scan_cpu(*args, gate=silu_z, gate_mode=2)
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2]
    return dict(value=nbytes / best / 1e9, unit="GB/s", cores=orc.num_threads(), kind="port",
                sample=f"full workload (batch {batch} x T {T} x d_inner {di} x d_state {ds}, f32, gated), median of "
                       f"{len(times)} runs of the oracle's restatement of the reference CPU scan; bytes counted as the "
                       f"GPU leg's algorithmic bytes so the ratio is a time ratio",
                ms_per_step=best * 1e3)


def cpu_prefill_sample(cfg_kw, sample_layers, sample_tokens, full_tokens, seed=42):
    """The oracle's restatement of the reference's CPU forward_prefill (PrefillMode::Parallel,
    src/mamba_ssm/cpu/prefill.rs:420-696) on a bounded sample: `sample_layers` of the model's layers over one sequence of
    `sample_tokens` tokens, all host cores; scaled linearly in layers and tokens (the pipeline is O(layers x T)) to the
    full workload.  A port (the Rust binary needs cargo, probed below), a baseline only."""
    import shutil
    import numpy as np
    import orc
    from mamba_rs_amd import MambaConfig
    cfg = MambaConfig(**{**cfg_kw, "n_layers": sample_layers})
    P = orc.M1Params(cfg.d_model, cfg.d_state, cfg.d_conv, cfg.expand, sample_layers, cfg.d_model, seed=seed)
    x = (np.random.default_rng(seed).standard_normal((sample_tokens, cfg.d_model)) * 0.02).astype(np.float32)
    cs, ss = orc.m1_zero_state(P)
    orc.m1_backbone_prefill(P, x[:8], cs, ss, identity_proj=True)          # warm-up
    times = []
    for _ in range(3):
        cs, ss = orc.m1_zero_state(P)
        t0 = time.perf_counter(); orc.m1_backbone_prefill(P, x, cs, ss, identity_proj=True); times.append(time.perf_counter() - t0)
    ts = sorted(times)[1]
    scale = (cfg_kw["n_layers"] / sample_layers) * (full_tokens / sample_tokens)
    return {"kind": "port", "cargo_on_box": shutil.which("cargo") is not None, "cores": orc.num_threads(),
            "sample": f"{sample_layers} of {cfg_kw['n_layers']} layers x {sample_tokens} tokens of one sequence, f32, median of 3",
            "sample_ms": ts * 1e3, "scaled_to_full_ms": ts * scale * 1e3, "tok_per_s": full_tokens / (ts * scale)}


DEFAULT_LEGS = "c1,lm,lm28,published,m1_kernels,m3,m3_engine"
MFMA_BF16_PEAK_TFLOPS = 2500.0


def m1_step_bytes(cfg, B, es, vocab=0):
    """Algorithmic bytes of one decode step of a Mamba-1 backbone: every layer's weights once, conv and SSM state read
    and written, the residual row; plus the tied head's table when a vocabulary is given."""
    dm, di, ds, dc, dr = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank()
    layer = es * (dm * 2 * di + di * (dr + 2 * ds) + dr * di + di * dm) + 2 * 4 * B * di * (ds + dc) + 2 * 4 * B * dm
    return cfg.n_layers * layer + ((vocab + 63) // 64 * 64) * dm * es


def m3_step_bytes(cfg, B, es):
    dm, di, nh, hd, ds, ip = cfg.d_model, cfg.d_inner(), cfg.nheads(), cfg.headdim, cfg.d_state, cfg.in_proj_out_dim()
    return cfg.n_layers * (es * (dm * ip + di * dm) + 2 * 4 * B * nh * (hd * ds + ds + hd) + 2 * 4 * B * dm)


def m3_prefill_roofline(cfg, batch, T, seconds, es=2):
    """A Mamba-3 prefill against the two rooflines: the chunked scan's bytes per layer (x, Q, K read + y written + the
    step scalars) and the matrix work (two projections + the scan's four contractions per chunk)."""
    M = batch * T
    dm, di, nh, hd, ds, ip = cfg.d_model, cfg.d_inner(), cfg.nheads(), cfg.headdim, cfg.d_state, cfg.in_proj_out_dim()
    nbytes = (4 * M * di * es + 12 * M * nh) * cfg.n_layers
    flops = (2.0 * M * (dm * ip + di * dm) + 4 * 2.0 * 64 * hd * ds * (M // 64) * nh) * cfg.n_layers
    return {"scan_algorithmic_bytes": nbytes, "hbm_frac": nbytes / seconds / 1e9 / HBM_PEAK_GBPS,
            "matrix_flop": flops, "mfma_frac": flops / seconds / 1e12 / MFMA_BF16_PEAK_TFLOPS}


def m1_prefill_roofline(cfg, batch, T, seconds, es=2):
    """A Mamba-1 prefill against the two rooflines: the bytes its own streaming kernels must move per layer (selective
    scan with the gate read, conv1d + SiLU: delta,u,z read + y written + B,C + state; x read + u written + window) and
    the matrix work of its four projections (2 M N K each, bf16 operands, f32 sums)."""
    M = batch * T
    dm, di, ds, dc, dr = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank()
    xd = dr + 2 * ds
    scan = scan_algorithmic_bytes(batch, T, di, ds, es, gated=True)
    conv = 2 * M * di * es + 2 * 4 * batch * di * dc + 4 * di * (dc + 1)
    flops = 2.0 * M * (dm * 2 * di + di * xd + dr * di + di * dm) * cfg.n_layers
    nbytes = (scan + conv) * cfg.n_layers
    return {"scan_conv_algorithmic_bytes": nbytes, "hbm_frac": nbytes / seconds / 1e9 / HBM_PEAK_GBPS,
            "gemm_flop": flops, "mfma_frac": flops / seconds / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "note": "hbm_frac: bytes of the scan and conv kernels of every layer / whole prefill time / 8 TB/s; mfma_frac: "
                    "projection flops / whole prefill time / 2.5 PFLOP/s (dense bf16); each is a share of one prefill that "
                    "does both kinds of work in sequence"}


def lm_leg(name, cfg_kw, vocab, prefill_bt, decode_b, decode_steps, seed=42, shared_layer=False, cpu_sample=None,
           with_generate=True, gemm_tuning=False, decode_graph=True):
    """Prefill tok/s and greedy-decode us/step of a random-init LM-shaped backbone (bf16 storage):
    token ids -> device embedding gather -> backbone (-> tied head -> argmax for decode).  With shared_layer the model's
    layers all hold one layer's random weights (timing only: the kernels and their operand sizes are those of the full
    model, the host-side initialisation is one layer's).  With gemm_tuning the prefill engine first times the GEMM
    library's kernels for its three projection shapes and keeps the fastest (set-up, outside the timed region); the
    untuned figure is reported beside the tuned one."""
    import numpy as np
    from mamba_rs_amd import GpuMambaBackbone, GpuMambaLM, MambaConfig, MambaWeights, WeightDtype
    cfg = MambaConfig(**cfg_kw)
    if shared_layer:
        w = MambaWeights.random_lm(MambaConfig(**{**cfg_kw, "n_layers": 1}), seed)
        w.layers = w.layers * cfg.n_layers
    else:
        w = MambaWeights.random_lm(cfg, seed)
    rng = np.random.default_rng(seed + 1)
    embed = (rng.standard_normal((vocab, cfg.d_model), dtype=np.float32) * np.float32(0.02))
    out = {"model": name}
    if shared_layer:
        out["weights"] = "one layer's random weights in every layer (timing only)"
    pb, pt = prefill_bt
    pre = GpuMambaBackbone.new_with_dtype(0, w, cfg, cfg.d_model, pb, WeightDtype.BF16)
    lm_p = GpuMambaLM(pre, embed)
    toks = rng.integers(0, vocab, (pb, pt)).astype(np.int32)
    lm_p.prefill(toks); pre.sync()                      # warm-up (library kernel selection, scratch)

    def timed_prefill():
        # untimed passes until the GPU has been under load for 150 ms (its clocks settle within about 50 ms), then three timed
        t_end = time.perf_counter() + 0.15
        while time.perf_counter() < t_end:
            pre.reset(); lm_p.prefill(toks); pre.sync()
        times = []
        for _ in range(3):
            pre.reset(); pre.sync()
            t0 = time.perf_counter(); lm_p.prefill(toks); pre.sync(); times.append(time.perf_counter() - t0)
        return sorted(times)[1]
    tp = timed_prefill()
    out["prefill"] = {"batch": pb, "seq_len": pt, "ms": tp * 1e3, "tok_per_s": pb * pt / tp}
    if gemm_tuning:
        t0 = time.perf_counter()
        pre.set_gemm_tuning(True)
        pre.reset(); lm_p.prefill(toks); pre.sync()     # the projection shapes are timed over the library's kernels here
        tune_s = time.perf_counter() - t0
        tt = timed_prefill()
        out["prefill"] = {"batch": pb, "seq_len": pt, "ms": tt * 1e3, "tok_per_s": pb * pt / tt, "vendor_gemm_kernels": "timed once, fastest kept",
                          "tuning_s": tune_s, "ms_with_default_vendor_kernels": tp * 1e3}
    out["prefill"]["roofline"] = m1_prefill_roofline(cfg, pb, pt, out["prefill"]["ms"] * 1e-3)
    lm_p.close(); pre.close()
    if cpu_sample:
        out["cpu_port_prefill"] = cpu_prefill_sample(cfg_kw, cpu_sample[0], cpu_sample[1], pb * pt, seed)
    dec_out = []
    for db in (decode_b if isinstance(decode_b, (list, tuple)) else [decode_b]):
        def timed_decode(tuned):
            dec = GpuMambaBackbone.new_with_dtype(0, w, cfg, cfg.d_model, db, WeightDtype.BF16)
            if tuned:
                dec.set_gemm_tuning(True)                  # takes effect in the eager step that precedes the capture
            lm_d = GpuMambaLM(dec, embed)
            lm_d.set_tokens(rng.integers(0, vocab, db).astype(np.int32))
            if decode_graph:
                lm_d.capture_graph()
            spin_steps(lm_d.decode_step, dec.sync)
            t0 = time.perf_counter()
            for _ in range(decode_steps):
                lm_d.decode_step()
            dec.sync()
            return dec, lm_d, (time.perf_counter() - t0) / decode_steps
        # from 65 rows (wide models) or 129 rows up the projections of a decode step go to the GEMM library as well
        tune_decode = gemm_tuning and db > 64
        td_default = None
        if tune_decode:
            dec, lm_d, td_default = timed_decode(False)
            lm_d.close(); dec.close()
        dec, lm_d, td = timed_decode(tune_decode)
        tk = lm_d.get_tokens()
        assert ((tk >= 0) & (tk < vocab)).all()
        step_bytes = m1_step_bytes(cfg, db, 2, vocab)
        entry = {"batch": db, "steps": decode_steps, "us_per_step": td * 1e6, "tok_per_s": db / td,
                 "algorithmic_bytes_per_step": step_bytes, "hbm_frac": step_bytes / td / 1e9 / HBM_PEAK_GBPS}
        if td_default is not None:
            entry["vendor_gemm_kernels"] = "timed once, fastest kept"
            entry["us_per_step_with_default_vendor_kernels"] = td_default * 1e6
        if not decode_graph:
            entry["launch"] = "kernel by kernel (no hipGraph)"
        if with_generate and decode_graph:
            # batched generation with the sampler in the loop: ragged prompts of 8..12 tokens, 128 new tokens per slot
            from mamba_rs_amd import SampleParams
            prompts = [[int(t) for t in rng.integers(0, vocab, 8 + (i % 5))] for i in range(db)]
            params = [SampleParams(temperature=0.8, top_k=50, top_p=0.9, max_tokens=128, seed=i) for i in range(db)]
            lm_d.generate_batch(prompts, params)                       # warm-up (captures the step)
            t0 = time.perf_counter(); gen = lm_d.generate_batch(prompts, params); tg = time.perf_counter() - t0
            n_gen = sum(len(g) for g in gen)
            entry["generate_batch"] = {"sampler": "temperature 0.8, top_k 50, top_p 0.9", "new_tokens": n_gen, "ms": tg * 1e3,
                                       "us_per_step": tg / (12 + 128) * 1e6, "gen_tok_per_s": n_gen / tg,
                                       "hbm_frac": step_bytes / (tg / (12 + 128)) / 1e9 / HBM_PEAK_GBPS}
        dec_out.append(entry)
        lm_d.close(); dec.close()
    out["decode"] = dec_out
    return out


def c1_leg():
    """The tiny CPU-runnable configuration (d_model 128, 2 layers, d_state 16, f32, batch 1, T 256; weights
    MambaWeights::init seed 42, input N(0,1)): the f32 engine's prefill and graph decode on the GPU, the oracle's
    restatement of the reference CPU prefill / step beside them, and the largest relative difference between the two."""
    import numpy as np
    import orc
    from mamba_rs_amd import GpuMambaBackbone, MambaConfig, MambaWeights
    cfg = MambaConfig(d_model=128, d_state=16, d_conv=4, expand=2, n_layers=2)
    T = 256
    w = MambaWeights.init(cfg, 128, 42)
    P = orc.M1Params(128, 16, 4, 2, 2, 128, seed=42)
    x = np.random.default_rng(42).standard_normal((1, T, 128)).astype(np.float32)
    eng = GpuMambaBackbone.new(0, w, cfg, 128, 1)
    got = eng.prefill_sequence(x)                     # warm-up; leaves the input on the device
    times = []
    for _ in range(5):
        eng.reset(); eng.sync()
        t0 = time.perf_counter(); eng.prefill_device(eng.prefill_input_ptr(), T); eng.sync(); times.append(time.perf_counter() - t0)
    tp = sorted(times)[2]
    cs, ss = orc.m1_zero_state(P)
    want = orc.m1_backbone_prefill(P, x[0], cs, ss)[-1]
    err = float(np.abs(got.reshape(-1) - want).max() / max(np.abs(want).max(), 1e-30))
    ctimes = []
    for _ in range(5):
        cs, ss = orc.m1_zero_state(P)
        t0 = time.perf_counter(); orc.m1_backbone_prefill(P, x[0], cs, ss); ctimes.append(time.perf_counter() - t0)
    tc = sorted(ctimes)[2]
    eng.reset(); eng.step(x[0, 0:1]); eng.capture_graph()
    spin_steps(eng.step_gpu_only, eng.sync)
    t0 = time.perf_counter()
    for _ in range(256):
        eng.step_gpu_only()
    eng.sync()
    td = (time.perf_counter() - t0) / 256
    t0 = time.perf_counter()
    for t in range(64):
        orc.m1_backbone_step(P, x[0, t], cs, ss)
    tcs = (time.perf_counter() - t0) / 64
    eng.close()
    roof = m1_prefill_roofline(cfg, 1, T, tp, es=4)
    roof["mfma_frac"] = None     # f32 projections do not run on the bf16 matrix path
    dm, di, ds, dc, dr = 128, 256, 16, 4, 8
    step_bytes = 2 * (4 * (dm * 2 * di + di * (dr + 2 * ds) + dr * di + di * dm) + 2 * 4 * di * (ds + dc) + 2 * 4 * dm)
    return {"config": "d_model 128, 2 layers, d_state 16, f32, batch 1, T 256",
            "gpu_prefill": {"ms": tp * 1e3, "tok_per_s": T / tp, "roofline": roof}, "gpu_decode_us_per_step": td * 1e6,
            "gpu_decode_hbm_frac": step_bytes / td / 1e9 / HBM_PEAK_GBPS,
            "cpu_port_prefill": {"ms": tc * 1e3, "tok_per_s": T / tc, "cores": orc.num_threads()},
            "cpu_port_decode_us_per_step": tcs * 1e6, "prefill_last_step_max_rel_diff_gpu_vs_cpu_port": err}


def default_configs_leg():
    """The reference's two default configurations (MambaConfig::default: d_model 128, 3 layers, src/config.rs:174-186;
    Mamba3Config::default: d_model 128, 4 layers, headdim 16, src/mamba3_siso/config.rs:132-150), f32, one step in a
    hipGraph: the quantity behind the reference's published "GPU step" figures (docs/mamba1-benchmarks.md:111-115,
    docs/mamba3-benchmarks.md:16; other hardware, quoted beside ours, never a ratio)."""
    import numpy as np
    from mamba_rs_amd import GpuMambaBackbone, GpuMamba3Backbone, MambaConfig, MambaWeights, Mamba3Config, Mamba3Weights

    def run(eng, x, n=400):
        eng.step(x); eng.capture_graph()
        spin_steps(eng.step_gpu_only, eng.sync)
        t0 = time.perf_counter()
        for _ in range(n):
            eng.step_gpu_only()
        eng.sync()
        eng.close()
        return (time.perf_counter() - t0) / n * 1e6

    out = {"published_rtx6000ada": {"m1_step_us_b1_graph": 79, "m1_step_us_b128_graph": 139, "m3_step_us_b1_graph": 87,
                                    "m3_synthetic_lm_tok_per_s_graph": {"f32": 5778, "bf16": 5824}}}
    c1 = MambaConfig(d_model=128, d_state=16, d_conv=4, expand=2, n_layers=3)
    c3 = Mamba3Config(d_model=128, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=4, rope_fraction=0.5, a_floor=1e-4)
    for B in (1, 128):
        x = np.random.default_rng(B).standard_normal((B, 128)).astype(np.float32)
        out[f"m1_step_us_b{B}"] = run(GpuMambaBackbone.new(0, MambaWeights.init(c1, 128, 42), c1, 128, B), x)
        out[f"m3_step_us_b{B}"] = run(GpuMamba3Backbone.new(0, Mamba3Weights.init(c3, 128, 42), c3, 128, B), x)
        out[f"m1_step_hbm_frac_b{B}"] = m1_step_bytes(c1, B, 4) / out[f"m1_step_us_b{B}"] / 1e3 / HBM_PEAK_GBPS
        out[f"m3_step_hbm_frac_b{B}"] = m3_step_bytes(c3, B, 4) / out[f"m3_step_us_b{B}"] / 1e3 / HBM_PEAK_GBPS
    # the reference's synthetic Mamba-3 LM (tests/bench_bf16_vs_f32.rs:148-215: d_model 256, 8 layers, headdim 16, vocab 256,
    # a_floor 0.0625; prompt [1..5], 100 greedy tokens, second run timed)
    from mamba_rs_amd import GpuMamba3LM, SampleParams, WeightDtype
    cl = Mamba3Config(d_model=256, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=8, rope_fraction=0.5, a_floor=0.0625)
    wl = Mamba3Weights.init(cl, 256, 0xB00B)
    wl.input_proj_w = np.zeros(0, np.float32); wl.input_proj_b = np.zeros(0, np.float32)   # the LM feeds embeddings straight in
    embed = ((np.random.default_rng(0xBEEF).random((256, 256), dtype=np.float32) - np.float32(0.5)) * np.float32(0.1))
    sp = SampleParams(temperature=0.0, max_tokens=100)
    lm_out = {}
    for name, dt in (("f32", WeightDtype.F32), ("bf16", WeightDtype.BF16)):
        bb = GpuMamba3Backbone.new_with_dtype(0, wl, cl, 256, 1, dt)
        lm = GpuMamba3LM(bb, embed)
        lm.generate([1, 2, 3, 4, 5], params=sp)
        t0 = time.perf_counter(); toks = lm.generate([1, 2, 3, 4, 5], params=sp); dt_s = time.perf_counter() - t0
        lm_out[name] = len(toks) / dt_s
        lm_out[name + "_hbm_frac"] = (m3_step_bytes(cl, 1, 4 if name == "f32" else 2) + 256 * 256 * (4 if name == "f32" else 2)) * lm_out[name] / 1e9 / HBM_PEAK_GBPS
        lm.close(); bb.close()
    out["m3_synthetic_lm_tok_per_s"] = lm_out
    return out


def published_configs_leg():
    """Configurations the reference publishes end-to-end figures for (docs/mamba1-benchmarks.md:23, 52-54, 77; measured
    there on an RTX 6000 Ada with real checkpoints; random-init weights of the same shapes here): 130m greedy decode at
    batch 1 in f32 and at batch 16 in bf16, and the 370m-shape parallel-scan prefill of one prompt of 256 / 1024 / 4096
    tokens in bf16."""
    import numpy as np
    from mamba_rs_amd import GpuMambaBackbone, GpuMambaLM, MambaConfig, MambaWeights, WeightDtype
    vocab = 50280
    rng = np.random.default_rng(11)
    out = {"published_rtx6000ada": {"130m_decode_tok_per_s_b1": {"f32": 725, "bf16": 1029}, "130m_bf16_decode_tok_per_s_b16_total": 5026,
                                    "370m_bf16_prefill_ms": {"256": 31.8, "1024": 87.9, "4096": 328.8}}}
    cfg = MambaConfig(d_model=768, d_state=16, d_conv=4, expand=2, n_layers=24)
    w = MambaWeights.random_lm(cfg, 42)
    embed = (rng.standard_normal((vocab, cfg.d_model), dtype=np.float32) * np.float32(0.02))
    for key, dt, B in (("130m_f32_decode_b1", WeightDtype.F32, 1), ("130m_bf16_decode_b16", WeightDtype.BF16, 16)):
        dec = GpuMambaBackbone.new_with_dtype(0, w, cfg, cfg.d_model, B, dt)
        lm = GpuMambaLM(dec, embed)
        lm.set_tokens(rng.integers(0, vocab, B).astype(np.int32))
        lm.capture_graph()
        spin_steps(lm.decode_step, dec.sync)
        t0 = time.perf_counter()
        for _ in range(128):
            lm.decode_step()
        dec.sync()
        td = (time.perf_counter() - t0) / 128
        out[key] = {"us_per_step": td * 1e6, "tok_per_s_total": B / td,
                    "hbm_frac": m1_step_bytes(cfg, B, dt.size_bytes(), vocab) / td / 1e9 / HBM_PEAK_GBPS}
        lm.close(); dec.close()
    c370 = MambaConfig(d_model=1024, d_state=16, d_conv=4, expand=2, n_layers=48)
    w370 = MambaWeights.random_lm(c370, 43)
    e370 = (rng.standard_normal((vocab, 1024), dtype=np.float32) * np.float32(0.02))
    pre = {}
    for T in (256, 1024, 4096):
        eng = GpuMambaBackbone.new_with_dtype(0, w370, c370, 1024, 1, WeightDtype.BF16)
        lm = GpuMambaLM(eng, e370)
        toks = rng.integers(0, vocab, (1, T)).astype(np.int32)
        lm.prefill(toks); eng.sync()
        times = []
        for _ in range(3):
            eng.reset(); eng.sync()
            t0 = time.perf_counter(); lm.prefill(toks); eng.sync(); times.append(time.perf_counter() - t0)
        pre[str(T)] = sorted(times)[1] * 1e3
        pre[str(T) + "_roofline"] = m1_prefill_roofline(c370, 1, T, sorted(times)[1])
        lm.close(); eng.close()
    out["370m_bf16_prefill_ms_b1"] = pre
    return out


def m1_kernels_leg():
    """The other Mamba-1 kernels of the path at the 130m shape (bf16 storage), each against its HBM roofline:
    causal conv1d + SiLU over batch 8 x T 2048 reading the x half of in_proj's rows in place, and the decode
    scan step (B/C gathered from the x_proj row, SiLU gate fused) at batch 64."""
    import torch
    from mamba_rs_amd import ops
    dev, bf = "cuda:0", torch.bfloat16
    B, T, di, ds, dc, dr = 8, 2048, 1536, 16, 4, 48
    g = torch.Generator(device=dev); g.manual_seed(5)

    def timeit(f, n, spin_ms=100.0):
        # the op runs untimed for spin_ms first (the GPU's clocks settle within about 50 ms of load), as the headline leg does
        t_end = time.perf_counter() + spin_ms * 1e-3
        f()
        while time.perf_counter() < t_end:
            for _ in range(50):
                f()
            torch.cuda.synchronize()
        for _ in range(3):
            f()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            f()
        b.record(); torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e3

    proj = torch.randn(B, T, 2 * di, device=dev, generator=g).to(bf)
    w = torch.randn(di, dc, device=dev, generator=g); bias = torch.randn(di, device=dev, generator=g)
    st = torch.zeros(B, di, dc, device=dev); u = torch.empty(B, T, di, device=dev, dtype=bf)
    us_conv = timeit(lambda: ops.conv1d_seq_silu(u, st, proj[:, :, :di], w, bias), 30)
    conv_bytes = 2 * B * T * di * 2 + 2 * 4 * B * di * dc + 4 * di * (dc + 1)
    Bd = 64
    h = torch.zeros(Bd, di, ds, device=dev); y = torch.empty(Bd, di, device=dev, dtype=bf)
    delta = torch.rand(Bd, di, device=dev, generator=g).mul(0.1).to(bf); uu = torch.randn(Bd, di, device=dev, generator=g).to(bf)
    xdbl = torch.randn(Bd, dr + 2 * ds, device=dev, generator=g).to(bf); gate = torch.randn(Bd, di, device=dev, generator=g).to(bf)
    a_neg = -torch.arange(1, ds + 1, device=dev, dtype=torch.float32).repeat(di, 1).contiguous(); D = torch.ones(di, device=dev)
    ops.ssm_step_gather_gate(h, y, delta, uu, xdbl, gate, a_neg, D, dr, dr + ds)
    torch.cuda.synchronize()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        for _ in range(24):
            ops.ssm_step_gather_gate(h, y, delta, uu, xdbl, gate, a_neg, D, dr, dr + ds)
    us_step = timeit(gr.replay, 30) / 24
    step_bytes = 2 * 4 * Bd * di * ds + 4 * Bd * di * 2 + 4 * di * ds
    # the headline scan once more per storage type (the reference ships f32, bf16 and f16 variants of the kernel),
    # and without the S4D-real shortcut (a general A: 16 exponentials per step instead of one)
    scan = {}
    inp = make_inputs(B, T, di, ds)
    tt = {k: torch.from_numpy(v).to(dev) for k, v in inp.items()}
    ws = torch.zeros(ops.ssm_scan_workspace_bytes(B, T, di, ds), dtype=torch.uint8, device=dev)
    hs = torch.zeros(B, di, ds, device=dev)
    for name, tdt, esz, fl in (("f32", torch.float32, 4, ops.A_S4D_REAL), ("f16", torch.float16, 2, ops.A_S4D_REAL),
                               ("bf16_general_A", bf, 2, 0)):
        dl, uu_, zz, Bm, Cm = (tt[k].to(tdt) for k in ("delta", "u", "z", "B", "C"))
        yy = torch.empty_like(dl)
        us_s = timeit(lambda: ops.ssm_scan_fwd(hs, yy, dl, uu_, Bm, Cm, tt["a_neg"], tt["D"], gate=zz, flags=ops.GATE_SILU | ops.SCAN_FLAGS_ZERO | fl, workspace=ws), 20)
        nb = scan_algorithmic_bytes(B, T, di, ds, esz, gated=True)
        scan[name] = {"us": us_s, "algorithmic_bytes": nb, "GBps": nb / us_s / 1e3, "hbm_frac": nb / us_s / 1e3 / HBM_PEAK_GBPS}
    return {"selective_scan_other_storage": scan,
            "conv1d_seq_silu": {"batch": B, "seq_len": T, "us": us_conv, "algorithmic_bytes": conv_bytes,
                                "GBps": conv_bytes / us_conv / 1e3, "hbm_frac": conv_bytes / us_conv / 1e3 / HBM_PEAK_GBPS},
            "ssm_step_gather_gate_b64": {"us_per_call_in_graph": us_step, "algorithmic_bytes": step_bytes,
                                         "GBps": step_bytes / us_step / 1e3, "hbm_frac": step_bytes / us_step / 1e3 / HBM_PEAK_GBPS}}


def m3_leg():
    """Mamba-3 SISO scan kernels at the 768-wide shape (24 heads x headdim 64, d_state 64, bf16):
    chunked SSD over batch 4 x 4096 (one layer) and the batch-1 decode step kernel."""
    import numpy as np
    import torch
    from mamba_rs_amd import ops
    from test_oracle_m3 import m3_inputs
    B, T, nh, hd, ds = 4, 4096, 24, 64, 64
    inp = m3_inputs(np.random.default_rng(3), B, T, nh, hd, ds)
    dev = "cuda:0"
    t = {k: torch.from_numpy(v).to(dev) for k, v in inp.items()}
    x, K, Q = (t[k].to(torch.bfloat16) for k in ("x", "K", "Q"))
    ssm = torch.zeros(B, nh, hd, ds, device=dev); kst = torch.zeros(B, nh, ds, device=dev); vst = torch.zeros(B, nh, hd, device=dev)
    y = torch.empty_like(x)

    def timeit(f, n, spin_ms=100.0):
        # the op runs untimed for spin_ms first (the GPU's clocks settle within about 50 ms of load), as the headline leg does
        t_end = time.perf_counter() + spin_ms * 1e-3
        f()
        while time.perf_counter() < t_end:
            for _ in range(20):
                f()
            torch.cuda.synchronize()
        for _ in range(3):
            f()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            f()
        b.record(); torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e3

    ws = torch.empty(ops.m3_ssd_workspace_bytes(B, T, nh, hd, ds), dtype=torch.uint8, device=dev)
    us = timeit(lambda: ops.m3_ssd_fwd(ssm, kst, vst, y, x, K, Q, t["dt"], t["trap"], t["a_val"], t["D"], workspace=ws), 10)
    nbytes = 4 * B * T * nh * hd * 2 + 3 * B * T * nh * 4
    al, be, ga = ops.m3_compute_abg(t["dt"], t["a_val"], t["trap"])
    x1, K1, Q1 = x[:1, 0].contiguous(), K[:1, 0].contiguous(), Q[:1, 0].contiguous()
    s1, k1, v1, y1 = ssm[:1].clone(), kst[:1].clone(), vst[:1].clone(), torch.empty_like(x[:1, 0])
    a1, b1, g1 = al[:1, 0].contiguous(), be[:1, 0].contiguous(), ga[:1, 0].contiguous()
    g = torch.cuda.CUDAGraph()
    ops.m3_step(s1, k1, v1, y1, x1, K1, Q1, a1, b1, g1, t["D"])
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        for _ in range(24):
            ops.m3_step(s1, k1, v1, y1, x1, K1, Q1, a1, b1, g1, t["D"])
    us_step = timeit(g.replay, 50) / 24
    prof, prof_src = profile_figures("m3_ssd_c4_bf16.md", "m3_ssd.hip", ["traffic_bytes_per_call", "mfma_busy_frac_full_pass", "mfma_busy_frac_state_pass"])
    flop = 4 * 2 * 64 * 64 * 64 * B * (T // 64) * nh
    step_state_bytes = 2 * 4 * nh * (hd * ds + ds + hd) + 4 * nh * hd * 2
    return {"ssd_prefill_layer": {"batch": B, "seq_len": T, "us": us, "algorithmic_bytes": nbytes, "GBps": nbytes / us / 1e3,
                                  "hbm_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS, "tok_per_s_layer": B * T / us * 1e6,
                                  "mfma_flop": flop, "mfma_frac": flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS,
                                  "measured_traffic_bytes": prof["traffic_bytes_per_call"],
                                  "traffic_over_algorithmic": (prof["traffic_bytes_per_call"] / nbytes) if prof["traffic_bytes_per_call"] else None,
                                  "measured_mfma_busy_frac": {"full_pass": prof["mfma_busy_frac_full_pass"], "state_pass": prof["mfma_busy_frac_state_pass"]},
                                  "counters_source": prof_src},
            "decode_step_kernel_b1": {"us_per_layer_call_in_graph": us_step, "algorithmic_bytes": step_state_bytes,
                                      "hbm_frac": step_state_bytes / us_step / 1e3 / HBM_PEAK_GBPS}}


def m3_engine_leg(steps=512, batches=(1, 16), prefill_bt=(4, 4096)):
    """Mamba-3 backbone at the 768-wide shape (24 layers, d_inner 1536, 24 heads x 64, d_state 64, 16 rope angles,
    bf16 storage): prefill tok/s over batch 4 x 4096 (inputs resident in the device input buffer) and decode us/step
    of the three-kernel layer chain in a hipGraph (the host writes nothing per step)."""
    import numpy as np
    from mamba_rs_amd import GpuMamba3Backbone, Mamba3Config, Mamba3Weights, WeightDtype
    cfg = Mamba3Config(d_model=768, d_state=64, expand=2, headdim=64, ngroups=1, n_layers=24, rope_fraction=0.5)
    rng = np.random.default_rng(7)
    w = Mamba3Weights.random_lm(cfg, 42)       # identity projection, as an LM backbone
    out = []
    dm, di, nh, hd, ds, ip = cfg.d_model, cfg.d_inner(), cfg.nheads(), cfg.headdim, cfg.d_state, cfg.in_proj_out_dim()
    pb, pt = prefill_bt
    pre = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 768, pb, WeightDtype.BF16)
    pre.prefill_sequence((rng.standard_normal((pb, pt, 768)) * 0.5).astype(np.float32))   # warm-up; leaves the input on the device
    t_end = time.perf_counter() + 0.15      # untimed passes until the clocks have settled under load, as in lm_leg
    while time.perf_counter() < t_end:
        pre.reset(); pre.prefill_device(pt); pre.sync()
    times = []
    for _ in range(3):
        pre.reset(); pre.sync()
        t0 = time.perf_counter(); pre.prefill_device(pt); pre.sync(); times.append(time.perf_counter() - t0)
    tp = sorted(times)[1]
    prefill = {"batch": pb, "seq_len": pt, "ms": tp * 1e3, "tok_per_s": pb * pt / tp, "roofline": m3_prefill_roofline(cfg, pb, pt, tp)}
    pre.close()
    for B in batches:
        eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 768, B, WeightDtype.BF16)
        eng.step((rng.standard_normal((B, 768)) * 0.5).astype(np.float32))
        eng.capture_graph()
        spin_steps(eng.step_gpu_only, eng.sync)
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step_gpu_only()
        eng.sync()
        td = (time.perf_counter() - t0) / steps
        step_bytes = m3_step_bytes(cfg, B, 2)
        entry = {"batch": B, "steps": steps, "us_per_step": td * 1e6, "algorithmic_bytes_per_step": step_bytes,
                 "hbm_frac": step_bytes / td / 1e9 / HBM_PEAK_GBPS}
        if B == 1:
            # the LM loop on top (tied 50280-entry head): 100 greedy tokens from a short prompt, as the reference's
            # synthetic Mamba-3 LM figure (docs/mamba3-benchmarks.md:28)
            from mamba_rs_amd import GpuMamba3LM, SampleParams
            vocab = 50280
            lm = GpuMamba3LM(eng, (rng.standard_normal((vocab, dm), dtype=np.float32) * np.float32(0.02)))
            prompt = [int(t) for t in rng.integers(0, vocab, 8)]
            sp = SampleParams(temperature=0.0, max_tokens=100)
            lm.generate(prompt, params=sp)
            t0 = time.perf_counter(); toks = lm.generate(prompt, params=sp); tg = time.perf_counter() - t0
            entry["lm_greedy_100_tokens"] = {"ms": tg * 1e3, "tok_per_s": len(toks) / tg,
                                             "hbm_frac": (step_bytes + (vocab + 63) // 64 * 64 * dm * 2) * len(toks) / tg / 1e9 / HBM_PEAK_GBPS}
            lm.close()
        out.append(entry)
        eng.close()
    return {"prefill": prefill, "decode": out}


def engine_legs(args, legs, tune):
    """The legs that drive the engines through the C ABI from numpy buffers: no torch in them."""
    extras = {}
    if "c1" in legs:
        extras["tiny_f32_cpu_config"] = c1_leg()
        extras["reference_default_configs_f32"] = default_configs_leg()
    if "lm" in legs:
        extras["lm_130m_shape_bf16"] = lm_leg("130m-shape", dict(d_model=768, d_state=16, d_conv=4, expand=2, n_layers=24), 50280,
                                              (8, 2048), [64, 1], 256, cpu_sample=(24, 256), gemm_tuning=tune,
                                              decode_graph=not args.lm_no_graph)
    if "published" in legs:
        extras["reference_published_configs"] = published_configs_leg()
    if "m3_engine" in legs:
        extras["mamba3_768_bf16"] = {"backbone": m3_engine_leg()}
    elif "m3_prefill" in legs:   # the backbone's prefill alone (not a default leg: the command behind its profile)
        extras["mamba3_768_bf16"] = {"backbone": m3_engine_leg(batches=())}
    if "lm28" in legs or args.big:
        extras["lm_2.8b_shape_bf16"] = lm_leg("2.8b-shape", dict(d_model=2560, d_state=16, d_conv=4, expand=2, n_layers=64), 50280,
                                              (4, 4096), [1, 16, 64, 128], 128, shared_layer=not args.big, cpu_sample=(2, 64),
                                              with_generate=False, gemm_tuning=tune, decode_graph=not args.lm_no_graph)
    return extras


def run_engine_legs_child(args, tune):
    """Runs the engine legs in a child process (started before this process has touched the GPU) and returns its JSON line,
    or {"failure": ...} -- the caller then runs the legs itself."""
    import subprocess
    cmd = [sys.executable, os.path.abspath(__file__), "--engine-legs-child", "--legs", args.legs, "--gemm-tune", "on" if tune else "off"]
    if args.big:
        cmd.append("--big")
    if args.lm_no_graph:
        cmd.append("--lm-no-graph")
    try:
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=1500)
        if r.returncode != 0:
            return {"failure": f"exit code {r.returncode}: {r.stderr.strip()[-300:]}"}
        res = json.loads(r.stdout.strip().splitlines()[-1])
        if res.get("torch_in_process"):
            return {"failure": "the child process imported torch"}
        return res
    except Exception as e:   # noqa: BLE001 - any failure of the child falls back to the in-process legs
        return {"failure": f"{type(e).__name__}: {e}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spinup-ms", type=float, default=250.0, help="untimed run of the op before the warm-up and timed steps (GPU clock ramp); 0 = none")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="only the headline scan line (no LM / Mamba-3 legs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 256 MiB device copy (a known-size kernel to scale rocprof FETCH_SIZE/WRITE_SIZE by)")
    ap.add_argument("--big", action="store_true", help="the 2.8b-shape LM leg with 64 independently initialised layers (minutes of host-side init) instead of one shared layer")
    ap.add_argument("--gemm-tune", choices=["auto", "on", "off"], default="auto",
                    help="prefill legs of the LM engines pick their vendor GEMM kernels by timing them (auto: in the full default run only)")
    ap.add_argument("--engine-legs", choices=["auto", "child", "inprocess"], default="auto",
                    help="where the engine legs (c1, lm, lm28, published, m3_engine) run.  torch bundles its own build of the vendor GEMM "
                         "library, and a process that imports torch first binds libmamba_hip.so to that copy; a host without torch, such "
                         "as the Rust binding, runs on the copy under /opt/rocm, whose kernels for the engines' library projections "
                         "(prefill; decode past the own chain's row limit) are faster.  'child' runs those legs, which need no torch, in "
                         "a process of their own before this one touches the GPU; 'inprocess' runs them here behind the torch legs; "
                         "'auto' = child in the full default run, inprocess when --legs, --no-cpu or --lm-no-graph narrows it (profiling)")
    ap.add_argument("--engine-legs-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--lm-no-graph", action="store_true",
                    help="the decode steps of the lm / lm28 legs launch kernel by kernel instead of replaying a hipGraph, and the "
                         "generation runs are skipped (for kernel traces of those steps)")
    ap.add_argument("--legs", default=DEFAULT_LEGS,
                    help="comma list of the extras to run: c1, lm, lm28, published, m1_kernels, m3, m3_engine (for profiling one leg at a time)")
    args = ap.parse_args()
    legs = {x.strip() for x in args.legs.split(",") if x.strip()}
    unknown = legs - {"c1", "lm", "lm28", "published", "m1_kernels", "m3", "m3_engine", "m3_prefill"}
    if unknown:
        print(f"bench.py: unknown --legs entries {sorted(unknown)}", file=sys.stderr)
        sys.exit(2)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)
    tune = args.gemm_tune == "on" or (args.gemm_tune == "auto" and legs == set(DEFAULT_LEGS.split(",")))
    if args.engine_legs_child:
        # the engine legs alone, in a process that never imports torch; one JSON line for the parent
        res = {"extras": engine_legs(args, legs, tune), "torch_in_process": "torch" in sys.modules,
               "libraries": loaded_libraries(("librocblas", "libhipblaslt", "libamdhip64"))}
        print(json.dumps(res))
        return
    child = None
    use_child = args.engine_legs == "child" or (args.engine_legs == "auto" and legs == set(DEFAULT_LEGS.split(",")) and not args.no_cpu
                                                 and not args.lm_no_graph)
    if use_child and not args.no_extras:
        child = run_engine_legs_child(args, tune)
    shape = (8, 2048, 1536, 16)
    batch, T, di, ds = shape
    nbytes = scan_algorithmic_bytes(batch, T, di, ds, 2, gated=True)
    inp = make_inputs(*shape)
    g = gpu_leg(args, inp, shape)
    gbps = nbytes / (g["ms_per_step"] * 1e-3) / 1e9
    traffic, issue_us, traffic_source = profiled_scan_traffic()
    us = g["ms_per_step"] * 1e3
    gen_us = g["general_a_ms_per_step"] * 1e3
    out = {
        "metric": "m1_selective_scan_hbm_GBps",
        "value": gbps,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": g["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "isolated Mamba-1 selective scan forward, batch 8 x T 2048 x d_inner 1536 x d_state 16, "
                               "bf16 storage, f32 compute, SiLU gate fused, S4D-real A",
                   "tokens_per_step": batch * T, "storage": "bf16", "compute": "f32",
                   "launches_per_step": 1, "two_launch_ms_per_step": g["two_launch_ms_per_step"],
                   "spinup_ms": args.spinup_ms, "ms_per_step_from_idle": g["first_calls_ms"],
                   "spinup_note": "the op runs untimed for spinup_ms before the W warm-up and K timed steps, so that the GPU's clocks are where "
                                  "sustained load puts them; ms_per_step_from_idle is the same W + K measurement taken first, straight from idle",
                   "general_A_ms_per_step": g["general_a_ms_per_step"],
                   "general_A_note": "the same launch without the S4D-real flag (a trained checkpoint's A): 16 exponentials per step instead of one"},
        "tokens_per_s": batch * T / (g["ms_per_step"] * 1e-3),
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernels": ["scan_fused_kernel"],
                     "algorithmic_bytes_per_launch": nbytes, "median_launch_ms": g["median_launch_ms"],
                     # what the two kernels are bound by in fact: the instruction issue of the SIMDs (f32 without packed math)
                     "valu": {"bound": "valu-issue",
                              "model": "1024 SIMDs; two plain instructions per issue window of 2.02 ns from two different waves, a "
                                       "DPP-operand instruction a whole window, v_exp / v_rcp / v_mfma_f32_4x4x1 two windows",
                              "bound_us_per_call": issue_us, "achieved_us_per_call": us,
                              "frac": (issue_us / us) if issue_us else None, "source": traffic_source},
                     # the same launch on the kernels a trained checkpoint's A takes (no S4D-real shortcut)
                     "general_A": {"bound": "hbm", "achieved": nbytes / gen_us / 1e3, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                   "frac": nbytes / gen_us / 1e3 / HBM_PEAK_GBPS, "ms_per_step": g["general_a_ms_per_step"]}},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_leg(inp, shape, nbytes)
    if not args.no_extras:
        extras = {}
        if "m1_kernels" in legs:
            extras["m1_kernels_130m_shape_bf16"] = m1_kernels_leg()
        if "m3" in legs:
            extras["mamba3_768_bf16"] = m3_leg()
        if child is not None and "extras" in child:
            eng, where = child["extras"], {"process": "child process without torch", "libraries": child.get("libraries")}
        else:
            eng = engine_legs(args, legs, tune)
            where = {"process": "this process, behind the torch legs", "libraries": loaded_libraries(("librocblas", "libhipblaslt", "libamdhip64"))}
            if child is not None:
                where["child_failure"] = child.get("failure")
        for k, v in eng.items():
            if k == "mamba3_768_bf16":
                extras.setdefault(k, {}).update(v)
            else:
                extras[k] = v
        where["note"] = ("the copies of the vendor libraries the engine legs ran on (see --engine-legs): their prefill projections and the "
                         "128-row decode of the 2.8b shape are the library's kernels; this package's own kernels do not depend on it")
        extras["engine_legs"] = where
        out["extras"] = extras
    print(json.dumps(out))


if __name__ == "__main__":
    main()
