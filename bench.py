#!/usr/bin/env python3
"""Decode benchmark of the HIP Llama-3 path on one MI355X.

A "step" is one greedy decode step (one token, batch 1) of a seeded random-init model whose weights are
resident in HBM: the embedding gather, five launches per layer, the lm_head and the argmax, replayed as one
captured HIP graph with the token fed back on the device.  The primary workload is BASELINE config 2
(Llama-3.2-1B-shaped, fp16, 512-token prompt, 256 decoded tokens); the north-star shape (Llama-3.1-8B-shaped,
int8 weight-only, batch 1) is measured in the same run and reported under "secondary".

Prints ONE JSON line.  `roofline` is for the dominant kernel family (the one-row linear kernel behind wo, w2 and
the lm_head): algorithmic bytes of those launches / their event-timed duration, measured in a separate eager pass
of the same step with an event pair around every launch.  `step_roofline` is the whole-token figure
(algorithmic bytes per token x tokens/s / 8 TB/s).  `cpu_baseline` times the CPU oracle (single thread, the way the
reference's CLANG device runs) on a bounded sample of the same weights and cross-checks its tokens against the GPU.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# `roofline.traffic` (HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counters) cannot be read from inside this process:
# it is null here, and the counter runs of `bench.py --traffic-probe` under rocprofv3 are summarised under profiles/.


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def linear_bytes(cfg, out_f, in_f):
    """weight (+ scale) bytes one one-row linear must stream"""
    q = cfg["quantize"]
    if q == "int8":
        return out_f * in_f + out_f * 2
    if q == "nf4":
        return out_f * in_f // 2 + (out_f * in_f // 64) * 2
    return out_f * in_f * 2


def kernel_bytes(cfg, T, attn_wo=False):
    """algorithmic HBM bytes per decode step of each kernel family at T visible positions; attn_wo: attention and wo of a
    layer are one launch (their bytes move from `attn_decode` and `linear` to `attn_wo`)"""
    from denograd_amd import synthetic
    d, V, L = cfg["dim"], cfg["vocab_size"], cfg["n_layers"]
    shp = synthetic.linear_shapes(cfg)
    lb = lambda name: linear_bytes(cfg, *shp[name])
    head_q = "int8" if cfg["quantize"] == "int8" else None
    head = (V * d + V * 2) if head_q == "int8" else V * d * 2
    act = 2
    out = {
        "qkv_rope": L * (lb("attention.wq") + lb("attention.wk") + lb("attention.wv") + d * act),
        "attn_decode": synthetic.kv_bytes_per_position(cfg) * T,
        "linear": L * (lb("attention.wo") + lb("feed_forward.w2")) + head + d * act,
        "ffn_gate": L * (lb("feed_forward.w1") + lb("feed_forward.w3") + d * act),
    }
    if attn_wo:
        out["attn_wo"] = out.pop("attn_decode") + L * lb("attention.wo")
        out["linear"] -= L * lb("attention.wo")
    return out


def read_only_launches(lib, cfg, T, attn_wo, reps=12):
    """Time jsgrad_hip_read_probe at the byte count of every weight-streaming launch of one decode step (cold data: the
    source window moves through 1 GiB).  Returns ms per step per kernel family, their sum, and the per-size table."""
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.tensor import Tensor

    L, d, V = cfg["n_layers"], cfg["dim"], cfg["vocab_size"]
    shp = synthetic.linear_shapes(cfg)
    lb = lambda name: linear_bytes(cfg, *shp[name])
    head = (V * d + V * 2) if cfg["quantize"] == "int8" else V * d * 2
    kv = synthetic.kv_bytes_per_position(cfg) * T // L
    launches = {   # family -> [(count per step, bytes)]
        "qkv_rope": [(L, lb("attention.wq") + lb("attention.wk") + lb("attention.wv"))],
        "ffn_gate": [(L, lb("feed_forward.w1") + lb("feed_forward.w3"))],
        "linear": [(L, lb("feed_forward.w2")), (1, head)],
    }
    if attn_wo:
        launches["attn_wo"] = [(L, lb("attention.wo") + kv)]
    else:
        launches["linear"].append((L, lb("attention.wo")))
        launches["attn_decode"] = [(L, kv)]

    span = 1 << 30
    src, sink = Tensor.empty((span,), "uint8"), Tensor.zeros((4,), "uint8")
    check(lib.jsgrad_hip_memset(src.ptr, 1, span))
    kid = ffi.PROF_KINDS["read_probe"]
    cache, off = {}, 0

    def probe(nbytes):
        nonlocal off
        nbytes = max(16, nbytes // 16 * 16)
        if nbytes not in cache:
            check(lib.jsgrad_hip_profile(1))
            for _ in range(reps + 2):
                off = (off + nbytes + (64 << 20)) % (span - nbytes) // 256 * 256
                check(lib.jsgrad_hip_read_probe(src.ptr + off, nbytes, sink.ptr))
            n, tot = C.c_int(), C.c_double()
            check(lib.jsgrad_hip_profile_read(kid, C.byref(n), C.byref(tot)))
            check(lib.jsgrad_hip_profile(0))
            cache[nbytes] = tot.value / n.value
        return cache[nbytes]

    fams = {k: sum(c * probe(b) for c, b in v) for k, v in launches.items()}
    return {"families": fams, "step_ms": sum(fams.values()), "sizes_us": {str(b): round(1e3 * t, 2) for b, t in sorted(cache.items())}}


def run_workload(name, prompt_len, steps, warmup, profile_steps=8, use_graph=True, blocker_steps=40, per_op_steps=64, fused_step=False,
                 prefill="serial", with_sampled=True):
    """prefill: "serial" feeds the prompt token by token as the reference does (llama3.ts:307-311); "rows" feeds it in one
    several-position pass (matrix-core GEMMs), which is what a long prompt takes in practice."""
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.llama3 import Llama3

    lib = ffi.load()
    ctx = prompt_len + warmup + steps + 3 * (profile_steps + blocker_steps) + (2 * per_op_steps if with_sampled or fused_step else 0) + 32
    cfg = synthetic.config(name, max_context=ctx)
    t0 = time.perf_counter()
    llm = Llama3.from_config(cfg, fused_step=fused_step).random_init(seed=0, tied=cfg["tied"])
    if not use_graph:
        llm.model.forward_jit = None     # the same kernels, launched one by one instead of replayed as a graph
    check(lib.jsgrad_hip_sync())
    log(f"[{name}] weights on device in {time.perf_counter() - t0:.1f}s")
    prompt = [int(t) for t in synthetic.random_prompt(cfg, prompt_len, seed=0)]
    t0 = time.perf_counter()
    llm.batched_prefill = prefill == "rows"
    llm._prefill(prompt[:-1])
    llm._call(prompt[-1])
    llm.start_pos += 1
    llm.model._rows = None       # the several-row scratch of a one-pass prefill is not needed any more
    log(f"[{name}] {'one-pass' if prefill == 'rows' else 'token-serial'} prefill of {prompt_len} tokens in {time.perf_counter() - t0:.2f}s")

    m = llm.model
    m.generate(warmup)
    llm.start_pos += warmup
    check(lib.jsgrad_hip_sync())
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.jsgrad_hip_event_create(C.byref(e0)))
    check(lib.jsgrad_hip_event_create(C.byref(e1)))
    t_first = llm.start_pos + 1
    w0 = time.perf_counter()
    check(lib.jsgrad_hip_event_record(e0))
    m.generate(steps)
    check(lib.jsgrad_hip_event_record(e1))
    check(lib.jsgrad_hip_sync())
    wall = time.perf_counter() - w0
    llm.start_pos += steps
    ms = C.c_float()
    check(lib.jsgrad_hip_event_elapsed_ms(e0, e1, C.byref(ms)))
    t_avg = t_first + (steps - 1) / 2.0          # mean number of visible positions over the timed steps
    tok_s = steps / wall

    # per-kernel durations: the same step, eager, with a start/stop event pair attached to every dispatch (the
    # dispatch's own begin/end stamps, as a kernel trace reports them).  Graph replays are queued first and not waited
    # for, so the eager launches run back to back like the replayed ones.
    def profiled(n_steps):
        check(lib.jsgrad_hip_profile(1))
        if use_graph:
            m.generate(blocker_steps)
            llm.start_pos += blocker_steps
        for _ in range(n_steps):
            m._step()
        kinds = {}
        for kname, kid in ffi.PROF_KINDS.items():
            n, tot = C.c_int(), C.c_double()
            check(lib.jsgrad_hip_profile_read(kid, C.byref(n), C.byref(tot)))
            if n.value:
                kinds[kname] = {"launches_per_step": n.value // n_steps, "ms_per_step": tot.value / n_steps}
        check(lib.jsgrad_hip_profile(0))
        llm.start_pos += n_steps
        return kinds

    fused = m._fused is not None
    kinds = profiled(profile_steps)
    sampled = None
    if not fused and with_sampled:
        # the same steps ending in the reference's default sampler (temperature 0.95, whole-vocabulary draw, llama3.ts:192)
        # instead of the greedy argmax: four small launches more per token
        m._set_sampling(0.95, 0, 0.0, 0.0, 0.0)
        m._step(); m._step(); m.generate(4)
        llm.start_pos += 6
        check(lib.jsgrad_hip_sync())
        w1 = time.perf_counter()
        m.generate(per_op_steps)
        check(lib.jsgrad_hip_sync())
        s_ms = 1e3 * (time.perf_counter() - w1) / per_op_steps
        llm.start_pos += per_op_steps
        sk = profiled(2).get("sample", {})
        sampled = {"temperature": 0.95, "tok_s": round(1e3 / s_ms, 2), "ms_per_step": round(s_ms, 4), "sampler_launches_per_step": sk.get("launches_per_step"),
                   "sampler_ms_per_step": round(sk.get("ms_per_step", 0.0), 4)}
        m._set_sampling(0.0, 0, 0.0, 0.0, 0.0)
    per_op = None
    if fused:
        # the same model through the one-launch-per-op path, for the per-family table and as a second data point
        saved, m._fused = m._fused, None
        if m.forward_jit is not None:
            m.forward_jit.reset()
        m._step(); m._step()
        llm.start_pos += 2
        check(lib.jsgrad_hip_sync())
        w1 = time.perf_counter()
        m.generate(per_op_steps)
        check(lib.jsgrad_hip_sync())
        per_op_ms = 1e3 * (time.perf_counter() - w1) / per_op_steps
        llm.start_pos += per_op_steps
        per_op = profiled(profile_steps)
        m._fused = saved
        if m.forward_jit is not None:
            m.forward_jit.reset()
    fam = per_op if fused else kinds
    kb = kernel_bytes(cfg, llm.start_pos, attn_wo="attn_wo" in fam)
    for kname, b_ in kb.items():
        k = fam[kname]
        k["bytes_per_step"] = int(b_)
        k["avg_us_per_launch"] = 1e3 * k["ms_per_step"] / k["launches_per_step"]
        k["GBps"] = b_ / (k["ms_per_step"] * 1e-3) / 1e9
    bytes_tok = synthetic.weight_bytes_per_token(cfg) + synthetic.kv_bytes_per_position(cfg) * t_avg
    # The measuring stick: a launch that only reads as many bytes as each weight-streaming launch of the step moves (cold
    # data, same event timing).  What the step would take if its launches did nothing but read.
    read_only = read_only_launches(lib, cfg, llm.start_pos, "attn_wo" in fam)
    for kname, r in read_only["families"].items():
        if kname in fam:
            fam[kname]["read_only_ms_per_step"] = r
    if fused:
        # one launch = one token: the step kernel is the dominant (only) kernel
        step_ms = kinds["decode_step"]["ms_per_step"]
        bytes_now = synthetic.weight_bytes_per_token(cfg) + synthetic.kv_bytes_per_position(cfg) * llm.start_pos
        achieved = bytes_now / (step_ms * 1e-3) / 1e9
        kern = "stream_step_kernel" if m._fused.mode == "stream" else "decode_step_kernel"
        roof = {"bound": "hbm", "kernel": f"{kern} (whole token: embedding, 5 phases x layers, lm_head, argmax)", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "bytes_per_launch": int(bytes_now), "avg_us_per_launch": round(step_ms * 1e3, 2)}
    else:
        # the lm_head on its own (the same event pairs, eager launches on cold-ish data), so that the `linear` family can be
        # reported per matrix: one lm_head launch of ~0.5 GB and L launches of w2 (and wo where it is a launch of its own)
        check(lib.jsgrad_hip_profile(1))
        for _ in range(6):
            m.output.call(m._ctx.h, out=m._ctx.logits, norm=m.norm)
        n_, tot_ = C.c_int(), C.c_double()
        check(lib.jsgrad_hip_profile_read(ffi.PROF_KINDS["linear"], C.byref(n_), C.byref(tot_)))
        check(lib.jsgrad_hip_profile(0))
        head_ms = tot_.value / max(1, n_.value)
        V, d, L = cfg["vocab_size"], cfg["dim"], cfg["n_layers"]
        head_b = (V * d + V * 2) if cfg["quantize"] == "int8" else V * d * 2
        rest_n = fam["linear"]["launches_per_step"] - 1
        rest_ms = max(1e-9, fam["linear"]["ms_per_step"] - head_ms)
        rest_b = kb["linear"] - head_b
        fam["linear"]["per_matrix"] = {
            "lm_head": {"launches_per_step": 1, "bytes_per_launch": int(head_b), "avg_us_per_launch": round(1e3 * head_ms, 2), "GBps": round(head_b / (head_ms * 1e-3) / 1e9, 1)}}
        if rest_n > 0:
            rest_name = "w2" if "attn_wo" in fam else "wo+w2"
            fam["linear"]["per_matrix"][rest_name] = {"launches_per_step": rest_n, "bytes_per_launch": int(rest_b / rest_n), "avg_us_per_launch": round(1e3 * rest_ms / rest_n, 2),
                                                      "GBps": round(rest_b / (rest_ms * 1e-3) / 1e9, 1)}
        # the dominant kernel: the weight-streaming family the step spends the most time in
        dom = max((k for k in kb if k in fam), key=lambda k: fam[k]["ms_per_step"])
        kern = {"linear": "gemv_kernel<EPI_STORE> (lm_head and the layer matrices that are launches of their own)", "ffn_gate": "gemv_kernel<EPI_SWIGLU> (ffn_norm + w1, w3 + SwiGLU)",
                "qkv_rope": "gemv_kernel<EPI_ROPE_KV> (attention_norm + wq, wk, wv + rotary + cache write)",
                "attn_wo": "attn_wo_kernel (decode attention + wo + residual)", "attn_decode": "attn_decode_kernel"}[dom]
        achieved = fam[dom]["GBps"]
        roof = {"bound": "hbm", "kernel": kern, "family": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "bytes_per_launch": int(kb[dom] / fam[dom]["launches_per_step"]), "avg_us_per_launch": round(fam[dom]["avg_us_per_launch"], 2),
                "ms_per_step": round(fam[dom]["ms_per_step"], 4),
                # the same launches as read-only kernels of the same sizes: the rate a launch of this size can reach at all
                "read_only_GBps": round(kb[dom] / (read_only["families"][dom] * 1e-3) / 1e9, 1),
                "families": {k: {"ms_per_step": round(fam[k]["ms_per_step"], 4), "GBps": round(fam[k]["GBps"], 1), "frac": round(fam[k]["GBps"] / HBM_PEAK_GBS, 4)}
                             for k in kb if k in fam}}
    rnd = lambda d: {k: {kk: (round(vv, 3) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in d.items()}
    res = {
        "name": name, "tok_s": tok_s, "ms_per_step": 1e3 * wall / steps, "event_ms_per_step": ms.value / steps,
        "roofline": roof,
        "step_roofline": {"bytes_per_token": int(bytes_tok), "achieved": round(bytes_tok * tok_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(bytes_tok * tok_s / 1e9 / HBM_PEAK_GBS, 4),
                          "read_only_launches_ms": round(read_only["step_ms"], 4), "read_only_sizes_us": read_only["sizes_us"]},
        "kernels": rnd(kinds),
        "config": {"workload": f"Llama-3 decode bs=1, {name}-shaped random init ({cfg['quantize']}), {prompt_len}-token prompt, {steps} greedy tokens",
                   "prompt": prompt_len, "decode": steps, "avg_visible_positions": t_avg, "max_context": ctx,
                   "launch": ("one persistent kernel per token" if fused else "one launch per fused op") + (", replayed as a HIP graph" if use_graph else ", eager")},
    }
    if sampled is not None:
        res["sampled"] = sampled
    if per_op is not None:
        res["per_op_path"] = {"tok_s": round(1e3 / per_op_ms, 2), "ms_per_step": round(per_op_ms, 4), "kernels": rnd(per_op)}
    return llm, cfg, res


def cpu_baseline(llm, cfg, budget_s=15.0, n_prompt=4):
    """Time the oracle on the host (1 thread) on the same weights and check its tokens against the GPU's."""
    import oracle as orc
    from denograd_amd import synthetic
    from denograd_amd.state import get_state_dict

    t0 = time.perf_counter()
    sd = {k: v.numpy() for k, v in get_state_dict(llm.model).items()}
    log(f"[cpu] weights copied to host in {time.perf_counter() - t0:.1f}s")
    ocfg = dict(cfg, max_context=64)
    cpu = orc.OracleModel(ocfg, sd)
    orc.set_threads(1)          # the reference's CLANG device runs one thread
    prompt = [int(t) for t in synthetic.random_prompt(cfg, n_prompt, seed=7)]
    t0 = time.perf_counter()
    cpu.forward([prompt[0]], 0, want_logits=False)
    per = time.perf_counter() - t0
    n_new = int(max(2, min(28, budget_s / per - len(prompt))))
    cpu.reset()
    t0 = time.perf_counter()
    toks_c = list(cpu.generate(prompt, n_new))
    dt = time.perf_counter() - t0
    n_fwd = len(prompt) + n_new - 1
    # the GPU on the same prompt from position 0 (stale cache rows past the current position are never read)
    llm.start_pos, llm.last_seen_toks = 0, []
    toks_g = llm.chat_tokens(prompt, n_new)["tokens"]
    same = sum(int(a == b) for a, b in zip(toks_g, toks_c))
    return {"value": round(n_fwd / dt, 4), "unit": "tok/s", "cores": 1, "kind": "port",
            "sample": f"{n_fwd} single-token forwards ({len(prompt)}-token prompt + {n_new} greedy tokens from position 0) of the same {cfg['name']} weights, "
                      f"C oracle (gcc -O2, fp16 storage, float accumulate), 1 thread of {os.cpu_count()} host cpus",
            "tokens_identical_to_gpu": f"{same}/{n_new}"}


MFMA_PEAK_TFLOPS = 2500.0    # MI355X dense fp16 matrix-core peak


def run_batched(name, bsz, prompt_len, steps):
    """Batched prefill (all prompts in one several-position pass, matrix-core GEMMs + causal attention), then batched
    greedy decode with the tokens fed back on the device.  Prefill is priced against the fp16 MFMA peak, decode against HBM."""
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.llama3 import Llama3

    lib = ffi.load()
    ctx = prompt_len + steps + 8
    cfg = synthetic.config(name, max_context=ctx)
    llm = Llama3.from_config(cfg).random_init(seed=0, tied=cfg["tied"])
    m = llm.model
    prompts = np.stack([synthetic.random_prompt(cfg, prompt_len, seed=100 + b) for b in range(bsz)]).astype(np.int32)
    m.forward_rows(prompts[:, :64], 0)                 # allocate caches / scratch, load code objects
    m.forward_rows(prompts, 0)                          # warm-up pass at full size
    check(lib.jsgrad_hip_sync())

    def read_kinds():
        kinds = {}
        for kname, kid in ffi.PROF_KINDS.items():
            n, tot = C.c_int(), C.c_double()
            check(lib.jsgrad_hip_profile_read(kid, C.byref(n), C.byref(tot)))
            if n.value:
                kinds[kname] = {"launches": n.value, "ms": round(tot.value, 3)}
        return kinds

    t0 = time.perf_counter()
    tok = m.forward_rows(prompts, 0)
    check(lib.jsgrad_hip_sync())
    prefill_s = time.perf_counter() - t0
    check(lib.jsgrad_hip_profile(1))
    tok = m.forward_rows(prompts, 0)
    pre_kinds = read_kinds()
    check(lib.jsgrad_hip_profile(0))

    d, L, H, KV, F, V = cfg["dim"], cfg["n_layers"], cfg["n_heads"], cfg["n_kv_heads"], cfg["hidden_dim"], cfg["vocab_size"]
    hd = d // H
    e_l = 2 * d * H * hd + 2 * d * KV * hd + 3 * d * F           # linear elements per layer
    rows = bsz * prompt_len
    lin_flop = 2.0 * L * e_l * rows + 2.0 * V * d * bsz           # lm_head on the last position only
    att_flop = 2.0 * prompt_len * prompt_len * H * hd * L * bsz  # causal: QK^T + PV over the lower triangle
    gemm_ms = pre_kinds.get("gemm", {}).get("ms", 0.0)
    prefill = {"tok_s": round(rows / prefill_s, 1), "seconds": round(prefill_s, 4), "tokens": rows,
               "flop": lin_flop + att_flop, "tflops": round((lin_flop + att_flop) / prefill_s / 1e12, 1),
               "roofline": {"bound": "mfma", "kernel": "gemm_kernel (all Linear layers of the pass)", "achieved": round(lin_flop / (gemm_ms * 1e-3) / 1e12, 1) if gemm_ms else None,
                            "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(lin_flop / (gemm_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4) if gemm_ms else None,
                            "traffic": None},
               "kernels": pre_kinds}

    # batched decode: one position per sequence per step (4 warm-up steps, the timed ones, 4 profiled ones)
    steps = max(steps, 9)
    pos = prompt_len
    for _ in range(4):
        tok = m.forward_rows(tok, pos); pos += 1
    check(lib.jsgrad_hip_sync())
    t0 = time.perf_counter()
    for _ in range(steps - 4 - 4):
        tok = m.forward_rows(tok, pos); pos += 1
    check(lib.jsgrad_hip_sync())
    dec_s = time.perf_counter() - t0
    n_dec = steps - 8
    check(lib.jsgrad_hip_profile(1))
    for _ in range(4):
        tok = m.forward_rows(tok, pos); pos += 1
    dec_kinds = read_kinds()
    check(lib.jsgrad_hip_profile(0))
    t_avg = prompt_len + 4 + n_dec / 2.0
    bytes_step = synthetic.weight_bytes_per_token(cfg) + bsz * synthetic.kv_bytes_per_position(cfg) * t_avg
    gpu_ms = sum(v["ms"] for v in dec_kinds.values()) / 4
    decode = {"tok_s": round(bsz * n_dec / dec_s, 1), "steps_s": round(n_dec / dec_s, 2), "ms_per_step": round(1e3 * dec_s / n_dec, 4),
              "kernel_ms_per_step": round(gpu_ms, 4), "bytes_per_step": int(bytes_step),
              "roofline": {"bound": "hbm", "achieved": round(bytes_step * n_dec / dec_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(bytes_step * n_dec / dec_s / 1e9 / HBM_PEAK_GBS, 4)},
              "kernels": {k: {"launches_per_step": v["launches"] // 4, "ms_per_step": round(v["ms"] / 4, 4)} for k, v in dec_kinds.items()}}
    return {"config": {"workload": f"Llama-3 {name}-shaped random init ({cfg['quantize']}), {bsz} sequences x {prompt_len}-token prompts in one pass, "
                                   f"then {steps} batched greedy steps", "batch": bsz, "prompt": prompt_len, "decode": steps, "max_context": ctx},
            "prefill": prefill, "decode": decode}


def traffic_probe(name, batch=1, position=0):
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.llama3 import Llama3
    from denograd_amd.tensor import Tensor
    lib = ffi.load()
    n = 512 << 20
    src, dst = Tensor.zeros((n,), "uint8"), Tensor.empty((n,), "uint8")
    check(lib.jsgrad_hip_sync())
    check(lib.jsgrad_hip_copy(dst.ptr, src.ptr, n))      # reads 512 MiB, writes 512 MiB
    check(lib.jsgrad_hip_sync())
    cfg = synthetic.config(name, max_context=position + 64)
    llm = Llama3.from_config(cfg).random_init(seed=0, tied=cfg["tied"])
    llm.model.forward_jit = None
    llm.start_pos = position      # the cache rows before it are whatever the allocation holds: the counters do not care
    for t in (1, 2, 3, 4):
        llm._call(t)
        llm.start_pos += 1
    check(lib.jsgrad_hip_sync())
    if batch > 1:      # two batched decode steps (the few-row kernels) after an 8-token batched prefill
        prompts = np.stack([synthetic.random_prompt(cfg, 8, seed=100 + b) for b in range(batch)]).astype(np.int32)
        tok = llm.model.forward_rows(prompts, 0)
        tok = llm.model.forward_rows(tok, 8)
        tok = llm.model.forward_rows(tok, 9)
        check(lib.jsgrad_hip_sync())


STAMP_NAMES = {0: "position word read", 10: "attention item starts", 11: "query rows in LDS", 12: "scores done", 13: "softmax done", 14: "P.V in the wavefronts' slots",
               15: "partial result stored", 16: "every chunk's (m, l) seen", 17: "merge weights ready", 18: "merged row stored", 1: "attention item done",
               2: "wo: hint of the attention row seen", 3: "wo: hint barrier", 4: "wo: attention row staged", 21: "wo rows done",
               5: "x requested, table written", 6: "first item requested", 7: "x arrived, squares summed", 9: "sum of squares exchanged",
               26: "... by the block's last wavefront", 27: "first item requested by the last wavefront", 28: "x arrived in the last wavefront",
               23: "x staged, first two items requested", 24: "first item used", 25: "second item used", 8: "end"}


def stamps(name, position, layers=8):
    """Time stamps taken INSIDE the kernels (a library built with `make TRACE=1`): the 100 MHz device clock kept in LDS by one
    thread of three blocks per launch and copied out when the block ends.  Runs a few eager decode steps of `name` (cut to
    `layers` layers) from `position` and prints, for the last attention launch and the last w1 | w3 launch, microseconds
    since the earliest stamp of that launch."""
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.llama3 import Llama3
    lib = ffi.load()
    raw = C.CDLL(ffi.LIB_PATH)
    if not hasattr(raw, "jsgrad_hip_gemv_trace"):
        raise SystemExit("this library has no time stamps: build it with `make -B -C denograd_amd/csrc TRACE=1`")
    cfg = synthetic.config(name, max_context=position + 64, n_layers=layers)
    llm = Llama3.from_config(cfg).random_init(seed=0, tied=cfg["tied"])
    m = llm.model
    m.forward_jit = None
    llm.start_pos = position
    for t in (1, 2, 3):
        llm._call(t)
        llm.start_pos += 1
    buf = (C.c_ulonglong * 128)()
    out = {}

    def read(entry, rows):
        fn = getattr(raw, entry)
        fn.argtypes, fn.restype = [C.c_void_p], C.c_int
        check(fn(buf))
        t4 = np.array(buf[:], dtype=np.uint64).reshape(4, 32)
        t, whole = t4[:3].astype(np.int64), t4[3]       # row 3: over all blocks of the launch (earliest start kept complemented)
        if not (t > 0).any():
            return None
        t0 = t[t > 0].min()
        res = {who: {STAMP_NAMES[s_]: round((int(t[r][s_]) - int(t0)) / 100.0, 2) for s_ in sorted(STAMP_NAMES, key=lambda k: t[r][k]) if t[r][s_] > 0}
               for r, who in enumerate(rows)}
        if whole[2]:
            us = lambda v: round((int(v) - int(t0)) / 100.0, 2)
            res["all blocks of the launch"] = {"latest block end": us(whole[2])}
        return res
    fused = m._ctx.fuse_attn_wo
    llm._call(4)
    llm.start_pos += 1
    if fused:
        out["attn_wo_kernel"] = read("jsgrad_hip_attn_wo_trace", ["block 0 (chunk 0 of kv head 0: merges)", "block n_kv_heads (chunk 1 of kv head 0, then wo rows)", "last block (wo rows only)"])
    else:
        out["attn_decode_kernel"] = read("jsgrad_hip_attn_decode_trace", ["chunk 0 of kv head 0 (merges)", "chunk 1 of kv head 0", "last chunk of the last kv head"])
    # the w1 | w3 launch of one layer, alone (the trace keeps the last launch of its translation unit)
    blk, ctx = m.layers[layers - 1], m._ctx
    f = blk.feed_forward
    sp = lambda l: l.scale.ptr if l.scale is not None else None
    check(lib.jsgrad_hip_ffn_gate(f.w1.kind, f.w1.weight.ptr, sp(f.w1), f.w3.weight.ptr, sp(f.w3), ctx.h.ptr, blk.ffn_norm.weight.ptr, blk.ffn_norm.eps, ctx.g.ptr,
                                  m.dim, m.hidden_dim, ffi.F16))
    out["gemv_kernel<EPI_SWIGLU> (w1 | w3)"] = read("jsgrad_hip_gemv_trace", ["block 0", "middle block", "last block"])
    return {"workload": name, "position": position, "layers": layers, "microseconds_since_first_stamp": out}


def run_rows_gemm(workload="8B-int8", rows=16, only=""):
    """The several-row Linear launches of one decode step of `rows` sequences, one shape at a time: wq|wk|wv (as one plain
    matrix of their combined height), wo, w1|w3 + SwiGLU, w2, lm_head.  Weights are rotated over cold copies (more than the
    256 MB of memory-side cache between two uses of a copy); time per launch from the event pair around each dispatch.
    `only`: comma-separated subset of the shape names (e.g. "lm_head" for a counter run on one kernel)."""
    from denograd_amd import ffi, synthetic
    from denograd_amd.ffi import check
    from denograd_amd.tensor import Tensor
    lib = ffi.load()
    cfg = synthetic.CONFIGS[workload]
    if cfg["quantize"] != "int8":
        raise SystemExit("--rows-gemm-only is written for int8 workloads")
    dim, hidden, vocab = cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
    hd = dim // cfg["n_heads"]
    shapes = {"qkv": (dim + 2 * cfg["n_kv_heads"] * hd, dim), "wo": (dim, dim), "w1w3": (hidden, dim), "w2": (dim, hidden), "lm_head": (vocab, dim)}
    out = {}
    for name, (o, i) in shapes.items():
        if only and name not in only.split(","):
            continue
        nb = o * i * (2 if name == "w1w3" else 1)
        ncopy = max(3, min(10, (2 << 30) // nb))
        def make():
            w = Tensor.empty((o, i), "int8")
            check(lib.jsgrad_hip_memset(w.ptr, 3, o * i))
            return w
        ws = [(make(), make() if name == "w1w3" else None) for _ in range(ncopy)]
        sc, x = Tensor.ones((o,), "float16"), Tensor.randn((rows, i), "float16", 2, 1.0)
        y, res = Tensor.empty((rows, o), "float16"), Tensor.randn((rows, o), "float16", 3, 1.0)
        def launch(k):
            a, b = ws[k % ncopy]
            if b is not None:
                check(lib.jsgrad_hip_gemm_ffn_gate(ffi.W_I8, a.ptr, sc.ptr, b.ptr, sc.ptr, x.ptr, rows, y.ptr, i, o))
            else:
                check(lib.jsgrad_hip_gemm(ffi.W_I8, a.ptr, sc.ptr, o, i, x.ptr, rows, y.ptr, res.ptr if name in ("wo", "w2") else None))
        for k in range(ncopy):
            launch(k)
        check(lib.jsgrad_hip_profile(1))
        for k in range(3 * ncopy):
            launch(k)
        n, tot = C.c_int(), C.c_double()
        check(lib.jsgrad_hip_profile_read(ffi.PROF_KINDS["gemm"], C.byref(n), C.byref(tot)))
        check(lib.jsgrad_hip_profile(0))
        us = 1e3 * tot.value / n.value
        out[name] = {"out_features": o * (2 if name == "w1w3" else 1), "in_features": i, "bytes": nb, "us": round(us, 2), "GBps": round(nb / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4)}
        del ws
    return {"workload": workload, "rows": rows, "shapes": out}


def run_formats(reps=5):
    """Load-time kernels of the checkpoint path, each on one lm_head-sized tensor (128256 x 2048 elements): GGML Q6_K ->
    float32, bfloat16 -> float16, and the q_proj row permutation.  HBM-bound byte work: bytes read + written per second."""
    from denograd_amd import ffi
    from denograd_amd.ffi import check
    from denograd_amd.tensor import Tensor

    lib = ffi.load()
    rows, cols = 128256, 2048
    n = rows * cols
    e0, e1 = C.c_void_p(), C.c_void_p()
    check(lib.jsgrad_hip_event_create(C.byref(e0)))
    check(lib.jsgrad_hip_event_create(C.byref(e1)))

    def timed(fn, nbytes):
        fn()
        check(lib.jsgrad_hip_event_record(e0))
        for _ in range(reps):
            fn()
        check(lib.jsgrad_hip_event_record(e1))
        ms = C.c_float()
        check(lib.jsgrad_hip_event_elapsed_ms(e0, e1, C.byref(ms)))
        us = 1e3 * ms.value / reps
        return {"bytes": int(nbytes), "us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    out = {}
    nb = lib.jsgrad_hip_ggml_nbytes(14, n)
    blocks = Tensor.empty((nb,), "uint8")
    check(lib.jsgrad_hip_memset(blocks.ptr, 0x11, nb))
    f32 = Tensor.empty((n,), "float32")
    out["ggml_q6k_dequant"] = timed(lambda: check(lib.jsgrad_hip_ggml_dequant(14, blocks.ptr, n, f32.ptr)), nb + 4 * n)
    h = Tensor.empty((rows, cols), "float16")
    out["bf16_to_f16"] = timed(lambda: check(lib.jsgrad_hip_cast(f32.ptr, ffi.BF16, h.ptr, ffi.F16, n)), 4 * n)
    h2 = Tensor.empty((rows, cols), "float16")
    out["hf_permute"] = timed(lambda: check(lib.jsgrad_hip_hf_permute(h.ptr, h2.ptr, rows, cols * 2, rows // 64)), 4 * n)
    out["tensor"] = f"{rows} x {cols} elements"
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--workload", default="1B", help="primary synthetic config (denograd_amd/synthetic.py)")
    ap.add_argument("--secondary", default="8B-int8", help="second workload measured in the same run ('' to skip)")
    ap.add_argument("--secondary-steps", type=int, default=128)
    ap.add_argument("--others", default="3B-int8:1024:64,8B-nf4:4096:64", help="further bs=1 decode legs as name:prompt:steps (the remaining BASELINE configurations; "
                    "their prompts are fed in one several-position pass); '' to skip")
    ap.add_argument("--batched", default="8B-int8", help="workload of the batched prefill + batched decode leg ('' to skip)")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--batch-prompt", type=int, default=2048)
    ap.add_argument("--batch-steps", type=int, default=128)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle baseline")
    ap.add_argument("--traffic-probe", action="store_true", help="for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: one 512 MiB device-to-device copy "
                    "(a plain copy kernel of known size, to scale the counters) followed by 4 eager decode steps of --workload; prints nothing")
    ap.add_argument("--traffic-batch", type=int, default=1, help="with --traffic-probe: also two batched decode steps of this many sequences")
    ap.add_argument("--traffic-position", type=int, default=0, help="with --traffic-probe: the position the four decode steps start from (attention then reads that many cache rows)")
    ap.add_argument("--stamps", action="store_true", help="with a library built by `make TRACE=1`: time stamps taken inside the attention and w1 | w3 kernels of --workload "
                    "at --traffic-position; prints their JSON")
    ap.add_argument("--fused-step", action="store_true", help="run each token as one persistent kernel (jsgrad_hip_decode_step) instead of one launch per fused op")
    ap.add_argument("--stream-step", action="store_true", help="run each token as one persistent kernel with streaming wavefronts (jsgrad_hip_stream_step)")
    ap.add_argument("--formats-only", action="store_true", help="only the load-time kernels of the checkpoint path (GGML dequantisation, casts, row permutation); prints their JSON")
    ap.add_argument("--rows-gemm-only", action="store_true", help="only the several-row Linear launches of a batched decode step (--batched workload, --batch rows), "
                    "one shape at a time over cold weights; prints their JSON")
    ap.add_argument("--rows-gemm-shapes", default="", help="with --rows-gemm-only: comma-separated subset of qkv,wo,w1w3,w2,lm_head")
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel eagerly instead of replaying a captured HIP graph "
                    "(rocprofv3 --kernel-trace on this image crashes inside hipGraphLaunch, so profiles are taken this way)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus must be 1")
        sys.exit(2)

    from denograd_amd import ffi
    from denograd_amd.device import Device
    if args.stamps:
        ffi.LIB_PATH = ffi.LIB_PATH.replace(".so", "_trace.so")      # the library `make TRACE=1` builds beside the product
    dev = Device.get("HIP").init()
    log(f"device: {dev.name}, {dev.cu_count} CUs")

    if args.traffic_probe:
        traffic_probe(args.workload, args.traffic_batch, args.traffic_position)
        return
    if args.stamps:
        print(json.dumps({"stamps": stamps(args.workload, args.traffic_position)}), flush=True)
        return
    if args.formats_only:
        print(json.dumps({"formats": run_formats()}), flush=True)
        return
    if args.rows_gemm_only:
        print(json.dumps({"rows_gemm": run_rows_gemm(args.batched or "8B-int8", args.batch, args.rows_gemm_shapes)}), flush=True)
        return
    step_mode = "stream" if args.stream_step else args.fused_step
    llm, cfg, res = run_workload(args.workload, args.prompt, args.steps, args.warmup, use_graph=not args.no_graph, fused_step=step_mode)
    cpu = None if args.no_cpu else cpu_baseline(llm, cfg)
    del llm
    secondary, cpu2 = None, None
    if args.secondary:
        llm2, cfg2, secondary = run_workload(args.secondary, args.prompt, args.secondary_steps, args.warmup, use_graph=not args.no_graph, fused_step=step_mode)
        cpu2 = None if args.no_cpu else cpu_baseline(llm2, cfg2, budget_s=12.0, n_prompt=2)
        del llm2
    others = {}
    for spec in filter(None, args.others.split(",")):
        oname, oprompt, osteps = spec.split(":")
        llm3, cfg3, r3 = run_workload(oname, int(oprompt), int(osteps), args.warmup, profile_steps=4, use_graph=not args.no_graph, fused_step=False,
                                      prefill="rows", with_sampled=False)
        del llm3
        others[oname] = {"value": round(r3["tok_s"], 2), "unit": "tok/s", "steps": int(osteps), "ms_per_step": round(r3["ms_per_step"], 4),
                         "dtype": f"{cfg3['quantize']} weights, f16 activations", "config": r3["config"], "roofline": r3["roofline"],
                         "step_roofline": r3["step_roofline"], "kernels": r3["kernels"]}

    out = {
        "metric": "decode tok/s bs=1 + % HBM roofline, Llama-3.2-1B fp16 & 8B int8",
        "value": round(res["tok_s"], 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "config": res["config"],
        "roofline": res["roofline"], "cpu_baseline": cpu,
        "step_roofline": res["step_roofline"], "kernels": res["kernels"], "event_ms_per_step": round(res["event_ms_per_step"], 4),
        "launch_mode": "eager" if args.no_graph else "hip_graph", "per_op_path": res.get("per_op_path"), "sampled": res.get("sampled"),
    }
    if secondary:
        out["secondary"] = {"value": round(secondary["tok_s"], 2), "unit": "tok/s", "steps": args.secondary_steps, "ms_per_step": round(secondary["ms_per_step"], 4),
                            "dtype": "i8 weights, f16 activations", "config": secondary["config"], "roofline": secondary["roofline"],
                            "step_roofline": secondary["step_roofline"], "kernels": secondary["kernels"], "per_op_path": secondary.get("per_op_path"),
                            "sampled": secondary.get("sampled"), "cpu_baseline": cpu2}
    if others:
        out["others"] = others
    if args.batched:
        out["batched"] = run_batched(args.batched, args.batch, args.batch_prompt, args.batch_steps)
    out["formats"] = run_formats()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
