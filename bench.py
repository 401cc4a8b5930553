#!/usr/bin/env python3
"""Decode throughput of the quantized llama hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b-q4k|stories-6l-q8_0] [--no-cpu-baseline]

One step = one greedy decode token at batch 1 (LM head + argmax, then the trunk for the chosen token).
The model is random-init from a seed in the packed GGUF format, resident in HBM before the timed region;
the prompt is prefilled outside the timed region, as the reference excludes prefill from tokens/s
(RealModelInferenceEngine.swift:6355, 6415-6419).  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X published HBM3E peak

WORKLOADS = {
    # BASELINE.json configs[3]
    "llama3-8b-q4k": dict(arch="LLAMA3_8B", fmt="q4_k", kv="f16", prompt=512, decode=256, seed=4,
                          describe="Llama-3-8B architecture, random-init, Q4_K linears + Q4_K lm_head, fp16 "
                                   "embedding/norms/KV; 512-token prompt then greedy decode at batch 1"),
    # BASELINE.json configs[1]
    "stories-6l-q8_0": dict(arch="STORIES_6L", fmt="q8_0", kv="f32", prompt=16, decode=128, seed=2,
                            describe="6-layer d=768 llama (12 heads x 64, FFN 2048, vocab 32000, ctx 256), all linears "
                                     "Q8_0; 16-token prompt then greedy decode at batch 1"),
}


def build_model(name: str):
    import espresso_amd.llama as ll
    import espresso_amd.synthetic as syn
    from espresso_amd import _lib
    w = WORKLOADS[name]
    cfg = ll.MultiModelConfig(**getattr(syn, w["arch"]))
    fmt = _lib.FORMAT_NAMES[w["fmt"]]
    kv = _lib.FORMAT_F16 if w["kv"] == "f16" else _lib.FORMAT_F32
    t0 = time.time()
    rt, packed = syn.build_runtime(cfg, fmt, seed=w["seed"], kv_format=kv, keep_packed=True)
    return cfg, rt, packed, time.time() - t0


def run_gpu(name: str, steps: int, warmup: int, graph: bool = True):
    import espresso_amd.llama as ll
    w = WORKLOADS[name]
    cfg, rt, packed, build_s = build_model(name)
    ll.set_graph_replay(rt, graph)
    if w["prompt"] + warmup + steps + 1 > cfg.max_seq:
        raise SystemExit(f"prompt {w['prompt']} + warmup {warmup} + steps {steps} does not fit context {cfg.max_seq}")
    prompt = np.random.default_rng(1000 + w["seed"]).integers(0, cfg.vocab, w["prompt"]).astype(np.uint32)
    t0 = time.perf_counter()
    rt.prefill(prompt)
    prefill_s = time.perf_counter() - t0
    warm_tokens = ll.continue_greedy(rt, warmup)
    # ---- timed region: exactly `steps` decode steps; every step ends with a device-to-host read of the
    # chosen token, so the region is bracketed by stream synchronisation on both sides
    rt.last_hidden()
    t0 = time.perf_counter()
    tokens = ll.continue_greedy(rt, steps)
    rt.last_hidden()
    elapsed = time.perf_counter() - t0
    # ---- instrumented pass (not part of `value`): HIP events around every GEMV/attention launch
    extra = min(32, cfg.max_seq - rt.visible() - 1)
    ll.set_kernel_timing(rt, True)
    ll.continue_greedy(rt, extra)
    kt = ll.kernel_times(rt)
    ll.set_kernel_timing(rt, False)
    timed = {k: ll.time_kernel_dispatch(rt, k, 8) for k in ("qkv", "wo", "gate_up", "down", "head")}
    b2b = {k: v[0] for k, v in timed.items()}
    own = {k: v[1] for k, v in timed.items()}
    # the prompt once more, now that every kernel has run before (the first walk above includes what a kernel's first launch costs)
    rt.reset()
    rt.last_hidden()
    t0 = time.perf_counter()
    rt.prefill(prompt)
    rt.last_hidden()
    prefill_again_s = time.perf_counter() - t0
    # and with every operand rounded to fp16 once (the faster, less exact block path)
    ll.set_split_activations(rt, False)
    rt.reset()
    rt.last_hidden()
    t0 = time.perf_counter()
    rt.prefill(prompt)
    rt.last_hidden()
    prefill_fp16_s = time.perf_counter() - t0
    ll.set_split_activations(rt, True)
    return dict(prefill_fp16_s=prefill_fp16_s, kernel_us=own, cfg=cfg, rt=rt, packed=packed, prompt=prompt, tokens=warm_tokens + tokens, elapsed=elapsed,
                build_s=build_s, prefill_s=prefill_s, prefill_again_s=prefill_again_s, kernel_times=kt, b2b_us=b2b, weight_bytes=rt.weight_bytes)


def cpu_baseline(name: str, gpu: dict) -> dict:
    """Times the CPU oracle (the C restatement of the reference's CPU-exact path) in the reference's default arithmetic - fp32
    activations into every matrix product - on a bounded sample of the same model: same packed bytes, dequantised to fp32 as the
    reference holds them.  The 6-layer model runs whole on one thread; the 8B model runs whole (all 32 layers, 32 GB of fp32
    weights) with the matrix-vector rows spread over the host cores this process may use, on a short prompt."""
    from oracle import oracle as orc
    from espresso_amd import _lib
    w = WORKLOADS[name]
    cfg, packed = gpu["cfg"], gpu["packed"]
    fmt = _lib.FORMAT_NAMES[w["fmt"]]
    host_cores = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = host_cores
    full = name == "stories-6l-q8_0"
    threads = 1 if full else max(1, min(16, usable))
    prompt = gpu["prompt"]
    n_prompt = len(prompt) if full else 32
    before = orc.get_threads()
    orc.set_threads(threads)
    try:
        t0 = time.perf_counter()
        rt = orc.runtime_from_packed(cfg, packed, fmt, cfg.n_layer, w["kv"] == "f16", cfg.max_seq if full else n_prompt + 24, gemv_inputs_fp16=False)
        t_load = time.perf_counter() - t0
        t0 = time.perf_counter()
        rt.prefill(prompt[:n_prompt].tolist())
        t_prefill = time.perf_counter() - t0
        n_tok = 32 if full else 16
        toks = []
        t0 = time.perf_counter()
        for _ in range(n_tok):
            t = rt.select_greedy(); toks.append(t); rt.advance(t)
        dt = time.perf_counter() - t0
        rt.close()
    finally:
        orc.set_threads(before)
    out = {"value": n_tok / dt, "unit": "tok/s", "cores": threads, "host_cores": host_cores, "usable_cores": usable, "kind": "port",
           "arithmetic": "reference default: fp32 activations, fp32 dequantised weights, fp32 sums"}
    if full:
        same = toks == gpu["tokens"][:n_tok]
        out["sample"] = (f"whole model, {n_tok} greedy tokens after the same {n_prompt}-token prompt on one thread; "
                         f"tokens identical to the GPU run: {same}")
    else:
        out["sample"] = (f"whole model (all {cfg.n_layer} layers, fp32 weights dequantised in {t_load:.1f} s), {n_tok} greedy tokens after the "
                         f"first {n_prompt} tokens of the prompt were walked ({t_prefill:.1f} s, {n_prompt / t_prefill:.1f} tok/s); matrix-vector "
                         f"rows over {threads} threads (the order of every row's sum is the single-threaded one)")
    return out


# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# workload (FETCH_SIZE scaled by 2.000, WRITE_SIZE by 1.000, the factors kernels of known size in the same runs gave);
# the runs and the per-kernel table are in profiles/q4k_gemv_decode_llama3_8b_pmc_traffic.txt.
TRAFFIC_FILE = "profiles/q4k_gemv_decode_llama3_8b_pmc_traffic.txt"
# the same kernel's mean duration in the committed rocprofv3 kernel trace (a profiled run with eager launches)
TRACE_FILE = "profiles/q4k_gemv_decode_llama3_8b_kernel_trace.txt"
TRAFFIC_SOURCE = TRAFFIC_FILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this workload; not measured in this run)"


def profile_figure(path: str, key: str):
    """A figure the committed profile summaries carry on a line of their own, `key = value`; None when the file or the line is absent."""
    try:
        with open(os.path.join(ROOT, path)) as f:
            for line in f:
                parts = line.split("=")
                if len(parts) == 2 and parts[0].strip() == key:
                    return float(parts[1].split()[0])
    except OSError:
        pass
    return None


def measured_traffic(workload: str, kernel: str):
    v = profile_figure(TRAFFIC_FILE, f"{workload}.{kernel}.hbm_bytes_per_launch")
    return int(v) if v is not None else None


def profile_kernel_us(workload: str, kernel: str):
    return profile_figure(TRACE_FILE, f"{workload}.{kernel}.mean_us")


# BASELINE.json configs[2]: weight-GEMV microbenchmark at the Llama-3-8B layer shapes
MICRO_SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]


def run_microbench(shapes=None, formats=("q4_k", "q4_0"), batches=(1, 2, 4, 8), launches=100) -> dict:
    """Isolated dequant-GEMV (matrix-core GEMV kernels: one to four rows, and five to eight rows in one pass) for Q4_K and Q4_0, weights
    rotated through enough copies that no launch finds them in the last-level cache."""
    import espresso_amd.ops as ops
    from espresso_amd import _lib
    rows_out = []
    for name in formats:
        fmt = _lib.FORMAT_NAMES[name]
        for rows, cols in (shapes or MICRO_SHAPES):
            blocks = ops.synth_weights(fmt, 7 + rows + cols, 0.02, rows * cols)
            m = ops.Matrix(fmt, blocks, rows, cols)
            rotate = max(2, min(64, int(600e6 // m.bytes) + 1))
            for batch in batches:
                t = m.time_gemv(batch, 10, launches, rotate)
                nbytes = m.bytes + batch * cols * 2 + batch * rows * 4
                rows_out.append({"format": name, "rows": rows, "cols": cols, "batch": batch, "mean_us": round(t["mean_us"], 2),
                                 "gbps": round(nbytes / t["mean_us"] / 1e3, 1), "frac_hbm_peak": round(nbytes / t["mean_us"] / 1e3 / HBM_PEAK_GBPS, 3),
                                 "bytes": nbytes})
            m.close()
    return {"metric": "dequant-GEMV HBM GB/s", "unit": "GB/s", "n_gpus": 1, "data": "synthetic",
            "how": f"mean of {launches} back-to-back launches between two HIP events after 10 warm-up launches; weights rotate "
                   "through copies totalling > 600 MB so every launch reads HBM; each mean includes the ~4 us a dependent launch costs",
            "results": rows_out}


def run_two_token(steps: int) -> dict:
    """BASELINE.json configs[4]: 6-layer fp16 target, 1-layer draft of the same width and vocabulary, both random-init;
    16-token prompts; the exact two-token loop until the context is full, at batch 1 and at batch 16 (sixteen sequences in
    lock step, 32-row passes on the matrix cores); in both, a pass is one captured graph with every decision on the device.  tok/s counts decode time only (the loop's own decode_ms; prefill excluded)."""
    import espresso_amd.llama as ll
    import espresso_amd.synthetic as syn
    from espresso_amd import _lib
    tcfg = ll.MultiModelConfig(**syn.STORIES_6L)
    dcfg = ll.MultiModelConfig(**dict(syn.STORIES_6L, n_layer=1))
    target, packed = syn.build_runtime(tcfg, _lib.FORMAT_F16, seed=1, max_sequences=16, keep_packed=True)
    draft, _ = syn.build_runtime(dcfg, _lib.FORMAT_F16, seed=9, max_sequences=16)
    rng = np.random.default_rng(1001)
    prompts = [rng.integers(0, tcfg.vocab, 16).astype(np.uint32) for _ in range(16)]
    n = min(steps, tcfg.max_seq - 16)

    def timed(t, d):
        ll.generate_two_token(t, d, prompts[0], 8)              # warm-up
        tokens, st = ll.generate_two_token(t, d, prompts[0], n)
        return tokens, st, len(tokens) / (st["decode_ms"] * 1e-3)

    def plain_rate(t):
        t.generate(prompts[0], 8)
        t0 = time.perf_counter()
        t.prefill(prompts[0])
        t_prefill = time.perf_counter() - t0
        t0 = time.perf_counter()
        toks, _ = t.generate(prompts[0], n)
        return toks, len(toks) / (time.perf_counter() - t0 - t_prefill)

    def report(tokens, st, rate, plain, plain_tok_s):
        return {"tok_s": rate, "passes": st["passes"], "accepted_future_tokens_per_pass": st["accepted_total"] / max(st["passes"], 1),
                "committed_exact_tokens_per_pass": st["committed_total"] / max(st["passes"], 1),
                "stream_identical_to_plain_greedy": tokens == plain[:len(tokens)], "plain_greedy_tok_s": plain_tok_s,
                "speedup_over_plain_greedy": rate / plain_tok_s}

    plain, plain_tok_s = plain_rate(target)
    tokens, stats, rate = timed(target, draft)
    # the target as its own draft: every proposal is accepted, but the draft costs as much as the target
    twin, _ = syn.build_runtime(tcfg, _lib.FORMAT_F16, seed=1)
    twin_tokens, twin_stats, twin_rate = timed(target, twin)
    twin.close()
    # a one-layer draft that always agrees: a target of the same shape and cost whose layers above the first add nothing
    # (zero output projections), drafted by its own first layer.  The scheme's ceiling with a draft of this size.
    agree = dict(packed, layers=[dict(L) for L in packed["layers"]])
    for L in agree["layers"][1:]:
        L["wo"] = np.zeros_like(np.asarray(L["wo"]))
        L["w2"] = np.zeros_like(np.asarray(L["w2"]))
    a_target, a_draft = ll.LlamaRuntime(tcfg, max_sequences=16), ll.LlamaRuntime(dcfg, max_sequences=16)
    ll.load_packed_weights(a_target, agree, _lib.FORMAT_F16)
    ll.load_packed_weights(a_draft, dict(agree, layers=agree["layers"][:1]), _lib.FORMAT_F16)
    a_plain, a_plain_tok_s = plain_rate(a_target)
    a_tokens, a_stats, a_rate = timed(a_target, a_draft)

    def batch_runs(t, d):
        runs = {}
        for label, dd in (("plain_greedy", None), ("two_token", d)):
            t.reset(); d.reset()
            ll.generate_batch(t, prompts, 4, draft=dd)           # warm-up
            t.reset(); d.reset()
            toks, st = ll.generate_batch(t, prompts, n, draft=dd)
            runs[label] = {"tokens": toks, "tok_s": sum(len(x) for x in toks) / (st["decode_ms"] * 1e-3), "stats": st}
        return runs

    batch = batch_runs(target, draft)
    a_batch = batch_runs(a_target, a_draft)
    a_target.close(); a_draft.close()
    b2, ab2 = batch["two_token"]["stats"], a_batch["two_token"]["stats"]
    return {"metric": "exact two-token decode tok/s (6L d768 fp16 target, 1L draft)", "value": rate, "unit": "tok/s",
            "n_gpus": 1, "steps": len(tokens), "data": "synthetic", "higher_is_better": True,
            "batch1": dict(report(tokens, stats, rate, plain, plain_tok_s),
                           target_as_its_own_draft=report(twin_tokens, twin_stats, twin_rate, plain, plain_tok_s),
                           one_layer_draft_that_always_agrees=report(a_tokens, a_stats, a_rate, a_plain, a_plain_tok_s)),
            "batch16": {"tok_s": batch["two_token"]["tok_s"], "passes": b2["passes"],
                        "accepted_future_tokens_per_pass_per_sequence": b2["accepted_total"] / max(b2["passes"], 1) / 16,
                        "committed_exact_tokens_per_pass_per_sequence": b2["committed_total"] / max(b2["passes"], 1) / 16,
                        "streams_identical_to_plain_greedy": batch["two_token"]["tokens"] == batch["plain_greedy"]["tokens"],
                        "plain_greedy_tok_s": batch["plain_greedy"]["tok_s"],
                        "one_layer_draft_that_always_agrees": {
                            "tok_s": a_batch["two_token"]["tok_s"], "passes": ab2["passes"],
                            "accepted_future_tokens_per_pass_per_sequence": ab2["accepted_total"] / max(ab2["passes"], 1) / 16,
                            "streams_identical_to_plain_greedy": a_batch["two_token"]["tokens"] == a_batch["plain_greedy"]["tokens"],
                            "plain_greedy_tok_s": a_batch["plain_greedy"]["tok_s"],
                            "speedup_over_plain_greedy": a_batch["two_token"]["tok_s"] / a_batch["plain_greedy"]["tok_s"]}},
            "note": "a random-init draft almost never agrees with a random-init target, so its acceptance is ~0 and those figures are "
                    "the cost of drafting and verifying; the target as its own draft accepts every proposal at twice the work per "
                    "pass; the one-layer draft that always agrees (a target whose upper layers add nothing, same shape and cost) "
                    "shows the ceiling for a draft of that size; whole batch, decode only"}


def run_two_token_8b(steps: int) -> dict:
    """The exact two-token loop on the headline model: 8B architecture, Q4_K, fp16 KV, 512-token prompt, batch 1, with a
    one-layer draft.  Random-init models never agree, so two drafts bracket the scheme: a random one (no proposal accepted:
    what drafting and the two-row verify cost) and the target's own first layer under a target whose upper layers add nothing
    (wo and w2 zero above layer 0: same shapes, same bytes, same time per step; every proposal accepted: the ceiling for a
    draft of this size)."""
    import espresso_amd.llama as ll
    import espresso_amd.synthetic as syn
    from espresso_amd import _lib
    w = WORKLOADS["llama3-8b-q4k"]
    fmt, kv = _lib.FORMAT_NAMES[w["fmt"]], _lib.FORMAT_F16
    tcfg = ll.MultiModelConfig(**syn.LLAMA3_8B)
    dcfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1))
    target, _ = syn.build_runtime(tcfg, fmt, seed=w["seed"], kv_format=kv, zero_upper_outputs=True)
    agreeing, _ = syn.build_runtime(dcfg, fmt, seed=w["seed"], kv_format=kv)
    random_draft, _ = syn.build_runtime(dcfg, fmt, seed=w["seed"] + 50, kv_format=kv)
    prompt = np.random.default_rng(1000 + w["seed"]).integers(0, tcfg.vocab, w["prompt"]).astype(np.uint32)
    n = min(steps, tcfg.max_seq - w["prompt"] - 2)
    target.generate(prompt, 8)
    t0 = time.perf_counter()
    target.prefill(prompt)
    t_prefill = time.perf_counter() - t0
    t0 = time.perf_counter()
    plain, _ = target.generate(prompt, n)
    plain_tok_s = len(plain) / (time.perf_counter() - t0 - t_prefill)

    def run(draft):
        ll.generate_two_token(target, draft, prompt, 8)
        tokens, st = ll.generate_two_token(target, draft, prompt, n)
        rate = len(tokens) / (st["decode_ms"] * 1e-3)
        return {"tok_s": rate, "passes": st["passes"], "accepted_future_tokens_per_pass": st["accepted_total"] / max(st["passes"], 1),
                "committed_exact_tokens_per_pass": st["committed_total"] / max(st["passes"], 1),
                "stream_identical_to_plain_greedy": tokens == plain[:len(tokens)], "speedup_over_plain_greedy": rate / plain_tok_s}

    out = {"metric": "exact two-token decode tok/s (8B-arch Q4_K target, 1-layer draft)", "unit": "tok/s", "n_gpus": 1, "data": "synthetic",
           "prompt_tokens": int(w["prompt"]), "steps": n, "plain_greedy_tok_s": plain_tok_s,
           "random_one_layer_draft": run(random_draft), "one_layer_draft_that_always_agrees": run(agreeing),
           "note": "decode time only (the loop's own decode_ms); the target's layers above the first have zero wo and w2, which changes "
                   "its tokens (those of its first layer) and not its cost"}
    target.close(); agreeing.close(); random_draft.close()
    return out


def run_stamps() -> dict:
    """Where the time of one Q4_K GEMV launch goes: every wavefront of one launch inside a back-to-back train over copies
    of the matrix that exceed the caches (weights from HBM, code and activations warm) records 100 MHz wall-clock stamps at its start, after the activations are
    staged, after its first weights were consumed and at its end.  Percentiles over the wavefronts, in microseconds
    from the first wavefront's start, beside the period to the next launch's first wavefront start: the difference is
    time in which no wavefront of either kernel runs (kernel end, dependency barrier, dispatch of the next grid)."""
    import espresso_amd.ops as ops
    from espresso_amd import _lib
    fmt = _lib.FORMAT_NAMES["q4_k"]
    out = []
    for name, rows, cols in (("q|k|v", 6144, 4096), ("wo", 4096, 4096), ("gate|up", 28672, 4096), ("down", 4096, 14336)):
        m = ops.Matrix(fmt, ops.synth_weights(fmt, 7 + rows + cols, 0.02, rows * cols), rows, cols)
        for kernel, mode in (("matrix-core", 1),):   # the stamped instantiations are the matrix-core ones
            ops.set_tuning("q4k_mfma", mode)
            runs = [ops.gemv_stamps(m, 1, 400) for _ in range(5)]
            st, period_us = sorted(runs, key=lambda r: r[1])[len(runs) // 2]      # the run with the median period
            t = (st.astype(np.float64) - float(st[:, 0].min())) / 100.0           # microseconds
            pct = lambda col: [round(float(np.percentile(t[:, col], q)), 2) for q in (0, 50, 90, 100)]
            out.append({"matrix": name, "rows": rows, "cols": cols, "kernel": kernel, "wavefronts": int(len(t)),
                        "start_us_min_p50_p90_max": pct(0), "staged_us": pct(1), "first_weights_consumed_us": pct(2), "end_us": pct(3),
                        "per_wavefront_busy_us_p50": round(float(np.median(t[:, 3] - t[:, 0])), 2),
                        "period_to_next_launch_us": round(period_us, 2), "period_us_all_runs": [round(r[1], 2) for r in runs],
                        "outside_the_wavefronts_us": round(period_us - float(t[:, 3].max()), 2),
                        "weight_bytes": int(rows * cols // 256 * 144),
                        "gbps_inside_the_wavefronts": round(rows * cols // 256 * 144 / float(t[:, 3].max()) / 1e3, 1)})
        ops.set_tuning("q4k_mfma", -1)
        m.close()
    return {"metric": "per-wavefront stamps of one Q4_K GEMV launch (Llama-3-8B shapes, one activation row, fp16 activations given, weights from HBM)",
            "unit": "us", "n_gpus": 1, "results": out}


def reader_ceiling(bytes_per_launch: int, gemv_back_to_back_us: float) -> dict:
    """A kernel with the matrix-core Q4_K GEMV's grid and loads that only reads: one launch's worth of bytes per launch
    (rotating buffers, back to back) and 1 GiB per launch (the steady state)."""
    import espresso_amd.ops as ops
    pair = 2304                                        # one weight tile: sixteen rows x 256 columns
    n = bytes_per_launch // pair * pair
    one = ops.hbm_read_probe_pairs(n, pair, 512, 8, max(2, int(1.2e9 // n)), 128)
    big = ops.hbm_read_probe_pairs((1 << 30) // pair * pair, pair, 512, 8, 2, 8)
    return {"bytes_per_launch": n, "mean_us": round(one["mean_us"], 2), "gbps": round(one["gbps"], 1),
            "gemv_back_to_back_over_reader": round(gemv_back_to_back_us / one["mean_us"], 3),
            "steady_state_gbps_1gib_launch": round(big["gbps"], 1),
            "note": "same grid (512 workgroups of 8 wavefronts), same 128-bit loads one 2304-byte tile ahead per wavefront, no arithmetic, "
                    "staging or epilogue; back-to-back dependent launches over buffers that rotate through > 1 GB"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="llama3-8b-q4k")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch kernels one at a time instead of replaying the captured per-token HIP graph "
                         "(for rocprofv3 kernel traces)")
    ap.add_argument("--microbench", action="store_true", help="weight-GEMV microbenchmark (Q4_K / Q4_0, batch 1, 2, 8) instead of decode")
    ap.add_argument("--stamps", action="store_true", help="per-wavefront time stamps inside one Q4_K GEMV launch, per decode shape and kernel")
    ap.add_argument("--two-token", action="store_true", help="exact two-token draft/verify decode on the 6-layer model instead of plain decode")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this path is a batch-1 decode on a single MI355X; run with --gpus 1")
    import espresso_amd.ops as ops
    ops.init()
    if args.microbench:
        print(json.dumps(run_microbench()))
        return
    if args.two_token:
        out = run_two_token(args.steps or 240)
        out["llama3-8b-q4k"] = run_two_token_8b(args.steps or 240)
        print(json.dumps(out))
        return
    if args.stamps:
        print(json.dumps(run_stamps()))
        return
    w = WORKLOADS[args.workload]
    steps = args.steps if args.steps is not None else w["decode"]
    gpu = run_gpu(args.workload, steps, args.warmup, graph=not args.no_graph)
    tok_s = steps / gpu["elapsed"]
    kt = gpu["kernel_times"]
    pair_us = kt.pop("event_pair", {"mean_us": 0.0})["mean_us"]   # an event pair around nothing
    dominant = max((k for k in kt if kt[k]["bytes_per_launch"]), key=lambda k: kt[k]["total_us"])
    d = dict(kt[dominant])
    # the dominant kernel again, without per-launch events: every layer's matrix in turn, back to back
    d["b2b_us"] = gpu["b2b_us"][dominant]
    d["kernel_us"] = gpu["kernel_us"][dominant]
    d["gbps"] = d["bytes_per_launch"] / d["kernel_us"] / 1e3
    n_layer = gpu["cfg"].n_layer
    per_token = {"qkv": n_layer, "wo": n_layer, "gate_up": n_layer, "down": n_layer, "head": 1}
    gemv_us = sum(gpu["b2b_us"][k] * n for k, n in per_token.items())
    gemv_bytes = sum(kt[k]["bytes_per_launch"] * n for k, n in per_token.items())
    gemv_kernel_us = sum(gpu["kernel_us"][k] * n for k, n in per_token.items())
    result = {
        "metric": "decode tok/s bs1 (%s)" % ("8B-arch Q4_K" if args.workload == "llama3-8b-q4k" else "6L d768 Q8_0"),
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": gpu["elapsed"] / steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": args.workload, "description": w["describe"], "prompt_tokens": w["prompt"],
                   "weight_bytes_per_token": gpu["weight_bytes"],
                   "token_bytes_over_hbm_peak_tok_s": HBM_PEAK_GBPS * 1e9 / gpu["weight_bytes"]},
        "roofline": {"bound": "hbm", "kernel": f"dequant-GEMV {dominant}", "achieved": d["gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": d["gbps"] / HBM_PEAK_GBPS, "traffic": measured_traffic(args.workload, dominant),
                     "traffic_source": TRAFFIC_SOURCE if measured_traffic(args.workload, dominant) is not None else None,
                     "profile": ({"mean_launch_us": profile_kernel_us(args.workload, dominant),
                                  "frac": d["bytes_per_launch"] / profile_kernel_us(args.workload, dominant) / 1e3 / HBM_PEAK_GBPS,
                                  "source": TRACE_FILE + " (rocprofv3 --kernel-trace of this command with --no-graph; not measured in this run)"}
                                 if profile_kernel_us(args.workload, dominant) else None),
                     "bytes_per_launch": d["bytes_per_launch"], "mean_launch_us": d["kernel_us"], "launches_timed": 8 * (1 if dominant == "head" else n_layer),
                     "all_gemv_gbps": gemv_bytes / gemv_us / 1e3 if gemv_us else 0.0,
                     "all_gemv_frac": gemv_bytes / gemv_us / 1e3 / HBM_PEAK_GBPS if gemv_us else 0.0,
                     "all_gemv_note": "a token's GEMV bytes over its GEMVs' back-to-back periods (kernel + the gap to the next launch); "
                                      "all_gemv_frac_kernel_durations: over the kernels' own durations (kernel_us), as a kernel trace adds them up",
                     "all_gemv_frac_kernel_durations": gemv_bytes / gemv_kernel_us / 1e3 / HBM_PEAK_GBPS if gemv_kernel_us else 0.0,
                     "per_kernel": {k: {"mean_us": round(v["mean_us"], 2), "gbps": round(v["gbps"], 1), "launches": v["launches"]}
                                    for k, v in kt.items()},
                     "how": "achieved/mean_launch_us: the dominant kernel launched for each layer's matrix in turn, 8 rounds on the "
                            "library stream after the timed region, every launch with a pair of HIP events of its own that take the "
                            "kernel's start and end (hipExtLaunchKernel): the mean kernel duration, the figure a rocprofv3 kernel trace "
                            "reports.  kernel_us: the same for the other GEMVs.  back_to_back_us: the same launches between two events "
                            "(kernel + the gap to the next launch).  per_kernel: an event pair around every launch of an instrumented "
                            "decode pass; each mean includes what a pair costs by itself (event_pair_us)",
                     "kernel_us": {k: round(x, 2) for k, x in gpu["kernel_us"].items()},
                     "event_pair_us": round(pair_us, 2), "back_to_back_us": {k: round(x, 2) for k, x in gpu["b2b_us"].items()},
                     "reader_same_grid": reader_ceiling(d["bytes_per_launch"], gpu["b2b_us"][dominant]),
                     "plain_read_kernel_gbps": round(ops.hbm_read_probe(1 << 30, 10), 1),
                     "plain_read_kernel_note": "a kernel that only streams 1 GiB with 128-bit loads, same process: the ceiling "
                                               "the memory system gives the simplest reader, to read `frac` against"},
        "model_build_s": round(gpu["build_s"], 1), "prefill_s": round(gpu["prefill_s"], 3),
        "prefill": {"tokens": w["prompt"], "tok_s": w["prompt"] / gpu["prefill_s"], "second_walk_s": round(gpu["prefill_again_s"], 4),
                    "second_walk_tok_s": w["prompt"] / gpu["prefill_again_s"],
                    "second_walk_fp16_operands_s": round(gpu["prefill_fp16_s"], 4),
                    "second_walk_fp16_operands_tok_s": w["prompt"] / gpu["prefill_fp16_s"],
                    "note": "tok_s: the first walk of the prompt in the process (kernels' first launches included); second_walk: the same prompt "
                            "again after a reset; fp16_operands: the same with esp_llama_set_split_activations(0), every operand rounded to fp16 once",
                    "path": ("blocks of up to 512 rows; Q4_K: MFMA GEMM with exact integer weights and activations as hi/lo fp16 pairs (twice the "
                             "MFMA work of the fp16-operand GEMM, logits within 2e-2 of the fp32 CPU walk at 32 layers); other formats: "
                             "dequant-fused fp16 MFMA GEMM") if w["prompt"] >= 32 else "token by token (prompts under 32 tokens)"},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, gpu)
    gpu["rt"].close()
    del gpu
    if not args.no_secondary:
        secondary = {}
        other = "stories-6l-q8_0" if args.workload == "llama3-8b-q4k" else None
        if other:
            ow = WORKLOADS[other]
            osteps = ow["decode"]
            g2 = run_gpu(other, osteps, args.warmup, graph=not args.no_graph)
            sec = {"metric": "decode tok/s bs1 (6L d768 Q8_0)", "value": osteps / g2["elapsed"], "unit": "tok/s",
                   "steps": osteps, "ms_per_step": g2["elapsed"] / osteps * 1e3, "workload": other,
                   "weight_bytes_per_token": g2["weight_bytes"],
                   "frac_hbm_peak_whole_token": g2["weight_bytes"] / (g2["elapsed"] / osteps) / 1e9 / HBM_PEAK_GBPS,
                   "per_kernel": {k: {"mean_us": round(v["mean_us"], 2), "gbps": round(v["gbps"], 1)} for k, v in g2["kernel_times"].items()},
                   "per_kernel_note": "raw HIP-event means, event-pair overhead (see event_pair) included"}
            if not args.no_cpu_baseline:
                sec["cpu_baseline"] = cpu_baseline(other, g2)
            g2["rt"].close()
            del g2
            secondary[other] = sec
        # BASELINE.json configs[2] (the two largest shapes; --microbench prints all four) and configs[4]
        secondary["gemv_microbench"] = run_microbench(shapes=[(14336, 4096), (4096, 14336)], launches=50)
        # BASELINE.json configs[1]: the 6-layer model's isolated Q8_0 shapes at batch 1 and 2 (the small ones fit the memory-side cache
        # even when rotated, and are launch-bound: about 3 us per dependent launch whatever they read)
        secondary["gemv_microbench_q8_0"] = run_microbench(shapes=[(768, 768), (2048, 768), (768, 2048), (32000, 768)], formats=("q8_0",),
                                                           batches=(1, 2), launches=50)
        secondary["two_token"] = run_two_token(240)
        secondary["two_token_8b"] = run_two_token_8b(240)
        result["secondary"] = secondary
    print(json.dumps(result))


if __name__ == "__main__":
    main()
