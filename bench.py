#!/usr/bin/env python3
"""Throughput of the engine on the Qwen2.5-7B shape with random weights, one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--no-points]
    python bench.py --workload 0.5b | 32b      (the baseline's other workloads, through the scheduler)

A step is one decode step of ``--batch`` sequences (default 8) whose prompts of 2,048
random ids were prefilled before; W steps are run untimed, then exactly K steps are timed
between device synchronisations. One JSON line is printed: ``value`` is decoded tokens per
second; ``prefill`` is one 2,048-token prompt in one step; ``roofline`` prices the decode
step against HBM bandwidth (every weight it uses once, plus the cache of the live
requests); ``points`` holds decode at batch 1, 64, 128 and 256 (tokens a second, and the fraction of
the HBM peak that the step's bytes over its time come to). Peaks: HBM 8 TB/s, dense bf16 MFMA
2.5 PFLOP/s, fp32 157.3 TFLOP/s. ``measured_peaks`` is what this device's own probes reach (a
streaming read, a copy, the matrix cores on random and on all-zero operands); ``kernels`` prices
every dominant part of the decode step (bytes / time) and of the prefill (flops / time) against both.
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

SHAPE_7B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=28, hidden_size=3584,
                num_attention_heads=28, num_key_value_heads=4, head_dim=128, intermediate_size=18944,
                vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")
# The other two workloads of the baseline: many requests of mixed lengths through the scheduler.
WORKLOADS = {
    "0.5b": dict(shape=dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=24, hidden_size=896,
                            num_attention_heads=14, num_key_value_heads=2, head_dim=64, intermediate_size=4864,
                            vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                            use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu"),
                 name="Qwen2.5-0.5B shape, random weights", requests=64, prompt_lo=16, prompt_hi=4096, new_tokens=128,
                 ctx=32768, budget=8192),
    "32b": dict(shape=dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=64, hidden_size=5120,
                           num_attention_heads=40, num_key_value_heads=8, head_dim=128, intermediate_size=27648,
                           vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
                           use_sliding_window=False, max_position_embeddings=8192, hidden_act="silu"),
                name="Qwen2.5-32B shape, random weights", requests=16, prompt_lo=4096, prompt_hi=4096, new_tokens=128,
                ctx=8192, budget=1024),
}
PROMPT, NEW, PAGE = 2048, 256, 16
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def matmul_params(c):
    E, F, QD, KD = c["hidden_size"], c["intermediate_size"], c["num_attention_heads"] * c["head_dim"], \
        c["num_key_value_heads"] * c["head_dim"]
    per_layer = E * (QD + 2 * KD) + QD * E + 2 * F * E + F * E
    return per_layer, c["vocab_size"] * E


def decode_bytes(c, elem, batch, mean_ctx):
    """Bytes one decode step has to read: every matrix, bias and norm once, and the keys and
    values of every live request."""
    per_layer, head = matmul_params(c)
    L, E = c["num_hidden_layers"], c["hidden_size"]
    KD = c["num_key_value_heads"] * c["head_dim"]
    QD = c["num_attention_heads"] * c["head_dim"]
    weights = (L * per_layer + head) * elem + (L * (2 * E + QD + 2 * KD) + E) * 4
    cache = batch * mean_ctx * 2 * KD * L * elem
    return weights + cache


def prefill_flops(c, T):
    per_layer, head = matmul_params(c)
    L, H, D = c["num_hidden_layers"], c["num_attention_heads"], c["head_dim"]
    return 2.0 * T * L * per_layer + L * 4.0 * D * H * T * (T + 1) / 2 + 2.0 * head


def part_work(c, elem, batch, mean_ctx, T):
    """What each timed part of a step has to move or compute, all layers together:
    ({part: bytes of a decode step}, {part: flops of a prefill of T tokens})."""
    L, E, F, V = c["num_hidden_layers"], c["hidden_size"], c["intermediate_size"], c["vocab_size"]
    H, D = c["num_attention_heads"], c["head_dim"]
    QD, KD = H * D, c["num_key_value_heads"] * D
    params = {"qkv": L * E * (QD + 2 * KD), "wo": L * QD * E, "gate_up": L * 2 * F * E, "down": L * F * E, "head": V * E}
    dec = {k: v * elem for k, v in params.items()}
    dec["attn"] = batch * mean_ctx * 2 * KD * L * elem
    pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
    pre["attn"] = L * 4.0 * D * H * T * (T + 1) / 2
    return dec, pre


def kernel_fractions(eng, stage, step_fn, n, shape, elem, batch, mean_ctx, peaks, short):
    """Times ``n`` steps of ``stage`` ("decode" or "prefill") by part (device events around each part's
    kernels, steps run eagerly) and prices every dominant part: bytes / time for a decode step's parts
    against HBM, flops / time for the prefill's against the matrix cores; against the published peak
    ("frac") and, if measured, against what this device's own probes reach ("frac_measured")."""
    eng.profile_start()
    for _ in range(n):
        step_fn()
    book = eng.profile_stop()[stage]
    dec_b, pre_f = part_work(shape, elem, batch, mean_ctx, PROMPT)
    out = {}
    if stage == "decode":
        for part, nbytes in dec_b.items():
            ms = book.get(part, 0.0) / n
            if ms > 0:
                e = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e-3 / HBM_PEAK, 4)}
                if peaks:
                    e["frac_measured"] = round(nbytes / ms / 1e6 / peaks["hbm_read_GBps"], 4)
                out["decode." + part] = e
        out["decode.other"] = {"us": round(sum(v for k, v in book.items() if k not in dec_b) / n * 1e3, 1)}
    else:
        for part, flops in pre_f.items():
            ms = book.get(part, 0.0) / n
            if ms > 0:
                e = {"us": round(ms * 1e3, 1), "TFLOPs": round(flops / ms / 1e9, 1), "frac": round(flops / ms / 1e-3 / FLOP_PEAK[short], 4)}
                if peaks and short == "bf16":
                    e["frac_measured"] = round(flops / ms / 1e9 / peaks["mfma_bf16_TFLOPs"], 4)
                out["prefill." + part] = e
        out["prefill.other"] = {"us": round(sum(v for k, v in book.items() if k not in pre_f) / n * 1e3, 1)}
    return out


def serve_workload(which, dtype, temp=0.0, budget=0):
    """``--workload 0.5b | 32b``: all requests are submitted at once and served by the scheduler
    (prompt portions under the token budget beside decoded tokens; greedy, or with ``--temp``
    the reference's default sampling at that temperature); the second of two runs is timed. One JSON line: prompt and generated tokens per second of wall time."""
    import numpy as np
    import torch
    import hf_cpu_amd
    import hf_cpu_amd.session as S
    w = dict(WORKLOADS[which])
    if budget:
        w["budget"] = budget
    cfg = hf_cpu_amd.config_from_dict(w["shape"])
    t0 = time.perf_counter()
    s = S.Session(cfg, dtype=dtype, ctx_max=w["ctx"], batch=w["budget"], page_size=PAGE, max_seqs=64,
                  kv_tokens=w["requests"] * (w["prompt_hi"] + w["new_tokens"] + PAGE), seed=0)
    torch.cuda.synchronize()
    print(f"[bench] weights and cache ready in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    prompts = [[int(t) for t in rng.integers(0, cfg.vocab_size, int(rng.integers(w["prompt_lo"], w["prompt_hi"] + 1)))]
               for _ in range(w["requests"])]
    for rep in range(2):
        steps0 = s.engine.steps_run
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        gens = s.generate(prompts, temp=temp, seed=1, max_tokens=w["new_tokens"])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        steps = s.engine.steps_run - steps0
        n_prompt, n_gen = sum(len(p) for p in prompts), sum(len(g.tokens) for g in gens)
        print(f"[bench] run {rep}: {n_prompt} prompt + {n_gen} generated tokens in {dt:.2f} s, {steps} steps, "
              f"{sum(g.preemptions for g in gens)} preemptions", file=sys.stderr, flush=True)
    sh = w["shape"]
    short = "bf16" if dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": f"tokens served per second, prompts and generated ({w['name']})", "value": round((n_prompt + n_gen) / dt, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 1, "ms_per_step": round(dt / steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {"model": w["name"], "num_hidden_layers": sh["num_hidden_layers"], "hidden_size": sh["hidden_size"],
                   "num_attention_heads": sh["num_attention_heads"], "num_key_value_heads": sh["num_key_value_heads"],
                   "head_dim": sh["head_dim"], "intermediate_size": sh["intermediate_size"], "vocab_size": sh["vocab_size"],
                   "requests": w["requests"], "prompt_tokens": n_prompt, "generated_tokens": n_gen,
                   "token_budget": w["budget"], "ctx": w["ctx"], "page_size": PAGE, "temp": temp, "parallelism": "none"},
        "generated_tok_per_s": round(n_gen / dt, 1)}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1, 64, 128 and 256")
    ap.add_argument("--prefill-reps", type=int, default=3)
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="run one phase only and print a short line (for profiling a phase by itself)")
    ap.add_argument("--context", type=int, default=PROMPT,
                    help="with --only decode: tokens every sequence holds before the timed steps (prefilled in portions "
                         "of 2,048); with --only prefill: the length of the prompt, computed in portions of 2,048; "
                         "the default run's is 2,048")
    ap.add_argument("--shape", choices=["7b", "0.5b", "32b"], default="7b",
                    help="with --only: the layer sizes of the step (the default measurement's are the 7B shape's)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the probes of the device's own peaks")
    ap.add_argument("--no-kernels", action="store_true", help="skip the timing by part")
    ap.add_argument("--workload", choices=["7b", "0.5b", "32b"], default="7b",
                    help="7b: the default measurement; 0.5b, 32b: the baseline's other workloads, served by the scheduler")
    ap.add_argument("--temp", type=float, default=0.0,
                    help="for --workload 0.5b | 32b: sample at this temperature (top-k 40, top-p 0.95, min-p 0.05) instead of greedy")
    ap.add_argument("--budget", type=int, default=0,
                    help="for --workload 0.5b | 32b: the scheduler's token budget of a step (0 = the workload's own)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus must be 1")
        return 2
    if args.workload != "7b":
        return serve_workload(args.workload, args.dtype, args.temp, args.budget)
    if args.context != PROMPT and args.only is None:
        print("bench.py: --context goes with --only decode | prefill (the default measurement has 2,048-token prompts)")
        return 2
    if args.shape != "7b" and args.only is None:
        print("bench.py: --shape goes with --only prefill | decode (the default measurement is of the 7B shape)")
        return 2
    if args.steps + args.warmup > NEW:
        print(f"bench.py: --steps + --warmup must not exceed the {NEW} new tokens of the workload")
        return 2

    import numpy as np
    import torch
    import hf_cpu_amd
    import hf_cpu_amd.session as S

    shape = dict(SHAPE_7B if args.shape == "7b" else WORKLOADS[args.shape]["shape"])
    layers_of_shape = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    cfg = hf_cpu_amd.config_from_dict(shape)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    elem = 2 if short == "bf16" else 4
    point_batches = () if args.no_points or args.only else (1, 64, 128, 256)
    biggest = max((args.batch,) + point_batches)
    t_load = time.perf_counter()
    s = S.Session(cfg, dtype=args.dtype, ctx_max=args.context + NEW, batch=PROMPT, page_size=PAGE, max_seqs=biggest,
                  kv_tokens=biggest * (args.context + NEW), seed=0)
    eng, ops = s.engine, s.ops
    torch.cuda.synchronize()
    print(f"[bench] weights and cache ready in {time.perf_counter() - t_load:.1f} s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)

    def prompt():
        return [int(t) for t in rng.integers(0, cfg.vocab_size, PROMPT)]

    peaks = None
    if not args.no_peaks and args.only is None:
        from hf_cpu_amd.probe import measure_peaks
        peaks = measure_peaks(ops)
        print(f"[bench] measured peaks: {peaks}", file=sys.stderr, flush=True)
    kernels = {}
    by_part = not args.no_kernels and args.only is None and args.steps + args.warmup + 4 <= NEW

    # ---- prefill: one prompt of 2,048 tokens in one step, logits for its last token ----
    times = []
    for rep in range(0 if args.only == "decode" else args.prefill_reps + 1):
        p = prompt()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.step([("prefill", p, [PROMPT - 1])])
        ops.argmax(logits).cpu()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        eng.release("prefill")
    if args.only == "decode":
        pre_s = float("nan")
    else:
        pre_s = sorted(times[1:])[len(times[1:]) // 2]        # the first run warms up
        print(f"[bench] prefill {PROMPT} tokens: {pre_s * 1e3:.1f} ms", file=sys.stderr, flush=True)
    if by_part:

        def one_prefill():
            eng.step([("prefill", prompt(), [PROMPT - 1])])
            eng.release("prefill")
        kernels.update(kernel_fractions(eng, "prefill", one_prefill, 2, shape, elem, 1, PROMPT, peaks, short))
    if args.only == "prefill" and args.context > PROMPT:
        # A long prompt in portions of 2,048 tokens, each a step of its own: what every portion costs (later
        # ones attend over all that lies before them), and the whole.
        whole = []
        for rep in range(2):
            per = []
            for at in range(0, args.context, PROMPT):
                n = min(PROMPT, args.context - at)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = eng.step([("long", prompt()[:n], [n - 1] if at + n == args.context else [])])
                if at + n == args.context:
                    ops.argmax(logits).cpu()
                torch.cuda.synchronize()
                per.append(time.perf_counter() - t0)
            eng.release("long")
            whole.append(per)
        per = whole[-1]
        total = sum(per)
        # flops: every portion's products, and attention over the causal part of the whole prompt
        L, H, D = shape["num_hidden_layers"], shape["num_attention_heads"], shape["head_dim"]
        per_layer, head = matmul_params(shape)
        flops = 2.0 * args.context * L * per_layer + L * 4.0 * D * H * args.context * (args.context + 1) / 2 + 2.0 * head
        print(json.dumps({"phase": "prefill", "shape": args.shape, "tokens": args.context, "portion": PROMPT,
                          "ms": round(total * 1e3, 2), "tok_per_s": round(args.context / total, 1),
                          "frac": round(flops / total / FLOP_PEAK[short], 4),
                          "first_portion_ms": round(per[0] * 1e3, 2), "last_portion_ms": round(per[-1] * 1e3, 2)}))
        return 0
    if args.only == "prefill":
        print(json.dumps({"phase": "prefill", "shape": args.shape, "tokens": PROMPT, "ms": round(pre_s * 1e3, 3)}))
        return 0


    def decode(batch, steps, warmup, by_part=False):
        ids = [("d", i) for i in range(batch)]
        last = []
        for r in ids:
            for at in range(0, args.context, PROMPT):            # the prompt in portions of 2,048 tokens
                n = min(PROMPT, args.context - at)
                logits = eng.step([(r, prompt()[:n], [n - 1] if at + n == args.context else [])])
            last.append(int(ops.argmax(logits).cpu()[0]))

        # The serving loop's way of decoding: a step takes its tokens from where the sampler left them on
        # the device, and the host reads every step's tokens one step late, while the next step runs.
        state = {"dev": torch.tensor(last, dtype=torch.int32, device=ops.device), "read": lambda: last}
        fed_rows = {i: i for i in range(batch)}

        def one():
            logits = eng.step([(r, [0], [0]) for r in ids], fed=(state["dev"], fed_rows))
            chosen = ops.argmax(logits)
            later = s.sampler._to_host_later(chosen)     # the copy is enqueued behind the choice; it is read a step late
            state["tokens"] = state["read"]()
            state["dev"], state["read"] = chosen, later
        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if by_part:                           # after the timed steps, at the context they ended with
            kernels.update(kernel_fractions(eng, "decode", one, 4, shape, elem, batch, PROMPT + warmup + steps + 2.5,
                                            peaks, short))
        for r in ids:
            eng.release(r)
        return dt

    dt = decode(args.batch, args.steps, args.warmup, by_part=by_part)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    print(f"[bench] decode batch {args.batch}: {ms_step:.3f} ms/step", file=sys.stderr, flush=True)
    if args.only == "decode":
        nbytes = decode_bytes(shape, elem, args.batch, args.context + args.warmup + (args.steps + 1) / 2.0)
        print(json.dumps({"phase": "decode", "shape": args.shape, "batch": args.batch, "context": args.context,
                          "ms_per_step": round(ms_step, 4),
                          "tok_per_s": round(value, 1), "GBps": round(nbytes / (dt / args.steps) / 1e9, 1)}))
        return 0
    mean_ctx = PROMPT + args.warmup + (args.steps + 1) / 2.0
    nbytes = decode_bytes(shape, elem, args.batch, mean_ctx)
    achieved = nbytes / (dt / args.steps) / 1e9
    points = {}
    for b in point_batches:
        k, w = min(args.steps, 32), min(args.warmup, 4)
        d = decode(b, k, w)
        points[f"decode_b{b}"] = round(b * k / d, 1)
        points[f"decode_b{b}_hbm_frac"] = round(decode_bytes(shape, elem, b, PROMPT + w + (k + 1) / 2.0) / (d / k) / HBM_PEAK, 4)
        print(f"[bench] decode batch {b}: {d / k * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    flops = prefill_flops(shape, PROMPT)
    line = {
        "metric": "decode tok/s at batch 8 (Qwen2.5-7B shape, 2048-token prompts)" if args.batch == 8
        else f"decode tok/s at batch {args.batch} (Qwen2.5-7B shape, 2048-token prompts)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic",
        "config": {"model": "Qwen2.5-7B shape, random weights", "num_hidden_layers": layers_of_shape,
                   "layers_run": shape["num_hidden_layers"], "hidden_size": shape["hidden_size"],
                   "num_attention_heads": shape["num_attention_heads"],
                   "num_key_value_heads": shape["num_key_value_heads"], "head_dim": shape["head_dim"],
                   "intermediate_size": shape["intermediate_size"], "vocab_size": shape["vocab_size"],
                   "tie_word_embeddings": False, "global_batch": args.batch, "seq_len": PROMPT + NEW,
                   "prompt_len": PROMPT, "new_tokens": NEW, "page_size": PAGE, "parallelism": "none"},
        "prefill": {"value": round(PROMPT / pre_s, 1), "tokens": PROMPT, "ms": round(pre_s * 1e3, 3),
                    "frac": round(flops / pre_s / FLOP_PEAK[short], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4)},
        "points": points,
    }
    if peaks:                                  # against what this device's own probes reach
        line["measured_peaks"] = peaks
        line["roofline"]["measured_peak"] = peaks["hbm_read_GBps"]
        line["roofline"]["frac_measured"] = round(achieved / peaks["hbm_read_GBps"], 4)
        if short == "bf16":
            line["prefill"]["frac_measured"] = round(flops / pre_s / 1e12 / peaks["mfma_bf16_TFLOPs"], 4)
    if kernels:
        line["kernels"] = kernels
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
