"""Shared by the tests: the two tiny configurations, model folders with weights that
make faults visible, traces in the four cuttings, and the comparison with the plain
implementation."""
import json
import os
import struct

import numpy as np

import plain

# The two tiny configurations differ in every size and option.
CONFIG_A = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=64,
                num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=176,
                vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                use_sliding_window=False, max_position_embeddings=128, hidden_act="silu")
CONFIG_B = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=3, hidden_size=96,
                num_attention_heads=3, num_key_value_heads=1, head_dim=32, intermediate_size=256,
                vocab_size=1000, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
                use_sliding_window=True, sliding_window=32, max_window_layers=1,
                max_position_embeddings=256, hidden_act="silu")
# Sizes that the kernels of the serving path take (widths that are multiples of 128, a head size of 64): the tiny
# configurations above run the plain kernels for most of a step.
CONFIG_C = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=256,
                num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=384,
                vocab_size=777, rope_theta=50000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                use_sliding_window=True, sliding_window=48, max_window_layers=1,
                max_position_embeddings=256, hidden_act="silu")
PAGE = {"A": 16, "B": 8, "C": 16}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}


def bf16_round(a):
    """float array -> the nearest bfloat16 values (ties to even), as float32."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32)


def make_weights(cfg, seed, sharp=True):
    """name -> float32 array. ``sharp``: scales that give activations of order one and
    peaked attention, after the reference's tiny-model writer (tools/mkmodel.pl:104-120:
    embeddings 0.5, Wq/Wk 1.2/sqrt(E), Wv 1/sqrt(E), Wo 1/sqrt(QD), bq/bk 0.3, bv 0.2,
    norms 1 + 0.1 N, gate 1.2/sqrt(E), up 1/sqrt(E), down 1/sqrt(F)). Otherwise N(0, 0.02)
    everywhere and norms 1 + 0.1 N."""
    rng = np.random.default_rng(seed)
    E, F, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    H, G = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    D = cfg.get("head_dim") or E // H
    QD, KD = H * D, G * D

    def n(shape, std):
        return (rng.standard_normal(shape) * (std if sharp else 0.02)).astype(np.float32)

    def norm(size):
        return (1.0 + 0.1 * rng.standard_normal(size)).astype(np.float32)
    w = {"model.embed_tokens.weight": n((V, E), 0.5)}
    for l in range(L):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"] = norm(E)
        w[p + "self_attn.q_proj.weight"] = n((QD, E), 1.2 / E ** 0.5)
        w[p + "self_attn.k_proj.weight"] = n((KD, E), 1.2 / E ** 0.5)
        w[p + "self_attn.v_proj.weight"] = n((KD, E), 1.0 / E ** 0.5)
        w[p + "self_attn.o_proj.weight"] = n((E, QD), 1.0 / QD ** 0.5)
        w[p + "self_attn.q_proj.bias"] = n((QD,), 0.3)
        w[p + "self_attn.k_proj.bias"] = n((KD,), 0.3)
        w[p + "self_attn.v_proj.bias"] = n((KD,), 0.2)
        w[p + "post_attention_layernorm.weight"] = norm(E)
        w[p + "mlp.gate_proj.weight"] = n((F, E), 1.2 / E ** 0.5)
        w[p + "mlp.up_proj.weight"] = n((F, E), 1.0 / E ** 0.5)
        w[p + "mlp.down_proj.weight"] = n((E, F), 1.0 / F ** 0.5)
    w["model.norm.weight"] = norm(E)
    if not cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = n((V, E), 1.0 / E ** 0.5)
    return w


def write_safetensors(path, tensors, dtype="F32"):
    """The tests' own writer (8-byte length, JSON header, raw data)."""
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        a = np.ascontiguousarray(a, dtype=np.float32)
        if dtype == "BF16":
            raw = (bf16_round(a).view(np.uint32) >> 16).astype("<u2").tobytes()
        elif dtype == "F16":
            raw = a.astype("<f2").tobytes()
        else:
            raw = a.astype("<f4").tobytes()
        header[name] = {"dtype": dtype, "shape": list(a.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)


def make_model_dir(path, cfg, seed, sharp=True, dtype="F32", weights=None):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    w = weights if weights is not None else make_weights(cfg, seed, sharp)
    write_safetensors(os.path.join(path, "model.safetensors"), w, dtype)
    return path


def random_requests(cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for i, n in enumerate(lengths)}


# ---- traces: lists of steps {"step", "entries": [{"id", "tokens", "want"}], "end"} ---------

def _step(i, entries, end=()):
    return {"step": i, "entries": [{"id": r, "tokens": list(t), "want": list(w)} for r, t, w in entries],
            "end": list(end)}


def trace_whole(reqs):
    """Each request alone and whole, logits at every place."""
    return [_step(i, [(r, toks, range(len(toks)))], [r]) for i, (r, toks) in enumerate(reqs.items())]


def trace_tail(reqs, tail=32):
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for r, toks in reqs.items():
        head = max(len(toks) - tail, 1)
        steps.append(_step(len(steps), [(r, toks[:head], range(head))]))
        for i in range(head, len(toks)):
            steps.append(_step(len(steps), [(r, toks[i:i + 1], [0])], [r] if i == len(toks) - 1 else []))
        if head == len(toks):
            steps[-1]["end"] = [r]
    return steps


def trace_portions(reqs, sizes=(5, 2, 9, 3, 2, 17, 4, 2, 31, 6)):
    """Portions of changing size, down to two tokens (a last single token if one is left)."""
    steps = []
    for k, (r, toks) in enumerate(reqs.items()):
        at, j = 0, k
        while at < len(toks):
            n = min(sizes[j % len(sizes)], len(toks) - at)
            j += 1
            last = at + n == len(toks)
            steps.append(_step(len(steps), [(r, toks[at:at + n], range(n))], [r] if last else []))
            at += n
    return steps


def trace_mixed(reqs, seed, max_live=4, decode_tail=12):
    """Up to ``max_live`` requests live at once; in a step some bring a portion of their
    prompt (2..24 tokens), some one token (their last ``decode_tail`` tokens go one by one),
    some sit the step out; a finished request ends and the next one starts."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs.items())
    live = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            r, toks = waiting.pop(0)
            live[r] = [toks, 0]
        entries, end = [], []
        for r, (toks, at) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue
            left = len(toks) - at
            n = 1 if left <= decode_tail else min(int(rng.integers(2, 25)), left - decode_tail)
            if n == 1 and left > decode_tail:
                n = min(2, left)
            entries.append((r, toks[at:at + n], range(n)))
            live[r][1] = at + n
            if at + n == len(toks):
                end.append(r)
                del live[r]
        if entries:
            steps.append(_step(len(steps), entries, end))
    return steps


def max_live_tokens(steps, round_to=64):
    """The --max-tokens a trace needs: the largest sum over live requests of their final
    lengths rounded up to ``round_to``... taken at every step (a request is live from its
    first step to the step that ends it)."""
    total = {}
    for s in steps:
        for e in s["entries"]:
            total[e["id"]] = total.get(e["id"], 0) + len(e["tokens"])
    live, best = set(), 0
    for s in steps:
        for e in s["entries"]:
            live.add(e["id"])
        best = max(best, sum(-(-total[r] // round_to) * round_to for r in live))
        for r in s["end"]:
            live.discard(r)
    return best


def wanted_places(steps):
    """For each step with wanted logits: [(request, position), ...] in row order."""
    at, out = {}, {}
    for s in steps:
        rows = []
        for e in s["entries"]:
            base = at.get(e["id"], 0)
            rows.extend((e["id"], base + w) for w in e["want"])
            at[e["id"]] = base + len(e["tokens"])
        if rows:
            out[s["step"]] = rows
    return out


def run_trace_in_engine(engine, steps):
    """{(request, position): logits row (numpy fp32)} by driving Engine.step."""
    places = wanted_places(steps)
    got = {}
    for s in steps:
        logits = engine.step([(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if s["step"] in places:
            rows = logits.float().cpu().numpy()
            assert rows.shape[0] == len(places[s["step"]])
            for row, key in zip(rows, places[s["step"]]):
                got[key] = row.copy()
        for r in s["end"]:
            engine.release(r)
    return got


def plain_logits(model_dir, reqs, round_weights_bf16=False):
    cfg, w = plain.read_model(model_dir)
    if round_weights_bf16:
        w = {k: (bf16_round(v).astype(np.float64) if v.ndim == 2 else v) for k, v in w.items()}
    return {r: plain.forward(cfg, w, toks) for r, toks in reqs.items()}


def compare(got, want, tol, what=""):
    """Every wanted row within ``tol`` times the request's largest |logit| of the plain
    implementation (max abs difference); reports the first wrong place in position order.
    Returns the worst relative difference."""
    worst = 0.0
    scale = {r: float(np.max(np.abs(v))) for r, v in want.items()}
    for (r, pos) in sorted(got, key=lambda k: (k[0], k[1])):
        err = float(np.max(np.abs(got[(r, pos)].astype(np.float64) - want[r][pos]))) / scale[r]
        worst = max(worst, err)
        assert err <= tol, (f"{what}: request {r} position {pos}: max |diff| / max |logit| = {err:.3e} "
                            f"> {tol:.1e}")
    return worst
