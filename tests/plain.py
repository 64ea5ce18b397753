"""The plain implementation: Qwen2 dense over whole sequences, in float64 numpy.

No cache, no batching, no kernels, one function for each part, written from the
reference's formulas (each function cites file:line under the reference's src/ or
tools/). It shares no code with the package: it reads config.json and
model.safetensors with its own few lines. The engine is compared with this.

Where the reference leaves a choice open the choice is stated in the function:
the sliding window (absent from the reference) and the rotary angle (closed form
in float64, as the reference's own oracle tools/ref-forward.pl:97 does, where its
engine uses a running fp32 product, src/model.c:472-476).
"""
import json
import math
import os
import struct

import numpy as np

# ---- reading a model folder (own reader: JSON header + raw little-endian data) -----------


def read_safetensors(path):
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        raw = data[b:e]
        if info["dtype"] == "F32":
            arr = np.frombuffer(raw, "<f4").astype(np.float64)
        elif info["dtype"] == "BF16":
            arr = (np.frombuffer(raw, "<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif info["dtype"] == "F16":
            arr = np.frombuffer(raw, "<f2").astype(np.float64)
        else:
            raise ValueError(f"{name}: dtype {info['dtype']}")
        out[name] = arr.reshape(info["shape"])
    return out


def read_model(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ---- parts -----------------------------------------------------------------------------

def embed(table, tokens):
    """x[t, :] = table[token[t], :], no scaling (src/model.c:566-571)."""
    return table[np.asarray(tokens)]


def rmsnorm(x, w, eps):
    """y = x * (1 / sqrt(mean(x*x) + eps)) * w over the last axis (src/mathx.c:65-75)."""
    mean = np.mean(x * x, axis=-1, keepdims=True)
    return (x * (1.0 / np.sqrt(mean + eps))) * w


def linear(x, W, b=None):
    """y[t, r] = dot(W[r, :], x[t, :]) + b[r]; W is [rows = out, cols = in]
    (src/model.c:408-424)."""
    y = x @ W.T
    return y if b is None else y + b


def rope_angles(positions, n_rot, base):
    """theta[p, i] = p * base^(-2i / n_rot), i < n_rot/2 (tools/ref-forward.pl:97;
    src/mathx.c:115-127 gives the per-step factor base^(-2/n_rot))."""
    i = np.arange(n_rot // 2, dtype=np.float64)
    return np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / n_rot)


def rope(v, positions, n_rot, base):
    """Rotates pairs (i, i + n_rot/2) of every head: a' = a*cos - b*sin, b' = a*sin + b*cos;
    dimensions from n_rot on pass through (src/model.c:478-493, the non-interleaved branch).
    v: [T, heads, D]."""
    th = rope_angles(positions, n_rot, base)
    c, s = np.cos(th)[:, None, :], np.sin(th)[:, None, :]
    half = n_rot // 2
    out = v.copy()
    a, b = v[..., :half], v[..., half:n_rot]
    out[..., :half] = a * c - b * s
    out[..., half:n_rot] = a * s + b * c
    return out


def softmax(s):
    """exp(s - max) / sum over the last axis (src/mathx.c:77-86)."""
    e = np.exp(s - np.max(s, axis=-1, keepdims=True))
    return e / np.sum(e, axis=-1, keepdims=True)


def visible(n, window):
    """mask[q, k]: key k is visible to query q iff k <= q (src/model.c:514, len = pos + 1)
    and, with a window W > 0, q - k < W (the reference has no window; this is the
    definition the engine's configuration documents)."""
    q = np.arange(n)[:, None]
    k = np.arange(n)[None, :]
    m = k <= q
    if window and window > 0:
        m &= (q - k) < window
    return m


def attention(q, k, v, window=0, scale=None):
    """q: [T, H, D]; k, v: [T, G, D]. Head h reads key/value head h // (H // G); scores
    dot(q, k) * scale with scale = 1/sqrt(D) applied after the dot; softmax over the
    visible keys; weighted sum of values (src/model.c:499-528)."""
    T, H, D = q.shape
    G = k.shape[1]
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    mask = visible(T, window)
    out = np.empty_like(q)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = np.where(mask, s, -np.inf)
        out[:, h, :] = softmax(s) @ v[:, g, :]
    return out


def silu(x):
    """x / (1 + exp(-x)) (src/mathx.c:34)."""
    return x / (1.0 + np.exp(-x))


def swiglu_mlp(x, Wg, Wu, Wd):
    """Wdown (silu(Wgate x) * (Wup x)) (src/model.c:612-621, 537)."""
    return linear(silu(linear(x, Wg)) * linear(x, Wu), Wd)


# ---- the model ---------------------------------------------------------------------------

def layer_window(cfg, l):
    if cfg.get("use_sliding_window") and l >= cfg.get("max_window_layers", cfg["num_hidden_layers"]):
        return cfg["sliding_window"]
    return 0


def attention_block(cfg, w, l, x, positions):
    """Norm, q/k/v with bias, rotary on q and k (not v), attention, output projection
    (src/model.c:580-607)."""
    p = f"model.layers.{l}.self_attn."
    H, G = cfg["num_attention_heads"], cfg.get("num_key_value_heads") or cfg["num_attention_heads"]
    D = cfg.get("head_dim") or cfg["hidden_size"] // H
    T = x.shape[0]
    q = linear(x, w[p + "q_proj.weight"], w[p + "q_proj.bias"]).reshape(T, H, D)
    k = linear(x, w[p + "k_proj.weight"], w[p + "k_proj.bias"]).reshape(T, G, D)
    v = linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).reshape(T, G, D)
    q = rope(q, positions, D, cfg["rope_theta"])
    k = rope(k, positions, D, cfg["rope_theta"])
    att = attention(q, k, v, layer_window(cfg, l)).reshape(T, H * D)
    return linear(att, w[p + "o_proj.weight"])


def forward(cfg, w, tokens, first_position=0):
    """Logits [T, V] of a whole sequence (src/model.c:545-640): embedding; per layer
    x += attention(norm(x)), x += mlp(norm(x)); final norm; head (the embedding matrix
    when no lm_head.weight is stored, src/model.c:156-158)."""
    eps = cfg["rms_norm_eps"]
    T = len(tokens)
    positions = np.arange(first_position, first_position + T)
    x = embed(w["model.embed_tokens.weight"], tokens)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        x = x + attention_block(cfg, w, l, rmsnorm(x, w[p + "input_layernorm.weight"], eps), positions)
        h = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])
    x = rmsnorm(x, w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(x, head)


# ---- sampling (src/sample.c) ---------------------------------------------------------------

MASK64 = (1 << 64) - 1


class Rng:
    """xorshift64* (src/sample.c:9-23)."""

    def __init__(self, seed):
        self.s = (seed * 0x9e3779b97f4a7c15 + 0x1234567) & MASK64
        if self.s == 0:
            self.s = 0x2545f4914f6cdd1d

    def uniform(self):
        x = self.s
        x ^= x >> 12
        x ^= (x << 25) & MASK64
        x ^= x >> 27
        self.s = x
        return np.float32(((x * 0x2545f4914f6cdd1d) & MASK64) >> 40) / np.float32(16777216.0)


def expf(x):
    """The reference's own exponential, src/mathx.c:7-32, one fp32 operation at a time: exp(x) =
    2^n exp(r), n = floor(x log2(e) + 1/2), r = x - n ln2 taken off in two parts, exp(r) by a
    polynomial of degree 7. The sampler's probabilities come from this routine (src/sample.c:99),
    and a draw can turn on their last bit."""
    f = np.float32
    x = f(x)
    if x != x:
        return x
    if x > f(88.3762626647949):
        x = f(88.3762626647949)
    if x < f(-87.3365478515625):
        return f(0.0)
    fx = f(math.floor(f(f(x * f(1.44269504088896341)) + f(0.5))))
    n = int(fx)
    x = f(x - f(fx * f(0.693359375)))
    x = f(x - f(fx * f(-2.12194440e-4)))
    z = f(x * x)
    y = f(1.9875691500e-4)
    for c in (1.3981999507e-3, 8.3334519073e-3, 4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1):
        y = f(f(y * x) + f(c))
    y = f(f(f(y * z) + x) + f(1.0))
    return f(y * f(math.ldexp(1.0, n)))


def sample(logits, temp, top_k, top_p, min_p, rng):
    """src/sample.c:66-117: greedy when temp <= 0 (first index of the maximum); else sort by
    (logit descending, id ascending), keep top_k, p = exp((l - max)/temp) normalised in fp32,
    min-p prefix, top-p prefix, draw r = u * sum and take the first prefix sum above r."""
    logits = np.asarray(logits, dtype=np.float32)
    if temp <= 0:
        return int(np.argmax(logits))
    order = sorted(range(len(logits)), key=lambda i: (-logits[i], i))
    if 0 < top_k < len(order):
        order = order[:top_k]
    f = np.float32
    mx = logits[order[0]]
    p = [expf(f(f(logits[i] - mx) / f(temp))) for i in order]
    total = f(0)
    for v in p:
        total = f(total + v)
    p = [f(v / total) for v in p]
    kept = len(p)
    if min_p > 0:
        kept = 0
        while kept < len(p) and p[kept] >= f(min_p) * p[0]:
            kept += 1
        kept = max(kept, 1)
    if 0 < top_p < 1:
        cum = f(0)
        for i in range(kept):
            cum = f(cum + p[i])
            if cum >= f(top_p):
                kept = i + 1
                break
    total = f(0)
    for i in range(kept):
        total = f(total + p[i])
    r = f(rng.uniform() * total)
    cum = f(0)
    for i in range(kept):
        cum = f(cum + p[i])
        if r < cum:
            return order[i]
    return order[kept - 1]


def logprob(logits, tok):
    """logit - max - log(sum(exp(l - max))) (src/sample.c:25-33)."""
    logits = np.asarray(logits, dtype=np.float64)
    mx = logits.max()
    return float(logits[tok] - mx - np.log(np.sum(np.exp(logits - mx))))
