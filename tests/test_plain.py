"""What pins the plain implementation beside the reference's text (no GPU): vectors the
reference's own tests hold, special cases that reduce to a library routine, invariants.
Each is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import torch

import helpers
import plain


def test_rmsnorm_vector_of_the_reference():
    """x = {1..5}, w = {1, 1, 2, 2, 0.5}, eps = 1e-6 -> x * w / sqrt(11 + 1e-6)
    (tests/test_kern.c:242-248). A mean taken as a sum, or eps outside the root, fails."""
    x = np.array([1, 2, 3, 4, 5.0])
    w = np.array([1, 1, 2, 2, 0.5])
    assert np.allclose(plain.rmsnorm(x, w, 1e-6), x * w / math.sqrt(11 + 1e-6), rtol=0, atol=1e-12)
    c = 3.0                                    # weight one on a vector of +-c gives +-c / sqrt(c^2 + eps)
    v = np.array([c, -c, c, -c])
    assert np.allclose(plain.rmsnorm(v, np.ones(4), 0.5), v / math.sqrt(c * c + 0.5))


def test_softmax_and_silu_vectors_of_the_reference():
    """softmax {1, 2, 3, 4}: sums to 1, increasing, neighbours in ratio e (tests/test_kern.c:249-253);
    silu(0) = 0, silu(1) = 0.7310585786 (tests/test_kern.c:33-34)."""
    s = plain.softmax(np.array([1, 2, 3, 4.0]))
    assert abs(s.sum() - 1) < 1e-12 and np.all(np.diff(s) > 0) and abs(s[3] / s[2] - math.e) < 1e-12
    assert plain.silu(np.array(0.0)) == 0.0 and abs(plain.silu(np.array(1.0)) - 0.7310585786) < 1e-9


def test_rope_frequencies_and_identity_at_zero():
    """theta_scale(1e6, 64), (1e4, 128), (1e4, 96) = base^(-2/n) (tests/test_kern.c:156-158);
    position 0 is the identity (cos_sin(0) = (1, 0), tests/test_kern.c:140-154)."""
    for base, n in ((1e6, 64), (1e4, 128), (1e4, 96)):
        th = plain.rope_angles([1], n, base)[0]
        assert abs(th[1] / th[0] - base ** (-2.0 / n)) < 1e-15 and th[0] == 1.0
    v = np.random.default_rng(0).standard_normal((1, 2, 16))
    assert np.array_equal(plain.rope(v, [0], 16, 1e4), v)


def test_rope_pairing_sign_and_invariants():
    """Pairs are (i, i + half): a unit vector on dimension 0 turns into dimensions 0 and half
    by (cos, sin) of the position (a rotation by +angle, src/model.c:488-490); interleaved
    pairing or a flipped sign fails. Norms of pairs are kept; <rope(q, p + s), rope(k, p' + s)>
    depends on p - p' alone."""
    D = 8
    v = np.zeros((1, 1, D))
    v[0, 0, 0] = 1.0
    out = plain.rope(v, [3], D, 1e4)[0, 0]
    assert abs(out[0] - math.cos(3)) < 1e-12 and abs(out[4] - math.sin(3)) < 1e-12
    assert np.allclose(out[[1, 2, 3, 5, 6, 7]], 0)
    rng = np.random.default_rng(1)
    q, k = rng.standard_normal((1, 1, 32)), rng.standard_normal((1, 1, 32))
    dots = [float((plain.rope(q, [9 + s], 32, 1e6) * plain.rope(k, [2 + s], 32, 1e6)).sum()) for s in (0, 5, 1000)]
    assert max(dots) - min(dots) < 1e-9
    r = plain.rope(q, [77], 32, 1e6)[0, 0]
    assert np.allclose(r[:16] ** 2 + r[16:] ** 2, q[0, 0, :16] ** 2 + q[0, 0, 16:] ** 2)
    part = plain.rope(q, [77], 16, 1e6)[0, 0]          # rot_dim < head_dim: the rest passes through
    assert np.array_equal(part[16:], q[0, 0, 16:]) and not np.allclose(part[:16], q[0, 0, :16])


def test_attention_reduces_to_library_routines():
    """Without a window, attention over a whole prompt equals the library's causal
    scaled-dot-product attention; with H = G it is plain multi-head attention; with a band
    mask it equals the library's with that mask. A scale applied twice, a mask off by one or
    a wrong head grouping fails."""
    rng = np.random.default_rng(2)
    T, H, G, D = 23, 6, 2, 16
    q, k, v = (rng.standard_normal(s) for s in ((T, H, D), (T, G, D), (T, G, D)))
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]
    tk = torch.from_numpy(np.repeat(k, H // G, axis=1)).permute(1, 0, 2)[None]
    tv = torch.from_numpy(np.repeat(v, H // G, axis=1)).permute(1, 0, 2)[None]
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    assert np.allclose(plain.attention(q, k, v), ref, atol=1e-12)
    W = 5
    i = torch.arange(T)
    band = (i[None, :] <= i[:, None]) & (i[:, None] - i[None, :] < W)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=band)[0].permute(1, 0, 2).numpy()
    assert np.allclose(plain.attention(q, k, v, window=W), ref, atol=1e-12)
    assert np.allclose(plain.attention(q, k, v, window=T), plain.attention(q, k, v), atol=0)    # window >= context
    # a single query at position 0 returns value row 0; equal scores return the mean of the values
    assert np.allclose(plain.attention(q[:1], k[:1], v[:1])[0, 0], v[0, 0])
    z = plain.attention(np.zeros((T, H, D)), k, v)
    assert np.allclose(z[-1, 0], v[:, 0].mean(axis=0)) and np.allclose(z[-1, 5], v[:, 1].mean(axis=0))
    # heads 1 and 4 of six on two key/value heads: h // (H / G) gives 0 and 1, h % G would give 1 and 0
    assert np.allclose(z[-1, 1], v[:, 0].mean(axis=0)) and np.allclose(z[-1, 4], v[:, 1].mean(axis=0))
    assert not np.allclose(z[-1, 1], v[:, 1].mean(axis=0))


def test_window_mask_edges():
    m = plain.visible(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True]      # 0 <= q - k < 3
    assert m[2].tolist() == [True, True, True, False, False, False]
    assert plain.visible(4, 0).tolist() == np.tril(np.ones((4, 4), bool)).tolist()


def test_linear_and_mlp_reduce_to_library_routines():
    rng = np.random.default_rng(3)
    x, W, b = rng.standard_normal((5, 7)), rng.standard_normal((3, 7)), rng.standard_normal(3)
    ref = torch.nn.functional.linear(torch.from_numpy(x), torch.from_numpy(W), torch.from_numpy(b)).numpy()
    assert np.allclose(plain.linear(x, W, b), ref)
    Wg, Wu, Wd = rng.standard_normal((11, 7)), rng.standard_normal((11, 7)), rng.standard_normal((7, 11))
    t = torch.from_numpy
    ref = (torch.nn.functional.silu(t(x) @ t(Wg).T) * (t(x) @ t(Wu).T)) @ t(Wd).T
    assert np.allclose(plain.swiglu_mlp(x, Wg, Wu, Wd), ref.numpy())


def test_model_level_properties(tmp_path):
    """x = 0 isolates the bias (q = bq); a tied model equals an untied one whose head is the
    embedding; the window changes nothing at positions below it and something beyond it;
    logits at a position depend on earlier tokens only."""
    cfg = dict(helpers.CONFIG_B)
    w = {k: v.astype(np.float64) for k, v in helpers.make_weights(cfg, 5).items()}
    toks = helpers.random_requests(cfg, [50], 1)["r0"]
    full = plain.forward(cfg, w, toks)
    assert full.shape == (50, 1000)
    cut = plain.forward(cfg, w, toks[:20])
    assert np.allclose(full[:20], cut, atol=1e-12)                        # causal
    off = plain.forward(dict(cfg, use_sliding_window=False), w, toks)
    assert np.allclose(full[:32], off[:32], atol=1e-12) and np.max(np.abs(full[40:] - off[40:])) > 1e-3
    wider = plain.forward(dict(cfg, max_window_layers=3), w, toks)       # no layer windowed
    assert np.allclose(wider, off, atol=1e-12)
    tied = dict(cfg, tie_word_embeddings=True)
    w_tied = {k: v for k, v in w.items() if k != "lm_head.weight"}
    w_same = dict(w_tied, **{"lm_head.weight": w["model.embed_tokens.weight"]})
    assert np.allclose(plain.forward(tied, w_tied, toks), plain.forward(cfg, w_same, toks), atol=0)
    p = "model.layers.0.self_attn."
    q = plain.linear(np.zeros((1, 96)), w[p + "q_proj.weight"], w[p + "q_proj.bias"])
    assert np.array_equal(q[0], w[p + "q_proj.bias"])


def test_sampler_of_the_plain_implementation():
    """Greedy takes the first index of the maximum (src/sample.c:72-77, src/sample.h:17); the
    random numbers are the reference's xorshift64* (first draws for seed 0 computed by hand from
    src/sample.c:9-23); temperature sampling follows the ordered pipeline."""
    assert plain.sample([1.0, 5.0, 5.0, 2.0], 0.0, 40, 0.95, 0.05, None) == 1
    r = plain.Rng(0)
    s = 0x1234567
    s ^= s >> 12
    s ^= (s << 25) & plain.MASK64
    s ^= s >> 27
    want = np.float32(((s * 0x2545f4914f6cdd1d) & plain.MASK64) >> 40) / np.float32(16777216.0)
    assert r.uniform() == want and 0 <= want < 1
    logits = np.log(np.array([0.5, 0.25, 0.125, 0.125], dtype=np.float64)).astype(np.float32)
    counts = np.zeros(4)
    rng = plain.Rng(42)
    for _ in range(4000):
        counts[plain.sample(logits, 1.0, 0, 1.0, 0.0, rng)] += 1
    assert np.all(np.abs(counts / 4000 - [0.5, 0.25, 0.125, 0.125]) < 0.03)
    assert all(plain.sample(logits, 1.0, 1, 1.0, 0.0, rng) == 0 for _ in range(20))       # top-k 1
    assert all(plain.sample(logits, 1.0, 0, 0.6, 0.0, rng) in (0, 1) for _ in range(50))  # top-p 0.6
    assert all(plain.sample(logits, 1.0, 0, 1.0, 0.4, rng) in (0, 1) for _ in range(50))  # min-p 0.4
    assert abs(plain.logprob(logits, 1) - math.log(0.25)) < 1e-6


def test_exponential_of_the_reference():
    """The checks that the reference's own test holds for its exponential (tests/test_kern.c:21-32):
    relative error below 4e-7 from -87 to 88 in steps of 0.0137, exp(0) = 1, exp(-100) = 0, a finite
    value for 1000. The product's vectorised routine gives the same bits as the plain one."""
    import math
    from host_draw import hfc_expf
    xs = np.arange(-87.0, 88.0, 0.0137, dtype=np.float32)
    got = np.array([plain.expf(x) for x in xs], dtype=np.float32)
    ref = np.exp(xs.astype(np.float64))
    assert np.max(np.abs(got.astype(np.float64) - ref) / ref) < 4e-7
    assert plain.expf(0.0) == 1.0 and plain.expf(-100.0) == 0.0 and math.isfinite(plain.expf(1000.0))
    assert np.array_equal(hfc_expf(xs), got)
    edge = np.array([0.0, -0.0, -100.0, 1000.0, -87.3365478515625, -87.33655, 88.3762626647949, 1e-30, -1e-30], np.float32)
    assert np.array_equal(hfc_expf(edge), np.array([plain.expf(x) for x in edge], dtype=np.float32))
    rng = np.random.default_rng(0)
    more = (rng.standard_normal(20000) * 20).astype(np.float32)
    assert np.array_equal(hfc_expf(more), np.array([plain.expf(x) for x in more], dtype=np.float32))


# ---- the arrangement of a layer (src/model.c:580-636) -----------------------------------------
# Each case makes all but one path of the layer vanish, so that the logits have a closed form made
# of parts that the tests above pin. A norm applied to the residual stream as well, a norm after
# the branch instead of before it, a dropped final norm, a branch that replaces the stream
# instead of adding to it, rotated values or a missing bias each fail at least one of them.

def _f64(cfg, seed):
    return {k: v.astype(np.float64) for k, v in helpers.make_weights(cfg, seed).items()}


def _head_of(cfg, w, x):
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return plain.linear(plain.rmsnorm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), head)


def _silence(w, cfg, keep=None):
    """o_proj = down_proj = 0 in every layer but ``keep``: those layers add nothing to the stream."""
    w = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        if l != keep:
            w[f"model.layers.{l}.self_attn.o_proj.weight"] = np.zeros_like(w[f"model.layers.{l}.self_attn.o_proj.weight"])
            w[f"model.layers.{l}.mlp.down_proj.weight"] = np.zeros_like(w[f"model.layers.{l}.mlp.down_proj.weight"])
    return w


def test_layers_that_add_nothing_leave_head_of_norm_of_embedding():
    """o_proj = down_proj = 0 everywhere: logits = head(norm(embed(tokens))) exactly (src/model.c:609, 623
    add zeros; src/model.c:629-636). Fails if the final norm is missing, if a layer's norm also
    replaces the stream, or if the stream is overwritten by a branch."""
    for name, cfg in helpers.CONFIGS.items():
        w = _silence(_f64(cfg, 11), cfg)
        toks = helpers.random_requests(cfg, [9], 2)["r0"]
        want = _head_of(cfg, w, plain.embed(w["model.embed_tokens.weight"], toks))
        assert np.array_equal(plain.forward(cfg, w, toks), want), name
        assert np.max(np.abs(want)) > 1e-3


def test_a_zero_input_norm_leaves_the_biases_and_the_unnormed_stream():
    """input_layernorm.weight = 0 in layer l: its attention sees h = 0, so q = bq, k = bk, v = bv at every
    position; every visible value is bv, so the attention output is bv of the query head's key/value head
    h // (H / G), and the stream grows by Wo times that, at every position alike (src/model.c:580-609).
    With that layer's down_proj = 0 and the other layers silent, logits = head(norm(embed + Wo rep(bv))).
    Fails if the norm sits behind the branch or on the stream, if values are rotated (bv would turn
    with the position), if a bias is dropped, or if heads are grouped by h % G."""
    for name, cfg in helpers.CONFIGS.items():
        H, G, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        for l in range(cfg["num_hidden_layers"]):
            w = _silence(_f64(cfg, 12), cfg, keep=l)
            p = f"model.layers.{l}."
            w[p + "input_layernorm.weight"] = np.zeros(cfg["hidden_size"])
            w[p + "mlp.down_proj.weight"] = np.zeros_like(w[p + "mlp.down_proj.weight"])
            toks = helpers.random_requests(cfg, [40], 3)["r0"]            # beyond B's window of 32
            bv = w[p + "self_attn.v_proj.bias"].reshape(G, D)
            rep = np.concatenate([bv[h // (H // G)] for h in range(H)])
            add = w[p + "self_attn.o_proj.weight"] @ rep
            want = _head_of(cfg, w, plain.embed(w["model.embed_tokens.weight"], toks) + add[None, :])
            got = plain.forward(cfg, w, toks, first_position=3)
            assert np.allclose(got, want, rtol=0, atol=1e-11), (name, l)
            assert np.max(np.abs(add)) > 1e-2
            # the attention block alone, given h = 0
            block = plain.attention_block(cfg, w, l, np.zeros((5, cfg["hidden_size"])), np.arange(4, 9))
            assert np.allclose(block, np.tile(add, (5, 1)), rtol=0, atol=1e-12)


def test_a_zero_post_attention_norm_silences_the_feed_forward():
    """post_attention_layernorm.weight = 0: the feed-forward sees 0 and adds Wdown (silu(0) * 0) = 0
    (src/model.c:611-623), so the logits are those of the model with that layer's down_proj = 0. Fails if
    the feed-forward reads the stream without its norm, or the norm of the other branch."""
    cfg = helpers.CONFIG_B
    w = _f64(cfg, 13)
    toks = helpers.random_requests(cfg, [21], 4)["r0"]
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        a = dict(w, **{p + "post_attention_layernorm.weight": np.zeros(cfg["hidden_size"])})
        b = dict(w, **{p + "mlp.down_proj.weight": np.zeros_like(w[p + "mlp.down_proj.weight"])})
        full = plain.forward(cfg, w, toks)
        assert np.array_equal(plain.forward(cfg, a, toks), plain.forward(cfg, b, toks))
        assert np.max(np.abs(full - plain.forward(cfg, b, toks))) > 1e-3


def test_one_layer_with_one_branch_is_that_branch_on_the_normed_stream():
    """One layer alive. With its o_proj = 0: logits = head(norm(e + mlp(norm2(e)))) (the feed-forward reads
    the norm of the stream as the attention left it, and adds to the un-normed stream). With its down_proj = 0
    and a single token: attention over one key returns its value, so logits = head(norm(e + Wo rep(Wv norm1(e) + bv)))."""
    for name, cfg in helpers.CONFIGS.items():
        H, G, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        eps = cfg["rms_norm_eps"]
        l = cfg["num_hidden_layers"] - 1
        p = f"model.layers.{l}."
        base = _silence(_f64(cfg, 14), cfg, keep=l)
        toks = helpers.random_requests(cfg, [6], 5)["r0"]
        e = plain.embed(base["model.embed_tokens.weight"], toks)
        w = dict(base, **{p + "self_attn.o_proj.weight": np.zeros_like(base[p + "self_attn.o_proj.weight"])})
        mlp = plain.swiglu_mlp(plain.rmsnorm(e, w[p + "post_attention_layernorm.weight"], eps),
                               w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        assert np.allclose(plain.forward(cfg, w, toks), _head_of(cfg, w, e + mlp), rtol=0, atol=1e-11), name
        w = dict(base, **{p + "mlp.down_proj.weight": np.zeros_like(base[p + "mlp.down_proj.weight"])})
        for pos in (0, 7):                                      # one token: the output is its own value, not rotated
            h1 = plain.rmsnorm(e[:1], w[p + "input_layernorm.weight"], eps)
            v = plain.linear(h1, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).reshape(G, D)
            rep = np.concatenate([v[h // (H // G)] for h in range(H)])
            want = _head_of(cfg, w, e[:1] + (w[p + "self_attn.o_proj.weight"] @ rep)[None, :])
            assert np.allclose(plain.forward(cfg, w, toks[:1], first_position=pos), want, rtol=0, atol=1e-11), (name, pos)
        # both branches alive, one token: the feed-forward reads the stream as the attention left it
        w = base
        h1 = plain.rmsnorm(e[:1], w[p + "input_layernorm.weight"], eps)
        v = plain.linear(h1, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).reshape(G, D)
        x1 = e[:1] + (w[p + "self_attn.o_proj.weight"] @ np.concatenate([v[h // (H // G)] for h in range(H)]))[None, :]
        x2 = x1 + plain.swiglu_mlp(plain.rmsnorm(x1, w[p + "post_attention_layernorm.weight"], eps),
                                   w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        assert np.allclose(plain.forward(cfg, w, toks[:1], first_position=3), _head_of(cfg, w, x2), rtol=0, atol=1e-11), name


def test_positions_enter_only_through_distances():
    """A shift of all positions changes nothing (rotary encodes distances; values and the stream carry no
    position): the logits of a sequence that starts at position 1000 are those of one that starts at 0."""
    for name, cfg in helpers.CONFIGS.items():
        w = _f64(cfg, 15)
        toks = helpers.random_requests(cfg, [45], 6)["r0"]
        a, b = plain.forward(cfg, w, toks), plain.forward(cfg, w, toks, first_position=1000)
        assert np.max(np.abs(a - b)) < 1e-8 * np.max(np.abs(a)), name
