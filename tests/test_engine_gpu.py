"""The engine against the plain implementation, in every way of cutting the work."""
import numpy as np
import pytest

import helpers
import plain

pytestmark = pytest.mark.gpu

# Largest |logit difference| allowed between the engine and the float64 plain implementation,
# as a fraction of the request's largest |logit|.
# fp32: rounding of a few hundred fused multiply-adds per value (measured: about 1e-6).
# bf16: activations and cache rounded to 8 bits of mantissa at every part (measured: 0.8e-2).
TOL = {"float32": 5e-6, "bfloat16": 2e-2}
KERNELS_AGREE = 2e-2     # bf16: another order of summation flips roundings of activations, which spread like any rounding
LENGTHS = {"A": [7, 19, 33, 70, 101], "B": [1, 40, 77, 100, 130], "C": [3, 48, 49, 120, 200]}


@pytest.fixture(scope="module", params=["A", "B", "C"])
def tiny(request, tmp_path_factory):
    name = request.param
    cfg = helpers.CONFIGS[name]
    d = helpers.make_model_dir(str(tmp_path_factory.mktemp("model" + name)), cfg, seed=ord(name))
    reqs = helpers.random_requests(cfg, LENGTHS[name], seed=7)
    return name, cfg, d, reqs, helpers.plain_logits(d, reqs)


def engine_for(model_dir, dtype, name, max_tokens, max_seqs=4):
    import hf_cpu_amd
    return hf_cpu_amd.load_engine(model_dir, dtype=dtype, page_tokens=helpers.PAGE[name],
                                  max_tokens=max_tokens, max_seqs=max_seqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cutting", ["whole", "tail", "portions", "mixed"])
def test_cuttings(gpu, tiny, dtype, cutting):
    name, cfg, d, reqs, want = tiny
    steps = {"whole": helpers.trace_whole, "tail": helpers.trace_tail, "portions": helpers.trace_portions,
             "mixed": lambda r: helpers.trace_mixed(r, seed=3)}[cutting](reqs)
    max_tokens = helpers.max_live_tokens(steps)
    engine = engine_for(d, dtype, name, max_tokens)
    got = helpers.run_trace_in_engine(engine, steps)
    assert len(got) == sum(len(t) for t in reqs.values())
    worst = helpers.compare(got, want, TOL[dtype], f"{name} {dtype} {cutting}")
    print(f"{name} {dtype} {cutting}: worst |diff| {worst:.3e}")
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    if cutting == "mixed":
        assert any(p.reused > 0 for p in engine.manager.pools), "the trace was meant to use pages again"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuttings_agree_with_each_other(gpu, tiny, dtype):
    """Beyond agreeing with the plain implementation, the cuttings agree among themselves
    far more closely: the same values are computed, only in other launches."""
    name, cfg, d, reqs, _ = tiny
    results = []
    for make in (helpers.trace_whole, helpers.trace_portions, lambda r: helpers.trace_mixed(r, seed=5)):
        steps = make(reqs)
        engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps))
        results.append(helpers.run_trace_in_engine(engine, steps))
    tol = 2e-5 if dtype == "float32" else 0.06
    for other in results[1:]:
        for key, row in results[0].items():
            err = float(np.max(np.abs(row - other[key])))
            assert err <= tol, f"{name} {dtype}: {key}: cuttings differ by {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_same_trace_twice_gives_the_same_bits(gpu, tiny, dtype):
    """No kernel adds with atomics or in an order that depends on timing: a mixed trace replayed
    in a second engine gives the same logits bit for bit."""
    name, cfg, d, reqs, _ = tiny
    steps = helpers.trace_mixed(reqs, seed=11)
    runs = []
    for _ in range(2):
        engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps))
        runs.append(helpers.run_trace_in_engine(engine, steps))
    assert runs[0].keys() == runs[1].keys()
    for key, row in runs[0].items():
        assert np.array_equal(row, runs[1][key]), f"{name} {dtype}: {key} differs between two runs"


def test_window_edge_shows(gpu, tmp_path):
    """Config B with one key made to stand out: a query far beyond the window must not see
    it in the windowed layers, one inside the window must. The plain implementation decides;
    a window off by one moves the logits by far more than the tolerance."""
    cfg = dict(helpers.CONFIG_B)
    w = helpers.make_weights(cfg, seed=11)
    for l in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{l}.self_attn.k_proj.bias"] *= 4.0      # large common key component
        w[f"model.layers.{l}.self_attn.q_proj.bias"] *= 4.0
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, 0, weights=w)
    reqs = helpers.random_requests(cfg, [31, 32, 33, 34, 64, 65, 97], seed=2)
    want = helpers.plain_logits(d, reqs)
    off = dict(cfg, use_sliding_window=False)
    d_off = helpers.make_model_dir(str(tmp_path / "off"), off, 0, weights=w)
    want_off = helpers.plain_logits(d_off, reqs)
    # the window matters: beyond it the two models differ clearly, inside it they are equal
    assert max(np.max(np.abs(want["r6"][40:] - want_off["r6"][40:])), 0) > 0.05
    assert np.max(np.abs(want["r6"][:32] - want_off["r6"][:32])) < 1e-9
    for steps in (helpers.trace_whole(reqs), helpers.trace_tail(reqs, 8), helpers.trace_mixed(reqs, 1)):
        engine = engine_for(d, "float32", "B", helpers.max_live_tokens(steps))
        helpers.compare(helpers.run_trace_in_engine(engine, steps), want, TOL["float32"], "window")


def test_far_key_among_hundreds(gpu, tmp_path):
    """One early token whose key every later query matches strongly in layer 0, so that its
    value must reach position 259 through 16 pages: a block table entry or a page offset that
    is wrong anywhere on the way moves the logits far beyond the tolerance.

    Construction: with rope_theta = 1e9 the pair (5, 13) of a head turns by less than 0.01 rad
    over 260 positions. Every query gets a large bias on dimension 5; key dimension 5 reads the
    direction e of the residual stream; token 77's embedding is e itself, other embeddings are
    random, so token 77's key stands out by about 8 : 1."""
    cfg = dict(helpers.CONFIG_A, max_position_embeddings=512, rope_theta=1e9)
    E, H, G, D = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    w = helpers.make_weights(cfg, seed=4)
    rng = np.random.default_rng(12)
    e = rng.standard_normal(E)
    e /= np.linalg.norm(e)
    w["model.embed_tokens.weight"][77] = (4.0 * e).astype(np.float32)
    for g in range(G):
        w["model.layers.0.self_attn.k_proj.weight"][g * D + 5] = e.astype(np.float32)
    for h in range(H):
        w["model.layers.0.self_attn.q_proj.bias"][h * D + 5] = 6.0
    toks = [t if t != 77 else 78 for t in helpers.random_requests(cfg, [260], seed=9)["r0"]]
    toks[3] = 77
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, 0, weights=w)
    reqs = {"r0": toks}
    want = helpers.plain_logits(d, reqs)
    other = helpers.plain_logits(d, {"r0": toks[:3] + [78] + toks[4:]})
    assert np.max(np.abs(want["r0"][200:] - other["r0"][200:])) > 1.0, "the far key was meant to matter"
    for steps in (helpers.trace_whole(reqs), helpers.trace_tail(reqs), helpers.trace_portions(reqs)):
        for dtype in ("float32", "bfloat16"):
            engine = engine_for(d, dtype, "A", helpers.max_live_tokens(steps))
            helpers.compare(helpers.run_trace_in_engine(engine, steps), want, TOL[dtype], "far key " + dtype)


def test_first_tokens_and_long_decode(gpu, tiny):
    """The first tokens of a sequence one by one from an empty cache, and a long run of
    single-token steps (every page edge is crossed in decode)."""
    name, cfg, d, reqs, want = tiny
    r = "r4"
    toks = reqs[r]
    steps = [{"step": i, "entries": [{"id": r, "tokens": [t], "want": [0]}], "end": []}
             for i, t in enumerate(toks)]
    steps[-1]["end"] = [r]
    for dtype in ("float32", "bfloat16"):
        engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps))
        got = helpers.run_trace_in_engine(engine, steps)
        helpers.compare(got, {r: want[r]}, TOL[dtype], f"{name} {dtype} token by token")


def test_step_refusals_leave_no_trace(gpu, tiny):
    from hf_cpu_amd.status import EngineError
    name, cfg, d, reqs, want = tiny
    engine = engine_for(d, "float32", name, 128, max_seqs=2)
    with pytest.raises(EngineError) as e:
        engine.step([("a", [1, cfg["vocab_size"]], [0])])
    assert e.value.code == "EINVAL" and "vocabulary" in str(e.value)
    with pytest.raises(EngineError) as e:
        engine.step([("a", [1, 2], [2])])
    assert e.value.code == "EINVAL"
    with pytest.raises(EngineError) as e:
        engine.step([("a", list(range(100)), []), ("b", list(range(100)), [])])     # 128 tokens of pages
    assert e.value.code == "ENOMEM"
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    with pytest.raises(EngineError) as e:
        engine.step([("a", [1], []), ("b", [1], []), ("c", [1], [])])                # 2 slots
    assert e.value.code == "ENOMEM"
    assert not engine.manager.held
    toks = reqs["r2"]
    got = helpers.run_trace_in_engine(engine, helpers.trace_whole({"r2": toks}))
    helpers.compare(got, want, TOL["float32"], "after refusals")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager(gpu, tiny, dtype):
    """Decode steps replayed from a captured graph against the same steps run eagerly: many
    replays, with eager steps of other shapes (a new prompt, a request that ends) in between,
    every replay compared. The graph is first replayed at its third step of a shape."""
    name, cfg, d, reqs, want = tiny
    import hf_cpu_amd
    runs = {}
    for graphs in (False, True):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=helpers.PAGE[name], max_tokens=1024,
                                        max_seqs=4, graphs=graphs)
        rows = []
        live = {r: 0 for r in ("r2", "r3", "r4")}
        for r in live:                                        # prompts: all but the last 25 tokens
            n = len(reqs[r]) - 25
            engine.step([(r, reqs[r][:n], [])])
            live[r] = n
        for i in range(25):
            if i == 9:                                        # an eager step of another shape in between
                engine.step([("r1", reqs["r1"], [0])])
            if i == 15:
                engine.release("r1")
            logits = engine.step([(r, [reqs[r][at]], [0]) for r, at in live.items()])
            rows.append(logits.float().cpu().numpy().copy())
            for r in live:
                live[r] += 1
        runs[graphs] = rows
        if graphs:
            assert engine.graph_replays >= 20
        else:
            assert engine.graph_replays == 0
    # A replay launches the kernels of the eager step with the same arguments: the same bits.
    for i, (a, b) in enumerate(zip(runs[False], runs[True])):
        assert np.array_equal(a, b), f"decode step {i}: graph and eager differ by {float(np.max(np.abs(a - b))):.3e}"
    got = {("r4", len(reqs["r4"]) - 25 + i): runs[True][i][2] for i in range(25)}
    helpers.compare(got, want, TOL[dtype], "graph replay")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_every_size_share_a_few_graphs(gpu, tmp_path, dtype):
    """Nineteen requests decoded together that end one after another, so that every batch size
    from 19 down to 1 occurs: every row against the plain implementation, and sizes above 8 are
    filled up to a multiple of 8 with rows of no request (they live on a page and in a slot that
    the manager never hands out), so that 24 and 16 are the only shapes captured for them. A
    second pass over the same sizes replays, and gives the bits of the first; the engine keeps
    only its most recently used graphs."""
    import hf_cpu_amd
    cfg = helpers.CONFIG_B
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, seed=3)
    n_req = 19
    lengths = [22 + (5 * i) % 13 + i for i in range(n_req)]               # request i ends after lengths[i] tokens
    reqs = helpers.random_requests(cfg, lengths, seed=31)
    want = helpers.plain_logits(d, reqs)
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=8, max_tokens=64 * n_req, max_seqs=n_req)
    engine.GRAPHS_KEPT = 4                      # fewer than the shapes that occur: graphs are dropped and captured again
    passes = []
    for again in range(2):
        got, sizes = {}, set()
        for r, toks in reqs.items():
            engine.step([(r, toks[:12], [])])
        at = {r: 12 for r in reqs}
        while at:
            live = list(at)
            logits = engine.step([(r, [reqs[r][at[r]]], [0]) for r in live]).float().cpu().numpy()
            sizes.add(len(live))
            for r, row in zip(live, logits):
                got[(r, at[r])] = row.copy()
                at[r] += 1
                if at[r] == len(reqs[r]):
                    del at[r]
                    engine.release(r)
        assert sizes == set(range(1, n_req + 1))
        helpers.compare(got, want, TOL[dtype], "batches of every size")
        passes.append(got)
    assert all(np.array_equal(passes[0][k], passes[1][k]) for k in passes[0])
    assert {key[0] for key in engine._graph_seen if key[0] > 8} <= {16, 24}
    assert 0 < len(engine._graphs) <= 4
    assert engine.graph_replays > 0
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)


@pytest.mark.parametrize("seed", range(20))
def test_random_configurations(gpu, tmp_path, seed):
    """Configurations drawn at random within what config.json allows (head sizes in steps of
    16, any number of heads and groups, widths and vocabularies that are no power of two and not
    even multiples of 8, windows, page sizes), each through a mixed trace with few pages, in
    both precisions against the plain implementation: the kernels either take a size or hand
    it to a kernel that does; they never give a wrong result."""
    import hf_cpu_amd
    rng = np.random.default_rng(100 + seed)
    D = int(rng.choice([16, 32, 48, 64, 80, 96, 128]))
    G = int(rng.choice([1, 2, 3, 4]))
    group = int(rng.choice([1, 2, 3, 4, 7]))
    window = int(rng.choice([0, 0, 7, 20, 33]))
    layers = int(rng.integers(1, 4))
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=layers,
               hidden_size=int(rng.choice([40, 56, 72, 100, 136, 150])), num_attention_heads=G * group,
               num_key_value_heads=G, head_dim=D, intermediate_size=int(rng.choice([64, 100, 192, 200, 330])),
               vocab_size=int(rng.integers(50, 1200)), rope_theta=float(rng.choice([1e4, 5e5, 1e6])),
               rms_norm_eps=float(rng.choice([1e-6, 1e-5, 3e-5])), tie_word_embeddings=bool(rng.integers(0, 2)),
               use_sliding_window=window > 0, sliding_window=window or 4096,
               max_window_layers=int(rng.integers(0, layers + 1)), max_position_embeddings=256, hidden_act="silu")
    page = int(rng.choice([4, 8, 16, 32]))
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, seed=seed)
    reqs = helpers.random_requests(cfg, [int(n) for n in rng.integers(1, 90, 5)], seed=seed)
    steps = helpers.trace_mixed(reqs, seed=seed, max_live=3)
    def run(dtype, plain_kernels=False):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=page,
                                        max_tokens=helpers.max_live_tokens(steps, round_to=max(64, page)), max_seqs=3)
        engine.ops.force_plain_gemm = engine.ops.force_plain_attention = plain_kernels
        got = helpers.run_trace_in_engine(engine, steps)
        assert not engine.manager.held
        engine.manager.check()
        return got
    helpers.compare(run("float32"), helpers.plain_logits(d, reqs), TOL["float32"], f"random configuration {seed} fp32 {cfg}")
    # bf16 rounds activations at the same places whichever kernels run. Against float64 (weights
    # rounded alike) widths as small as 40 average less of that rounding away than the two fixed
    # configurations do: the bound is 3e-2 here. A kernel's fault shows between the kernels:
    # the matrix-core kernels against the plain ones, on the same roundings.
    want = helpers.plain_logits(d, reqs, round_weights_bf16=True)
    got, got_plain = run("bfloat16"), run("bfloat16", plain_kernels=True)
    helpers.compare(got, want, 3e-2, f"random configuration {seed} bf16 {cfg}")
    helpers.compare(got_plain, want, 3e-2, f"random configuration {seed} bf16 with plain kernels {cfg}")
    worst = max(float(np.max(np.abs(got[k] - got_plain[k]))) / float(np.max(np.abs(want[k[0]]))) for k in got)
    assert worst <= KERNELS_AGREE, f"random configuration {seed}: kernels differ by {worst:.2e} {cfg}"
    print(f"random configuration {seed}: matrix-core and plain kernels differ by {worst:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoded_tokens_between_prompt_portions_keep_their_places(gpu, tiny, dtype):
    """A step whose entries alternate prompt portions of 16 tokens and more with single tokens: the
    engine lays the short ones first (attention takes them as a step of their own), the logits still
    come back in the order of the entries and of their wanted places."""
    name, cfg, d, reqs, want = tiny
    ids = [r for r in reqs if len(reqs[r]) >= 33][:3]
    if len(ids) < 3:
        pytest.skip("needs three requests of 33 tokens or more")
    a, b, c = ids
    engine = engine_for(d, dtype, name, max_tokens=512)
    engine.step([(a, reqs[a][:20], []), (c, reqs[c][:5], [])])
    entries = [(b, reqs[b][:30], [29, 0]), (a, [reqs[a][20]], [0]), (c, reqs[c][5:25], [3, 19]), (a + "x", reqs[a][:1], [0])]
    rows = engine.step(entries).float().cpu().numpy()
    places = [(b, 29), (b, 0), (a, 20), (c, 8), (c, 24), (a, 0)]
    assert rows.shape[0] == len(places)
    got = {((r, p) if i < 5 else ("first", 0)): row for i, ((r, p), row) in enumerate(zip(places, rows))}
    first = got.pop(("first", 0))
    helpers.compare(got, want, TOL[dtype], f"{name} {dtype} alternating entries")
    scale = float(np.max(np.abs(want[a])))
    assert float(np.max(np.abs(first - want[a][0]))) / scale <= TOL[dtype]
    # and the requests go on from there
    more = engine.step([(a, [reqs[a][21]], [0]), (b, reqs[b][30:33], [2])]).float().cpu().numpy()
    helpers.compare({(a, 21): more[0], (b, 32): more[1]}, want, TOL[dtype], f"{name} {dtype} the step after")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_truncate_then_other_tokens(gpu, tiny, dtype):
    """A request is cut back (src/model.c:305) inside a page and to a page's edge, and fed other tokens:
    the logits are those of the sequence as it then reads. With a window (configuration B) a cut that
    would need pages the window has given back is refused and changes nothing; one that does not is
    served, across the window's edge."""
    from hf_cpu_amd.status import EngineError
    import plain
    name, cfg, d, reqs, _ = tiny
    P = helpers.PAGE[name]
    rng = np.random.default_rng(5)
    toks = reqs["r3"]                                             # 70 (A) or 100 (B) tokens
    pcfg, w = plain.read_model(d)
    engine = engine_for(d, dtype, name, 256)
    engine.step([("t", toks, [])])
    # B's window of 32 lets go of pages as the request grows: only short cuts stay possible there
    cuts = [len(toks) - 3, len(toks) - P - 5, (len(toks) - 2 * P) // P * P] if name == "A" else [len(toks) - 3, len(toks) + 3]
    seq = list(toks)
    for cut in cuts:
        more = [int(t) for t in rng.integers(0, cfg["vocab_size"], 7)]
        engine.truncate("t", cut)
        assert engine.length("t") == cut
        engine.manager.check()
        seq = seq[:cut] + more
        got = engine.step([("t", more[:5], [0, 4])]).float().cpu().numpy()
        got = np.concatenate([got, engine.step([("t", more[5:6], [0])]).float().cpu().numpy(),
                              engine.step([("t", more[6:], [0])]).float().cpu().numpy()])
        want = plain.forward(pcfg, w, seq)
        scale = float(np.max(np.abs(want)))
        for row, pos in zip(got, (cut, cut + 4, cut + 5, cut + 6)):
            err = float(np.max(np.abs(row - want[pos]))) / scale
            assert err <= TOL[dtype], f"{name} {dtype}: cut to {cut}, position {pos}: {err:.3e}"
    if name == "B":                                               # window 32: pages before position len - 32 are gone
        before = (engine.length("t"), [list(t) for t in engine.manager.held["t"].tables])
        with pytest.raises(EngineError) as e:
            engine.truncate("t", 20)
        assert e.value.code == "ENOTSUP"
        assert (engine.length("t"), [list(t) for t in engine.manager.held["t"].tables]) == before
    engine.release("t")
    engine.manager.check()
    assert all(p.n_held == 0 for p in engine.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_what_a_page_held_before_does_not_matter(gpu, tiny, dtype):
    """Every row of the cache starts as NaN (as if each page's last owner had overflowed): a step reads
    only rows that it or an earlier step of the same request wrote, and what it reads beside them
    (rows past a request's end, pages a window has given back, whole blocks of keys fetched for a few)
    has weight zero and must not reach the result: 0 x NaN is NaN. Mixed trace, pages used again."""
    name, cfg, d, reqs, want = tiny
    steps = helpers.trace_mixed(reqs, seed=11)
    engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps))
    for view in engine.storage.views:
        if hasattr(view, "k"):
            view.k.fill_(float("nan"))
            view.v.fill_(float("inf"))
    got = helpers.run_trace_in_engine(engine, steps)
    assert all(np.isfinite(row).all() for row in got.values()), "a stale row of the cache reached the logits"
    helpers.compare(got, want, TOL[dtype], f"{name} {dtype} on a cache of NaN")
    assert any(p.reused > 0 for p in engine.manager.pools)
    # and with the pages poisoned again between a prompt and its decoded tokens: only rows of live requests are kept
    whole = helpers.trace_tail({"r2": reqs["r2"]}, tail=8)
    engine = engine_for(d, dtype, name, 256)
    got, places = {}, helpers.wanted_places(whole)
    for i, s in enumerate(whole):
        rows = engine.step([(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).float().cpu().numpy()
        for row, key in zip(rows, places[s["step"]]):
            got[key] = row.copy()
        if i == 0:
            h = engine.manager.held["r2"]
            for g, group in enumerate(engine.manager.groups):
                own = [p for p in h.tables[g] if p >= 0]
                for e in group.entries:
                    view = engine.storage.views[e]
                    P = view.page_tokens
                    keep_k = {p: view.k[p * P:(p + 1) * P].clone() for p in own}
                    keep_v = {p: view.v[p * P:(p + 1) * P].clone() for p in own}
                    view.k.fill_(float("inf"))
                    view.v.fill_(float("nan"))
                    for p in own:
                        view.k[p * P:(p + 1) * P] = keep_k[p]
                        view.v[p * P:(p + 1) * P] = keep_v[p]
    helpers.compare(got, {"r2": want["r2"]}, TOL[dtype], f"{name} {dtype} decoding beside poisoned pages")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_taken_from_the_device(gpu, tiny, dtype):
    """``Engine.step(fed=...)``: the single token of some entries comes from an int32 tensor on the device,
    at rows the caller names, instead of from the host. A mixed step whose entries are ordered long portion,
    fed decoder, short portion, fed decoder (inside the step requests with few tokens are laid first, so the
    places the tokens go to are not the entries' order), with rows taken from a shuffled tensor; then a plain
    decode step of more requests than the engine decodes without filling the batch up, replayed from a graph.
    Each gives the bits of the same step with the tokens given by the host. Rows outside the tensor and
    entries with two tokens are refused."""
    import torch
    from hf_cpu_amd.status import EngineError
    name, cfg, d, reqs, _ = tiny
    V = cfg["vocab_size"]
    rng = np.random.default_rng(9)
    prompts = {f"q{i}": [int(t) for t in rng.integers(0, V, n)] for i, n in enumerate([5, 9, 3, 12, 6, 7, 4, 8, 10, 11, 2])}
    many = list(prompts)
    junk = 10 ** 6

    def run(feed):
        eng = engine_for(d, dtype, name, 64 * 16, max_seqs=13)
        eng.step([(r, prompts[r], []) for r in many])
        long_a, short_b = [int(t) for t in rng0.integers(0, V, 30)], [int(t) for t in rng0.integers(0, V, 4)]
        tok = {r: int(rng0.integers(0, V)) for r in many}
        pool = torch.full((64,), junk, dtype=torch.int32, device="cuda")
        where = {r: int(p) for r, p in zip(many, rng0.permutation(64))}
        for r in many:
            pool[where[r]] = tok[r]
        out = []
        # long portion, fed decoder, short portion, fed decoder
        entries = [("A", long_a, [0, 29]), ("q0", [tok["q0"]], [0]), ("B", short_b, [3]), ("q1", [tok["q1"]], [0])]
        if feed:
            entries[1] = ("q0", [junk], [0])
            entries[3] = ("q1", [junk], [0])
            out.append(eng.step(entries, fed=(pool, {1: where["q0"], 3: where["q1"]})).float().cpu().numpy().copy())
        else:
            out.append(eng.step(entries).float().cpu().numpy().copy())
        # plain decode steps of eleven requests (filled up to sixteen rows), several so that a graph replays
        for _ in range(4):
            tok = {r: int(rng0.integers(0, V)) for r in many}
            for r in many:
                pool[where[r]] = tok[r]
            if feed:
                got = eng.step([(r, [junk], [0]) for r in many], fed=(pool, {i: where[r] for i, r in enumerate(many)}))
            else:
                got = eng.step([(r, [tok[r]], [0]) for r in many])
            out.append(got.float().cpu().numpy().copy())
        return eng, out, pool

    rng0 = np.random.default_rng(4)
    _, by_host, _ = run(False)
    rng0 = np.random.default_rng(4)
    eng, by_device, pool = run(True)
    for i, (a, b) in enumerate(zip(by_host, by_device)):
        assert a.shape == b.shape and np.array_equal(a, b), f"step {i}"
    assert eng.graph_replays > 0
    with pytest.raises(EngineError):
        eng.step([("q0", [1], [0])], fed=(pool, {0: 64}))
    with pytest.raises(EngineError):
        eng.step([("q0", [1, 2], [1])], fed=(pool, {0: 3}))
    with pytest.raises(EngineError):
        eng.step([("q0", [1], [0])], fed=(pool.long(), {0: 3}))
    eng.manager.check()


@pytest.mark.parametrize("rows", [(1 << 24) - 32, (1 << 24) + 1024])    # (the storage keeps one page more than the pool hands out)
def test_pages_at_the_far_end_of_a_cache_of_many_gigabytes(gpu, tmp_path, rows):
    """A pool so large that a layer's keys are 2^32 elements: the matrix-core attention reaches the cache with 32-bit
    element offsets and 24-bit row numbers, so just below that size it must still be right at the pool's last pages,
    and from that size on the calls go to the plain kernels, which count in 64 bits. The pool's free stack is turned
    over, so that the requests get the highest page ids; a mixed trace against the plain implementation."""
    import torch
    import hf_cpu_amd
    cfg = dict(helpers.CONFIG_C, num_hidden_layers=1, num_key_value_heads=4, use_sliding_window=False)
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, seed=5)
    reqs = helpers.random_requests(cfg, [40, 70, 33], seed=8)
    steps = helpers.trace_mixed(reqs, seed=2, max_live=3, decode_tail=6)
    want = helpers.plain_logits(d, reqs, round_weights_bf16=True)
    engine = hf_cpu_amd.load_engine(d, dtype="bfloat16", page_tokens=16, max_tokens=rows, max_seqs=3, max_context=128)
    k = next(v for v in engine.storage.views if v is not None).k
    assert k.shape[0] >= rows and (k.numel() >= 1 << 32) == (rows >= 1 << 24)
    for pool in engine.manager.pools:
        pool._free.reverse()                                # the highest page ids first
    got = helpers.run_trace_in_engine(engine, steps)
    worst = helpers.compare(got, want, 2e-2, f"a cache of {rows} rows")
    print(f"a cache of {rows} rows of 256 keys, pages from the far end: worst relative difference {worst:.2e}")
    engine.manager.check()
    del engine, k
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,tol", [("bfloat16", 2e-2), ("float32", 1e-5)])
def test_a_step_of_seventy_thousand_tokens(gpu, tmp_path, dtype, tol):
    """400 requests with prompts of 174 to 180 tokens in ONE step: more tokens and more requests than any grid
    dimension of 65,535 holds, so every launcher's way of counting blocks is exercised (rows of a norm, tiles of a
    product, tiles and requests of attention). Every 25th request and the last, first and last position, against
    the plain implementation."""
    import hf_cpu_amd
    cfg = dict(helpers.CONFIG_C, num_hidden_layers=1)
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, seed=9)
    rng = np.random.default_rng(0)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], 180 - (i % 7))] for i in range(400)}
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=400 * 192, max_seqs=400, max_context=192)
    logits = engine.step([(r, toks, [0, len(toks) - 1]) for r, toks in reqs.items()]).float().cpu().numpy()
    assert sum(len(t) for t in reqs.values()) > 70000
    pcfg, w = plain.read_model(d)
    if dtype == "bfloat16":
        w = {k: (helpers.bf16_round(v).astype(np.float64) if v.ndim == 2 else v) for k, v in w.items()}
    for j, (r, toks) in enumerate(reqs.items()):
        if j % 25 and j != len(reqs) - 1:
            continue
        want = plain.forward(pcfg, w, toks)
        for jj, at in enumerate((0, len(toks) - 1)):
            err = float(np.max(np.abs(logits[2 * j + jj] - want[at])) / np.max(np.abs(want)))
            assert err < tol, f"request {r} position {at}: {err:.2e}"
    engine.manager.check()
