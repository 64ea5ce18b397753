"""Each part alone, a schedule that is more than a list of layers, and toy parts that are
registered, built and stepped without touching the package: a mixer with state of its own, a
feed-forward with routing, another position encoding."""
import dataclasses
import json
import math
import os
import types

import numpy as np
import pytest
import torch

import helpers
import plain
import hf_cpu_amd
from hf_cpu_amd import PartSpec, ScheduleEntry, register_architecture, register_part
from hf_cpu_amd.engine import Engine
from hf_cpu_amd.parts import FixedState, PagedKV, ParamSpec, Part
from hf_cpu_amd.registry import make_part

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).cuda()


class Harness:
    """A cache and step inputs for parts that are run outside a model."""

    def __init__(self, ops, needs, page=4, n_pages=64, slots=4):
        dtype = ops.act_dtype
        stub = types.SimpleNamespace(cache_needs=lambda: needs, dtype=dtype, vocab_size=1000)
        self.engine = Engine(stub, ops, page_tokens=page, n_pages=n_pages, max_seqs=slots)

    def inputs(self, entries):
        m = self.engine.manager
        entries = [hf_cpu_amd.engine.Entry(r, t, []) for r, t in entries]
        for e in entries:
            if e.req_id not in m.held:
                m.admit(e.req_id)
            m.reserve(e.req_id, len(e.tokens))
        step = self.engine._inputs(entries)
        for e in entries:
            m.commit(e.req_id, len(e.tokens))
        return step

    @property
    def views(self):
        return self.engine.storage.views


def bind(part, params, ops):
    part.bind_all({k: dev(v) for k, v in params.items()}, ops)
    return part


def test_norm_part(ops32):
    rng = np.random.default_rng(0)
    part = make_part("norm", PartSpec("rmsnorm", dict(size=50, eps=1e-3, prefix="n.")))
    assert [(s.name, s.shape, s.kind) for s in part.param_specs()] == [("n.weight", (50,), "vector")]
    w = rng.standard_normal(50).astype(np.float32)
    bind(part, {"n.weight": w}, ops32)
    x = rng.standard_normal((6, 50)).astype(np.float32)
    out = torch.empty((6, 50), device="cuda")
    part.forward(ops32, dev(x), out)
    assert np.max(np.abs(out.cpu().numpy() - plain.rmsnorm(x.astype(np.float64), w, 1e-3))) < 1e-5


def test_feed_forward_part(ops32):
    rng = np.random.default_rng(1)
    E, F = 40, 72
    part = make_part("feed_forward", PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=F, prefix="m.")))
    p = {"m.gate_proj.weight": rng.standard_normal((F, E)) / 6, "m.up_proj.weight": rng.standard_normal((F, E)) / 6,
         "m.down_proj.weight": rng.standard_normal((E, F)) / 8}
    p = {k: v.astype(np.float32) for k, v in p.items()}
    bind(part, p, ops32)
    h = rng.standard_normal((5, E)).astype(np.float32)
    x = rng.standard_normal((5, E)).astype(np.float32)
    tx = dev(x)
    part.forward(ops32, None, dev(h), tx)
    want = x + plain.swiglu_mlp(h.astype(np.float64), *(p[k].astype(np.float64) for k in p))
    assert np.max(np.abs(tx.cpu().numpy() - want)) < 2e-5


def attention_reference(p, prefix, h, positions, H, G, D, theta, window, rot=None, Dv=None):
    T = h.shape[0]
    Dv = Dv or D
    q = plain.linear(h, p[prefix + "q_proj.weight"], p[prefix + "q_proj.bias"]).reshape(T, H, D)
    k = plain.linear(h, p[prefix + "k_proj.weight"], p[prefix + "k_proj.bias"]).reshape(T, G, D)
    v = plain.linear(h, p[prefix + "v_proj.weight"], p[prefix + "v_proj.bias"]).reshape(T, G, Dv)
    q, k = plain.rope(q, positions, rot or D, theta), plain.rope(k, positions, rot or D, theta)
    if Dv == D:
        att = plain.attention(q, k, v, window)
    else:       # value heads of their own size: the same weights on other values (scores do not see the values)
        att = np.zeros((T, H, Dv))
        for lo in range(0, Dv, D):
            part = np.zeros((T, G, D))
            part[..., :min(D, Dv - lo)] = v[..., lo:lo + D]
            att[..., lo:lo + D] = plain.attention(q, k, part, window)[..., :min(D, Dv - lo)]
    return plain.linear(att.reshape(T, H * Dv), p[prefix + "o_proj.weight"])


@pytest.mark.parametrize("H,G,D,window,rot,Dv", [(4, 2, 16, 0, 16, None), (6, 3, 32, 9, 32, None), (2, 2, 48, 0, 32, None),
                                                 (4, 2, 16, 0, 16, 24), (6, 2, 32, 11, 32, 8)])
def test_attention_part_alone(ops32, ops16, H, G, D, window, rot, Dv):
    """One attention mixer with its cache: a prompt in two portions, then single tokens; two
    requests side by side. The reference is attention over each whole sequence. The third
    case rotates only part of each head and has a width that is no multiple of 64; the last two have
    value heads of another size than the keys' (the cache's value rows are then narrower or wider than
    its key rows: a group of its own in the manager, the plain kernels on the device), also in bf16."""
    rng = np.random.default_rng(H * D)
    E, theta = 56, 5e4
    spec = PartSpec("attention", dict(hidden_size=E, n_heads=H, n_kv_heads=G, head_dim=D, qkv_bias=True,
                                      window=window, prefix="a.", **({} if Dv is None else {"v_head_dim": Dv}),
                                      position=PartSpec("rotary", dict(head_dim=D, rot_dim=rot, theta=theta))))
    part = make_part("mixer", spec)
    assert part.cache_need() == PagedKV(G * D, G * (Dv or D), window)
    p = {s.name: (rng.standard_normal(s.shape) * (0.3 if s.kind == "vector" else 1.2 / math.sqrt(s.shape[1])))
         .astype(np.float32) for s in part.all_param_specs()}
    bind(part, p, ops32)
    p64 = {k: v.astype(np.float64) for k, v in p.items()}
    hs = {r: rng.standard_normal((n, E)).astype(np.float32) for r, n in (("a", 21), ("b", 13))}
    want = {r: attention_reference(p64, "a.", h.astype(np.float64), range(len(h)), H, G, D, theta, window, rot, Dv)
            for r, h in hs.items()}
    har = Harness(ops32, [part.cache_need()])
    cuts = [[("a", 0, 9)], [("a", 9, 19), ("b", 0, 12)], [("a", 19, 20), ("b", 12, 13)], [("a", 20, 21)]]
    for cut in cuts:
        step = har.inputs([(r, [0] * (e - s)) for r, s, e in cut])
        h = np.concatenate([hs[r][s:e] for r, s, e in cut])
        x = torch.zeros((h.shape[0], E), device="cuda")
        part.forward(ops32, step, dev(h), har.views[0], x)
        ref = np.concatenate([want[r][s:e] for r, s, e in cut])
        err = np.max(np.abs(x.cpu().numpy() - ref))
        assert err < 5e-5, f"cut {cut}: {err:.3e}"
    if Dv is None:
        return
    part16 = make_part("mixer", spec)
    part16.bind_all({k: dev(v, torch.float32 if v.ndim == 1 else torch.bfloat16) for k, v in p.items()}, ops16)
    r64 = {k: (helpers.bf16_round(v).astype(np.float64) if v.ndim == 2 else v.astype(np.float64)) for k, v in p.items()}
    har = Harness(ops16, [part16.cache_need()])
    for cut in cuts:
        step = har.inputs([(r, [0] * (e - s)) for r, s, e in cut])
        h = helpers.bf16_round(np.concatenate([hs[r][s:e] for r, s, e in cut]))
        x = torch.zeros((h.shape[0], E), device="cuda")
        part16.forward(ops16, step, dev(h, torch.bfloat16), har.views[0], x)
        ops16.settle()
        whole = {r: attention_reference(r64, "a.", helpers.bf16_round(hh).astype(np.float64), range(len(hh)), H, G, D, theta, window, rot, Dv)
                 for r, hh in hs.items()}
        ref = np.concatenate([whole[r][s:e] for r, s, e in cut])
        err = np.max(np.abs(x.cpu().numpy() - ref)) / np.max(np.abs(ref))
        assert err < 2e-2, f"bf16, cut {cut}: {err:.3e}"


def toy_plan_factory():
    """Registers a toy mixer that keeps a running average per request in a state slot, and an
    architecture whose layers differ: attention + gated mlp, then the toy mixer + gated mlp,
    with a schedule that runs layer 0 twice and lets the second run of it read the first
    run's cache. Nothing in the package is edited for this."""

    @register_part("mixer", "toy_ema")
    class ToyEma(Part):
        """s <- decay * s + (1 - decay) * h_t per request, in token order; x_t += W s."""

        def __init__(self, hidden_size, decay, prefix=""):
            super().__init__(prefix)
            self.E, self.decay = hidden_size, decay

        def param_specs(self):
            return [ParamSpec(self.prefix + "mix.weight", (self.E, self.E), "matrix", ("normal", 0.2))]

        def cache_need(self):
            return FixedState(self.E)

        def bind(self, params, ops):
            self.w = params[self.prefix + "mix.weight"]

        def forward(self, ops, step, h, cache, x, write_cache=True):
            q_start = step.host["q_start"]
            for s in range(step.n_seqs):
                slot = int(step.host["seq_slot"][s])
                state = cache.state[slot]
                for t in range(int(q_start[s]), int(q_start[s + 1])):
                    state.mul_(self.decay).add_(h[t].float(), alpha=1 - self.decay)
                    x[t] += self.w.float() @ state

    @register_part("mixer", "toy_ema_kernel")
    class ToyEmaKernel(ToyEma):
        """The same mixer with a kernel of its own, from a library that is not the package's
        (tests/toy_kernels/toy_ema.hip): the step's shape is all the host looks at, so steps that use it
        may be captured into graphs."""
        graph_safe = True
        _lib = None

        @classmethod
        def lib(cls):
            if cls._lib is None:
                from ctypes import c_float, c_int, c_void_p as P
                from hf_cpu_amd.kernels import load_extension
                from hf_cpu_amd.kernels.build import build_extension
                here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "toy_kernels")
                path = os.path.join(here, "libtoy.so")
                if not os.path.exists(path):
                    build_extension([os.path.join(here, "toy_ema.hip")], path)
                cls._lib = load_extension(path, {"toy_ema": [P, c_int, P, P, c_int, P, P, P, c_int, c_int, c_float, P]})
            return cls._lib

        def forward(self, ops, step, h, cache, x, write_cache=True):
            code = {torch.float32: 0, torch.bfloat16: 1}
            ops.call(self.lib().toy_ema, h.data_ptr(), code[h.dtype], cache.state.data_ptr(), self.w.data_ptr(),
                     code[self.w.dtype], x.data_ptr(), step.q_start.data_ptr(), step.seq_slot.data_ptr(), step.n_seqs,
                     self.E, self.decay, what="toy_ema")

    @dataclasses.dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        vocab_size: int
        hidden_size: int
        decay: float
        mixer_kind: str = "toy_ema"

        @classmethod
        def from_dict(cls, obj, origin="config.json"):
            return cls(obj["architectures"][0], obj["vocab_size"], obj["hidden_size"], obj["decay"],
                       obj.get("mixer_kind", "toy_ema"))

    def toy_plan(cfg):
        E = cfg.hidden_size

        def layer(l, mixer):
            pre = f"layers.{l}."
            return hf_cpu_amd.LayerPlan.of(
                pre, PartSpec("prenorm", dict(hidden_size=E)),
                norm1=PartSpec("rmsnorm", dict(size=E, eps=1e-5, prefix=pre + "norm1.")), mixer=mixer,
                norm2=PartSpec("rmsnorm", dict(size=E, eps=1e-5, prefix=pre + "norm2.")),
                feed_forward=PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=2 * E, prefix=pre + "mlp.")))
        att = PartSpec("attention", dict(hidden_size=E, n_heads=2, n_kv_heads=1, head_dim=16, qkv_bias=False,
                                         window=0, prefix="layers.0.attn.",
                                         position=PartSpec("rotary", dict(head_dim=16, rot_dim=16, theta=1e4))))
        toy = PartSpec(cfg.mixer_kind, dict(hidden_size=E, decay=cfg.decay, prefix="layers.1.ema."))
        return hf_cpu_amd.ModelPlan(
            hidden_size=E, vocab_size=cfg.vocab_size,
            embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab_size, hidden_size=E, prefix="embed.")),
            layers=(layer(0, att), layer(1, toy)),
            schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0)),
            final_norm=PartSpec("rmsnorm", dict(size=E, eps=1e-5, prefix="final.")),
            head=PartSpec("linear", dict(vocab_size=cfg.vocab_size, hidden_size=E, tied=True,
                                         tied_to="embed.weight", prefix="head.")))
    register_architecture("ToyEmaForCausalLM", ToyConfig, toy_plan)
    return ToyConfig


def toy_reference(w, toks, decay):
    """The toy model over a whole sequence, written out directly."""
    E = w["embed.weight"].shape[1]
    T = len(toks)
    x = w["embed.weight"][toks]

    def mlp(x, pre):
        return plain.swiglu_mlp(plain.rmsnorm(x, w[pre + "norm2.weight"], 1e-5), w[pre + "mlp.gate_proj.weight"],
                                w[pre + "mlp.up_proj.weight"], w[pre + "mlp.down_proj.weight"])

    def attn(x, own_kv=None):
        h = plain.rmsnorm(x, w["layers.0.norm1.weight"], 1e-5)
        q = plain.rope(plain.linear(h, w["layers.0.attn.q_proj.weight"]).reshape(T, 2, 16), range(T), 16, 1e4)
        if own_kv is None:
            k = plain.rope(plain.linear(h, w["layers.0.attn.k_proj.weight"]).reshape(T, 1, 16), range(T), 16, 1e4)
            v = plain.linear(h, w["layers.0.attn.v_proj.weight"]).reshape(T, 1, 16)
        else:
            k, v = own_kv
        out = plain.linear(plain.attention(q, k, v).reshape(T, 32), w["layers.0.attn.o_proj.weight"])
        return out, (k, v)
    a, kv = attn(x)
    x = x + a
    x = x + mlp(x, "layers.0.")
    h = plain.rmsnorm(x, w["layers.1.norm1.weight"], 1e-5)
    s = np.zeros(E)
    outs = []
    for t in range(T):
        s = decay * s + (1 - decay) * h[t]
        outs.append(w["layers.1.ema.mix.weight"] @ s)
    x = x + np.array(outs)
    x = x + mlp(x, "layers.1.")
    a, _ = attn(x, own_kv=kv)                     # layer 0 again, reading the cache of its first run
    x = x + a
    x = x + mlp(x, "layers.0.")
    return plain.linear(plain.rmsnorm(x, w["final.weight"], 1e-5), w["embed.weight"])


def make_toy_model(tmp_path, mixer_kind="toy_ema"):
    toy_plan_factory()
    cfg = {"architectures": ["ToyEmaForCausalLM"], "vocab_size": 90, "hidden_size": 24, "decay": 0.8,
           "mixer_kind": mixer_kind}
    d = str(tmp_path / ("toy_" + mixer_kind))
    os.makedirs(d)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    model = hf_cpu_amd.Model.from_config(hf_cpu_amd.config_from_dict(cfg))
    assert [type(n).__name__ for n in model.cache_needs()] == ["PagedKV", "FixedState", "NoneType"]
    rng = np.random.default_rng(3)
    w = {}
    for s in model.param_specs():
        if s.optional:
            continue
        std = {"embed.weight": 0.5}.get(s.name, 0.3 if s.kind == "matrix" else 0.1)
        w[s.name] = ((1.0 if s.kind == "vector" else 0.0) + rng.standard_normal(s.shape) * std).astype(np.float32)
    helpers.write_safetensors(os.path.join(d, "model.safetensors"), w)
    return d, w, rng


@pytest.mark.parametrize("mixer_kind", ["toy_ema", "toy_ema_kernel"])
def test_toy_mixer_with_state_and_a_schedule_that_repeats(gpu, tmp_path, mixer_kind):
    """The toy mixer in eager tensor arithmetic, and the same with a kernel of its own that the test
    brings in a library of its own (no file of the package knows either)."""
    d, w, rng = make_toy_model(tmp_path, mixer_kind)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 90, n)] for i, n in enumerate([5, 23, 40, 31])}
    w64 = {k: v.astype(np.float64) for k, v in w.items()}
    want = {r: toy_reference(w64, t, 0.8) for r, t in reqs.items()}
    for steps in (helpers.trace_whole(reqs), helpers.trace_portions(reqs), helpers.trace_mixed(reqs, seed=2, max_live=3)):
        engine = hf_cpu_amd.load_engine(d, dtype="float32", page_tokens=8, max_tokens=helpers.max_live_tokens(steps),
                                        max_seqs=3)
        got = helpers.run_trace_in_engine(engine, steps)
        helpers.compare(got, want, 2e-5, "toy model")
        assert not engine.manager.held


def test_toy_mixer_with_a_kernel_of_its_own_replays_from_graphs(gpu, tmp_path):
    """The toy mixer's own kernel declares itself safe to capture: decode steps of a model that holds
    it are replayed from graphs, and give what the model written out directly gives."""
    d, w, rng = make_toy_model(tmp_path, "toy_ema_kernel")
    w64 = {k: v.astype(np.float64) for k, v in w.items()}
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 90, 30)] for i in range(3)}
    want = {r: toy_reference(w64, t, 0.8) for r, t in reqs.items()}
    engine = hf_cpu_amd.load_engine(d, dtype="float32", page_tokens=8, max_tokens=192, max_seqs=3)
    assert engine.use_graphs
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:6], "want": [5]} for r, t in reqs.items()], "end": []}]
    for i in range(6, 30):
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": [t[i]], "want": [0]} for r, t in reqs.items()],
                      "end": list(reqs) if i == 29 else []})
    got = helpers.run_trace_in_engine(engine, steps)
    helpers.compare(got, want, 2e-5, "toy model, decode steps from graphs")
    assert engine.graph_replays >= 20


def toy_greedy(w64, prompt, n, decay=0.8):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(toy_reference(w64, toks, decay)[-1])))
    return toks[len(prompt):]


def test_toy_mixer_through_the_scheduler_with_forks_and_a_tight_cache(gpu, tmp_path):
    """A model with per-request state of fixed size served by the scheduler: continuations forked from
    one prompt take a copy of its state; a cache too small for everybody throws requests out, whose
    state starts from zero again when they come back. Every sequence ends with the tokens that the
    model written out directly gives it."""
    import hf_cpu_amd.session as S
    d, w, rng = make_toy_model(tmp_path, "toy_ema_kernel")
    w64 = {k: v.astype(np.float64) for k, v in w.items()}
    prompts = [[int(t) for t in rng.integers(0, 90, n)] for n in (9, 17, 5, 12)]
    want = [toy_greedy(w64, p, 14) for p in prompts]
    s = S.Session(d, dtype="float32", ctx_max=48, batch=8, page_size=4, max_seqs=4, kv_tokens=72)
    gens = s.generate(prompts, n=2, temp=0.0, max_tokens=14)
    assert len(gens) == 8 and all(g.error is None and g.stop == "length" for g in gens)
    for i, g in enumerate(gens):
        assert g.tokens == want[i // 2], f"sequence {i} (prompt {i // 2}): {g.tokens} != {want[i // 2]}"
    assert sum(g.preemptions for g in gens) > 0, "the cache was meant to be too small for everybody"
    s.engine.manager.check()
    assert not s.engine.manager.held


def blocks_plan_factory():
    """Registers three toy arrangements of a layer, none of which is the package's: one with four norms
    (a norm before and after each branch), one whose mixer and feed-forward read the same normed input
    and are added together, and one that has a mixer and nothing else. The layer plan names the parts
    each needs; the package's model passes them through as a mapping."""

    @register_part("block", "toy_four_norms")
    class FourNorms(Part):
        def __init__(self, hidden_size, prefix=""):
            super().__init__(prefix)
            self.E = hidden_size

        def branch(self, ops, x, pre, post, run):
            h = torch.empty((x.shape[0], self.E), dtype=ops.act_dtype, device=x.device)
            pre.forward(ops, x, h)
            y = torch.zeros_like(x)
            run(h, y)
            ops.settle(y)
            out = torch.empty_like(h)
            post.forward(ops, y, out)
            x += out.float()

        def forward(self, ops, step, x, parts, caches, write_cache=True):
            ops.settle(x)
            self.branch(ops, x, parts["norm_in"], parts["norm_mixed"],
                        lambda h, y: parts["mixer"].forward(ops, step, h, caches.get("mixer"), y, write_cache))
            self.branch(ops, x, parts["norm_mid"], parts["norm_out"],
                        lambda h, y: parts["feed_forward"].forward(ops, step, h, y))

    @register_part("block", "toy_parallel")
    class Parallel(Part):
        def __init__(self, hidden_size, prefix=""):
            super().__init__(prefix)
            self.E = hidden_size

        def forward(self, ops, step, x, parts, caches, write_cache=True):
            h = torch.empty((x.shape[0], self.E), dtype=ops.act_dtype, device=x.device)
            parts["norm"].forward(ops, x, h)
            ops.settle(x)
            parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)
            parts["feed_forward"].forward(ops, step, h, x)            # the same input: both branches start at one norm

    @register_part("block", "toy_mixer_only")
    class MixerOnly(Part):
        def __init__(self, hidden_size, prefix=""):
            super().__init__(prefix)
            self.E = hidden_size

        def forward(self, ops, step, x, parts, caches, write_cache=True):
            h = torch.empty((x.shape[0], self.E), dtype=ops.act_dtype, device=x.device)
            parts["norm"].forward(ops, x, h)
            ops.settle(x)
            parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)

    @dataclasses.dataclass(frozen=True)
    class BlocksConfig:
        architecture: str
        vocab_size: int
        hidden_size: int

        @classmethod
        def from_dict(cls, obj, origin="config.json"):
            return cls(obj["architectures"][0], obj["vocab_size"], obj["hidden_size"])

    def blocks_plan(cfg):
        E = cfg.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", dict(size=E, eps=1e-5, prefix=name + "."))

        def attention(l, window=0):
            return PartSpec("attention", dict(hidden_size=E, n_heads=2, n_kv_heads=2, head_dim=16, qkv_bias=False,
                                              window=window, prefix=f"layers.{l}.attn.",
                                              position=PartSpec("rotary", dict(head_dim=16, rot_dim=16, theta=1e4))))

        def mlp(l):
            return PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=2 * E, prefix=f"layers.{l}.mlp."))
        layers = (
            hf_cpu_amd.LayerPlan.of("layers.0.", PartSpec("toy_four_norms", dict(hidden_size=E)),
                                    norm_in=norm("layers.0.n0"), mixer=attention(0), norm_mixed=norm("layers.0.n1"),
                                    norm_mid=norm("layers.0.n2"), feed_forward=mlp(0), norm_out=norm("layers.0.n3")),
            hf_cpu_amd.LayerPlan.of("layers.1.", PartSpec("toy_parallel", dict(hidden_size=E)),
                                    norm=norm("layers.1.n0"), mixer=attention(1, window=7), feed_forward=mlp(1)),
            hf_cpu_amd.LayerPlan.of("layers.2.", PartSpec("toy_mixer_only", dict(hidden_size=E)),
                                    norm=norm("layers.2.n0"), mixer=attention(2)),
        )
        return hf_cpu_amd.ModelPlan(
            hidden_size=E, vocab_size=cfg.vocab_size,
            embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab_size, hidden_size=E, prefix="embed.")),
            layers=layers, schedule=tuple(ScheduleEntry(l) for l in range(3)),
            final_norm=norm("final"),
            head=PartSpec("linear", dict(vocab_size=cfg.vocab_size, hidden_size=E, tied=True, tied_to="embed.weight",
                                         prefix="head.")))
    register_architecture("ToyBlocksForCausalLM", BlocksConfig, blocks_plan)


def blocks_reference(w, toks):
    """The model of blocks_plan_factory over a whole sequence, written out directly (float64)."""
    T = len(toks)
    x = w["embed.weight"][toks]

    def norm(x, name):
        return plain.rmsnorm(x, w[name + ".weight"], 1e-5)

    def attn(h, l, window=0):
        pre = f"layers.{l}.attn."
        q = plain.rope(plain.linear(h, w[pre + "q_proj.weight"]).reshape(T, 2, 16), range(T), 16, 1e4)
        k = plain.rope(plain.linear(h, w[pre + "k_proj.weight"]).reshape(T, 2, 16), range(T), 16, 1e4)
        v = plain.linear(h, w[pre + "v_proj.weight"]).reshape(T, 2, 16)
        return plain.linear(plain.attention(q, k, v, window).reshape(T, 32), w[pre + "o_proj.weight"])

    def mlp(h, l):
        pre = f"layers.{l}.mlp."
        return plain.swiglu_mlp(h, w[pre + "gate_proj.weight"], w[pre + "up_proj.weight"], w[pre + "down_proj.weight"])
    x = x + norm(attn(norm(x, "layers.0.n0"), 0), "layers.0.n1")
    x = x + norm(mlp(norm(x, "layers.0.n2"), 0), "layers.0.n3")
    h = norm(x, "layers.1.n0")
    x = x + attn(h, 1, window=7) + mlp(h, 1)
    x = x + attn(norm(x, "layers.2.n0"), 2)
    return plain.linear(norm(x, "final"), w["embed.weight"])


def test_toy_blocks_with_four_norms_with_parallel_branches_and_without_a_feed_forward(gpu, tmp_path):
    """Layers that are not 'norm, mixer, norm, feed-forward': the plan names each layer's parts, the
    block gets them as a mapping. Whole, in portions and mixed, against the model written out."""
    blocks_plan_factory()
    cfg = {"architectures": ["ToyBlocksForCausalLM"], "vocab_size": 80, "hidden_size": 24}
    d = str(tmp_path / "blocks")
    os.makedirs(d)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    model = hf_cpu_amd.Model.from_config(hf_cpu_amd.config_from_dict(cfg))
    assert sorted(model.layers[0].named) == ["feed_forward", "mixer", "norm_in", "norm_mid", "norm_mixed", "norm_out"]
    assert sorted(model.layers[2].named) == ["mixer", "norm"]
    needs = model.cache_needs()
    assert [n.window for n in needs] == [0, 7, 0] and model.cache_slots == [{"mixer": 0}, {"mixer": 1}, {"mixer": 2}]
    rng = np.random.default_rng(9)
    w = {}
    for s in model.param_specs():
        if s.optional:
            continue
        std = {"embed.weight": 0.5}.get(s.name, 0.3 if s.kind == "matrix" else 0.1)
        w[s.name] = ((1.0 if s.kind == "vector" else 0.0) + rng.standard_normal(s.shape) * std).astype(np.float32)
    helpers.write_safetensors(os.path.join(d, "model.safetensors"), w)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 80, n)] for i, n in enumerate([4, 21, 38, 30])}
    w64 = {k: v.astype(np.float64) for k, v in w.items()}
    want = {r: blocks_reference(w64, t) for r, t in reqs.items()}
    for steps in (helpers.trace_whole(reqs), helpers.trace_portions(reqs), helpers.trace_mixed(reqs, seed=6, max_live=3)):
        engine = hf_cpu_amd.load_engine(d, dtype="float32", page_tokens=8, max_tokens=helpers.max_live_tokens(steps),
                                        max_seqs=3)
        got = helpers.run_trace_in_engine(engine, steps)
        helpers.compare(got, want, 2e-5, "toy blocks")
        assert not engine.manager.held


def routed_plan_factory():
    """Registers a toy feed-forward with routing (top-1 of four experts, the router in fp32), two toy
    position encodings (a learned vector per position added to queries and keys; a slope per head times the
    distance added to the scores) and an
    architecture that uses them in some layers and the package's parts in others. Nothing in
    the package is edited for this; the toy parts use the package's products and cache store
    and plain tensor arithmetic for the rest."""

    @register_part("position", "toy_learned")
    class ToyLearned(Part):
        """q_t += table[pos_t], k_t += table[pos_t] for every head; values as they are."""

        def __init__(self, head_dim, max_positions, prefix=""):
            super().__init__(prefix)
            self.head_dim, self.n = head_dim, max_positions

        def param_specs(self):
            return [ParamSpec(self.prefix + "pos.weight", (self.n, self.head_dim), "matrix", ("normal", 0.5))]

        def bind(self, params, ops):
            self.table = params[self.prefix + "pos.weight"]

        def store(self, ops, step, qkv, n_heads, n_kv_heads, cache, write):
            ops.settle()                                       # the product before may have left partial sums
            add = self.table[step.positions.long()].to(qkv.dtype)
            for h in range(n_heads + n_kv_heads):              # queries, then keys
                qkv[:, h * self.head_dim:(h + 1) * self.head_dim] += add
            if write:
                ops.rope_store(qkv, step.positions, None, 0, n_heads, n_kv_heads, self.head_dim, cache,
                               step.group(cache.group).slot_map)

    @register_part("position", "toy_slopes")
    class ToySlopes(Part):
        """Queries and keys as they are; the score of key j for the query at p gets slope_h * (j - p) added: an
        encoding that enters the scores, through the attention part's ``score_slopes`` hook."""

        def __init__(self, head_dim, slopes, prefix=""):
            super().__init__(prefix)
            self.head_dim, self.slopes = head_dim, tuple(slopes)

        def bind(self, params, ops):
            self.score_slopes = hf_cpu_amd.memory.to_device(torch.tensor(self.slopes, dtype=torch.float32), ops.device,
                                                            "toy slopes")

        def store(self, ops, step, qkv, n_heads, n_kv_heads, cache, write):
            if write:
                ops.rope_store(qkv, step.positions, None, 0, n_heads, n_kv_heads, self.head_dim, cache,
                               step.group(cache.group).slot_map)

    @register_part("feed_forward", "toy_routed")
    class ToyRouted(Part):
        """x_t += p_e * down_e(relu(up_e(h_t))) with e = argmax of the router's logits and p_e its
        softmax probability, both in fp32."""

        def __init__(self, hidden_size, intermediate_size, n_experts, prefix=""):
            super().__init__(prefix)
            self.E, self.F, self.n = hidden_size, intermediate_size, n_experts

        def param_specs(self):
            out = [ParamSpec(self.prefix + "router.weight", (self.n, self.E), "matrix", ("normal", 0.5))]
            for e in range(self.n):
                out.append(ParamSpec(f"{self.prefix}experts.{e}.up.weight", (self.F, self.E), "matrix", ("normal", 0.3)))
                out.append(ParamSpec(f"{self.prefix}experts.{e}.down.weight", (self.E, self.F), "matrix", ("normal", 0.3)))
            return out

        def bind(self, params, ops):
            self.router = params[self.prefix + "router.weight"]
            self.up = [params[f"{self.prefix}experts.{e}.up.weight"] for e in range(self.n)]
            self.down = [params[f"{self.prefix}experts.{e}.down.weight"] for e in range(self.n)]

        def forward(self, ops, step, h, x):
            T = h.shape[0]
            logits = torch.empty((T, self.n), dtype=torch.float32, device=h.device)
            ops.gemm(h, self.router, logits)
            ops.settle()
            prob, expert = torch.softmax(logits, dim=1).max(dim=1)
            for e in range(self.n):
                rows = torch.nonzero(expert == e).flatten()
                if rows.numel() == 0:
                    continue
                he = h.index_select(0, rows).contiguous()
                mid = torch.empty((rows.numel(), self.F), dtype=h.dtype, device=h.device)
                ops.gemm(he, self.up[e], mid)
                out = torch.empty((rows.numel(), self.E), dtype=torch.float32, device=h.device)
                ops.gemm(torch.relu(mid), self.down[e], out)
                ops.settle()
                x.index_add_(0, rows, out * prob[rows, None])

    @dataclasses.dataclass(frozen=True)
    class RoutedConfig:
        architecture: str
        vocab_size: int
        hidden_size: int
        n_experts: int
        max_positions: int

        @classmethod
        def from_dict(cls, obj, origin="config.json"):
            return cls(obj["architectures"][0], obj["vocab_size"], obj["hidden_size"], obj["n_experts"],
                       obj["max_positions"])

    def routed_plan(cfg):
        E = cfg.hidden_size

        def attention(l, position, window):
            return PartSpec("attention", dict(hidden_size=E, n_heads=3, n_kv_heads=1, head_dim=16, qkv_bias=True,
                                              window=window, prefix=f"layers.{l}.attn.", position=position))

        def layer(l, mixer, ffn):
            pre = f"layers.{l}."
            return hf_cpu_amd.LayerPlan.of(
                pre, PartSpec("prenorm", dict(hidden_size=E)),
                norm1=PartSpec("rmsnorm", dict(size=E, eps=1e-6, prefix=pre + "norm1.")), mixer=mixer,
                norm2=PartSpec("rmsnorm", dict(size=E, eps=1e-6, prefix=pre + "norm2.")), feed_forward=ffn)
        learned = PartSpec("toy_learned", dict(head_dim=16, max_positions=cfg.max_positions, prefix="layers.0.attn."))
        rotary = PartSpec("rotary", dict(head_dim=16, rot_dim=8, theta=100.0))
        slopes = PartSpec("toy_slopes", dict(head_dim=16, slopes=TOY_SLOPES))
        dense = PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=40, prefix="layers.0.mlp."))
        dense2 = PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=24, prefix="layers.2.mlp."))
        routed = PartSpec("toy_routed", dict(hidden_size=E, intermediate_size=24, n_experts=cfg.n_experts,
                                             prefix="layers.1.moe."))
        return hf_cpu_amd.ModelPlan(
            hidden_size=E, vocab_size=cfg.vocab_size,
            embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab_size, hidden_size=E, prefix="embed.")),
            layers=(layer(0, attention(0, learned, 0), dense), layer(1, attention(1, rotary, 9), routed),
                    layer(2, attention(2, slopes, 0), dense2)),
            schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)),
            final_norm=PartSpec("rmsnorm", dict(size=E, eps=1e-6, prefix="final.")),
            head=PartSpec("linear", dict(vocab_size=cfg.vocab_size, hidden_size=E, tied=False, prefix="head.")))
    register_architecture("ToyRoutedForCausalLM", RoutedConfig, routed_plan)


TOY_SLOPES = (0.5, 0.125, 0.03125)


def routed_reference(w, toks, n_experts):
    """The toy model over a whole sequence, written out directly (float64)."""
    T = len(toks)
    x = w["embed.weight"][toks]

    def attn(x, l, window):
        pre = f"layers.{l}.attn."
        h = plain.rmsnorm(x, w[f"layers.{l}.norm1.weight"], 1e-6)
        q = plain.linear(h, w[pre + "q_proj.weight"], w[pre + "q_proj.bias"]).reshape(T, 3, 16)
        k = plain.linear(h, w[pre + "k_proj.weight"], w[pre + "k_proj.bias"]).reshape(T, 1, 16)
        v = plain.linear(h, w[pre + "v_proj.weight"], w[pre + "v_proj.bias"]).reshape(T, 1, 16)
        if l == 0:
            q = q + w[pre + "pos.weight"][:T, None, :]
            k = k + w[pre + "pos.weight"][:T, None, :]
        elif l == 1:
            q, k = plain.rope(q, range(T), 8, 100.0), plain.rope(k, range(T), 8, 100.0)
        else:                                                  # scores with slope_h * (j - p), written out
            att = np.empty_like(q)
            dist = np.arange(T)[None, :] - np.arange(T)[:, None]
            for h in range(3):
                sc = (q[:, h, :] @ k[:, 0, :].T) / 4.0 + TOY_SLOPES[h] * dist
                att[:, h, :] = plain.softmax(np.where(dist <= 0, sc, -np.inf)) @ v[:, 0, :]
            return plain.linear(att.reshape(T, 48), w[pre + "o_proj.weight"])
        return plain.linear(plain.attention(q, k, v, window).reshape(T, 48), w[pre + "o_proj.weight"])
    x = x + attn(x, 0, 0)
    x = x + plain.swiglu_mlp(plain.rmsnorm(x, w["layers.0.norm2.weight"], 1e-6), w["layers.0.mlp.gate_proj.weight"],
                             w["layers.0.mlp.up_proj.weight"], w["layers.0.mlp.down_proj.weight"])
    x = x + attn(x, 1, 9)
    h = plain.rmsnorm(x, w["layers.1.norm2.weight"], 1e-6)
    logits = h @ w["layers.1.moe.router.weight"].T
    prob = plain.softmax(logits)
    used = set()
    for t in range(T):
        e = int(np.argmax(logits[t]))
        used.add(e)
        mid = np.maximum(w[f"layers.1.moe.experts.{e}.up.weight"] @ h[t], 0.0)
        x[t] = x[t] + prob[t, e] * (w[f"layers.1.moe.experts.{e}.down.weight"] @ mid)
    x = x + attn(x, 2, 0)
    x = x + plain.swiglu_mlp(plain.rmsnorm(x, w["layers.2.norm2.weight"], 1e-6), w["layers.2.mlp.gate_proj.weight"],
                             w["layers.2.mlp.up_proj.weight"], w["layers.2.mlp.down_proj.weight"])
    out = plain.linear(plain.rmsnorm(x, w["final.weight"], 1e-6), w["head.weight"])
    return out, used


def test_toy_routed_feed_forward_and_toy_position_encoding(gpu, tmp_path):
    """Another feed-forward (with routing) and two other position encodings (one added to queries and
    keys, one that enters the scores), registered from here, in a model whose three layers differ in
    position encoding, window and feed-forward: whole, in portions and mixed with few pages, against the
    model written out directly."""
    routed_plan_factory()
    cfg = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 70, "hidden_size": 20, "n_experts": 4,
           "max_positions": 64}
    d = str(tmp_path / "routed")
    os.makedirs(d)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    model = hf_cpu_amd.Model.from_config(hf_cpu_amd.config_from_dict(cfg))
    needs = model.cache_needs()
    assert [type(n).__name__ for n in needs] == ["PagedKV"] * 3 and [n.window for n in needs] == [0, 9, 0]
    names = {s.name for s in model.param_specs()}
    assert "layers.1.moe.experts.3.down.weight" in names and "layers.0.attn.pos.weight" in names
    rng = np.random.default_rng(5)
    w = {}
    for s in model.param_specs():
        if s.optional:
            continue
        std = {"embed.weight": 0.5, "layers.1.moe.router.weight": 1.0}.get(s.name, 0.3 if s.kind == "matrix" else 0.1)
        w[s.name] = ((1.0 if s.kind == "vector" and s.name.endswith("norm1.weight") or s.name.endswith("norm2.weight")
                      or s.name == "final.weight" else 0.0) + rng.standard_normal(s.shape) * std).astype(np.float32)
    helpers.write_safetensors(os.path.join(d, "model.safetensors"), w)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 70, n)] for i, n in enumerate([6, 25, 44, 33])}
    w64 = {k: v.astype(np.float64) for k, v in w.items()}
    want, used = {}, set()
    for r, t in reqs.items():
        want[r], u = routed_reference(w64, t, 4)
        used |= u
    assert len(used) >= 3, "the inputs were meant to reach most experts"
    for steps in (helpers.trace_whole(reqs), helpers.trace_portions(reqs), helpers.trace_mixed(reqs, seed=4, max_live=3)):
        engine = hf_cpu_amd.load_engine(d, dtype="float32", page_tokens=4, max_tokens=helpers.max_live_tokens(steps),
                                        max_seqs=3)
        got = helpers.run_trace_in_engine(engine, steps)
        helpers.compare(got, want, 2e-5, "toy routed model")
        assert not engine.manager.held
