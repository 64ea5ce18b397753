"""The typed configuration of the Qwen2 dense architecture.

Every size and constant of the model comes from here, and every field comes from
a key of config.json. The quantities are the ones the reference reads from GGUF
metadata in ``hfc_model_load`` (src/model.c:119-139) and checks in
src/model.c:141-145; the sliding-window keys have no counterpart there.
"""
from dataclasses import dataclass, asdict

from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader


@dataclass(frozen=True)
class Qwen2Config:
    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    use_sliding_window: bool
    sliding_window: int          # 0 when no layer is windowed
    max_window_layers: int
    hidden_act: str
    eos_token_ids: tuple
    torch_dtype: str

    # ---- derived -------------------------------------------------------
    @property
    def q_size(self):
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_key_value_heads * self.head_dim

    def layer_window(self, layer):
        """The window of a layer in tokens, or 0 if it attends to every earlier
        token. Layer ``l`` is windowed iff ``use_sliding_window`` and
        ``l >= max_window_layers``; a key is then visible iff
        ``0 <= pos_q - pos_k < sliding_window``."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return 0

    def to_dict(self):
        """The config.json content that reads back as this configuration."""
        d = asdict(self)
        d["architectures"] = [d.pop("architecture")]
        d["model_type"] = "qwen2"
        eos = d.pop("eos_token_ids")
        if eos:
            d["eos_token_id"] = list(eos) if len(eos) > 1 else eos[0]
        if not self.use_sliding_window:
            d["sliding_window"] = None
        return d

    # ---- model options of a session ---------------------------------------
    @classmethod
    def apply_options(cls, obj, options):
        """``obj`` (config.json's object) with the options a session gives in the engine's own words.
        ``window`` = N replaces the file's window for the layers that may have one
        (``use_sliding_window``, ``sliding_window``); 0 turns it off."""
        obj = dict(obj)
        for name, value in options.items():
            if name == "window":
                obj["use_sliding_window"] = int(value) > 0
                if int(value) > 0:
                    obj["sliding_window"] = int(value)
                    obj.pop("layer_types", None)     # spelled from max_window_layers again when read
            else:
                fail(ENOTSUP, f"architecture '{(obj.get('architectures') or ['?'])[0]}' has no model option '{name}'")
        return obj

    # ---- reading -------------------------------------------------------
    @classmethod
    def from_dict(cls, obj, origin="config.json"):
        r = KeyReader(obj, origin)
        arch = r.str_list("architectures")
        if len(arch) != 1:
            fail(EFORMAT, f"{origin}: key 'architectures' must name exactly one architecture")
        L = r.integer("num_hidden_layers")
        E = r.integer("hidden_size")
        F = r.integer("intermediate_size")
        H = r.integer("num_attention_heads")
        G = r.integer("num_key_value_heads", default=H, hi=10 ** 5)     # src/model.c:126-127
        D = r.integer("head_dim", default=E // H)                       # src/model.c:130-131
        V = r.integer("vocab_size", hi=1 << 24)                          # src/model.c:148-153
        eps = r.number("rms_norm_eps", lo=0.0, hi=1.0)                   # src/model.c:134-136
        if r.has("rope_theta"):
            theta = r.number("rope_theta", lo=0.0, hi=1e12)              # src/model.c:137-139
            scaling = obj.get("rope_scaling")
        else:
            rp = KeyReader(obj.get("rope_parameters") or {}, origin + ":rope_parameters")
            theta = rp.number("rope_theta", lo=0.0, hi=1e12)
            scaling = rp.obj
        if scaling:
            kind = scaling.get("rope_type", scaling.get("type", "default"))
            if kind != "default":
                fail(ENOTSUP, f"{origin}: rope scaling of type '{kind}' is not supported")
        act = r.string("hidden_act", default="silu")
        if act != "silu":
            fail(ENOTSUP, f"{origin}: hidden_act '{act}' is not supported (only 'silu')")
        use_win = r.boolean("use_sliding_window", default=False)
        mwl = r.integer("max_window_layers", default=L, lo=0)
        win = r.integer("sliding_window", default=0, lo=1, hi=1 << 30) if use_win else 0
        if use_win and r.has("layer_types"):
            kinds = r.str_list("layer_types")
            want = tuple("sliding_attention" if l >= mwl else "full_attention" for l in range(L))
            if kinds != want:
                fail(ENOTSUP, f"{origin}: 'layer_types' does not follow 'max_window_layers' ({mwl})")
        cfg = cls(
            architecture=arch[0], vocab_size=V, hidden_size=E, intermediate_size=F,
            num_hidden_layers=L, num_attention_heads=H, num_key_value_heads=G, head_dim=D,
            rms_norm_eps=eps, rope_theta=theta,
            max_position_embeddings=r.integer("max_position_embeddings", default=0, lo=0, hi=1 << 30),
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            use_sliding_window=use_win, sliding_window=win, max_window_layers=mwl,
            hidden_act=act,
            eos_token_ids=r.int_list("eos_token_id", default=()),
            torch_dtype=r.string("torch_dtype", default=r.string("dtype", default="bfloat16")),
        )
        cfg.validate(origin)
        return cfg

    def validate(self, origin="config"):
        """Geometry checks of src/model.c:141-145, plus the window's."""
        H, G, D = self.num_attention_heads, self.num_key_value_heads, self.head_dim
        if H % G != 0:
            fail(EFORMAT, f"{origin}: num_attention_heads {H} is not a multiple of num_key_value_heads {G}")
        if D < 2 or D % 2 != 0:
            fail(EFORMAT, f"{origin}: head_dim {D} must be even and at least 2")
        if H * D > 1 << 20 or G * D > 1 << 20:
            fail(EFORMAT, f"{origin}: heads x head_dim is implausibly large")
        if self.use_sliding_window:
            if self.sliding_window <= 0:
                fail(EFORMAT, f"{origin}: use_sliding_window needs a positive sliding_window")
            if self.max_window_layers > self.num_hidden_layers:
                fail(EFORMAT, f"{origin}: max_window_layers {self.max_window_layers} exceeds "
                              f"num_hidden_layers {self.num_hidden_layers}")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab_size:
                fail(EFORMAT, f"{origin}: eos_token_id {e} is outside the vocabulary")
