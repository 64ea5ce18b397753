"""Softmax attention over a paged key/value cache, with grouped heads and an
optional window."""
import math

import torch

from .. import memory

from ..registry import make_part, register_part
from ..status import EINVAL, fail
from .base import PagedKV, ParamSpec, Part


@register_part("mixer", "attention")
class Attention(Part):
    """``q = Wq h + bq`` etc. (src/model.c:581-585); position encoding on q and k;
    for query head ``h`` the key/value head is ``h / (heads / kv_heads)``; scores
    ``dot(q, k) * scale`` over the visible keys, softmax in fp32, weighted sum of
    values (src/model.c:499-528); ``x += Wo att`` (src/model.c:606-609).

    A key at ``pk`` is visible to a query at ``pq`` iff ``0 <= pq - pk`` and, when
    ``window > 0``, ``pq - pk < window``.

    A position encoding that enters the scores instead of the queries and keys has an
    attribute ``score_slopes`` (fp32 on the device, one per query head): the score then is
    ``dot(q, k) * scale + score_slopes[h] * (pk - pq)``.
    """
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, hidden_size, n_heads, n_kv_heads, head_dim, qkv_bias, window, position,
                 scale=None, out_bias=False, v_head_dim=None, prefix=""):
        """``v_head_dim``: the size of a value head where it is not ``head_dim`` (key rows of the cache are
        then ``n_kv_heads * head_dim`` wide, value rows ``n_kv_heads * v_head_dim``, and the output
        projection reads ``n_heads * v_head_dim`` columns; such a mixer runs the plain kernels)."""
        super().__init__(prefix)
        if n_heads % n_kv_heads:
            fail(EINVAL, f"attention: {n_heads} heads are not a multiple of {n_kv_heads} key/value heads")
        self.E, self.H, self.G, self.D = hidden_size, n_heads, n_kv_heads, head_dim
        self.Dv = head_dim if v_head_dim is None else int(v_head_dim)
        self.QD, self.KD = n_heads * head_dim, n_kv_heads * head_dim
        self.VD, self.OD = n_kv_heads * self.Dv, n_heads * self.Dv
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # src/model.c:507
        self.position = make_part("position", position)
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    def sub_parts(self):
        return [self.position]

    def param_specs(self):
        p = self.prefix
        specs = [ParamSpec(p + "q_proj.weight", (self.QD, self.E)),
                 ParamSpec(p + "k_proj.weight", (self.KD, self.E)),
                 ParamSpec(p + "v_proj.weight", (self.VD, self.E)),
                 ParamSpec(p + "o_proj.weight", (self.E, self.OD))]
        if self.qkv_bias:
            specs += [ParamSpec(p + "q_proj.bias", (self.QD,), "vector"),
                      ParamSpec(p + "k_proj.bias", (self.KD,), "vector"),
                      ParamSpec(p + "v_proj.bias", (self.VD,), "vector")]
        if self.out_bias:
            specs.append(ParamSpec(p + "o_proj.bias", (self.E,), "vector"))
        return specs

    def cache_need(self):
        return PagedKV(self.KD, self.VD, self.window)

    def bind(self, params, ops):
        p = self.prefix
        # One matrix for the three projections that share an input: rows of q, then k, then v.
        mats = [params[p + n + "_proj.weight"] for n in "qkv"]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        if self.qkv_bias:
            self.b_qkv = memory.cat([params[p + n + "_proj.bias"] for n in "qkv"], 0, f"{p}q, k and v biases in one vector")
        self.w_o = params[p + "o_proj.weight"]
        self.short_request_rows = ops.prompt_rows     # where the attention kernels for decoded tokens and for prompt portions part
        if self.out_bias:
            self.b_o = params[p + "o_proj.bias"]

    def forward(self, ops, step, h, cache, x, write_cache=True):
        T = h.shape[0]
        width = self.QD + self.KD + self.VD if write_cache else self.QD
        qkv = ops.scratch("qkv", (T, width), ops.act_dtype)
        # a product that split K is added up inside the next kernel (position.store, the next norm)
        with ops.section("qkv"):
            ops.gemm(h, self.w_qkv[:width], qkv, bias=None if self.b_qkv is None else self.b_qkv[:width], defer=True)
        if self.Dv == self.D:
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache)
        else:                                   # only a position part that knows of value heads of another size can serve
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache, v_head_dim=self.Dv)
        att = ops.scratch("att", (T, self.OD), ops.act_dtype)
        with ops.section("attn"):
            ops.paged_attention(qkv, self.H, self.G, self.D, cache, step, self.window, self.scale, att,
                                slopes=getattr(self.position, "score_slopes", None), v_head_dim=self.Dv)
        with ops.section("wo"):
            ops.gemm(att, self.w_o, x, bias=self.b_o, accumulate=True, defer=True)
