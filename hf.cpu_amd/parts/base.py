"""What every part has in common, and the interface of each role.

A part is built from its sizes and constants alone (``PartSpec.args``) and a name
prefix. It declares its tensors (``param_specs``), receives them on the device
(``bind``) and computes (``forward``) with the kernels it is handed. No part knows
which model it is in.

Interfaces by role (``step`` is the engine's StepInputs, ``ops`` its kernels):

  embedding     forward(ops, step, out_x)                    tokens -> fp32 residual stream [T, E]
  norm          forward(ops, x, out, rows=None)              fp32 [T, E] -> activation dtype [T or R, E]
  position      store(ops, step, qkv, heads, kv_heads, cache, write[, v_head_dim=...])    acts on packed q | k | v rows
  mixer         cache_need(); forward(ops, step, h, cache, x, write_cache=True)     x += mixer(h)
  feed_forward  forward(ops, step, h, x)                                             x += ffn(h)
  block         forward(ops, step, x, parts, caches, write_cache)    parts: {name: part} as the plan names them;
                                                                     caches: {name: cache view} of those that keep one
  head          forward(ops, h, out_logits)                  activation [R, E] -> fp32 [R, V]
"""
from dataclasses import dataclass


@dataclass(frozen=True)
class ParamSpec:
    """One tensor of the checkpoint. ``kind``: "matrix" (a matrix-product operand,
    held in the compute dtype unless stored in 32-bit), "vector" (widened to fp32),
    "table" (integers, held as int32). ``init`` is the random-weights rule:
    ("normal", std) or ("one_plus_normal", std)."""
    name: str
    shape: tuple
    kind: str = "matrix"
    init: tuple = ("normal", 0.02)
    optional: bool = False


@dataclass(frozen=True)
class PagedKV:
    """A mixer's need for storage that grows with the sequence: one key row and one
    value row per token, kept for every earlier token (``window == 0``) or for the
    last ``window`` tokens only."""
    k_width: int
    v_width: int
    window: int = 0


@dataclass(frozen=True)
class FixedState:
    """A mixer's need for per-request storage of fixed size: ``n_floats`` fp32
    values per request, zero when the request is admitted."""
    n_floats: int


class Part:
    role = None
    kind = None
    # True if forward() only enqueues kernels whose arguments depend on the step's shape, never
    # on its values (no host-side loop over the step's tokens, no read-back): only then may the
    # engine capture a step into a graph and replay it. Parts say so themselves; the default is no.
    graph_safe = False
    # True if forward() reads its input activations (the norm's output it is handed) through ``ops.gemm`` alone: the
    # block may then ask the norm in front of it to be lazy (``Ops.rmsnorm``), which saves a kernel in decode steps.
    lazy_input_ok = False
    # A part whose kernels treat requests that bring fewer than this many tokens to a step differently from the
    # others (decoded tokens beside prompt portions) says so here: the step function then lays those requests first
    # (``StepInputs.n_short_seqs``), so that the part can take the two groups as steps of their own. 0: no such line.
    short_request_rows = 0

    def __init__(self, prefix=""):
        self.prefix = prefix

    def param_specs(self):
        return []

    def bind(self, params, ops):
        """``params`` maps each declared name that was found to its device tensor."""

    def sub_parts(self):
        """Parts this part owns (their tensors are declared and bound through it)."""
        return []

    def all_param_specs(self):
        specs = list(self.param_specs())
        for p in self.sub_parts():
            specs.extend(p.all_param_specs())
        return specs

    def bind_all(self, params, ops):
        for p in self.sub_parts():
            p.bind_all(params, ops)
        self.bind(params, ops)
