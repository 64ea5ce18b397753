"""The kernels as methods on tensors.

A matrix product with few rows splits its K range over the machine and leaves partial sums in
the workspace. With ``defer=True`` the product does not add them up itself: the next kernel
that reads the output does (``rmsnorm`` for the residual stream, ``rope_store`` for q/k/v), which
saves a launch and a pass over memory per product in decode. The pending state lives here; every
method that could disturb it settles it first, and a part that touches a tensor with anything
but these methods calls ``settle`` before.


``Ops`` belongs to one device and one compute dtype. Every method checks shapes,
dtypes and layout on the host, hands raw pointers to the library on the current
stream, and raises EngineError if the library refuses the call. Nothing here
computes with a library routine or on the CPU.
"""
import contextlib
import ctypes
import sys
from dataclasses import dataclass

import torch

from .. import memory
from ..status import EINVAL, ENOTSUP, EngineError, fail
from .lib import last_error, library

F32, BF16 = 0, 1
WORKSPACE_BYTES = 64 << 20           # partial sums of matrix products whose K is split
_CODE = {torch.float32: F32, torch.bfloat16: BF16}
_ELEMENT_BYTES = {torch.float32: 4, torch.bfloat16: 2, torch.float16: 2, torch.int32: 4, torch.int64: 8, torch.uint8: 1}


def _code(t):
    if t.dtype not in _CODE:
        fail(EINVAL, f"tensor dtype {t.dtype} is neither float32 nor bfloat16")
    return _CODE[t.dtype]


def _rows(t, what):
    """A 2-D tensor whose rows are contiguous; returns its row stride."""
    if t.dim() != 2 or t.stride(1) != 1:
        fail(EINVAL, f"{what}: expected a matrix with contiguous rows, got shape {tuple(t.shape)} "
                     f"strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _ints(t, what, n=None):
    if t.dtype != torch.int32 or not t.is_contiguous() or (n is not None and t.numel() < n):
        fail(EINVAL, f"{what}: expected a contiguous int32 tensor of at least {n} elements")
    return t.data_ptr()


@dataclass
class Pending:
    """A matrix product whose partial sums ([splits][M][N] fp32 in the workspace) wait to be added up."""
    out: torch.Tensor
    splits: int
    bias: object
    accumulate: bool


@dataclass
class LazyProduct:
    """A product into the residual stream that has not been launched yet: ``x += a @ w.T + bias``. If the next
    thing asked for is the norm of ``x``, product, residual sum and the norm's weight go into one kernel."""
    a: torch.Tensor
    w: torch.Tensor
    x: torch.Tensor
    bias: object
    section: object = None   # while timing: the section in which it was asked for (its time is booked there)


@dataclass
class LazyRope:
    """A rotation of queries and keys and a store of keys and values that has not been launched: if attention over
    the same rows of decoded tokens is asked for next, one kernel does all of it (``hfa_decode_attention``)."""
    args: tuple              # what rope_store was called with
    qkv: torch.Tensor
    cache: object


@dataclass
class Scaled:
    """A norm's output that holds ``x * weight`` only, not yet divided by the root mean square: the products that
    read it scale their sums by ``rsqrt(sum(ssq) / width + eps)`` instead. ``x``, ``weight`` and ``eps`` make it whole
    again (the plain norm kernel) if something else wants to read it."""
    out: torch.Tensor
    x: torch.Tensor
    weight: torch.Tensor
    eps: float
    ssq: torch.Tensor
    source_changed: bool = False       # x has gone on since: products may still read `out`, nothing can make it whole


class _NoSection:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SECTION = _NoSection()


class _Section:
    """Device time between entering and leaving, booked under a name."""

    def __init__(self, ops, name):
        self.ops, self.name = ops, name

    def __enter__(self):
        stack = self.ops._section_stack
        self.parent = stack[-1] if stack else None
        stack.append(self.name)
        self.start = torch.cuda.Event(enable_timing=True)
        self.start.record()
        return self

    def __exit__(self, *exc):
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        self.ops._section_stack.pop()
        self.ops._sections.append((self.name, self.start, end, self.parent))
        return False


class Ops:
    def __init__(self, act_dtype=torch.bfloat16, device="cuda:0"):
        if not torch.cuda.is_available():
            fail(ENOTSUP, "no GPU is visible: the engine runs on gfx950 only and has no CPU path")
        if act_dtype not in _CODE:
            fail(EINVAL, f"compute dtype {act_dtype} is neither float32 nor bfloat16")
        self.device = torch.device(device)
        self.act_dtype = act_dtype
        self.lib = library()
        self.prompt_rows = int(self.lib.hfa_attention_prompt_rows())   # see StepInputs and paged_attention
        self._scratch = {}
        self._shared = {}
        self._scratch_views = {}             # (name, shape, dtype) -> the view handed out last time
        self._stream_handle = None
        self.scratch_generation = 0
        self.workspace = memory.empty(WORKSPACE_BYTES, torch.uint8, self.device, "workspace of the matrix products")
        self.attn_workspace = memory.empty(WORKSPACE_BYTES, torch.uint8, self.device, "workspace of attention")
        self._pending = None
        self._lazy = None                    # a LazyProduct
        self._lazy_rope = None               # a LazyRope
        self._rope_tables = {}               # (positions, frequencies, tokens) -> cosines and sines of a pass's angles
        self._scaled = {}                    # data_ptr of a norm's output -> Scaled
        self.rows_parts = int(self.lib.hfa_gemm_rows_parts())
        self.fuse_rows = True                # tests switch it off to compare with the chain of separate kernels
        self.rows_always = False             # tests: every shape that the kernel of gemm_rows.hip takes goes through it
        self._splits_out = ctypes.c_int(0)
        self._sections = None                # while timing: (name, start event, end event, enclosing section) of every section left
        self._section_stack = []
        self.force_plain_gemm = False        # tests set these to compare the matrix-core paths with the plain ones
        self.force_plain_attention = False
        self._said_cache_too_large = False

    # ---- timing (the reference's hfc_prof_enable / hfc_prof_take, src/model.h:75-79) ----
    def section(self, name):
        """``with ops.section("qkv"): ...`` books the device time of the kernels enqueued inside
        under ``name`` while timing is on; otherwise it costs nothing."""
        return _NO_SECTION if self._sections is None else _Section(self, name)

    def timing(self, on):
        self._sections = [] if on else None
        self._section_stack = []

    def take_times(self):
        """Milliseconds per section name since the last call; waits for the device."""
        out = {}
        if self._sections:
            torch.cuda.synchronize(self.device)
            for name, start, end, parent in self._sections:
                ms = start.elapsed_time(end)
                out[name] = out.get(name, 0.0) + ms
                if parent is not None and parent != "total":       # (what "total" encloses is taken off it by the caller)
                    out[parent] = out.get(parent, 0.0) - ms
            self._sections = []
        return out

    # ---- plumbing ----------------------------------------------------------
    def _stream(self):
        s = self._stream_handle
        return s if s is not None else torch.cuda.current_stream(self.device).cuda_stream

    @contextlib.contextmanager
    def on_current_stream(self):
        """Inside, every kernel goes to the stream that is current on entry: asked for once
        instead of once per kernel (a forward pass enqueues hundreds)."""
        before = self._stream_handle
        self._stream_handle = torch.cuda.current_stream(self.device).cuda_stream
        self._scaled.clear()                 # what an earlier pass left in its work buffers is of no use to this one
        self._rope_tables.clear()
        try:
            yield self
        finally:
            self._stream_handle = before

    def _check(self, rc):
        if rc != 0:
            raise EngineError(EINVAL if rc == 1 else ENOTSUP, last_error())

    def call(self, entry_point, *args, what=None):
        """Launches an entry point of an extension library (``kernels.lib.load_extension``) on the step's
        stream: ``args`` are its arguments but the last, the stream. What was deferred is done first,
        since the kernel may read any tensor. Raises EngineError unless it returns 0."""
        self.settle()
        for sc in list(self._scaled.values()):               # and a norm's output that was left undivided is made whole
            if not sc.source_changed:
                self._whole(sc.out)
        rc = entry_point(*args, self._stream())
        if rc != 0:
            raise EngineError(EINVAL if rc == 1 else ENOTSUP,
                              f"{what or getattr(entry_point, '__name__', 'extension kernel')} returned {rc}")

    def shared(self, key, make):
        """A constant tensor that several parts want (``make()`` builds it the first time ``key`` is asked for)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]

    def scratch(self, name, shape, dtype):
        """A named work buffer that is reused from step to step; its contents are
        undefined on return. The same name always aliases the same memory."""
        key = (name, tuple(shape), dtype)
        view = self._scratch_views.get(key)
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = max(n, 1) * _ELEMENT_BYTES[dtype]
        buf = self._scratch.get(name)
        if buf is None or buf.numel() < nbytes:
            if torch.cuda.is_current_stream_capturing():
                fail(EINVAL, f"work buffer '{name}' would have to grow while a graph is being captured")
            buf = memory.empty(max(nbytes, 256), torch.uint8, self.device, f"work buffer '{name}'")
            self._scratch[name] = buf
            self.scratch_generation += 1          # captured graphs hold the old address
            self._scratch_views = {k: v for k, v in self._scratch_views.items() if k[0] != name}
        view = buf[:nbytes].view(dtype).view(*shape)
        if len(self._scratch_views) < 4096:
            self._scratch_views[key] = view
        return view

    # ---- kernels -----------------------------------------------------------
    def embed(self, table, tokens, out_x):
        self.settle()
        self._source_changes(out_x)
        T = out_x.shape[0]
        if out_x.dtype != torch.float32 or not out_x.is_contiguous() or not table.is_contiguous() \
                or table.shape[1] != out_x.shape[1]:
            fail(EINVAL, "embed: the output must be contiguous fp32 with the table's width")
        self._check(self.lib.hfa_embed(table.data_ptr(), _code(table), _ints(tokens, "embed tokens", T),
                                       out_x.data_ptr(), T, table.shape[1], table.shape[0], self._stream()))

    def rmsnorm(self, x, weight, eps, out, rows=None, lazy=False):
        """``out[r] = norm(x[rows[r]])``. ``lazy``: the caller promises that ``out`` is read by ``gemm`` alone. Then,
        if the product that completes ``x`` waits to be launched (``gemm(..., accumulate=True, defer=True)`` of few rows),
        one kernel does product, residual sum and ``out = x * weight``, and the division by the root mean square is
        left to the products that read ``out`` (see ``Scaled``)."""
        R = out.shape[0]
        E = x.shape[1]
        if x.dtype != torch.float32 or weight.dtype != torch.float32 or not x.is_contiguous() \
                or not out.is_contiguous() or out.shape[1] != E or weight.numel() != E:
            fail(EINVAL, "rmsnorm: x and weight must be fp32, contiguous, and of one width with out")
        if rows is None and R != x.shape[0]:
            fail(EINVAL, "rmsnorm: without row indices the output must have x's rows")
        z = self._lazy
        if lazy and rows is None and z is not None and z.x.data_ptr() == x.data_ptr() and z.x.shape == x.shape \
                and out.dtype == torch.bfloat16:
            self._lazy = None
            self._source_changes(x, keep=out)
            ssq = self.scratch(f"ssq@{out.data_ptr()}", (self.rows_parts * 32,), torch.float32)
            self._rows_resid(z, weight, out, ssq)
            self._scaled[out.data_ptr()] = Scaled(out, x, weight, float(eps), ssq)
            return
        self._scaled.pop(out.data_ptr(), None)
        pend = self._take_pending(x) if rows is None else None
        if pend is None:
            self.settle()
        self._check(self.lib.hfa_rmsnorm(x.data_ptr(), weight.data_ptr(), out.data_ptr(), _code(out),
                                         None if rows is None else _ints(rows, "rmsnorm rows", R),
                                         R, E, float(eps), None if pend is None else self.workspace.data_ptr(),
                                         0 if pend is None else pend.splits,
                                         None if pend is None or pend.bias is None else pend.bias.data_ptr(),
                                         self._stream()))

    def _take_pending(self, tensor):
        """The pending product if it is the residual sum of ``tensor`` (whole, contiguous), else None."""
        p = self._pending
        if p is not None and p.accumulate and p.out.data_ptr() == tensor.data_ptr() \
                and p.out.shape == tensor.shape and tensor.is_contiguous():
            self._pending = None
            return p
        return None

    def abandon(self):
        """Forgets a deferred product (after a step that failed: its partial sums are of no use)."""
        self._pending = None
        self._lazy = None
        self._lazy_rope = None
        self._scaled.clear()

    # ---- products of few rows that finish their outputs themselves (csrc/gemm_rows.hip) -----------------------
    def _rows_mode(self, a, w, out, bias, accumulate, swiglu):
        """The mode in which ``hfa_gemm_rows`` takes this product, or None."""
        if not self.fuse_rows or self.force_plain_gemm or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 \
                or a.dim() != 2 or w.dim() != 2 or a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
            return None
        M, K = a.shape
        mode = 1 if accumulate else 2 if swiglu else 0
        N = w.shape[0] // 2 if swiglu else w.shape[0]
        if (a.data_ptr() | w.data_ptr()) & 15 or not self.lib.hfa_gemm_rows_supports(
                mode, M, N, K, _rows(a, "gemm a"), _rows(w, "gemm w")):
            return None
        if accumulate:
            # Every block of that kernel reads all the activations, and a block of a narrow product owns few weight
            # rows to set against them: from 17 rows up a long K (the down projection) is quicker through the kernels
            # that cut K over the blocks, with the norm as a kernel of its own (7B shape, 32 rows: 58 against 50 us).
            if M > 16 and M * K > 128 << 10 and not self.rows_always:
                return None
            return mode if out.dtype == torch.float32 else None
        if swiglu:
            return mode if out.dtype == torch.bfloat16 and bias is None else None
        return mode

    def _rows_call(self, mode, a, w, N, bias, scaled=None, out=None, x=None, ssq_out=None, g=None, xg=None, act=None):
        M, K = a.shape
        null = ctypes.c_void_p(None)

        def ptr(t):
            return null if t is None else t.data_ptr()
        self._check(self.lib.hfa_gemm_rows(
            mode, a.data_ptr(), _rows(a, "gemm a"), w.data_ptr(), _rows(w, "gemm w"), M, N, K, ptr(bias),
            ptr(None if scaled is None else scaled.ssq), self.rows_parts, 1.0 / K, 0.0 if scaled is None else scaled.eps,
            ptr(out), 0 if out is None else _rows(out, "gemm out"), 0 if out is None else _code(out),
            ptr(x), 0 if x is None else _rows(x, "gemm out"), ptr(ssq_out), ptr(g),
            ptr(xg), 0 if xg is None else _rows(xg, "norm out"), ptr(act), 0 if act is None else _rows(act, "gemm out"),
            self._stream()))

    def _rows_resid(self, z, g=None, xg=None, ssq=None):
        """Launches a LazyProduct; with ``g`` and ``xg`` the kernel also leaves ``xg = x * g`` and the sums of squares.
        While timing, its time goes to the section in which the product was asked for, not to the one that launches it."""
        if self._sections is not None and z.section is not None and \
                (not self._section_stack or self._section_stack[-1] != z.section):
            with _Section(self, z.section):
                return self._rows_resid_now(z, g, xg, ssq)
        return self._rows_resid_now(z, g, xg, ssq)

    def _rows_resid_now(self, z, g, xg, ssq):
        if ssq is None:
            ssq = self.scratch("ssq@none", (self.rows_parts * 32,), torch.float32)
        self._rows_call(1, z.a, z.w, z.w.shape[0], z.bias, x=z.x, ssq_out=ssq, g=g, xg=xg)

    def _whole(self, t):
        """Makes a norm's output that was left undivided (``Scaled``) whole before something other than ``gemm`` reads it."""
        sc = self._scaled.pop(t.data_ptr(), None)
        if sc is not None:
            if sc.source_changed:
                fail(EINVAL, "a norm's output that was asked for lazily is read by something other than a product after "
                             "the normed tensor has changed: ask for the norm without lazy=True, or settle() its output first")
            self._check(self.lib.hfa_rmsnorm(sc.x.data_ptr(), sc.weight.data_ptr(), sc.out.data_ptr(), _code(sc.out), None,
                                             sc.out.shape[0], sc.out.shape[1], sc.eps, None, 0, None, self._stream()))

    def _source_changes(self, x, keep=None):
        """``x`` is about to change: norm outputs that were left undivided can no longer be made whole from it
        (products can still read them: x * weight and the sums of squares stay). ``keep``: one that is about to be
        overwritten is dropped."""
        for key, sc in list(self._scaled.items()):
            if sc.x.data_ptr() == x.data_ptr():
                if keep is not None and key == keep.data_ptr():
                    del self._scaled[key]
                else:
                    sc.source_changed = True

    def settle(self, tensor=None):
        """Adds up a deferred product now (all of them if ``tensor`` is None, else only one that
        writes ``tensor``), and makes ``tensor`` whole if it is a norm's output that was left undivided."""
        lr = self._lazy_rope
        if lr is not None and (tensor is None or lr.qkv.data_ptr() == tensor.data_ptr()):
            self._lazy_rope = None
            self.rope_store(*lr.args, lazy=False)
        z = self._lazy
        if z is not None and (tensor is None or z.x.data_ptr() == tensor.data_ptr()):
            self._lazy = None
            self._source_changes(z.x)
            self._rows_resid(z)
        if tensor is not None:
            self._whole(tensor)
        p = self._pending
        if p is None or (tensor is not None and p.out.data_ptr() != tensor.data_ptr()):
            return
        self._pending = None
        M, N = p.out.shape
        self._check(self.lib.hfa_gemm_finish(self.workspace.data_ptr(), p.splits,
                                             None if p.bias is None else p.bias.data_ptr(), p.out.data_ptr(),
                                             _code(p.out), _rows(p.out, "gemm out"), 1 if p.accumulate else 0, 0,
                                             M, N, self._stream()))

    def gemm(self, a, w, out, bias=None, accumulate=False, defer=False, swiglu=False):
        """out (+)= a @ w.T + bias, fp32 accumulation. ``defer``: if the kernel split K, leave the
        partial sums for the next kernel that reads ``out`` (see the module's text).
        ``swiglu``: w's rows come in blocks of 32 gate, 32 up (``interleave_gate_up``) and
        out = silu(gate) * up has half as many columns."""
        self.settle()
        lda, ldw, ldo = _rows(a, "gemm a"), _rows(w, "gemm w"), _rows(out, "gemm out")
        M, K = a.shape
        N = w.shape[0]
        if w.shape[1] != K or tuple(out.shape) != (M, N // 2 if swiglu else N):
            fail(EINVAL, f"gemm: shapes a{tuple(a.shape)} w{tuple(w.shape)} out{tuple(out.shape)} do not fit")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N or not bias.is_contiguous()):
            fail(EINVAL, "gemm: the bias must be contiguous fp32 with one value per output column")
        scaled = self._scaled.get(a.data_ptr())
        if scaled is not None and scaled.out.shape != a.shape:
            scaled = None
        mode = self._rows_mode(a, w, out, bias, accumulate, swiglu)
        if mode is not None and not (mode == 1 and scaled is not None):
            self._scaled.pop(out.data_ptr(), None)
            if mode == 1:                            # into the residual stream
                z = LazyProduct(a, w, out, bias, self._section_stack[-1] if self._section_stack else None)
                if defer:
                    self._lazy = z                   # the next norm of `out` may take it along
                else:
                    self._source_changes(out)
                    self._rows_resid(z)
            elif mode == 2:
                self._rows_call(2, a, w, N // 2, None, scaled=scaled, act=out)
            elif defer and out.dtype == torch.bfloat16 and M * N * 4 <= self.workspace.numel():
                # 32-bit sums for the kernel that follows (the rotation of queries and keys): one plane of the workspace
                plane = self.workspace[:M * N * 4].view(torch.float32).view(M, N)
                self._rows_call(0, a, w, N, bias, scaled=scaled, out=plane)
                self._pending = Pending(out, 1, None, False)
            else:
                self._rows_call(0, a, w, N, bias, scaled=scaled, out=out)
            return
        if scaled is not None:
            self._whole(a)
        self._scaled.pop(out.data_ptr(), None)
        if accumulate:
            self._source_changes(out)
        self._splits_out.value = 0
        self._check(self.lib.hfa_gemm(a.data_ptr(), _code(a), lda, w.data_ptr(), _code(w), ldw,
                                      None if bias is None else bias.data_ptr(), out.data_ptr(), _code(out), ldo,
                                      1 if accumulate else 0, 1 if swiglu else 0, M, N, K, self.workspace.data_ptr(),
                                      self.workspace.numel(), 1 if defer else 0, ctypes.byref(self._splits_out),
                                      1 if self.force_plain_gemm else 0, self._stream()))
        if self._splits_out.value:
            self._pending = Pending(out, self._splits_out.value, bias, accumulate)

    def can_fuse_swiglu(self, w_gate, w_up):
        """Whether gate and up may be interleaved for ``gemm(..., swiglu=True)``: bf16 on the
        matrix cores, a feature count that is a multiple of 32."""
        F, E = w_gate.shape
        return (self.act_dtype == torch.bfloat16 and w_gate.dtype == torch.bfloat16 and w_up.dtype == torch.bfloat16
                and F % 32 == 0 and E % 8 == 0 and not self.force_plain_gemm)

    @staticmethod
    def interleave_gate_up(w_gate, w_up):
        """[2F, E]: rows 0..31 of gate, rows 0..31 of up, rows 32..63 of gate, ..."""
        F, E = w_gate.shape
        return torch.stack([w_gate.view(F // 32, 32, E), w_up.view(F // 32, 32, E)], dim=1).reshape(2 * F, E).contiguous()

    def rope_store(self, qkv, positions, inv_freq, rot_dim, n_heads, n_kv_heads, head_dim, cache, slot_map,
                   v_head_dim=None, lazy=True):
        """Rotates q (and k) inside ``qkv`` and, if ``slot_map`` is given, stores k and v
        rows into ``cache.k`` / ``cache.v`` at the rows it names (values transposed inside
        their page, see csrc/api.h). ``v_head_dim``: the size of a value head if it is not ``head_dim``.
        When ``qkv`` is still the 32-bit plane that a product of few rows left and the shape allows it, the call
        waits (``lazy``): attention over the same rows may take it along (``paged_attention``)."""
        v_head_dim = head_dim if v_head_dim is None else int(v_head_dim)
        row_width = (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim
        pend = self._pending
        if lazy and self.fuse_rows and pend is not None and pend.splits == 1 and pend.bias is None and not pend.accumulate \
                and pend.out.data_ptr() == qkv.data_ptr() and pend.out.shape == qkv.shape and qkv.shape[1] == row_width \
                and qkv.dtype == torch.bfloat16 and slot_map is not None and n_kv_heads and v_head_dim == head_dim \
                and qkv.is_contiguous() and getattr(cache, "k", None) is not None and cache.k.dtype == torch.bfloat16 \
                and cache.k.numel() < 1 << 32 and cache.k.shape[0] < 1 << 24 \
                and self.lib.hfa_decode_attention_supports(n_heads, n_kv_heads, head_dim, rot_dim, cache.page_tokens,
                                                           cache.k.shape[1], row_width, n_heads * head_dim):
            self._lazy_rope = LazyRope((qkv, positions, inv_freq, rot_dim, n_heads, n_kv_heads, head_dim, cache, slot_map,
                                        v_head_dim), qkv, cache)
            return
        if pend is not None and not pend.accumulate and pend.out.data_ptr() == qkv.data_ptr() \
                and pend.out.shape == qkv.shape and qkv.shape[1] == row_width:
            self._pending = None
            if qkv.dtype == torch.bfloat16 and qkv.shape[0] >= 512 and rot_dim > 0:
                # A prompt portion: the kernel for many tokens does not add up partial sums; finishing
                # the product first and then taking that kernel is the quicker way.
                self._pending = pend
                self.settle()
                pend = None
        else:
            pend = None
            self.settle()
        ld = _rows(qkv, "rope_store qkv")
        T = qkv.shape[0]
        if qkv.shape[1] < row_width:
            fail(EINVAL, "rope_store: the rows are narrower than the heads they should hold")
        k_ptr = v_ptr = None
        if n_kv_heads and slot_map is not None:
            for c, width in ((cache.k, n_kv_heads * head_dim), (cache.v, n_kv_heads * v_head_dim)):
                if c.dtype != qkv.dtype or c.dim() != 2 or c.shape[1] != width or not c.is_contiguous():
                    fail(EINVAL, "rope_store: the cache must have the activations' dtype and one row of "
                                 f"{width} values per token")
            k_ptr, v_ptr = cache.k.data_ptr(), cache.v.data_ptr()
        self._check(self.lib.hfa_rope_store(
            qkv.data_ptr(), _code(qkv), ld, None if positions is None else _ints(positions, "positions", T),
            None if inv_freq is None else inv_freq.data_ptr(), rot_dim, n_heads, n_kv_heads, head_dim, v_head_dim,
            k_ptr, v_ptr, None if slot_map is None else _ints(slot_map, "slot_map", T),
            getattr(cache, "page_tokens", 0) or 0, T, None if pend is None else self.workspace.data_ptr(),
            0 if pend is None else pend.splits,
            None if pend is None or pend.bias is None else pend.bias.data_ptr(), self._stream()))

    def paged_attention(self, q, n_heads, n_kv_heads, head_dim, cache, step, window, scale, out, slopes=None,
                        v_head_dim=None):
        """Attention of the first ``n_heads * head_dim`` columns of ``q`` over ``cache``. ``slopes``
        (fp32, one per query head): the score of key j for the query at p gets ``slopes[h] * (j - p)``
        added, for position encodings that enter the scores; the plain kernel then runs, as it does when
        value heads have a size of their own (``v_head_dim``; ``out`` then has that many columns a head)."""
        v_head_dim = head_dim if v_head_dim is None else int(v_head_dim)
        self._scaled.pop(out.data_ptr(), None)               # whatever `out` held, it is no norm's lazy output any more
        lr = self._lazy_rope
        if lr is not None and lr.qkv.data_ptr() == q.data_ptr() and lr.cache is cache and slopes is None \
                and step.max_q_len == 1 and step.n_seqs == q.shape[0] and not self.force_plain_attention \
                and out.dtype == torch.bfloat16 and v_head_dim == head_dim and lr.args[4:7] == (n_heads, n_kv_heads, head_dim) \
                and cache.k.numel() < 1 << 32 and cache.k.shape[0] < 1 << 24:
            return self._decode_attention(lr, step, window, scale, out)
        self.settle()
        if slopes is not None and (slopes.dtype != torch.float32 or slopes.numel() != n_heads or not slopes.is_contiguous()
                                   or slopes.device != q.device):
            fail(EINVAL, "paged_attention: slopes must be contiguous fp32 on the device, one per query head")
        T = q.shape[0]
        ldq, ldo = _rows(q, "attention q"), _rows(out, "attention out")
        g = step.group(cache.group)
        if cache.k.dtype != q.dtype or out.dtype != q.dtype:
            fail(EINVAL, "paged_attention: queries, cache and output must share a dtype")
        if cache.k.shape[1] != n_kv_heads * head_dim or cache.v.shape[1] != n_kv_heads * v_head_dim:
            fail(EINVAL, "paged_attention: the cache rows do not hold n_kv_heads * head_dim keys and n_kv_heads * v_head_dim values")
        _ints(step.token_slot, "token_slot", T)
        _ints(step.positions, "positions", T)
        _ints(step.q_start, "q_start", step.n_seqs + 1)
        # the matrix-core kernels address the cache with 32-bit element offsets and 24-bit row numbers
        too_large = cache.k.numel() >= 1 << 32 or cache.k.shape[0] >= 1 << 24
        plain = self.force_plain_attention or slopes is not None or too_large
        if too_large and q.dtype == torch.bfloat16 and not self._said_cache_too_large:
            self._said_cache_too_large = True        # right, but many times slower: say so once
            print(f"[hf_cpu_amd] a layer's cache of {cache.k.shape[0]} rows x {cache.k.shape[1]} is beyond what the "
                  "matrix-core attention addresses (2^24 rows, 2^32 elements): the plain attention kernels run; "
                  "a smaller --kv-tokens brings the fast ones back", file=sys.stderr, flush=True)

        def call(first, n_tokens, q_start, n_seqs, max_q_len):
            self._check(self.lib.hfa_paged_attention(
                q.data_ptr() + first * ldq * q.element_size(), _code(q), ldq, cache.k.data_ptr(), cache.v.data_ptr(),
                cache.k.shape[1], cache.v.shape[1], g.block_table.data_ptr(), g.block_table.shape[1],
                step.token_slot.data_ptr() + 4 * first, step.positions.data_ptr() + 4 * first, q_start.data_ptr(), n_seqs,
                max_q_len, step.max_seq_len, out.data_ptr() + first * ldo * out.element_size(), ldo, n_tokens, n_heads,
                n_kv_heads, head_dim, v_head_dim, cache.page_tokens, int(window), float(scale),
                None if slopes is None else slopes.data_ptr(), self.attn_workspace.data_ptr(),
                self.attn_workspace.numel(), 1 if plain else 0, self._stream()))

        # Decoded tokens beside prompt portions: one call would send all of them to the kernel for prompt
        # portions, which walks a request's keys in one piece (a decoded token with a long context would
        # take as long as thousands of prompt tokens). The step lays requests with few tokens first, so
        # each part is a step of its own: the first goes to the kernel that cuts the keys into chunks.
        n_short = getattr(step, "n_short_seqs", 0)
        if not plain and q.dtype == torch.bfloat16 and step.max_q_len >= self.prompt_rows and 0 < n_short < step.n_seqs:
            ts = step.n_short_tokens
            _ints(step.q_start_long, "q_start_long", step.n_seqs - n_short + 1)
            call(0, ts, step.q_start, n_short, step.max_short_q_len)
            call(ts, T - ts, step.q_start_long, step.n_seqs - n_short, step.max_q_len)
        else:
            call(0, T, step.q_start, step.n_seqs, step.max_q_len)

    def _decode_attention(self, lr, step, window, scale, out):
        """Rotation, the store of the new keys and values and attention over the cache for decoded tokens, in one
        kernel: the queued ``rope_store`` (``lr``) and this call together."""
        qkv, positions, inv_freq, rot_dim, n_heads, n_kv_heads, head_dim, cache, slot_map, _ = lr.args
        T = qkv.shape[0]
        table = None
        if rot_dim:
            key = (positions.data_ptr(), inv_freq.data_ptr(), T, rot_dim)
            table = self._rope_tables.get(key)
            if table is None:                # the angles of this pass's tokens, once for all its layers
                table = self.scratch(f"rope_table@{inv_freq.data_ptr()}", (T, rot_dim), torch.float32)
                self._check(self.lib.hfa_rope_table(_ints(positions, "positions", T), inv_freq.data_ptr(), rot_dim // 2,
                                                    table.data_ptr(), T, self._stream()))
                self._rope_tables[key] = table
        g = step.group(cache.group)
        self._lazy_rope = None
        self._pending = None                 # the 32-bit plane of q, k and v is read here
        self._check(self.lib.hfa_decode_attention(
            self.workspace.data_ptr(), qkv.shape[1], None if table is None else table.data_ptr(), cache.k.data_ptr(),
            cache.v.data_ptr(), cache.k.shape[1], _ints(slot_map, "slot_map", T), g.block_table.data_ptr(),
            g.block_table.shape[1], _ints(step.token_slot, "token_slot", T), _ints(step.positions, "positions", T),
            _ints(step.q_start, "q_start", T + 1), T, step.max_seq_len, out.data_ptr(), _rows(out, "attention out"),
            n_heads, n_kv_heads, head_dim, cache.page_tokens, int(window), float(scale), self.attn_workspace.data_ptr(),
            self.attn_workspace.numel(), self._stream()))

    def swiglu(self, gate_up, out):
        self.settle()
        self._scaled.pop(out.data_ptr(), None)
        T, F2 = gate_up.shape
        if not gate_up.is_contiguous() or not out.is_contiguous() or tuple(out.shape) != (T, F2 // 2) \
                or out.dtype != gate_up.dtype or F2 % 2:
            fail(EINVAL, "swiglu: expected contiguous [T, 2F] in and [T, F] out of one dtype")
        self._check(self.lib.hfa_swiglu(gate_up.data_ptr(), out.data_ptr(), _code(out), T, F2 // 2, self._stream()))

    def scatter_i32(self, dst, idx, val):
        n = idx.numel()
        if n:
            self._check(self.lib.hfa_scatter_i32(_ints(dst, "scatter dst"), _ints(idx, "scatter idx"),
                                                 _ints(val, "scatter val", n), n, self._stream()))

    def move_i32(self, dst, dst_idx, src, src_idx):
        """dst[dst_idx[i]] = src[src_idx[i]] for int32 tensors on the device."""
        n = dst_idx.numel()
        if n:
            if src_idx.numel() != n:
                fail(EINVAL, "move_i32: as many places to read as to write")
            self._check(self.lib.hfa_move_i32(_ints(dst, "move dst"), _ints(dst_idx, "move dst_idx"), _ints(src, "move src"),
                                              _ints(src_idx, "move src_idx", n), n, self._stream()))

    def argmax(self, logits, out=None):
        self.settle()
        R, V = logits.shape
        if logits.dtype != torch.float32:
            fail(EINVAL, "argmax: logits must be fp32")
        if out is None:
            out = memory.empty(R, torch.int32, logits.device, "argmax output")
        self._check(self.lib.hfa_argmax(logits.data_ptr(), _rows(logits, "argmax logits"), _ints(out, "argmax out", R),
                                        R, V, self.workspace.data_ptr(), self.workspace.numel(), self._stream()))
        return out

    def order_rows(self, logits, rows=None):
        """(ids [n, V] int32, values [n, V] fp32): every candidate of the chosen rows (all rows if
        ``rows`` is None) in the order (logit descending, id ascending)."""
        self.settle()
        R, V = logits.shape
        if logits.dtype != torch.float32:
            fail(EINVAL, "order_rows: logits must be fp32")
        n = R if rows is None else int(rows.numel())
        ids = memory.empty((n, V), torch.int32, logits.device, "ordered ids")
        vals = memory.empty((n, V), torch.float32, logits.device, "ordered values")
        need = int(self.lib.hfa_order_rows_scratch(n, V))
        scratch = self.scratch("order_rows", (need,), torch.uint8)
        self._check(self.lib.hfa_order_rows(logits.data_ptr(), _rows(logits, "order_rows logits"),
                                            None if rows is None else _ints(rows, "order_rows rows", n), ids.data_ptr(),
                                            vals.data_ptr(), n, V, scratch.data_ptr(), need, self._stream()))
        return ids, vals

    def draw_rows(self, ids, vals, params, cuts):
        """tokens [n] int32 drawn from rows that ``order_rows`` put in order: ``params`` [n, 4] fp32 =
        (temp, top_p, min_p, uniform number), ``cuts`` [n] int32 = candidates left by top-k. ``vals``
        is overwritten with the probabilities."""
        n, V = vals.shape
        if vals.dtype != torch.float32 or not vals.is_contiguous() or ids.shape != vals.shape:
            fail(EINVAL, "draw_rows: expected contiguous fp32 values and ids of one shape")
        if params.dtype != torch.float32 or not params.is_contiguous() or tuple(params.shape) != (n, 4):
            fail(EINVAL, f"draw_rows: expected [{n}, 4] fp32 parameters")
        tokens = memory.empty((n,), torch.int32, vals.device, "drawn tokens")
        self._check(self.lib.hfa_draw_rows(vals.data_ptr(), _ints(ids, "draw_rows ids", n * V), n, V, params.data_ptr(),
                                           _ints(cuts, "draw_rows cuts", n), tokens.data_ptr(), self._stream()))
        return tokens

    def topk(self, logits, k, want_stats=True):
        """(ids [R, k] int32, values [R, k] fp32, stats [R, 2] fp32 = max and log-sum-exp
        above the max), candidates in the order (logit descending, id ascending)."""
        self.settle()
        R, V = logits.shape
        if logits.dtype != torch.float32:
            fail(EINVAL, "topk: logits must be fp32")
        ids = memory.empty((R, max(k, 1)), torch.int32, logits.device, "top-k ids")
        vals = memory.empty((R, max(k, 1)), torch.float32, logits.device, "top-k values")
        stats = memory.empty((R, 2), torch.float32, logits.device, "row statistics") if want_stats else None
        self._check(self.lib.hfa_topk(logits.data_ptr(), _rows(logits, "topk logits"), ids.data_ptr(), vals.data_ptr(),
                                      None if stats is None else stats.data_ptr(), R, V, k, self._stream()))
        return ids[:, :k], vals[:, :k], stats
