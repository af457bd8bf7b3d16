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
    def embed(self, table, tokens, out_x, scale=None, positions=None, inv_freq=None):
        """``out_x[t] = table[tokens[t]]``; with ``scale`` the row is multiplied by it, and with ``positions`` and
        ``inv_freq`` (fp32, one per pair of columns) a sinusoidal vector is added: column 2i gets ``sin(p inv_freq[i])``,
        column 2i + 1 the cosine."""
        self.settle()
        self._source_changes(out_x)
        T = out_x.shape[0]
        if out_x.dtype != torch.float32 or not out_x.is_contiguous() or not table.is_contiguous() \
                or table.shape[1] != out_x.shape[1]:
            fail(EINVAL, "embed: the output must be contiguous fp32 with the table's width")
        if scale is None and positions is None:
            self._check(self.lib.hfa_embed(table.data_ptr(), _code(table), _ints(tokens, "embed tokens", T),
                                           out_x.data_ptr(), T, table.shape[1], table.shape[0], self._stream()))
            return
        if positions is not None and (inv_freq is None or inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous()
                                      or inv_freq.numel() < (table.shape[1] + 1) // 2):
            fail(EINVAL, "embed: a position vector needs one fp32 frequency for every pair of columns")
        self._check(self.lib.hfa_embed_pos(table.data_ptr(), _code(table), _ints(tokens, "embed tokens", T),
                                           None if positions is None else _ints(positions, "positions", T),
                                           None if positions is None else inv_freq.data_ptr(), out_x.data_ptr(), T, table.shape[1],
                                           table.shape[0], 1.0 if scale is None else float(scale), self._stream()))

    def rmsnorm_add(self, y, weight, eps, out, gate=None, gate_bias=None, scale=1.0, accumulate=True):
        """``out (+)= scale * rmsnorm(y * sigmoid(gate + gate_bias)) * weight``, all in fp32 (``gate`` None: ``y`` as it is;
        ``accumulate`` False: ``out`` is overwritten): the norm of a branch's result on its way into the stream."""
        self.settle()
        self._source_changes(out)
        self._scaled.pop(out.data_ptr(), None)
        R, E = y.shape
        if y.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (R, E) or weight.dtype != torch.float32 \
                or weight.numel() != E or not weight.is_contiguous():
            fail(EINVAL, "rmsnorm_add: y, out and weight must be fp32 and of one width")
        if gate is not None and (tuple(gate.shape) != (R, E) or (gate_bias is not None and (gate_bias.dtype != torch.float32
                                                                                            or gate_bias.numel() != E))):
            fail(EINVAL, "rmsnorm_add: the gate has y's shape, its bias one fp32 value a column")
        if gate is None and gate_bias is not None:
            fail(EINVAL, "rmsnorm_add: a gate's bias without the gate")
        if gate is not None:
            self._whole(gate)
        self._check(self.lib.hfa_rmsnorm_add(
            y.data_ptr(), _rows(y, "norm in"), None if gate is None else gate.data_ptr(), 0 if gate is None else _code(gate),
            0 if gate is None else _rows(gate, "norm gate"), None if gate_bias is None else gate_bias.data_ptr(), weight.data_ptr(),
            out.data_ptr(), _rows(out, "norm out"), R, E, float(eps), float(scale), 1 if accumulate else 0, self._stream()))

    def polynorm(self, z, coef, eps, out):
        """``out = a N(z) + b N(z^2) + c N(z^3) + e`` row by row, ``N(u) = u / sqrt(mean(u^2) + eps)``, ``coef`` = (a, b, c, e)
        as four fp32 values on the device; sums and powers in fp32."""
        self.settle()
        self._whole(z)
        self._scaled.pop(out.data_ptr(), None)
        if z.shape != out.shape or z.dim() != 2 or coef.dtype != torch.float32 or coef.numel() != 4 or not coef.is_contiguous():
            fail(EINVAL, "polynorm: input and output of one shape, four fp32 coefficients")
        self._check(self.lib.hfa_polynorm(z.data_ptr(), _code(z), _rows(z, "polynorm in"), coef.data_ptr(), out.data_ptr(), _code(out),
                                          _rows(out, "polynorm out"), z.shape[0], z.shape[1], float(eps), self._stream()))

    def scale_rows(self, x, s):
        """``x *= s`` on fp32 rows, in place."""
        self.settle(x)
        if x.dtype != torch.float32 or x.dim() != 2:
            fail(EINVAL, "scale_rows: expected an fp32 matrix")
        if x.shape[0]:
            self._check(self.lib.hfa_scale_rows(x.data_ptr(), _rows(x, "scale_rows"), x.shape[0], x.shape[1], float(s), self._stream()))

    def head_norm_store(self, qkv, n_heads, n_kv_heads, head_dim, v_head_dim, q_weight, k_weight, eps, q_out, cache, slot_map):
        """Rows ``[q | k | v]`` (fp32 or bf16): every q head and every k head is RMS-normed over its ``head_dim`` values with a
        weight of that size which all heads share (None: the part stays as it is); q goes to ``q_out`` ([T, heads * head_dim],
        the cache's dtype), k and v to ``cache`` at the rows ``slot_map`` names (values transposed inside their page)."""
        self.settle()
        self._whole(qkv)
        self._scaled.pop(q_out.data_ptr(), None)
        T = qkv.shape[0]
        QD, KD, VD = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * v_head_dim
        for w, what in ((q_weight, "q"), (k_weight, "k")):
            if w is not None and (w.dtype != torch.float32 or w.numel() != head_dim or not w.is_contiguous()):
                fail(EINVAL, f"head_norm_store: the {what} weight must be {head_dim} contiguous fp32 values")
        if qkv.shape[1] < QD + KD + VD or tuple(q_out.shape) != (T, QD) or q_out.dtype != cache.k.dtype:
            fail(EINVAL, "head_norm_store: rows of q, k and v in; queries of the cache's dtype out")
        for c, width in ((cache.k, KD), (cache.v, VD)):
            if c.dim() != 2 or c.shape[1] != width or not c.is_contiguous():
                fail(EINVAL, f"head_norm_store: the cache must have one row of {width} values per token")
        self._check(self.lib.hfa_head_norm_store(
            qkv.data_ptr(), _code(qkv), _rows(qkv, "qkv"), n_heads, n_kv_heads, head_dim, v_head_dim,
            None if q_weight is None else q_weight.data_ptr(), None if k_weight is None else k_weight.data_ptr(), float(eps),
            q_out.data_ptr(), _rows(q_out, "queries"), cache.k.data_ptr(), cache.v.data_ptr(), _code(cache.k),
            _ints(slot_map, "slot_map", T), cache.page_tokens, T, self._stream()))

    def talk_mix(self, cross, talk, n_heads, n_kv_heads, v_head_dim, out, gate=None):
        """``out[t, h] = sigmoid(gate[t, h]) * sum_g talk[h, g] A[t, g, group of h]``: the heads' attention weights mixed after
        the softmax, as the same mix of what each head's weights give on the values of h's group. ``cross`` is
        ``paged_attention(..., cross_values=True)``'s output, ``talk`` fp32 [heads, heads]; ``gate`` None: no gate."""
        self.settle()
        self._scaled.pop(out.data_ptr(), None)
        T = out.shape[0]
        OD = n_heads * v_head_dim
        if tuple(cross.shape) != (T, n_kv_heads * OD) or not cross.is_contiguous() or out.shape[1] != OD \
                or talk.dtype != torch.float32 or tuple(talk.shape) != (n_heads, n_heads) or not talk.is_contiguous():
            fail(EINVAL, "talk_mix: cross [T, groups * heads * v_head_dim], talk fp32 [heads, heads], out [T, heads * v_head_dim]")
        if gate is not None:
            self._whole(gate)
            if gate.shape[0] != T or gate.shape[1] != OD:
                fail(EINVAL, "talk_mix: the gate has the output's shape")
        self._check(self.lib.hfa_talk_mix(cross.data_ptr(), _code(cross), talk.data_ptr(), None if gate is None else gate.data_ptr(),
                                          0 if gate is None else _code(gate), 0 if gate is None else _rows(gate, "gate"),
                                          out.data_ptr(), _code(out), _rows(out, "talk_mix out"), T, n_heads, n_kv_heads, v_head_dim,
                                          self._stream()))

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

    def _rows_call(self, mode, a, w, N, bias, scaled=None, out=None, x=None, ssq_out=None, g=None, xg=None, act=None, out_act=0):
        M, K = a.shape
        null = ctypes.c_void_p(None)

        def ptr(t):
            return null if t is None else t.data_ptr()
        self._check(self.lib.hfa_gemm_rows(
            mode, a.data_ptr(), _rows(a, "gemm a"), w.data_ptr(), _rows(w, "gemm w"), M, N, K, ptr(bias),
            ptr(None if scaled is None else scaled.ssq), self.rows_parts, 1.0 / K, 0.0 if scaled is None else scaled.eps,
            ptr(out), 0 if out is None else _rows(out, "gemm out"), 0 if out is None else _code(out), int(out_act),
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

    def gemm(self, a, w, out, bias=None, accumulate=False, defer=False, swiglu=False, activation=None):
        """out (+)= a @ w.T + bias, fp32 accumulation. ``defer``: if the kernel split K, leave the
        partial sums for the next kernel that reads ``out`` (see the module's text).
        ``swiglu``: w's rows come in blocks of 32 gate, 32 up (``interleave_gate_up``) and
        out = silu(gate) * up has half as many columns. ``activation``: ``out = act(a @ w.T + bias)`` (see ``activation``)."""
        act = 0
        if activation is not None:
            if accumulate or swiglu or defer:
                fail(EINVAL, "gemm: an activation goes with a plain output that is finished at once")
            if activation not in self.ACTIVATIONS:
                fail(ENOTSUP, f"activation '{activation}' is not one of {', '.join(sorted(self.ACTIVATIONS))}")
            act = self.ACTIVATIONS[activation]           # the product's last lines apply it
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
                self._rows_call(0, a, w, N, bias, scaled=scaled, out=out, out_act=act)
            return
        if scaled is not None:
            self._whole(a)
        self._scaled.pop(out.data_ptr(), None)
        if accumulate:
            self._source_changes(out)
        self._splits_out.value = 0
        self._check(self.lib.hfa_gemm(a.data_ptr(), _code(a), lda, w.data_ptr(), _code(w), ldw,
                                      None if bias is None else bias.data_ptr(), out.data_ptr(), _code(out), ldo,
                                      1 if accumulate else 0, 1 + act if act else 1 if swiglu else 0, M, N, K, self.workspace.data_ptr(),
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
        # rows of q, k and v of a layer that stores, or rows of q alone of a layer that reads what another layer stored
        stores = slot_map is not None and n_kv_heads > 0
        reads = slot_map is None and n_kv_heads == 0 and getattr(cache, "k", None) is not None and cache.k.shape[1] % head_dim == 0
        if lazy and self.fuse_rows and pend is not None and pend.splits == 1 and pend.bias is None and not pend.accumulate \
                and pend.out.data_ptr() == qkv.data_ptr() and pend.out.shape == qkv.shape and qkv.shape[1] == row_width \
                and qkv.dtype == torch.bfloat16 and (stores or reads) and v_head_dim == head_dim \
                and qkv.is_contiguous() and getattr(cache, "k", None) is not None and cache.k.dtype == torch.bfloat16 \
                and cache.k.numel() < 1 << 32 and cache.k.shape[0] < 1 << 24 \
                and self.lib.hfa_decode_attention_supports(n_heads, n_kv_heads or cache.k.shape[1] // head_dim, head_dim, rot_dim,
                                                           cache.page_tokens, cache.k.shape[1], row_width, n_heads * head_dim):
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
                        v_head_dim=None, mask_chunk=0, sink=False, cross_values=False, softcap=0.0, weights="softmax", head_bias=None):
        """Attention of the first ``n_heads * head_dim`` columns of ``q`` over ``cache``. ``slopes``
        (fp32, one per query head): the score of key j for the query at p gets ``slopes[h] * (j - p)``
        added, for position encodings that enter the scores; the plain kernel then runs, as it does when
        value heads have a size of their own (``v_head_dim``; ``out`` then has that many columns a head).
        ``mask_chunk`` > 0: a query sees only the keys of its own run of that many positions, counted from 0.
        ``sink``: the softmax's denominator holds one more term of score 0 that has no value. ``cross_values``: every
        head's weights are applied to the values of every key/value group; ``out`` is ``[T, groups * heads * v_head_dim]``,
        round r of head h (at ``(r * heads + h) * v_head_dim``) being its weights on the values of group (h's group + r) mod
        groups (see ``talk_mix``). ``softcap`` c > 0: a score becomes ``c tanh(score / c)`` before the weights are formed.
        ``weights`` ``"sigmoid"``: no softmax; a visible key weighs ``sigmoid(score + head_bias[h])`` (``head_bias``: fp32, one per
        query head, or None), and the weights are not normalised over the keys (on the matrix cores where a softmax would be; a cap under a softmax takes the plain kernel)."""
        v_head_dim = head_dim if v_head_dim is None else int(v_head_dim)
        mask_chunk = int(mask_chunk)
        if weights not in ("softmax", "sigmoid") or (weights == "sigmoid" and (sink or cross_values)):
            fail(ENOTSUP, f"paged_attention: weights '{weights}' are softmax or sigmoid (the latter without a sink term or mixed heads)")
        if head_bias is not None and (weights != "sigmoid" or head_bias.dtype != torch.float32 or head_bias.numel() != n_heads
                                      or not head_bias.is_contiguous() or head_bias.device != q.device):
            fail(EINVAL, "paged_attention: head_bias goes with sigmoid weights and is contiguous fp32 on the device, one per query head")
        softcap = float(softcap or 0.0)
        shaped_scores = softcap != 0.0 or weights != "softmax"
        plain_scores = softcap != 0.0 and weights == "softmax"        # what only the plain kernel computes
        self._scaled.pop(out.data_ptr(), None)               # whatever `out` held, it is no norm's lazy output any more
        lr = self._lazy_rope
        if lr is not None and lr.qkv.data_ptr() == q.data_ptr() and lr.cache is cache and slopes is None and not sink \
                and not cross_values and not shaped_scores \
                and step.max_q_len == 1 and step.n_seqs == q.shape[0] and not self.force_plain_attention \
                and out.dtype == torch.bfloat16 and v_head_dim == head_dim and lr.args[4] == n_heads and lr.args[6] == head_dim \
                and lr.args[5] in (0, n_kv_heads) and cache.k.shape[1] == n_kv_heads * head_dim \
                and cache.k.numel() < 1 << 32 and cache.k.shape[0] < 1 << 24:
            return self._decode_attention(lr, step, window, scale, out, mask_chunk, n_kv_heads)
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
        if cross_values and out.shape[1] != n_kv_heads * n_heads * v_head_dim:
            fail(EINVAL, "paged_attention: with cross_values the output holds groups * heads * v_head_dim columns")
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
                n_kv_heads, head_dim, v_head_dim, cache.page_tokens, int(window), mask_chunk, float(scale),
                None if slopes is None else slopes.data_ptr(), 1 if sink else 0, 1 if cross_values else 0, softcap,
                1 if weights == "sigmoid" else 0, None if head_bias is None else head_bias.data_ptr(), self.attn_workspace.data_ptr(),
                self.attn_workspace.numel(), 1 if plain else 0, self._stream()))

        # Decoded tokens beside prompt portions: one call would send all of them to the kernel for prompt
        # portions, which walks a request's keys in one piece (a decoded token with a long context would
        # take as long as thousands of prompt tokens). The step lays requests with few tokens first, so
        # each part is a step of its own: the first goes to the kernel that cuts the keys into chunks.
        n_short = getattr(step, "n_short_seqs", 0)
        if not plain and not plain_scores and v_head_dim == head_dim and q.dtype == torch.bfloat16 \
                and step.max_q_len >= self.prompt_rows and 0 < n_short < step.n_seqs:
            ts = step.n_short_tokens
            _ints(step.q_start_long, "q_start_long", step.n_seqs - n_short + 1)
            call(0, ts, step.q_start, n_short, step.max_short_q_len)
            call(ts, T - ts, step.q_start_long, step.n_seqs - n_short, step.max_q_len)
        else:
            call(0, T, step.q_start, step.n_seqs, step.max_q_len)

    def _decode_attention(self, lr, step, window, scale, out, mask_chunk=0, kv_heads=None):
        """Rotation, the store of the new keys and values and attention over the cache for decoded tokens, in one
        kernel: the queued ``rope_store`` (``lr``) and this call together."""
        qkv, positions, inv_freq, rot_dim, n_heads, n_kv_heads, head_dim, cache, slot_map, _ = lr.args
        n_kv_heads = n_kv_heads or kv_heads          # a layer that only reads: its rows hold no keys, the cache says how many heads
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
            cache.v.data_ptr(), cache.k.shape[1], None if slot_map is None else _ints(slot_map, "slot_map", T), g.block_table.data_ptr(),
            g.block_table.shape[1], _ints(step.token_slot, "token_slot", T), _ints(step.positions, "positions", T),
            _ints(step.q_start, "q_start", T + 1), T, step.max_seq_len, out.data_ptr(), _rows(out, "attention out"),
            n_heads, n_kv_heads, head_dim, cache.page_tokens, int(window), int(mask_chunk), float(scale),
            self.attn_workspace.data_ptr(),
            self.attn_workspace.numel(), self._stream()))

    def swiglu(self, gate_up, out):
        self.settle()
        self._scaled.pop(out.data_ptr(), None)
        T, F2 = gate_up.shape
        if not gate_up.is_contiguous() or not out.is_contiguous() or tuple(out.shape) != (T, F2 // 2) \
                or out.dtype != gate_up.dtype or F2 % 2:
            fail(EINVAL, "swiglu: expected contiguous [T, 2F] in and [T, F] out of one dtype")
        self._check(self.lib.hfa_swiglu(gate_up.data_ptr(), out.data_ptr(), _code(out), T, F2 // 2, self._stream()))

    # ---- norms in groups, queries and keys normed whole, mixers with per-request state -------------------------------
    GATES = {None: 0, "silu_before": 1, "sigmoid_after": 2, "silu_after": 3}

    def group_rmsnorm(self, x, weight, eps, groups, out, rows=None, gate=None, gate_kind=None, row_scale=None):
        """``out[r] = norm(x[rows[r]])``: the row is cut into ``groups`` equal runs, each divided by its own root mean
        square (``eps`` inside the root), the whole times ``weight``; sums in fp32. ``gate`` (a matrix with the rows of
        ``out``) with ``gate_kind`` ``silu_before`` (the row times silu(gate) is normed), ``sigmoid_after`` (the normed
        row is multiplied by sigmoid(gate)) or ``silu_after`` (by silu(gate)). ``row_scale`` (fp32 [rows, groups]): run g of row r is multiplied by
        ``row_scale[r, g]`` before everything else (a recurrence's denominator, a head at a time)."""
        self.settle()
        self._whole(x)
        self._scaled.pop(out.data_ptr(), None)
        R, E = out.shape
        if gate_kind not in self.GATES or (gate is None) != (gate_kind is None):
            fail(EINVAL, f"group_rmsnorm: a gate comes with its kind, one of {', '.join(k for k in self.GATES if k)}")
        if x.shape[1] != E or weight.dtype != torch.float32 or weight.numel() != E or not weight.is_contiguous() or E % int(groups):
            fail(EINVAL, f"group_rmsnorm: rows of {x.shape[1]}, {weight.numel()} fp32 weights, rows of {E} out, {groups} equal runs")
        if rows is None and R != x.shape[0]:
            fail(EINVAL, "group_rmsnorm: without row indices the output must have x's rows")
        if gate is not None and (gate.shape[0] != R or gate.shape[1] != E or rows is not None):
            fail(EINVAL, "group_rmsnorm: the gate has the output's shape, and no rows are gathered with it")
        if row_scale is not None and (rows is not None or row_scale.dtype != torch.float32 or not row_scale.is_contiguous()
                                      or tuple(row_scale.shape) != (R, int(groups))):
            fail(EINVAL, "group_rmsnorm: row_scale is fp32 [rows, groups], and no rows are gathered with it")
        self._check(self.lib.hfa_group_rmsnorm(
            x.data_ptr(), _code(x), _rows(x, "norm in"), weight.data_ptr(), out.data_ptr(), _code(out), _rows(out, "norm out"),
            None if rows is None else _ints(rows, "norm rows", R), R, E, int(groups), float(eps),
            None if gate is None else gate.data_ptr(), 0 if gate is None else _code(gate),
            0 if gate is None else _rows(gate, "norm gate"), self.GATES[gate_kind],
            None if row_scale is None else row_scale.data_ptr(), self._stream()))

    PAIRINGS = {"split_half": 0, "interleaved": 1}

    def qkv_prepare(self, qkv, positions, inv_freq, rot_dim, pairing, n_heads, n_kv_heads, head_dim, v_head_dim, cache, slot_map,
                    q_norm=None, k_norm=None, eps=0.0, v_blend=None, v_other=None, v_keep=None):
        """What lies between the q/k/v product and attention when ``rope_store`` does not do: rows ``[q | k | v]``;
        ``q_norm`` / ``k_norm`` (fp32 weights over the whole q part / k part): RMS norm of that part before the rotation;
        rotation of the first ``rot_dim`` dimensions of each head in ``pairing`` (``split_half``: i with i + rot_dim/2;
        ``interleaved``: 2i with 2i + 1); ``v_blend`` (a scalar on the device) and ``v_other`` ([T, values]):
        ``v <- (1 - v_blend) v + v_blend v_other``; ``v_keep`` ([T, values]) receives the values as projected. Keys and
        values go to ``cache`` at ``slot_map`` (values transposed inside their page)."""
        self.settle()
        self._whole(qkv)
        if pairing not in self.PAIRINGS:
            fail(ENOTSUP, f"rotary pairing '{pairing}' is not one of {', '.join(self.PAIRINGS)}")
        T = qkv.shape[0]
        QD, KD, VD = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * v_head_dim
        if qkv.shape[1] < QD + KD + VD:
            fail(EINVAL, "qkv_prepare: the rows are narrower than the heads they should hold")
        for w, n, what in ((q_norm, QD, "q_norm"), (k_norm, KD, "k_norm")):
            if w is not None and (w.dtype != torch.float32 or w.numel() != n or not w.is_contiguous()):
                fail(EINVAL, f"qkv_prepare: {what} must be {n} contiguous fp32 weights")
        for t, what in ((v_other, "v_other"), (v_keep, "v_keep")):
            if t is not None and (t.dtype != qkv.dtype or tuple(t.shape) != (T, VD) or not t.is_contiguous()):
                fail(EINVAL, f"qkv_prepare: {what} must be [{T}, {VD}] of the rows' dtype")
        if (v_blend is None) != (v_other is None) or (v_blend is not None and (v_blend.dtype != torch.float32 or v_blend.numel() != 1)):
            fail(EINVAL, "qkv_prepare: blending needs one fp32 weight on the device and the other values")
        k_ptr = v_ptr = None
        if slot_map is not None:
            for c, width in ((cache.k, KD), (cache.v, VD)):
                if c.dtype != qkv.dtype or c.dim() != 2 or c.shape[1] != width or not c.is_contiguous():
                    fail(EINVAL, f"qkv_prepare: the cache must have the activations' dtype and one row of {width} values per token")
            k_ptr, v_ptr = cache.k.data_ptr(), cache.v.data_ptr()

        def ptr(t):
            return None if t is None else t.data_ptr()
        self._check(self.lib.hfa_qkv_prepare(
            qkv.data_ptr(), _code(qkv), _rows(qkv, "qkv"), None if rot_dim == 0 else _ints(positions, "positions", T),
            None if rot_dim == 0 else inv_freq.data_ptr(), int(rot_dim), self.PAIRINGS[pairing], n_heads, n_kv_heads, head_dim,
            v_head_dim, ptr(q_norm), ptr(k_norm), float(eps), ptr(v_blend), ptr(v_other), ptr(v_keep), k_ptr, v_ptr,
            None if slot_map is None else _ints(slot_map, "slot_map", T), getattr(cache, "page_tokens", 0) or 0, T, self._stream()))

    def causal_conv(self, x, taps, bias, state, step, out, activation=None):
        """``out[t, c] = act(bias[c] + sum_j taps[c, j] x[t - (K - 1) + j, c])`` along each request's tokens (fp32 out);
        the K - 1 inputs before a request's first token of this step come from its row of ``state`` ([slots, >= (K - 1) C]
        fp32, oldest input first), which then receives the step's last K - 1 inputs. ``activation``: ``silu`` or None."""
        self.settle()
        self._whole(x)
        T, C = out.shape
        K = taps.shape[1]
        if taps.dtype != torch.float32 or not taps.is_contiguous() or taps.shape[0] != C or x.shape[0] != T or x.shape[1] != C \
                or out.dtype != torch.float32 or state.dtype != torch.float32 or state.stride(1) != 1 or state.shape[1] < (K - 1) * C \
                or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != C or not bias.is_contiguous())):
            fail(EINVAL, "causal_conv: taps [channels, taps] and bias fp32, fp32 output and state, one width for all")
        if activation not in (None, "silu"):
            fail(ENOTSUP, f"causal_conv: activation '{activation}' is neither silu nor None")
        self._check(self.lib.hfa_causal_conv(
            x.data_ptr(), _code(x), _rows(x, "conv in"), taps.data_ptr(), None if bias is None else bias.data_ptr(), C, K,
            state.data_ptr(), state.stride(0), _ints(step.q_start, "q_start", step.n_seqs + 1),
            _ints(step.seq_slot, "seq_slot", step.n_seqs), step.n_seqs, step.max_q_len, out.data_ptr(), _rows(out, "conv out"),
            self.ACTIVATIONS["silu"] if activation else 0, self._stream()))

    @staticmethod
    def scan_state_floats(n_heads, qk_dim, v_dim, normalizer=False):
        """The fp32 values of a request's state row that ``linear_scan`` needs for ``n_heads`` states of ``qk_dim`` x ``v_dim``:
        the kernel keeps them in the order its lanes read them, both sizes padded to what a block walks (the library's
        ``hfa_linear_scan_state_floats``, mirrored here so that a cache can be planned without the library). ``normalizer``
        (exponential gates): one more column a head, and the running maximum once for every block of columns."""
        lanes = 16 if qk_dim >= 64 else 8 if qk_dim > 16 else 4
        per = -(-qk_dim // lanes)
        per = 4 if per <= 4 else 8 if per <= 8 else 16
        columns = 256 // lanes
        if normalizer:
            blocks = -(-(v_dim + 1) // columns)
            return n_heads * lanes * per * blocks * columns + n_heads * blocks
        return n_heads * lanes * per * (-(-v_dim // columns) * columns)

    def linear_scan(self, q, k, v, qk_heads, qk_dim, n_heads, v_dim, state, step, y, decay=None, step_size=None,
                    step_bias=None, a_log=None, skip=None, exp_gates=None, q_scale=1.0, denom=None):
        """The recurrence over a matrix state per head, along each request's tokens from its row of ``state`` ([slots, >=
        ``scan_state_floats``] fp32, in the kernel's own order, left there for the next step): ``S <- a_t S + k_t (b_t v_t)^T``, ``y_t = S^T q_t +
        skip[h] v_t`` (fp32). Head h reads queries and keys of head ``h // (n_heads / qk_heads)``. With ``decay`` (fp32, one
        per head): ``a_t = decay[h]``, ``b_t = 1``. With ``step_size`` ([T, heads]), ``step_bias`` and ``a_log`` (fp32 per head):
        ``dt = softplus(step_size + step_bias)``, ``a_t = exp(-exp(a_log) dt)``, ``b_t = dt``. With ``exp_gates`` = (i [T, heads],
        f [T, heads], i_bias, f_bias (fp32 per head), cap): exponential input gates and sigmoid forget gates, both soft-capped,
        under a running maximum m that is kept beside the states (``scan_state_floats(..., normalizer=True)``):
        ``li = cap tanh((i + i_bias) / cap)``, ``lf = logsigmoid(cap tanh((f + f_bias) / cap))``, ``m_t = max(lf + m, li)``,
        ``a_t = exp(lf + m - m_t)``, ``b_t = exp(li - m_t)``; the state carries ``n_t = a_t n + b_t k_t`` as one more column and
        ``denom`` (fp32 [T, heads]) receives ``1 / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)``, by which the reader multiplies
        ``y``. ``q_scale`` multiplies the queries."""
        self.settle()
        for t in (q, k, v):
            self._whole(t)
        T = y.shape[0]
        gate = 0 if decay is not None else 2 if exp_gates is not None else 1
        gi = gf = gib = gfb = None
        cap = 0.0
        if gate == 2:
            gi, gf, gib, gfb, cap = exp_gates
            step_size, step_bias = gi, gib
            if gf.dtype != gi.dtype or gf.shape != gi.shape or _rows(gf, "scan f") != _rows(gi, "scan i") or gfb.dtype != torch.float32 \
                    or gfb.numel() != n_heads or denom is None or denom.dtype != torch.float32 or tuple(denom.shape) != (T, n_heads) \
                    or not denom.is_contiguous() or skip is not None or not cap > 0.0:
                fail(EINVAL, "linear_scan: exponential gates are (i, f, i_bias, f_bias, cap > 0) with i and f alike, and denom fp32 [T, heads]")
        if q.dtype != k.dtype or q.dtype != v.dtype or y.dtype != torch.float32 or state.dtype != torch.float32 \
                or state.stride(1) != 1 or q.shape[0] != T or k.shape[0] != T or v.shape[0] != T or y.shape[1] != n_heads * v_dim:
            fail(EINVAL, "linear_scan: q, k and v of one dtype and the step's rows, fp32 output and state")
        for t, what in ((decay, "decay"), (step_bias, "step_bias"), (a_log, "a_log"), (skip, "skip")):
            if t is not None and (t.dtype != torch.float32 or t.numel() != n_heads or not t.is_contiguous()):
                fail(EINVAL, f"linear_scan: {what} must be one fp32 value a head")
        if state.shape[1] < self.scan_state_floats(n_heads, qk_dim, v_dim, normalizer=gate == 2) or qk_dim > 256:
            fail(EINVAL, f"linear_scan: a state row of {state.shape[1]} values for {n_heads} states of {qk_dim} x {v_dim} (at most 256 rows)")
        if gate == 2 and step_size.shape[0] != T:
            fail(EINVAL, "linear_scan: the gates' inputs have the step's rows")
        if gate == 1 and (step_size is None or step_bias is None or a_log is None or step_size.shape[0] != T):
            fail(EINVAL, "linear_scan: without a fixed decay give step_size, step_bias and a_log")

        def ptr(t):
            return None if t is None else t.data_ptr()
        self._check(self.lib.hfa_linear_scan(
            q.data_ptr(), _rows(q, "scan q"), k.data_ptr(), _rows(k, "scan k"), qk_heads, qk_dim, v.data_ptr(), _rows(v, "scan v"),
            n_heads, v_dim, _code(q), gate, ptr(decay), ptr(step_size), 0 if step_size is None else _code(step_size),
            0 if step_size is None else _rows(step_size, "scan step"), ptr(step_bias), ptr(a_log), ptr(skip), state.data_ptr(),
            state.stride(0), _ints(step.q_start, "q_start", step.n_seqs + 1), _ints(step.seq_slot, "seq_slot", step.n_seqs),
            step.n_seqs, y.data_ptr(), _rows(y, "scan out"), ptr(gf), ptr(gfb), float(cap), float(q_scale), ptr(denom), self._stream()))

    def delta_scan(self, q, k, v, qk_heads, qk_dim, n_heads, v_dim, a, dt_bias, a_log, b, state, step, y, q_scale=1.0, unit_eps=1e-6):
        """The gated delta rule over a matrix state per head, along each request's tokens from its row of ``state`` (fp32,
        ``scan_state_floats`` values in ``linear_scan``'s order): ``g_t = exp(-exp(a_log[h]) softplus(a[t, h] + dt_bias[h]))``, one
        decay per key channel (``a`` [T, heads * qk_dim], ``dt_bias`` [heads * qk_dim]); ``S <- g_t * S`` row by row;
        ``u = sigmoid(b[t, h]) (v_t - S^T k_t)``; ``S <- S + k_t u^T``; ``y_t = S^T q_t``. ``q_t`` and ``k_t`` are first divided
        by ``sqrt(sum of squares + unit_eps)`` and ``q_t`` multiplied by ``q_scale``. Head h reads queries and keys of head
        ``h // (n_heads / qk_heads)``. Every input is fp32, as is every operation."""
        self.settle()
        T = y.shape[0]
        for t, what in ((q, "q"), (k, "k"), (v, "v"), (a, "a"), (b, "b"), (y, "y"), (state, "state")):
            if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or (what != "state" and t.shape[0] != T):
                fail(EINVAL, f"delta_scan: {what} must be an fp32 matrix with the step's rows")
        if dt_bias.dtype != torch.float32 or dt_bias.numel() != n_heads * qk_dim or not dt_bias.is_contiguous() \
                or a_log.dtype != torch.float32 or a_log.numel() != n_heads or not a_log.is_contiguous():
            fail(EINVAL, "delta_scan: dt_bias is one fp32 value a (head, key channel), a_log one a head")
        if state.shape[1] < self.scan_state_floats(n_heads, qk_dim, v_dim) or qk_dim > 256 or y.shape[1] != n_heads * v_dim \
                or a.shape[1] < n_heads * qk_dim or b.shape[1] < n_heads:
            fail(EINVAL, f"delta_scan: a state row of {state.shape[1]} values for {n_heads} states of {qk_dim} x {v_dim} (at most 256 rows)")
        self._check(self.lib.hfa_delta_scan(
            q.data_ptr(), _rows(q, "scan q"), k.data_ptr(), _rows(k, "scan k"), qk_heads, qk_dim, v.data_ptr(), _rows(v, "scan v"),
            n_heads, v_dim, a.data_ptr(), _rows(a, "scan a"), dt_bias.data_ptr(), a_log.data_ptr(), b.data_ptr(), _rows(b, "scan b"),
            float(q_scale), float(unit_eps), state.data_ptr(), state.stride(0), _ints(step.q_start, "q_start", step.n_seqs + 1),
            _ints(step.seq_slot, "seq_slot", step.n_seqs), step.n_seqs, int(step.max_q_len), y.data_ptr(), _rows(y, "scan out"), self._stream()))

    def channel_scan(self, q, k, v, n_heads, qk_dim, v_dim, gate, gate_bias, state, step, y, lower=None, tau=None, q_act=None,
                     q_scale=1.0):
        """A recurrence with a decay per key channel, along each request's tokens from its row of ``state`` (fp32,
        ``scan_state_floats`` values in ``linear_scan``'s order): ``S <- diag(a_t) S + k_t v_t^T``, ``y_t = S^T (q_scale q_t)`` (fp32).
        The decays are formed in fp32 from ``z = gate[t] + gate_bias`` ([T, heads * qk_dim], the bias fp32 or None). With ``lower``
        (fp32 [heads * qk_dim]): ``a = lower + (1 - lower) sigmoid(z)`` and ``k_t = 1 - a_t`` (``k`` is None: the forget gate decides
        what is written). With ``tau``: ``a = sigmoid(z)^(1 / tau)``, keys from ``k``. ``q_act`` ``"silu"``: the queries pass silu first."""
        self.settle()
        for t in (q, k, v, gate):
            if t is not None:
                self._whole(t)
        T = y.shape[0]
        form = 0 if lower is not None else 1
        if (lower is None) == (tau is None) or (form == 1) != (k is not None):
            fail(EINVAL, "channel_scan: either lower bounds and no keys, or tau and keys")
        if q.dtype != v.dtype or (k is not None and k.dtype != q.dtype) or y.dtype != torch.float32 or state.dtype != torch.float32 \
                or state.stride(1) != 1 or q.shape[0] != T or v.shape[0] != T or gate.shape[0] != T or y.shape[1] != n_heads * v_dim:
            fail(EINVAL, "channel_scan: q, k and v of one dtype and the step's rows, fp32 output and state")
        for t, what in ((gate_bias, "gate_bias"), (lower, "lower")):
            if t is not None and (t.dtype != torch.float32 or t.numel() != n_heads * qk_dim or not t.is_contiguous()):
                fail(EINVAL, f"channel_scan: {what} must be one fp32 value a (head, key channel)")
        if state.shape[1] < self.scan_state_floats(n_heads, qk_dim, v_dim) or qk_dim > 256:
            fail(EINVAL, f"channel_scan: a state row of {state.shape[1]} values for {n_heads} states of {qk_dim} x {v_dim} (at most 256 rows)")
        if q_act not in (None, "silu"):
            fail(ENOTSUP, f"channel_scan: the queries pass silu or nothing, not '{q_act}'")

        def ptr(t):
            return None if t is None else t.data_ptr()
        # the decays once a (token, head, channel), not once more in every block of a head's columns
        inv_tau = 0.0 if tau is None else 1.0 / float(tau)
        decays = self.scratch("channel_decays", (T, n_heads * qk_dim), torch.float32)
        self._check(self.lib.hfa_channel_decay(gate.data_ptr(), _code(gate), _rows(gate, "scan gate"), ptr(gate_bias), form, ptr(lower), inv_tau,
                                               decays.data_ptr(), _rows(decays, "decays"), T, n_heads * qk_dim, self._stream()))
        self._check(self.lib.hfa_channel_scan(
            q.data_ptr(), _rows(q, "scan q"), ptr(k), 0 if k is None else _rows(k, "scan k"), v.data_ptr(), _rows(v, "scan v"), _code(q),
            decays.data_ptr(), _rows(decays, "decays"), 1 if form == 0 else 0, self.ACTIVATIONS["silu"] if q_act else 0, n_heads, qk_dim,
            v_dim, float(q_scale), state.data_ptr(), state.stride(0), _ints(step.q_start, "q_start", step.n_seqs + 1),
            _ints(step.seq_slot, "seq_slot", step.n_seqs), step.n_seqs, y.data_ptr(), _rows(y, "scan out"), self._stream()))

    def scale_add(self, y, out, scale=1.0, columns=None, accumulate=True):
        """``out (+)= scale * columns * y`` in fp32, ``columns`` an fp32 vector with one factor a column (None: 1): a branch's
        result on its way into the stream."""
        self.settle()
        self._source_changes(out)
        self._scaled.pop(out.data_ptr(), None)
        R, E = y.shape
        if y.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (R, E) \
                or (columns is not None and (columns.dtype != torch.float32 or columns.numel() != E or not columns.is_contiguous())):
            fail(EINVAL, "scale_add: y, out and the columns' factors must be fp32 and of one width")
        self._check(self.lib.hfa_scale_add(y.data_ptr(), _rows(y, "scale_add in"), None if columns is None else columns.data_ptr(),
                                           float(scale), out.data_ptr(), _rows(out, "scale_add out"), R, E, 1 if accumulate else 0,
                                           self._stream()))

    def gate_mul(self, x, gate, out, kind="sigmoid"):
        """``out = x * act(gate)`` element by element, formed in fp32; ``kind`` is ``sigmoid`` or ``silu``. ``out`` may be ``x``."""
        self.settle()
        self._whole(x)
        self._whole(gate)
        self._scaled.pop(out.data_ptr(), None)
        if kind not in ("sigmoid", "silu") or x.shape != gate.shape or x.shape != out.shape or x.dim() != 2:
            fail(EINVAL, "gate_mul: x, gate and out of one shape; the gate's function is sigmoid or silu")
        self._check(self.lib.hfa_gate_mul(x.data_ptr(), _code(x), _rows(x, "gate_mul x"), gate.data_ptr(), _code(gate), _rows(gate, "gate"),
                                          out.data_ptr(), _code(out), _rows(out, "gate_mul out"), x.shape[0], x.shape[1],
                                          self.ACTIVATIONS[kind], self._stream()))

    def head_products(self, a, w, out, n_heads):
        """``out[t * H + h, :] = w[h] @ a[t * H + h, :K]``: a product per head, every head with a matrix of its own. ``a`` is
        ``[T * H, >= K]`` (the heads' rows of all tokens, a token's heads one after the other), ``w`` ``[H, N, K]`` and ``out``
        ``[T * H, >= N]``; both are usually views of ``[T, H * width]`` matrices. The heads are the experts of the grouped product
        that the mixture of experts runs (``hfa_moe_plan``, ``hfa_moe_gemm``): one launch for all heads, on the matrix cores
        where the sizes allow."""
        self.settle()
        self._whole(a)
        self._scaled.pop(out.data_ptr(), None)
        R, H = a.shape[0], int(n_heads)
        if w.dim() != 3 or not w.is_contiguous() or w.shape[0] != H or R % H or out.shape[0] != R or a.shape[1] < w.shape[2] \
                or out.shape[1] < w.shape[1] or (w.dtype != a.dtype and w.dtype != torch.float32):
            fail(EINVAL, "head_products: a [T * heads, >= K], w [heads, N, K] contiguous, out [T * heads, >= N]")
        N, K = int(w.shape[1]), int(w.shape[2])
        code, wcode = _code(a), _code(w)
        plain = 1 if self.force_plain_gemm else 0
        tile_rows = 32 if plain else int(self.lib.hfa_moe_tile_rows(code, wcode, R, H, N, K))
        max_tiles = R // tile_rows + H
        key = ("head ids", H)
        ids = self._shared.get(key)
        if ids is None or ids.shape[0] * H < R:           # head h is the h-th choice of every token
            if torch.cuda.is_current_stream_capturing():
                fail(EINVAL, "head_products: the table of heads would have to grow while a graph is being captured")
            rows = max(1024, 2 * (R // H))
            if ids is not None:                           # captured graphs may still read the smaller table: it stays alive
                self._shared[key + (ids.shape[0],)] = ids
            ids = memory.to_device(torch.arange(H, dtype=torch.int32).repeat(rows, 1), self.device, "the heads as choices of every token")
            self._shared[key] = ids
        row_pair = self.scratch("heads_row_pair", (R,), torch.int32)
        tiles = self.scratch("heads_tiles", (3 * max_tiles + 1,), torch.int32)
        n_tiles = tiles[3 * max_tiles:]
        self._check(self.lib.hfa_moe_plan(ids.data_ptr(), R, H, tile_rows, row_pair.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr(),
                                          self._stream()))
        self._check(self.lib.hfa_moe_gemm(a.data_ptr(), _rows(a, "head rows"), code, 1, w.data_ptr(), wcode, row_pair.data_ptr(),
                                          tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, out.data_ptr(), _rows(out, "head out"),
                                          _code(out), 1, None, 0, N, K, plain, 0, 0.0, 0.0, 0.0, self._stream()))

    def latent_pack(self, down, q, weight, eps, packed, n_heads, dim, rot, latent, folded=None):
        """The rows that ``rope_store`` and ``paged_attention`` take for attention through latents with one key/value head
        (key ``[rotated part | latent]``, value the latent): from ``down`` (fp32 [T, latent + rot]: the latent before its norm, then
        the key's part to be rotated) and ``q`` ([T, heads * (dim + rot)], a head being ``[dim | rot]``) it writes
        ``packed[t] = [heads x (rot | latent: left alone) | rot | latent | latent]``, the latent RMS-normed with ``weight``. ``folded``
        (``[T, heads * latent]``): the heads' queries with the keys' expansion folded in, copied into the heads' latent parts."""
        self.settle()
        self._whole(q)
        if folded is not None and (folded.shape[0] != down.shape[0] or folded.shape[1] < n_heads * latent or folded.dtype != q.dtype):
            fail(EINVAL, "latent_pack: the folded queries are [T, heads * latent] of the queries' dtype")
        T = down.shape[0]
        if down.dtype != torch.float32 or down.shape[1] < latent + rot or q.shape[0] != T or q.shape[1] < n_heads * (dim + rot) \
                or packed.shape[0] != T or packed.shape[1] < n_heads * (rot + latent) + rot + 2 * latent \
                or weight.dtype != torch.float32 or weight.numel() != latent or not weight.is_contiguous():
            fail(EINVAL, "latent_pack: rows of the latent and the rotated part (fp32), the heads' queries, an fp32 weight of the latent's size")
        self._check(self.lib.hfa_latent_pack(down.data_ptr(), _rows(down, "latent rows"), q.data_ptr(), _code(q), _rows(q, "queries"),
                                             weight.data_ptr(), float(eps), packed.data_ptr(), _code(packed), _rows(packed, "packed rows"),
                                             T, n_heads, dim, rot, latent, None if folded is None else folded.data_ptr(),
                                             0 if folded is None else _rows(folded, "folded queries"), self._stream()))

    # ---- layer norm, plain activations, soft cap -----------------------------------------------------------------
    def layernorm(self, x, weight, bias, eps, out, rows=None):
        """``out[r] = (x[rows[r]] - mean) / sqrt(var + eps) * weight + bias`` in fp32 (``bias`` None: no shift). A
        deferred product into ``x`` (the residual sum before the norm) is added up by the same kernel."""
        R, E = out.shape[0], x.shape[1]
        if x.dtype != torch.float32 or weight.dtype != torch.float32 or not x.is_contiguous() or not out.is_contiguous() \
                or out.shape[1] != E or weight.numel() != E or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != E)):
            fail(EINVAL, "layernorm: x, weight and bias must be fp32, contiguous, and of one width with out")
        if rows is None and R != x.shape[0]:
            fail(EINVAL, "layernorm: without row indices the output must have x's rows")
        self._scaled.pop(out.data_ptr(), None)
        pend = self._take_pending(x) if rows is None else None
        if pend is None:
            self.settle()
        else:
            self._source_changes(x)
        self._check(self.lib.hfa_layernorm(
            x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(), _code(out),
            None if rows is None else _ints(rows, "layernorm rows", R), R, E, float(eps),
            None if pend is None else self.workspace.data_ptr(), 0 if pend is None else pend.splits,
            None if pend is None or pend.bias is None else pend.bias.data_ptr(), x.shape[0], self._stream()))

    ACTIVATIONS = {"gelu_erf": 1, "gelu_tanh": 2, "relu2": 3, "silu": 4, "sigmoid": 5}

    def activation(self, kind, src, out):
        """``out = act(src)`` elementwise, computed in fp32: ``gelu_erf``, ``gelu_tanh``, ``relu2`` (relu squared), ``silu``
        or ``sigmoid``."""
        if kind not in self.ACTIVATIONS:
            fail(ENOTSUP, f"activation '{kind}' is not one of {', '.join(sorted(self.ACTIVATIONS))}")
        self.settle()
        self._whole(src)
        self._scaled.pop(out.data_ptr(), None)
        if src.shape != out.shape or src.dtype != out.dtype or src.dim() != 2:
            fail(EINVAL, "activation: input and output must be matrices of one shape and dtype")
        self._check(self.lib.hfa_activation(src.data_ptr(), _rows(src, "activation in"), out.data_ptr(), _rows(out, "activation out"),
                                            _code(out), src.shape[0], src.shape[1], self.ACTIVATIONS[kind], self._stream()))

    def softcap(self, x, cap):
        """``x <- cap * tanh(x / cap)`` on fp32 rows, in place."""
        self.settle(x)
        if x.dtype != torch.float32 or x.dim() != 2:
            fail(EINVAL, "softcap: expected an fp32 matrix")
        if x.shape[0]:
            self._check(self.lib.hfa_softcap(x.data_ptr(), _rows(x, "softcap"), x.shape[0], x.shape[1], float(cap), self._stream()))

    # ---- mixture of experts ------------------------------------------------------------------------------------------
    SCORINGS = {"softmax": 0, "sigmoid": 1, "softmax_chosen": 2}

    def moe_route(self, logits, top, n_groups, keep, scoring="softmax", renorm=True, out_scale=1.0):
        """(ids [T, top] int32, weights [T, top] fp32) from fp32 router logits [T, E]: see ``hfa_moe_route``. ``scoring``
        ``softmax_chosen``: the experts with the largest logits, weighted (with ``renorm``) by the softmax over the chosen
        logits alone."""
        self.settle()
        T, E = logits.shape
        if logits.dtype != torch.float32 or scoring not in self.SCORINGS:
            fail(EINVAL, f"moe_route: fp32 logits and a scoring among {', '.join(self.SCORINGS)}")
        ids = self.scratch("moe_ids", (T, top), torch.int32)
        wts = self.scratch("moe_weights", (T, top), torch.float32)
        self._check(self.lib.hfa_moe_route(logits.data_ptr(), _rows(logits, "router logits"), T, E, int(top), int(n_groups), int(keep),
                                           self.SCORINGS[scoring], 1 if renorm else 0, float(out_scale),
                                           ids.data_ptr(), wts.data_ptr(), self._stream()))
        return ids, wts

    def moe_experts(self, h, ids, weights, w_up, w_down, act, x, gated=None, weight_on="input"):
        """``x[t] += sum_k weights[t, k] * w_down[ids[t, k]] act(w_up[ids[t, k]] h[t])``: ``w_up`` is [E, F, width],
        ``w_down`` [E, width, F]. The pairs are put in expert order on the device, each expert's rows go through the
        two products in tiles, and the weighted results are added to ``x`` (fp32) choice by choice.

        ``gated`` = (alpha, limit, shift, interleaved): the experts are gated units whose weight scales their input. ``w_up``
        then is [E, 2F, width], an expert's gate rows before its up rows, or, ``interleaved`` (F a multiple of 32), in blocks of
        32 gate rows and 32 up rows (``interleave_experts``); with ``c = weights[t, k]``, ``g = min(c Wgate h, limit)``, ``u =
        clamp(c Wup h, -limit, limit)`` (``limit`` <= 0: unbounded) the expert gives ``Wdown (g sigmoid(alpha g) (u + shift))``,
        unweighted; ``act`` is ignored. Interleaved, the up product's last lines form the activation from its 32-bit sums;
        otherwise the sums pass through memory and a kernel of its own forms it. ``weight_on`` ``"output"`` (gated experts only;
        experts without a gate always weigh their output): c = 1 inside the expert, and the down product's rows are multiplied
        by the pair's weight instead."""
        self.settle()
        self._whole(h)
        self._source_changes(x)
        T, W = h.shape
        E, F, _ = w_up.shape
        if gated is not None:
            if F % 2:
                fail(EINVAL, "moe_experts: gated experts hold gate and up rows in one matrix of 2F rows")
            F //= 2
        F_up = w_up.shape[1]
        top = ids.shape[1]
        n_pairs = T * top
        if gated is None and act not in self.ACTIVATIONS:
            fail(ENOTSUP, f"activation '{act}' is not one of {', '.join(sorted(self.ACTIVATIONS))}")
        if tuple(w_up.shape) != (E, F_up, W) or tuple(w_down.shape) != (E, W, F) or not w_up.is_contiguous() or not w_down.is_contiguous() \
                or w_up.dtype != w_down.dtype or (w_up.dtype != h.dtype and w_up.dtype != torch.float32) or x.dtype != torch.float32 or tuple(x.shape) != (T, W) \
                or not x.is_contiguous() or tuple(weights.shape) != (T, top) or weights.dtype != torch.float32:
            fail(EINVAL, "moe_experts: the experts' matrices, the activations and the residual stream do not fit")
        code, wcode = _code(h), _code(w_up)              # matrices stored in 32-bit stay so beside bf16 activations
        plain = 1 if self.force_plain_gemm else 0
        # one size of tile for both products: rows are put into tiles once
        tile_rows = 32 if plain else min(int(self.lib.hfa_moe_tile_rows(code, wcode, n_pairs, E, F_up, W)),
                                         int(self.lib.hfa_moe_tile_rows(code, wcode, n_pairs, E, W, F)))
        max_tiles = n_pairs // tile_rows + E
        row_pair = self.scratch("moe_row_pair", (n_pairs,), torch.int32)
        tiles = self.scratch("moe_tiles", (3 * max_tiles + 1,), torch.int32)
        n_tiles = tiles[3 * max_tiles:]
        self._check(self.lib.hfa_moe_plan(_ints(ids, "moe ids", n_pairs), n_pairs, E, tile_rows, row_pair.data_ptr(), tiles.data_ptr(),
                                          n_tiles.data_ptr(), self._stream()))
        mid = self.scratch("moe_act", (n_pairs, F), h.dtype)
        y = self.scratch("moe_out", (n_pairs, W), torch.float32)
        if gated is not None:
            alpha, limit, shift, interleaved = gated
            w_in, w_out = (weights, None) if weight_on == "input" else (None, weights)
            # A row or two an expert (a few decoded tokens): the experts' matrices are streamed once, by blocks that own 32 of
            # their rows each; blocks that own a gate block and its up block are half as many and stream slower (835 against
            # 900 us for the experts of a step of 8 tokens, 64 experts of 1,024 x 4,096; at 64 tokens 1,440 against 1,395),
            # so there the activation stays a kernel of its own.
            streamed = not plain and tile_rows == 32 and code == BF16 and wcode == BF16 and W % 64 == 0 and n_pairs <= 2 * E
            if interleaved and not streamed:
                self._check(self.lib.hfa_moe_gemm(h.data_ptr(), _rows(h, "moe h"), code, top, w_up.data_ptr(), wcode, row_pair.data_ptr(),
                                                  tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, mid.data_ptr(), F, code, 0,
                                                  None if w_in is None else w_in.data_ptr(), 0, F_up, W, plain, 1, float(alpha),
                                                  float(limit), float(shift), self._stream()))
            else:
                self._gated_in_two(h, code, top, w_up, wcode, row_pair, tiles, n_tiles, max_tiles, tile_rows, mid, w_in, n_pairs,
                                   F, F_up, W, plain, alpha, limit, shift, interleaved)
            self._check(self.lib.hfa_moe_gemm(mid.data_ptr(), F, code, 0, w_down.data_ptr(), wcode, row_pair.data_ptr(), tiles.data_ptr(),
                                              n_tiles.data_ptr(), max_tiles, tile_rows, y.data_ptr(), W, F32, 1,
                                              None if w_out is None else w_out.data_ptr(), 0, W, F,
                                              plain, 0, 0.0, 0.0, 0.0, self._stream()))
            self._check(self.lib.hfa_moe_combine(y.data_ptr(), x.data_ptr(), T, top, W, self._stream()))
            return
        self._plain_experts(h, code, top, w_up, w_down, wcode, row_pair, tiles, n_tiles, max_tiles, tile_rows, mid, y, weights, act, F, W,
                            plain, x, T)

    def _gated_in_two(self, h, code, top, w_up, wcode, row_pair, tiles, n_tiles, max_tiles, tile_rows, mid, weights, n_pairs, F, F_up, W,
                      plain, alpha, limit, shift, interleaved):
        """The up product of gated experts as 32-bit sums, then the activation as a kernel of its own."""
        sums = self.scratch("moe_gate_up", (n_pairs, F_up), torch.float32)      # 32-bit sums: the weight scales them exactly
        self._check(self.lib.hfa_moe_gemm(h.data_ptr(), _rows(h, "moe h"), code, top, w_up.data_ptr(), wcode, row_pair.data_ptr(),
                                          tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, sums.data_ptr(), F_up, F32, 0,
                                          None, 0, F_up, W, plain, 0, 0.0, 0.0, 0.0, self._stream()))
        self._check(self.lib.hfa_moe_gated_act(sums.data_ptr(), F_up, row_pair.data_ptr(), None if weights is None else weights.data_ptr(),
                                               mid.data_ptr(), code, F,
                                               n_pairs, F, float(alpha), float(limit), float(shift), 1 if interleaved else 0,
                                               self._stream()))

    def _plain_experts(self, h, code, top, w_up, w_down, wcode, row_pair, tiles, n_tiles, max_tiles, tile_rows, mid, y, weights, act, F, W,
                       plain, x, T):
        """Experts without a gate: the activation in the up product's last lines, the weights in the down product's."""
        self._check(self.lib.hfa_moe_gemm(h.data_ptr(), _rows(h, "moe h"), code, top, w_up.data_ptr(), wcode, row_pair.data_ptr(),
                                          tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, mid.data_ptr(), F, code, 0, None,
                                          self.ACTIVATIONS[act], F, W, plain, 0, 0.0, 0.0, 0.0, self._stream()))
        self._check(self.lib.hfa_moe_gemm(mid.data_ptr(), F, code, 0, w_down.data_ptr(), wcode, row_pair.data_ptr(), tiles.data_ptr(),
                                          n_tiles.data_ptr(), max_tiles, tile_rows, y.data_ptr(), W, F32, 1, weights.data_ptr(), 0, W, F,
                                          plain, 0, 0.0, 0.0, 0.0, self._stream()))
        self._check(self.lib.hfa_moe_combine(y.data_ptr(), x.data_ptr(), T, top, W, self._stream()))

    @staticmethod
    def interleave_experts(w_gate, w_up):
        """[E, 2F, width] from [E, F, width] twice: of every expert rows 0..31 of gate, rows 0..31 of up, rows 32..63 of gate, ..."""
        E, F, W = w_gate.shape
        return torch.stack([w_gate.view(E, F // 32, 32, W), w_up.view(E, F // 32, 32, W)], dim=2).reshape(E, 2 * F, W).contiguous()

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
