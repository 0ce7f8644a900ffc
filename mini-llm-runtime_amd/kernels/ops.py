"""Python side of the HIP kernels: one `Kernels` object per element type.

Every method checks on the host that its operands lie on the GPU, are contiguous, have the
element type and the shapes that the kernel and its grid assume, and only then launches on
torch's current stream.  A kernel that cannot take a size refuses it here with a clear error.
There is no other implementation behind these methods: without the compiled extension, or
without a GPU, they raise.
"""
from __future__ import annotations

import ctypes

import torch

from . import build
from .profile import timed

_c_int = ctypes.c_int
_c_float = ctypes.c_float
_c_size_t = ctypes.c_size_t
_ptr = ctypes.c_void_p

MAX_HEAD_DIM = 256          # the attention and rotation kernels keep head_dim / 64 values per lane
ATTENTION_TILE_KEYS = 64
LIBRARY_GEMM_MIN_ROWS = 16    # above this many rows the bfloat16 engine's projections go to the library
LIBRARY_GEMM_WORKSPACE = 128 << 20   # bytes of scratch memory that the library may use
PREFILL_MAX_PAGES = 2048      # page ids of one group that the prompt-portion attention kernel keeps in LDS
TILES_MAX_HEAD_DIM = 128      # the 32x32-tile kernel for prompt portions keeps two sets of accumulators per lane
TILES_COLUMNS = (128, 64)     # (token, head) columns of one of its workgroups: the usual and the small one
TILES_PAIRING = {"auto": 0, "single": 1, "pairs": 2}
MFMA_MAX_PAGES = 4096         # page ids of one key range that the single-token attention kernel keeps in LDS
MAX_KEY_SPLITS = 1024         # the merge of key splits keeps one weight per split in LDS


class KernelError(RuntimeError):
    pass


def _p(t):
    return _ptr(t.data_ptr()) if t is not None else _ptr(0)


try:
    _raw_stream = torch._C._cuda_getCurrentRawStream          # the current stream's handle without a Stream object
except AttributeError:                                         # pragma: no cover
    _raw_stream = None


_device_index = getattr(torch._C, "_cuda_getDevice", None)    # (the current device's index without torch.cuda's wrapper)


def _stream():
    """Handle of torch's current stream on the current device."""
    if _raw_stream is not None:
        return _ptr(_raw_stream(_device_index() if _device_index is not None else torch.cuda.current_device()))
    return _ptr(torch.cuda.current_stream().cuda_stream)


def _need(cond, message):
    """`message` is a string or, where building it costs time, a function that returns one."""
    if not cond:
        raise KernelError(message() if callable(message) else message)


def _tensor(t, name, dtype, shape=None, ndim=None):
    # one cheap test on the way that every launch takes; the message is only put together on failure
    try:
        if (t.is_cuda and t.dtype is dtype and t.is_contiguous() and (ndim is None or t.dim() == ndim)
                and (shape is None or t.shape == shape or t.shape == tuple(shape))):
            return t
    except AttributeError:                                # (no tensor: said below)
        pass
    _need(isinstance(t, torch.Tensor), f"{name}: expected a tensor")
    _need(t.is_cuda, f"{name}: must lie on the GPU (there is no CPU path)")
    _need(t.dtype == dtype, f"{name}: expected {dtype}, got {t.dtype}")
    _need(t.is_contiguous(), f"{name}: must be contiguous")
    _need(ndim is None or t.dim() == ndim, f"{name}: expected {ndim} dimensions, got {tuple(t.shape)}")
    raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _ok(code, what):
    if code != 0:
        raise KernelError(f"{what}: launch failed with code {code}")


def _size(t):
    return 0 if t is None else t.numel() * t.element_size()


def _gemm_work(self, a, w, out, *rest, **kw):
    return _size(a) + _size(w) + _size(out), 2 * a.shape[0] * w.shape[0] * w.shape[1]


def _rows_prenorm_work(self, h, delta, weight, out, ss):
    return 2 * _size(h) + _size(delta) + _size(out), 0


def _prenormed_work(self, x, ss, eps, w, out, *rest, **kw):
    return _size(x) + _size(ss) + _size(w) + _size(out), 2 * x.shape[0] * w.shape[0] * w.shape[1]


def _residual_work(self, a, w, h, *rest, **kw):
    return _size(a) + _size(w) + 2 * _size(h), 2 * a.shape[0] * w.shape[0] * w.shape[1]


def _norm_work(self, h, delta, weight, out, eps, rows=None, write_h=True):
    n, width = out.shape[0], h.shape[1]
    moved = n * width * 4 + _size(out)
    if delta is not None:
        moved += n * width * (delta.element_size() + (4 if write_h else 0))
    return moved, 0


def _embed_work(self, ids, table, h):
    return _size(h) + h.numel() * table.element_size(), 0


def _rope_work(self, qkv, *rest, **kw):
    return 2 * _size(qkv), 0


def _tensors_work(*names):
    def work(self, *args, **kw):
        return sum(_size(a) for a in args if isinstance(a, torch.Tensor)), 0
    return work


class Kernels:
    def __init__(self, dtype, library_gemm=True):
        _need(dtype in (torch.float32, torch.bfloat16), f"no kernels for element type {dtype}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine's kernels are HIP only")
        self.dtype = dtype
        self.library_gemm = library_gemm
        self._library_workspace = None      # scratch memory of the vendor library's products, allocated once
        self._libs = {}
        self.profiler = None                # a `Profiler`: every launch is then bracketed by events

    # -- libraries ---------------------------------------------------------------------------
    def prepare(self, names):
        """Build (if need be) and load several libraries at once."""
        typed = [n for n in names if build.HIP_LIBRARIES[n][2]]
        untyped = [n for n in names if not build.HIP_LIBRARIES[n][2]]
        if typed:
            build.ensure_built(typed, self.dtype)
        if untyped:
            build.ensure_built(untyped)
        for n in names:
            self._lib(n)

    def _lib(self, name):
        lib = self._libs.get(name)
        if lib is None:
            lib = build.load(name, self.dtype)
            self._libs[name] = lib
        return lib

    # -- row-wise ----------------------------------------------------------------------------
    @timed("embed", _embed_work)
    def embed_gather(self, ids, table, h):
        """h[m] = float(table[ids[m]])."""
        rows = ids.numel()
        _tensor(ids, "ids", torch.int32, ndim=1)
        _tensor(table, "table", self.dtype, ndim=2)
        vocab, width = table.shape
        _tensor(h, "h", torch.float32, (rows, width))
        fn = self._lib("elementwise").mlr_embed_gather
        _ok(fn(_p(ids), _p(table), _p(h), _c_int(rows), _c_int(width), _c_int(vocab), _stream()),
            "embed_gather")

    @timed("norm", _norm_work)
    def add_rmsnorm(self, h, delta, weight, out, eps, rows=None, write_h=True):
        """x = h[src] + delta[src] (delta may be None); h[src] = x when write_h; out[r] =
        rmsnorm(x) * weight, src = rows[r] or r."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        if rows is not None:
            _tensor(rows, "rows", torch.int32, ndim=1)
            n_out = rows.numel()
        else:
            n_out = m
        _tensor(out, "out", self.dtype, (n_out, width))
        fn = self._lib("elementwise").mlr_add_rmsnorm
        _ok(fn(_p(h), _p(delta), _p(weight), _p(out), _p(rows), _c_int(n_out), _c_int(width),
               _c_float(eps), _c_int(1 if (write_h and delta is not None) else 0), _stream()),
            "add_rmsnorm")

    @timed("check")
    def status_reset(self, status):
        """status = (0, INT_MAX): nothing seen yet.  A kernel, so that a captured step can hold it."""
        _tensor(status, "status", torch.int32, (2,))
        _ok(self._lib("elementwise").mlr_status_reset(_p(status), _stream()), "status_reset")

    @timed("check")
    def finite_check(self, h, delta, layer, status):
        """ORs into status[0] which kinds of non-finite values h + delta holds (1: NaN, 2: infinity) and keeps
        in status[1] the smallest (layer << 20 | row) that held one."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(status, "status", torch.int32, (2,))
        _need(0 <= layer < 2047, "finite_check: layer index out of range")
        _ok(self._lib("elementwise").mlr_finite_check(_p(h), _p(delta), _c_int(m), _c_int(width), _c_int(layer),
                                                      _p(status), _stream()), "finite_check")

    @timed("norm", _tensors_work())
    def residual_add(self, h, delta):
        _tensor(h, "h", torch.float32, ndim=2)
        _tensor(delta, "delta", self.dtype, tuple(h.shape))
        fn = self._lib("elementwise").mlr_residual_add
        _ok(fn(_p(h), _p(delta), _c_size_t(h.numel()), _stream()), "residual_add")

    @timed("norm", _tensors_work())
    def residual_add_float(self, h, extra):
        """h += extra, both float (the embedding's output joining the stream again)."""
        _tensor(h, "h", torch.float32, ndim=2)
        _tensor(extra, "extra", torch.float32, tuple(h.shape))
        _ok(self._lib("elementwise").mlr_residual_add_float(_p(h), _p(extra), _c_size_t(h.numel()), _stream()),
            "residual_add_float")

    @timed("activation", _tensors_work())
    def silu_mul(self, gate_up, act):
        """act[m, f] = silu(gate_up[m, f]) * gate_up[m, F + f]."""
        _tensor(gate_up, "gate_up", self.dtype, ndim=2)
        m, two_f = gate_up.shape
        _need(two_f % 2 == 0, "gate_up: the width must be even")
        _tensor(act, "act", self.dtype, (m, two_f // 2))
        fn = self._lib("elementwise").mlr_silu_mul
        _ok(fn(_p(gate_up), _p(act), _c_int(m), _c_int(two_f // 2), _stream()), "silu_mul")

    GATED_ACTS = {"silu": 0, "gelu_tanh": 1}

    @timed("activation", _tensors_work())
    def gated_act_mul(self, gate_up, act, kind):
        """act[m, f] = kind(gate_up[m, f]) * gate_up[m, F + f]; kind: silu, or gelu_tanh,
        0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))."""
        _need(kind in self.GATED_ACTS, f"gated_act_mul: activation {kind!r} ({', '.join(self.GATED_ACTS)})")
        _tensor(gate_up, "gate_up", self.dtype, ndim=2)
        m, two_f = gate_up.shape
        _need(two_f % 2 == 0, "gate_up: the width must be even")
        _tensor(act, "act", self.dtype, (m, two_f // 2))
        _ok(self._lib("elementwise").mlr_gated_act_mul(_p(gate_up), _p(act), _c_int(m), _c_int(two_f // 2),
                                                       _c_int(self.GATED_ACTS[kind]), _stream()), "gated_act_mul")

    @timed("embed", _tensors_work())
    def pair_embed(self, ids, positions, slots, table, pairs, live, stage, h, buckets, mul_prev, mul_cur):
        """h[m] = float(table[ids[m]]) + float(pairs[row]), row = (token before * mul_prev + ids[m] * mul_cur) mod
        buckets, or row `buckets` at position 0.  The token before: the row above when it is the same request's
        previous position, else live[slot] (int32 [slots, 1]); a request's last row leaves its token in stage[slot]."""
        rows = ids.numel()
        for name, t in (("ids", ids), ("positions", positions), ("slots", slots)):
            _tensor(t, name, torch.int32, (rows,))
        _tensor(table, "table", self.dtype, ndim=2)
        vocab, width = table.shape
        _tensor(pairs, "pairs", self.dtype, (buckets + 1, width))
        _tensor(live, "live", torch.int32, ndim=2)
        _tensor(stage, "stage", torch.int32, tuple(live.shape))
        _need(live.shape[1] == 1 and buckets >= 1, "pair_embed: one token a slot, and at least one bucket")
        _tensor(h, "h", torch.float32, (rows, width))
        _ok(self._lib("elementwise").mlr_pair_embed(_p(ids), _p(positions), _p(slots), _p(table), _p(pairs), _p(live),
                                                    _p(stage), _p(h), _c_int(rows), _c_int(width), _c_int(vocab),
                                                    _c_int(buckets), ctypes.c_longlong(mul_prev), ctypes.c_longlong(mul_cur),
                                                    _stream()), "pair_embed")

    GATE_KINDS = {"silu": 0, "sigmoid": 1}

    @timed("activation", _tensors_work())
    def gate_mul(self, x, gate, out, kind="sigmoid", scale=1.0):
        """out = scale * x * kind(gate); gate: columns of a row-major matrix; out may be x."""
        _tensor(x, "x", self.dtype, ndim=2)
        m, width = x.shape
        stride = self._columns(gate, "gate", self.dtype, m, width)
        _tensor(out, "out", self.dtype, (m, width))
        _need(kind in self.GATE_KINDS, f"gate_mul: gate {kind!r}")
        _ok(self._lib("elementwise").mlr_gate_mul(_p(x), _p(gate), ctypes.c_long(stride), _p(out), _c_int(m), _c_int(width),
                                                  _c_int(self.GATE_KINDS[kind]), _c_float(scale), _stream()), "gate_mul")

    @timed("norm", _tensors_work())
    def rmsnorm_columns(self, x, weight, out, eps):
        """out = x / sqrt(mean(x^2) + eps) * weight, row by row, x being columns of a row-major matrix; 32-bit inside."""
        _need(isinstance(x, torch.Tensor) and x.dim() == 2, "rmsnorm_columns: x must be a matrix")
        rows, width = x.shape
        stride = self._columns(x, "x", self.dtype, rows, width)
        _tensor(weight, "weight", torch.float32, (width,))
        _tensor(out, "out", self.dtype, (rows, width))
        _ok(self._lib("elementwise").mlr_rmsnorm_columns(_p(x), ctypes.c_long(stride), _p(weight), _p(out), _c_int(rows),
                                                         _c_int(width), _c_float(eps), _stream()), "rmsnorm_columns")

    @timed("norm", _tensors_work())
    def scaled_sum(self, a, b, out, sa, sb):
        """out = sa * a + sb * b, the sum taken in 32-bit; out may be a or b."""
        _tensor(a, "a", self.dtype)
        _tensor(b, "b", self.dtype, tuple(a.shape))
        _tensor(out, "out", self.dtype, tuple(a.shape))
        _ok(self._lib("elementwise").mlr_scaled_sum(_p(a), _p(b), _p(out), _c_float(sa), _c_float(sb), _c_size_t(a.numel()),
                                                    _stream()), "scaled_sum")

    # -- projections -------------------------------------------------------------------------
    @timed("gemm", _gemm_work)
    def gemm(self, a, w, out):
        """out[M, N] = a[M, K] . w[N, K]^T; out has the element type or is float32."""
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        n, k2 = w.shape
        _need(k == k2, lambda: f"gemm: inner sizes differ ({k} and {k2})")
        _need(out.dtype in (self.dtype, torch.float32), lambda: f"gemm: output type {out.dtype} not supported")
        _tensor(out, "out", out.dtype, (m, n))
        if self.library_gemm and self.dtype == torch.bfloat16 and m > LIBRARY_GEMM_MIN_ROWS and \
                (out.dtype == torch.float32 or not self.streams_weight(m, k)):
            # many rows: a plain matrix product, handed to the vendor library (hipBLASLt), as the reference
            # hands its projections to cuBLAS (src/minillm/cuda/matrix.cpp:11-37).  (Float outputs are
            # logits, a vocabulary wide: there the library wins from 17 rows on at any inner size.)
            ws = self.reserve_library_workspace(a.device)
            _ok(self._lib("library_gemm").mlr_library_gemm(_p(a), _p(w), _p(out), _c_int(m), _c_int(n), _c_int(k),
                                                           _c_int(1 if out.dtype == torch.float32 else 0),
                                                           _p(ws), _c_size_t(ws.numel()), _stream()), "library_gemm")
            return
        fn = self._lib("gemm").mlr_gemm
        _ok(fn(_p(a), _p(w), _p(out), _c_int(m), _c_int(n), _c_int(k),
               _c_int(1 if out.dtype == torch.float32 else 0), _stream()), "gemm")

    def reserve_library_workspace(self, device):
        """The vendor library's scratch memory, allocated once."""
        if self._library_workspace is None:
            self._library_workspace = torch.empty(LIBRARY_GEMM_WORKSPACE, dtype=torch.uint8, device=device)
        return self._library_workspace

    def library_workspace_bytes(self):
        return 0 if self._library_workspace is None else self._library_workspace.numel()

    def streams_weight(self, rows, k):
        """Whether a projection of this many rows and inner size goes to the kernels that stream the weight
        once into the matrix cores, and not to the vendor library: up to 16 rows always; up to 64 rows while
        the rows, which every workgroup reads again, stay small beside its strip of the weight (measured on
        weights that do not sit in a cache: k = 1024 up to 64 rows, k = 2048 up to 32)."""
        if self.dtype != torch.bfloat16:
            return False
        if not self.library_gemm:
            return rows <= 64
        return rows <= LIBRARY_GEMM_MIN_ROWS or (rows <= 64 and k * ((rows + 15) // 16) <= 4096)

    def gated_silu_fused(self, rows, k=None):
        """Whether `gemm_gated_silu` is the path for this many rows and inner size: the bfloat16 engine, where
        `streams_weight` says so (elsewhere the library's product and a separate activation are faster), and
        without the library any number of rows when the inner size is a multiple of 64."""
        if self.dtype == torch.bfloat16 and rows > 64 and k is not None and k % 64 == 0 and rows * k < 2 ** 31:
            # many rows: the wide kernel's gated form.  Beside the library it is the faster way while the inner
            # size is short (measured against the library's product followed by the activation kernel, at 128
            # to 2048 rows: 0.58-0.95 of their time at k = 1024, 0.84-1.07 at k = 2048, 1.01-1.40 beyond)
            return not self.library_gemm or k <= 1024 or (k <= 2048 and rows <= 256)
        return self.streams_weight(rows, k if k is not None else 1 << 30)

    @timed("gemm", _gemm_work)
    def gemm_gated_silu(self, a, w, out):
        """out[M, N] = silu(a . w[:N]^T) * (a . w[N:]^T), w = [gate; up] stacked: up to 64 rows, or any number
        when the inner size is a multiple of 64 (the wide kernel's gated form)."""
        _need(self.dtype == torch.bfloat16, "gemm_gated_silu: bfloat16 only")
        _need(a.shape[0] <= 64 or (a.shape[1] % 64 == 0 and a.numel() < 2 ** 31 and w.numel() < 2 ** 31),
              "gemm_gated_silu: more than 64 rows need an inner size that is a multiple of 64 (and matrices "
              "below 2^31 elements)")
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        two_n, k2 = w.shape
        _need(k == k2 and two_n % 2 == 0, "gemm_gated_silu: sizes do not fit")
        _tensor(out, "out", self.dtype, (m, two_n // 2))
        fn = self._lib("gemm").mlr_gemm_gated_silu
        _ok(fn(_p(a), _p(w), _p(out), _c_int(m), _c_int(two_n // 2), _c_int(k), _stream()), "gemm_gated_silu")

    @timed("gemm", _gemm_work)
    def gemm_gated_clamped(self, a, w, out, limit, slope):
        """out[M, N] = g sigmoid(slope g) (u + 1), g = min(a . w[:N]^T, limit), u = clamp(a . w[N:]^T, -limit, limit):
        the clamped gate fused into the weight-streaming projection, up to 64 rows (bfloat16)."""
        _need(self.dtype == torch.bfloat16 and a.shape[0] <= 64, "gemm_gated_clamped: bfloat16, up to 64 rows")
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        two_n, k2 = w.shape
        _need(k == k2 and two_n % 2 == 0 and limit > 0, "gemm_gated_clamped: sizes do not fit")
        _tensor(out, "out", self.dtype, (m, two_n // 2))
        fn = self._lib("gemm").mlr_gemm_gated_clamped
        _ok(fn(_p(a), _p(w), _p(out), _c_int(m), _c_int(two_n // 2), _c_int(k), _c_float(limit), _c_float(slope), _stream()),
            "gemm_gated_clamped")

    @timed("gemm", _gemm_work)
    def gemm_gated_gelu_tanh(self, a, w, out):
        """out[M, N] = gelu_tanh(a . w[:N]^T) * (a . w[N:]^T), w = [gate; up] stacked: the tanh form of gelu fused into
        the weight-streaming projection, up to 64 rows (bfloat16)."""
        _need(self.dtype == torch.bfloat16 and a.shape[0] <= 64, "gemm_gated_gelu_tanh: bfloat16, up to 64 rows")
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        two_n, k2 = w.shape
        _need(k == k2 and two_n % 2 == 0, "gemm_gated_gelu_tanh: sizes do not fit")
        _tensor(out, "out", self.dtype, (m, two_n // 2))
        _ok(self._lib("gemm").mlr_gemm_gated_gelu_tanh(_p(a), _p(w), _p(out), _c_int(m), _c_int(two_n // 2), _c_int(k),
                                                       _stream()), "gemm_gated_gelu_tanh")

    # -- an RMSNorm handed from one projection to the next (few rows) ------------------------------
    HANDOFF_MAX_ROWS = 16

    def handoff_supported(self, rows):
        """Whether the projections before and after a norm can share it between them: the bfloat16 engine, up to
        16 rows.  The projection before the norm adds its sums to the residual stream h and leaves
        x = bf16(h * norm_w) and partial sums of squares of h's rows (`gemm_residual`); the projection after it
        multiplies its finished sums by the rows' scale rsqrt(mean(h^2) + eps) (`gemm_prenormed`): the scale is
        a factor per row, so the product with it commutes with the projection."""
        return self.dtype == torch.bfloat16 and 1 <= rows <= self.HANDOFF_MAX_ROWS

    @staticmethod
    def handoff_parts(width):
        """Partial sums of squares a row that `gemm_residual` leaves for an output `width` wide."""
        return (width + 15) // 16

    @timed("norm", _rows_prenorm_work)
    def rows_prenorm(self, h, delta, weight, out, ss):
        """h += delta (delta may be None); out = T(h * weight), without the norm's scale; ss[r, 0] = sum(h[r]^2)."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        _tensor(out, "out", self.dtype, (m, width))
        _tensor(ss, "ss", torch.float32, (m, 1))
        fn = self._lib("elementwise").mlr_rows_prenorm
        _ok(fn(_p(h), _p(delta), _p(weight), _p(out), _p(ss), _c_int(m), _c_int(width), _stream()), "rows_prenorm")

    @timed("gemm", _prenormed_work)
    def gemm_prenormed(self, x, ss, eps, w, out, gated=False):
        """out = rsqrt(sum(ss[m]) / K + eps) * (x . w^T), x being T(h * norm_w) [M, K] and ss [M, parts] partial
        sums of squares of h's rows; gated=True (w = [gate; up] stacked): silu(scale * gate) * (scale * up)."""
        _tensor(x, "x", self.dtype, ndim=2)
        m, k = x.shape
        _need(self.handoff_supported(m), "gemm_prenormed: bfloat16, at most 16 rows")
        _tensor(ss, "ss", torch.float32, ndim=2)
        _need(ss.shape[0] == m and ss.shape[1] >= 1, "gemm_prenormed: one row of partial sums per row of x")
        _tensor(w, "w", self.dtype, ndim=2)
        n = w.shape[0] // 2 if gated else w.shape[0]
        _need(w.shape[1] == k and (not gated or w.shape[0] % 2 == 0), "gemm_prenormed: weight does not fit")
        _tensor(out, "out", self.dtype, (m, n))
        fn = self._lib("gemm").mlr_gemm_prenormed
        _ok(fn(_p(x), _p(ss), _c_int(ss.shape[1]), _c_float(eps), _c_int(k), _p(w), _p(out), _c_int(m), _c_int(n),
               _c_int(k), _c_int(1 if gated else 0), _stream()), "gemm_prenormed")

    @timed("gemm", _residual_work)
    def gemm_residual(self, a, w, h, next_w=None, x_out=None, ss_out=None):
        """h += a . w^T (32-bit, in place).  With next_w (the weights of the norm that follows) also
        x_out = T(h * next_w) and ss_out[m, p] = the sum of squares of h[m, 16 p : 16 p + 16]."""
        _tensor(a, "a", self.dtype, ndim=2)
        m, k = a.shape
        _need(self.handoff_supported(m), "gemm_residual: bfloat16, at most 16 rows")
        _tensor(w, "w", self.dtype, ndim=2)
        n = w.shape[0]
        _need(w.shape[1] == k, "gemm_residual: inner sizes differ")
        _tensor(h, "h", torch.float32, (m, n))
        if next_w is not None:
            _tensor(next_w, "next_w", torch.float32, (n,))
            _tensor(x_out, "x_out", self.dtype, (m, n))
            _tensor(ss_out, "ss_out", torch.float32, (m, self.handoff_parts(n)))
        fn = self._lib("gemm").mlr_gemm_residual
        _ok(fn(_p(a), _p(w), _p(h), _p(next_w), _p(x_out if next_w is not None else None),
               _p(ss_out if next_w is not None else None), _c_int(m), _c_int(n), _c_int(k), _stream()), "gemm_residual")

    # -- attention ---------------------------------------------------------------------------
    def _check_cache(self, k_pages, v_pages, kv_heads, head_dim, page_size):
        _tensor(k_pages, "k_pages", self.dtype, ndim=4)
        _need(k_pages.shape[1:] == (kv_heads, page_size, head_dim),
              lambda: f"k_pages: expected [pages, {kv_heads}, {page_size}, {head_dim}], got {tuple(k_pages.shape)}")
        _tensor(v_pages, "v_pages", self.dtype, (k_pages.shape[0], kv_heads, head_dim, page_size))

    @timed("rope_kv", _rope_work)
    def qk_norm_rope_kv(self, qkv, q_out, k_pages, v_pages, block_table, slots, positions, q_norm_w,
                        k_norm_w, eps, rope, q_heads, kv_heads, head_dim, page_size, write_cache=True,
                        interleaved=False):
        """Per head: RMSNorm of q and k (weights may be None), rotation by `rope` [max_positions, rot_dim]
        (cosines | sines; may be None) of the head's first rot_dim channels in pairs (j, j + rot_dim / 2), or
        (2 j, 2 j + 1) when `interleaved`; q into q_out, k and v into their pages."""
        _need(head_dim % 2 == 0 and 2 <= head_dim <= MAX_HEAD_DIM,
              lambda: f"head_dim {head_dim}: the rotation kernel takes even sizes up to {MAX_HEAD_DIM}")
        width = (q_heads + 2 * kv_heads) * head_dim
        _tensor(qkv, "qkv", self.dtype, ndim=2)
        m = qkv.shape[0]
        _need(qkv.shape[1] == width, lambda: f"qkv: expected width {width}, got {qkv.shape[1]}")
        _tensor(q_out, "q_out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        if q_norm_w is not None:
            _tensor(q_norm_w, "q_norm_w", torch.float32, (head_dim,))
            _tensor(k_norm_w, "k_norm_w", torch.float32, (head_dim,))
        rot_dim = head_dim
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            rot_dim = rope.shape[1]
            _need(2 <= rot_dim <= head_dim and rot_dim % 2 == 0,
                  lambda: f"rope: the table's width {rot_dim} must be even and at most head_dim {head_dim}")
        fn = self._lib("rope_kv").mlr_qk_norm_rope_kv
        _ok(fn(_p(qkv), _c_int(width), _p(q_out), _p(k_pages), _p(v_pages), _p(block_table),
               _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(q_norm_w), _p(k_norm_w),
               _c_float(eps), _p(rope), _c_int(m), _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim),
               _c_int(page_size), _c_int(1 if write_cache else 0), _c_int(rot_dim), _c_int(1 if interleaved else 0),
               _stream()), "qk_norm_rope_kv")

    @staticmethod
    def attention_partial_numel(rows, q_heads, head_dim, max_splits):
        """Floats of scratch memory for the partial results of split attention: per (row, head, split) the
        unnormalised output, its maximum and its sum (the prompt-portion kernel keeps them 16 bytes apart)."""
        return rows * q_heads * max_splits * (head_dim + 4)

    @timed("attention")
    def paged_attention(self, q, k_pages, v_pages, block_table, slots, positions, out, q_heads,
                        kv_heads, head_dim, page_size, scale, window=None, split_keys=0, max_splits=1,
                        partial=None):
        """out[m, h] = softmax over the keys seen by token m (positions <= its own, within the
        window) of q.k * scale, times v; keys and values from the pages of slots[m]."""
        _need(1 <= head_dim <= MAX_HEAD_DIM,
              lambda: f"head_dim {head_dim}: the attention kernel takes up to {MAX_HEAD_DIM}")
        _need(q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits),
                  "partial buffer too small")
            group = q_heads // kv_heads
            _need(((group + 7) // 8) * max_splits <= 65535 and max_splits <= MAX_KEY_SPLITS,
                  "too many key splits for the grid")
        fn = self._lib("attention").mlr_paged_attention
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(partial), _c_int(m), _c_int(q_heads), _c_int(kv_heads),
               _c_int(head_dim), _c_int(page_size), _c_int(window or 0), _c_float(scale),
               _c_int(split_keys), _c_int(max_splits), _stream()), "paged_attention")

    def mfma_attention_supported(self, q_heads, kv_heads, head_dim, page_size):
        """The matrix-core attention kernel serves the bfloat16 engine for pages that are a multiple of
        16 tokens, head sizes that are a multiple of 16 and up to 16 query heads per kv head."""
        return (self.dtype == torch.bfloat16 and page_size % 16 == 0 and head_dim % 16 == 0
                and head_dim <= MAX_HEAD_DIM and q_heads % kv_heads == 0 and q_heads // kv_heads <= 16)

    @timed("attention")
    def attention_mfma(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                       groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, split_keys=0,
                       max_splits=1, partial=None, partial_rows=None):
        """As `paged_attention`, on the matrix cores.  The batch rows are covered by `groups` groups of
        consecutive rows of one request each (group_row0[i], group_ntok[i]), at most 16 // (q_heads //
        kv_heads) tokens a group.  `partial_rows`: the caller vouches that every group's rows lie below this
        batch row (the partial results are indexed by batch row and need not reach further); default: all rows."""
        _need(self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_mfma: sizes not supported (bfloat16, page_size % 16 == 0, head_dim % 16 == 0, "
              "at most 16 query heads per kv head)")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535 and max_splits <= MAX_KEY_SPLITS, "too many kv heads or key splits for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            reach = m if partial_rows is None else partial_rows
            _need(0 < reach <= m and partial.numel() >= self.attention_partial_numel(reach, q_heads, head_dim, max_splits),
                  "partial buffer too small")
        _need((split_keys // page_size + 2 if max_splits > 1 else block_table.shape[1]) <= MFMA_MAX_PAGES,
              "attention_mfma: a workgroup's key range spans more than 4096 pages; split the keys")
        fn = self._lib("attention").mlr_attention_mfma
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(partial), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(m),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0),
               _c_float(scale), _c_int(split_keys), _c_int(max_splits), _stream()), "attention_mfma")

    @staticmethod
    def max_key_splits():
        return MAX_KEY_SPLITS

    @staticmethod
    def mfma_longest_context(page_size):
        """The most keys that one workgroup of `attention_mfma` / `attention_decode_fused` can walk (it keeps
        their page ids in LDS; a key split that does not start at a page's edge touches one page more)."""
        return (MFMA_MAX_PAGES - 2) * page_size

    def decode_fusion_supported(self, q_heads, kv_heads, head_dim, page_size):
        """Attention for single new tokens that norms, rotates and caches inside itself: the matrix-core
        kernel's sizes and head sizes that are multiples of 64."""
        return self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim % 64 == 0

    @timed("attention")
    def attention_decode_fused(self, qkv, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                               groups, q_heads, kv_heads, head_dim, page_size, scale, q_norm_w, k_norm_w, eps, rope,
                               partial, window=None, split_keys=0, max_splits=1):
        """For a batch in which every group is ONE new token of a request (the caller vouches for that):
        per-head RMSNorm of q and k (weights may both be None), rotation by `rope` (may be None), attention
        over the cached keys and the token's own, and the write of the token's key and value into their
        pages, in two launches.  `qkv` holds the raw projections; `partial` is needed also without splits."""
        _need(self.decode_fusion_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_decode_fused: sizes not supported")
        width = (q_heads + 2 * kv_heads) * head_dim
        _tensor(qkv, "qkv", self.dtype, ndim=2)
        m = qkv.shape[0]
        _need(qkv.shape[1] == width, lambda: f"qkv: expected width {width}, got {qkv.shape[1]}")
        _need(groups == m, "attention_decode_fused: one group per row")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need((q_norm_w is None) == (k_norm_w is None), "q and k norm weights come together")
        if q_norm_w is not None:
            _tensor(q_norm_w, "q_norm_w", torch.float32, (head_dim,))
            _tensor(k_norm_w, "k_norm_w", torch.float32, (head_dim,))
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            _need(rope.shape[1] == head_dim, "rope: table width must equal head_dim")
        max_splits = max(1, max_splits)
        _need(kv_heads <= 65535 and max_splits <= MAX_KEY_SPLITS, "too many kv heads or key splits for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
        _tensor(partial, "partial", torch.float32, ndim=1)
        _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits), "partial buffer too small")
        _need((split_keys // page_size + 2 if max_splits > 1 else block_table.shape[1]) <= MFMA_MAX_PAGES,
              "attention_decode_fused: a workgroup's key range spans more than 4096 pages; split the keys")
        fn = self._lib("attention").mlr_attention_decode_fused
        _ok(fn(_p(qkv), _c_int(width), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]),
               _p(slots), _p(positions), _p(out), _p(partial), _p(group_row0), _p(group_ntok), _c_int(groups),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0),
               _c_float(scale), _c_int(split_keys), _c_int(max_splits), _p(q_norm_w), _p(k_norm_w), _c_float(eps),
               _p(rope), _stream()), "attention_decode_fused")

    def prefill_attention_supported(self, q_heads, kv_heads, head_dim, page_size, max_context=0):
        """The LDS-staged kernel for prompt portions: as the matrix-core kernel, head sizes up to 192 and
        contexts of at most 2048 pages (it keeps a group's page ids in LDS)."""
        return (self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim <= 192
                and max_context <= PREFILL_MAX_PAGES * page_size)

    @timed("attention")
    def attention_prefill(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                          groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, max_context=None):
        """Attention for prompt portions: groups of up to 4 * (16 // (q_heads // kv_heads)) consecutive rows
        of one request each; keys and values of a group are staged once through LDS."""
        _need(self.prefill_attention_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_prefill: sizes not supported")
        _need(block_table.shape[1] <= PREFILL_MAX_PAGES or max_context is not None,
              "attention_prefill: give max_context when the block table is wider than the kernel's page cache")
        _need((max_context or 0) <= PREFILL_MAX_PAGES * page_size, "attention_prefill: context too long")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        fn = self._lib("attention").mlr_attention_prefill
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(q_heads),
               _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0), _c_float(scale),
               _stream()), "attention_prefill")

    def tiles_attention_supported(self, q_heads, kv_heads, head_dim, page_size, max_context=0, num_pages=0,
                                  split_keys=0):
        """The 32x32-tile kernel for prompt portions: bfloat16, head sizes up to 128 in steps of 16, pages
        of a power of two of keys, at most 16 query heads per kv head, contexts of at most 2048 pages (it
        keeps a group's page ids in LDS), a cache of fewer than 2^32 elements per layer (32-bit offsets)."""
        stride = kv_heads * page_size * head_dim
        return (self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim <= TILES_MAX_HEAD_DIM
                and page_size & (page_size - 1) == 0
                and (split_keys > 0 or max_context <= PREFILL_MAX_PAGES * page_size)
                and stride < 2 ** 24 and num_pages < 2 ** 24 and stride * num_pages < 2 ** 32)

    @staticmethod
    def tiles_sizes_supported(q_heads, kv_heads, head_dim, page_size):
        """The part of `tiles_attention_supported` that the model's sizes and the page size decide (bfloat16 engine)."""
        return (page_size % 16 == 0 and page_size & (page_size - 1) == 0 and head_dim % 16 == 0
                and head_dim <= TILES_MAX_HEAD_DIM and q_heads % kv_heads == 0 and q_heads // kv_heads <= 16)

    @staticmethod
    def tiles_longest_context(page_size):
        """The most keys that one workgroup of `attention_tiles` can walk (it keeps their page ids in LDS;
        a key split that does not start at a page's edge touches one page more)."""
        return (PREFILL_MAX_PAGES - 2) * page_size

    @staticmethod
    def tiles_group_tokens(q_heads, kv_heads, columns=TILES_COLUMNS[0]):
        """The most tokens of a group of `attention_tiles` with workgroups of `columns` columns."""
        return columns // (q_heads // kv_heads)

    @timed("attention")
    def attention_tiles(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                        groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, max_context=None,
                        columns=TILES_COLUMNS[0], split_keys=0, max_splits=1, partial=None, pairing="auto"):
        """Attention for prompt portions: groups of up to columns // (q_heads // kv_heads) consecutive rows
        of one request each (columns = 128, or 64 for batches that would not fill the GPU with the larger
        workgroups); keys and values of a group are staged once through LDS in blocks of 64.  With
        max_splits > 1 a group's keys are split over workgroups in ranges of split_keys (a multiple of 64)
        and merged through `partial`.  `pairing`: whether a workgroup of 128 columns (without splits) takes two
        groups, an early and a late one of a prompt, which evens out their key ranges: "auto" unless that would
        leave compute units idle, "single" never, "pairs" always.  The caller vouches for the groups (consecutive rows of one request,
        no more tokens than `tiles_group_tokens`)."""
        _need(columns in TILES_COLUMNS, lambda: f"attention_tiles: columns must be one of {TILES_COLUMNS}")
        _need(pairing in TILES_PAIRING, lambda: f"attention_tiles: pairing must be one of {sorted(TILES_PAIRING)}")
        _need(self.tiles_attention_supported(q_heads, kv_heads, head_dim, page_size, num_pages=k_pages.shape[0]),
              "attention_tiles: sizes not supported")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(max_splits <= MAX_KEY_SPLITS and groups <= 65535, "too many key splits or groups for the grid")
            _need(split_keys // page_size + 2 <= PREFILL_MAX_PAGES, "attention_tiles: a split spans too many pages")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits),
                  "partial buffer too small")
        else:
            _need(block_table.shape[1] <= PREFILL_MAX_PAGES or max_context is not None,
                  "attention_tiles: give max_context when the block table is wider than the kernel's page cache")
            _need((max_context or 0) <= PREFILL_MAX_PAGES * page_size, "attention_tiles: context too long")
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        fn = self._lib("attention_tiles").mlr_attention_tiles
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(columns),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(k_pages.shape[0]),
               _c_int(window or 0), _c_float(scale), _c_int(split_keys), _c_int(max_splits), _p(partial),
               _c_int(TILES_PAIRING[pairing]), _stream()), "attention_tiles")

    # -- a layer whose two branches read the same input ----------------------------------------------
    @timed("norm", _tensors_work())
    def add2_rmsnorm2(self, h, d1, d2, w1, w2, out1, out2, eps):
        """x = h + d1 + d2 (either may be None), written back to h; out1 = rmsnorm(x) * w1 and, when given,
        out2 = rmsnorm(x) * w2: two norms of one input share its root mean square."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        for name, d in (("d1", d1), ("d2", d2)):
            if d is not None:
                _tensor(d, name, self.dtype, (m, width))
        _tensor(w1, "w1", torch.float32, (width,))
        _tensor(out1, "out1", self.dtype, (m, width))
        _need((w2 is None) == (out2 is None), "add2_rmsnorm2: the second norm needs a weight and an output")
        if w2 is not None:
            _tensor(w2, "w2", torch.float32, (width,))
            _tensor(out2, "out2", self.dtype, (m, width))
        fn = self._lib("elementwise").mlr_add2_rmsnorm2
        _ok(fn(_p(h), _p(d1), _p(d2), _p(w1), _p(w2), _p(out1), _p(out2), _c_int(m), _c_int(width), _c_float(eps),
               _stream()), "add2_rmsnorm2")

    @timed("norm", _tensors_work())
    def residual_add2(self, h, d1, d2=None):
        """h += d1 + d2 (d2 may be None), the sum of the two taken in 32-bit first."""
        _tensor(h, "h", torch.float32, ndim=2)
        _tensor(d1, "d1", self.dtype, tuple(h.shape))
        if d2 is not None:
            _tensor(d2, "d2", self.dtype, tuple(h.shape))
        fn = self._lib("elementwise").mlr_residual_add2
        _ok(fn(_p(h), _p(d1), _p(d2), _c_size_t(h.numel()), _stream()), "residual_add2")

    @timed("activation", _tensors_work())
    def clamped_glu(self, gate_up, act, limit, slope):
        """act = g * sigmoid(slope * g) * (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit);
        gate_up = [gate | up] side by side."""
        _tensor(gate_up, "gate_up", self.dtype, ndim=2)
        m, two_f = gate_up.shape
        _need(two_f % 2 == 0, "gate_up: the width must be even")
        _tensor(act, "act", self.dtype, (m, two_f // 2))
        fn = self._lib("elementwise").mlr_clamped_glu
        _ok(fn(_p(gate_up), _p(act), _c_int(m), _c_int(two_f // 2), _c_float(limit), _c_float(slope), _stream()),
            "clamped_glu")

    def _columns(self, t, name, dtype, rows, width):
        """A block of `width` columns of a row-major matrix (a view `x[:, a:b]` or a whole matrix): its row stride."""
        _need(isinstance(t, torch.Tensor) and t.is_cuda and t.dtype is dtype and t.dim() == 2
              and tuple(t.shape) == (rows, width) and (t.stride(1) == 1 or width == 1) and t.stride(0) >= width,
              lambda: f"{name}: expected {dtype} columns [{rows}, {width}] of a row-major matrix on the GPU")
        return t.stride(0)

    @timed("norm", _tensors_work())
    def gated_part_norm(self, y, gate, weight, out, part, eps, gate_first, gate_kind="silu"):
        """y float [rows, width] in parts of `part` values, each over its root mean square, times
        weight[i % len(weight)]; the activation of `gate` (columns of a matrix) multiplies before the norm
        (`gate_first`) or after it."""
        _tensor(y, "y", torch.float32, ndim=2)
        m, width = y.shape
        stride = self._columns(gate, "gate", self.dtype, m, width)
        _tensor(weight, "weight", torch.float32, ndim=1)
        period = weight.numel()
        _need(part >= 1 and width % part == 0 and period in (part, width), "gated_part_norm: sizes do not fit")
        _need(gate_kind in ("silu", "sigmoid"), "gated_part_norm: unknown gate")
        _tensor(out, "out", self.dtype, (m, width))
        fn = self._lib("elementwise").mlr_gated_part_norm
        _ok(fn(_p(y), _p(gate), ctypes.c_long(stride), _p(weight), _p(out), _c_int(m), _c_int(width), _c_int(part),
               _c_int(period), _c_float(eps), _c_int(1 if gate_first else 0), _c_int(0 if gate_kind == "silu" else 1),
               _stream()), "gated_part_norm")

    # -- mixers with a state of fixed size ------------------------------------------------------------
    CONV_MAX_TAPS = 8
    RECURRENCE_MAX_KEYS = 256

    @timed("conv", _tensors_work())
    def causal_conv(self, x, weight, bias, out, live, stage, state_offset, slots, positions, silu=True, write_state=True):
        """out[r, c] = act(bias[c] + sum_j weight[c, j] * input j - (taps - 1) tokens from r), a request's earlier
        inputs taken from the step's rows or from its state: `live`/`stage` [slots, floats] hold them from
        `state_offset` on as [taps - 1][channels]."""
        rows, channels = x.shape
        xs = self._columns(x, "x", self.dtype, rows, channels)
        _tensor(weight, "weight", torch.float32, ndim=2)
        taps = weight.shape[1]
        _need(weight.shape[0] == channels and 1 <= taps <= self.CONV_MAX_TAPS, "causal_conv: weight must be [channels, 1..8 taps]")
        if bias is not None:
            _tensor(bias, "bias", torch.float32, (channels,))
        os_ = self._columns(out, "out", self.dtype, rows, channels)
        self._check_state(live, stage, state_offset, (taps - 1) * channels)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        fn = self._lib("recurrence").mlr_causal_conv
        at = state_offset * 4
        _ok(fn(_p(x), ctypes.c_long(xs), _p(weight), _p(bias), _p(out), ctypes.c_long(os_), _ptr(live.data_ptr() + at),
               _ptr(stage.data_ptr() + at), ctypes.c_long(live.stride(0)), _p(slots), _p(positions), _c_int(rows),
               _c_int(channels), _c_int(taps), _c_int(1 if silu else 0), _c_int(1 if write_state else 0), _stream()),
            "causal_conv")

    @staticmethod
    def _check_state(live, stage, offset, count):
        for name, t in (("live", live), ("stage", stage)):
            _need(isinstance(t, torch.Tensor) and t.is_cuda and t.dtype is torch.float32 and t.dim() == 2
                  and t.is_contiguous(), f"{name}: the state must be float32 [slots, floats] on the GPU")
        _need(live.shape == stage.shape and 0 <= offset and offset + count <= live.shape[1],
              "the state does not hold what the kernel reads and writes")

    @timed("activation", _tensors_work())
    def gla_log_decay(self, z, bias, out, tau):
        """out = log(sigmoid(z + bias)^(1 / tau)), 32-bit."""
        _tensor(z, "z", self.dtype, ndim=2)
        rows, width = z.shape
        _tensor(bias, "bias", torch.float32, (width,))
        _tensor(out, "out", torch.float32, (rows, width))
        _need(tau > 0, "gla_log_decay: tau must be positive")
        fn = self._lib("recurrence").mlr_gla_log_decay
        _ok(fn(_p(z), _p(bias), _p(out), _c_int(rows), _c_int(width), _c_float(1.0 / tau), _stream()), "gla_log_decay")

    @timed("activation", _tensors_work())
    def mamba_step(self, raw, dt_bias, a_log, dt, log_decay):
        """dt = softplus(raw + dt_bias), log_decay = -exp(a_log) * dt, 32-bit; raw: columns [rows, heads]."""
        rows, heads = raw.shape
        stride = self._columns(raw, "raw", self.dtype, rows, heads)
        _tensor(dt_bias, "dt_bias", torch.float32, (heads,))
        _tensor(a_log, "a_log", torch.float32, (heads,))
        _tensor(dt, "dt", torch.float32, (rows, heads))
        _tensor(log_decay, "log_decay", torch.float32, (rows, heads))
        fn = self._lib("recurrence").mlr_mamba_step
        _ok(fn(_p(raw), ctypes.c_long(stride), _p(dt_bias), _p(a_log), _p(dt), _p(log_decay), _c_int(rows), _c_int(heads),
               _stream()), "mamba_step")

    @timed("recurrence", _tensors_work())
    def linear_recurrence(self, q, k, v, log_decay, out, live, stage, state_offset, seg_first, seg_count, segments, slots,
                          heads, n_keys, n_values, heads_per_group=1, v_scale=None, skip=None, q_scale=1.0,
                          write_state=True, piece_state=None, piece_decay=None, activation=None):
        """Per request of the step and head, from the live state: S_t = diag(exp(log_decay_t)) S_(t-1) + k_t (v_scale_t
        v_t)^T, out_t = S_t^T (q_scale q_t) + skip[head] v_t.  q, k: columns [rows, (heads / heads_per_group) * n_keys];
        v: columns [rows, heads * n_values]; log_decay float [rows, heads * n_keys] (a decay per key channel) or
        [rows, heads] (one per head); v_scale float [rows, heads]; the state [heads][n_keys][n_values] floats from
        `state_offset` on in a slot's row of `live`/`stage`.
        With `piece_state` float [segments * heads * n_keys * n_values] and `piece_decay` float [segments * heads *
        n_keys]: `seg_first`/`seg_count` name PIECES of requests (a request's pieces one after the other), which run
        side by side in three passes; the result differs from the token-by-token order by 32-bit rounding.
        log_decay float [heads]: one constant decay a head.  `activation` "silu": q, k and v pass it as they are read."""
        rows = v.shape[0]
        groups = heads // heads_per_group
        _need(heads >= 1 and heads_per_group >= 1 and heads % heads_per_group == 0, "linear_recurrence: heads and groups")
        _need(1 <= n_keys <= self.RECURRENCE_MAX_KEYS, f"linear_recurrence: 1..{self.RECURRENCE_MAX_KEYS} key channels a head")
        qs = self._columns(q, "q", self.dtype, rows, groups * n_keys)
        ks = self._columns(k, "k", self.dtype, rows, groups * n_keys)
        vs = self._columns(v, "v", self.dtype, rows, heads * n_values)
        _need(activation in (None, "silu"), f"linear_recurrence: activation {activation!r}")
        if log_decay.dim() == 1:                # the same decays for every token
            _tensor(log_decay, "log_decay", torch.float32, (heads,))
            per_channel, decay_stride = False, 0
        else:
            _tensor(log_decay, "log_decay", torch.float32, ndim=2)
            per_channel = log_decay.shape[1] == heads * n_keys
            _need(tuple(log_decay.shape) in ((rows, heads * n_keys), (rows, heads)),
                  "log_decay: [rows, heads * keys], [rows, heads] or [heads]")
            decay_stride = log_decay.shape[1]
            if n_keys == 1:
                per_channel = True              # (the two layouts coincide)
        if v_scale is not None:
            _tensor(v_scale, "v_scale", torch.float32, (rows, heads))
        if skip is not None:
            _tensor(skip, "skip", torch.float32, (heads,))
        _tensor(out, "out", torch.float32, (rows, heads * n_values))
        self._check_state(live, stage, state_offset, heads * n_keys * n_values)
        _tensor(seg_first, "seg_first", torch.int32, (segments,))
        _tensor(seg_count, "seg_count", torch.int32, (segments,))
        _tensor(slots, "slots", torch.int32, (rows,))
        _need(segments <= 65535 * 32 and heads <= 65535, "linear_recurrence: too many requests or heads for the grid")
        _need((piece_state is None) == (piece_decay is None), "linear_recurrence: piece_state and piece_decay go together")
        if piece_state is not None:
            _tensor(piece_state, "piece_state", torch.float32, ndim=1)
            _tensor(piece_decay, "piece_decay", torch.float32, ndim=1)
            _need(piece_state.numel() >= segments * heads * n_keys * n_values and piece_decay.numel() >= segments * heads * n_keys,
                  "linear_recurrence: the pieces' buffers are too small")
        fn = self._lib("recurrence").mlr_linear_recurrence
        at = state_offset * 4
        _ok(fn(_p(q), ctypes.c_long(qs), _p(k), ctypes.c_long(ks), _p(v), ctypes.c_long(vs), _p(log_decay),
               ctypes.c_long(decay_stride), _c_int(1 if per_channel else 0), _p(v_scale),
               ctypes.c_long(heads if v_scale is not None else 0), _p(skip), _c_float(q_scale), _p(out),
               _ptr(live.data_ptr() + at), _ptr(stage.data_ptr() + at), ctypes.c_long(live.stride(0)), _p(seg_first),
               _p(seg_count), _p(slots), _c_int(segments), _c_int(heads), _c_int(heads_per_group), _c_int(n_keys),
               _c_int(n_values), _c_int(1 if write_state else 0), _p(piece_state), _p(piece_decay),
               _c_int(1 if activation == "silu" else 0), _stream()), "linear_recurrence")

    @timed("activation", _tensors_work())
    def channel_log_decay(self, z, bias, a_log, out, heads, n_keys):
        """out = -exp(a_log[head]) * softplus(z + bias): the logarithm of a decay per key channel, 32-bit;
        z float [rows, heads * n_keys], bias float [heads * n_keys] or None, a_log float [heads]."""
        _tensor(z, "z", torch.float32, ndim=2)
        rows = z.shape[0]
        _need(z.shape[1] == heads * n_keys, "channel_log_decay: z must be [rows, heads * keys]")
        if bias is not None:
            _tensor(bias, "bias", torch.float32, (heads * n_keys,))
        _tensor(a_log, "a_log", torch.float32, (heads,))
        _tensor(out, "out", torch.float32, (rows, heads * n_keys))
        _ok(self._lib("recurrence").mlr_channel_log_decay(_p(z), _p(bias), _p(a_log), _p(out), _c_int(rows), _c_int(heads),
                                                          _c_int(n_keys), _stream()), "channel_log_decay")

    @timed("recurrence", _tensors_work())
    def delta_rule(self, q, k, v, log_decay, beta_raw, out, live, stage, state_offset, seg_first, seg_count, segments, slots,
                   heads, n_keys, n_values, heads_per_group=1, q_scale=1.0, unit_norm=True, unit_eps=1e-6, write_state=True,
                   decay_per_head=False):
        """Per request of the step and head, from the live state: S <- diag(exp(log_decay_t)) S; u = beta_t (v_t - S^T k_t);
        S <- S + k_t u^T; out_t = S^T q_t, with beta = sigmoid(beta_raw).  q, k: columns [rows, (heads / heads_per_group) *
        n_keys], made unit vectors per head inside (x / sqrt(sum x^2 + unit_eps); `unit_norm` False: taken as they
        are) and q multiplied by q_scale; v: columns [rows, heads * n_values]; log_decay float [rows, heads * n_keys], or
        with `decay_per_head` [rows, heads] (one decay for all key channels of a head);
        beta_raw float columns [rows, heads]; the state [heads][n_keys][n_values] floats from `state_offset` on in a
        slot's row of `live`/`stage`."""
        rows = v.shape[0]
        _need(heads >= 1 and heads_per_group >= 1 and heads % heads_per_group == 0, "delta_rule: heads and groups")
        groups = heads // heads_per_group
        _need(1 <= n_keys <= self.RECURRENCE_MAX_KEYS, f"delta_rule: 1..{self.RECURRENCE_MAX_KEYS} key channels a head")
        qs = self._columns(q, "q", self.dtype, rows, groups * n_keys)
        ks = self._columns(k, "k", self.dtype, rows, groups * n_keys)
        vs = self._columns(v, "v", self.dtype, rows, heads * n_values)
        _tensor(log_decay, "log_decay", torch.float32, (rows, heads if decay_per_head else heads * n_keys))
        bs = self._columns(beta_raw, "beta_raw", torch.float32, rows, heads)
        _tensor(out, "out", torch.float32, (rows, heads * n_values))
        self._check_state(live, stage, state_offset, heads * n_keys * n_values)
        _tensor(seg_first, "seg_first", torch.int32, (segments,))
        _tensor(seg_count, "seg_count", torch.int32, (segments,))
        _tensor(slots, "slots", torch.int32, (rows,))
        _need(segments <= 65535 * 32 and heads <= 65535, "delta_rule: too many requests or heads for the grid")
        at = state_offset * 4
        _ok(self._lib("recurrence").mlr_delta_rule(
            _p(q), ctypes.c_long(qs), _p(k), ctypes.c_long(ks), _p(v), ctypes.c_long(vs), _p(log_decay), _p(beta_raw),
            ctypes.c_long(bs), _p(out), _ptr(live.data_ptr() + at), _ptr(stage.data_ptr() + at), ctypes.c_long(live.stride(0)),
            _p(seg_first), _p(seg_count), _p(slots), _c_int(segments), _c_int(heads), _c_int(heads_per_group), _c_int(n_keys),
            _c_int(n_values), _c_int(1 if write_state else 0), _c_int(1 if unit_norm else 0), _c_float(q_scale),
            _c_float(unit_eps), _c_int(1 if decay_per_head else 0), _stream()), "delta_rule")

    DELTA_CHUNK_MAX_KEYS = 128

    def delta_chunk_tokens(self):
        """Tokens in a chunk of `delta_rule_chunked`."""
        return int(self._lib("recurrence").mlr_delta_chunk_tokens())

    def delta_chunk_floats(self, chunks, heads, n_keys, n_values):
        """Floats of scratch memory that `delta_rule_chunked` needs for so many chunks."""
        fn = self._lib("recurrence").mlr_delta_chunk_floats
        fn.restype = ctypes.c_long
        return int(chunks) * int(heads) * int(fn(_c_int(n_keys), _c_int(n_values)))

    @timed("recurrence", _tensors_work())
    def delta_rule_chunked(self, q, k, v, log_decay, beta_raw, out, live, stage, state_offset, seg_first, seg_count, segments,
                           slots, chunk_first, chunk_count, chunks, scratch, heads, n_keys, n_values, heads_per_group=1,
                           q_scale=1.0, unit_norm=True, unit_eps=1e-6, write_state=True, decay_per_head=False):
        """`delta_rule` over chunks of tokens: `chunk_first`/`chunk_count` cut every request of the step into chunks of
        at most `delta_chunk_tokens()` tokens (a request's chunks one after the other, the requests in the order of
        `seg_first`); what a chunk does to ANY state it might start from is worked out for all chunks side by side,
        then a request's chunks are applied in their order.  Up to DELTA_CHUNK_MAX_KEYS key channels a head; the
        result differs from the token-by-token order by 32-bit rounding."""
        rows = v.shape[0]
        _need(heads >= 1 and heads_per_group >= 1 and heads % heads_per_group == 0, "delta_rule_chunked: heads and groups")
        groups = heads // heads_per_group
        _need(1 <= n_keys <= self.DELTA_CHUNK_MAX_KEYS, f"delta_rule_chunked: 1..{self.DELTA_CHUNK_MAX_KEYS} key channels a head")
        qs = self._columns(q, "q", self.dtype, rows, groups * n_keys)
        ks = self._columns(k, "k", self.dtype, rows, groups * n_keys)
        vs = self._columns(v, "v", self.dtype, rows, heads * n_values)
        _tensor(log_decay, "log_decay", torch.float32, (rows, heads if decay_per_head else heads * n_keys))
        bs = self._columns(beta_raw, "beta_raw", torch.float32, rows, heads)
        _tensor(out, "out", torch.float32, (rows, heads * n_values))
        self._check_state(live, stage, state_offset, heads * n_keys * n_values)
        _tensor(seg_first, "seg_first", torch.int32, (segments,))
        _tensor(seg_count, "seg_count", torch.int32, (segments,))
        _tensor(chunk_first, "chunk_first", torch.int32, (chunks,))
        _tensor(chunk_count, "chunk_count", torch.int32, (chunks,))
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(scratch, "scratch", torch.float32, ndim=1)
        _need(scratch.numel() >= self.delta_chunk_floats(chunks, heads, n_keys, n_values), "delta_rule_chunked: scratch too small")
        _need(segments <= 65535 * 32 and heads <= 65535 and chunks >= segments, "delta_rule_chunked: requests, chunks or heads")
        at = state_offset * 4
        _ok(self._lib("recurrence").mlr_delta_rule_chunked(
            _p(q), ctypes.c_long(qs), _p(k), ctypes.c_long(ks), _p(v), ctypes.c_long(vs), _p(log_decay), _p(beta_raw),
            ctypes.c_long(bs), _p(out), _ptr(live.data_ptr() + at), _ptr(stage.data_ptr() + at), ctypes.c_long(live.stride(0)),
            _p(seg_first), _p(seg_count), _p(slots), _c_int(segments), _p(chunk_first), _p(chunk_count), _c_int(chunks),
            _p(scratch), _c_int(heads), _c_int(heads_per_group), _c_int(n_keys), _c_int(n_values),
            _c_int(1 if write_state else 0), _c_int(1 if unit_norm else 0), _c_float(q_scale), _c_float(unit_eps),
            _c_int(1 if decay_per_head else 0), _stream()), "delta_rule_chunked")

    # -- differential attention -----------------------------------------------------------------------
    DIFF_MAX_HEAD_DIM = 256
    DIFF_MAX_VALUE_DIM = 256

    def _check_diff_cache(self, k_pages, v_pages, kv_heads, head_dim, value_dim, page_size):
        _tensor(k_pages, "k_pages", self.dtype, ndim=4)
        _tensor(v_pages, "v_pages", self.dtype, ndim=4)
        pages = k_pages.shape[0]
        _need(tuple(k_pages.shape) == (pages, kv_heads, page_size, 2 * head_dim), "k_pages: [pages, kv_heads, page, 2 * head_dim]")
        _need(tuple(v_pages.shape) == (pages, kv_heads, value_dim, page_size), "v_pages: [pages, kv_heads, value_dim, page]")

    @timed("rope_kv", _tensors_work())
    def diff_kv_write(self, k, v, k_pages, v_pages, block_table, slots, positions, kv_heads, head_dim, value_dim, page_size):
        """The step's keys (both maps) and values into their pages."""
        rows = k.shape[0]
        ks = self._columns(k, "k", self.dtype, rows, kv_heads * 2 * head_dim)
        vs = self._columns(v, "v", self.dtype, rows, kv_heads * value_dim)
        self._check_diff_cache(k_pages, v_pages, kv_heads, head_dim, value_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        fn = self._lib("diff_attention").mlr_diff_kv_write
        _ok(fn(_p(k), ctypes.c_long(ks), _p(v), ctypes.c_long(vs), _p(k_pages), _p(v_pages), _p(block_table),
               _c_int(block_table.shape[1]), _p(slots), _p(positions), _c_int(rows), _c_int(kv_heads), _c_int(2 * head_dim),
               _c_int(value_dim), _c_int(page_size), _stream()), "diff_kv_write")

    @timed("rope_kv", _tensors_work())
    def diff_qkv_prep(self, q, k, v, k_pages, v_pages, block_table, slots, positions, rope, q_heads, kv_heads, head_dim,
                      value_dim, page_size, write_cache=True, interleaved=False):
        """The step's queries and keys (both maps of every head) turned by their positions, the keys and values into
        their pages.  q: columns [rows, q_heads * 2 * head_dim], turned in place; rope float [positions, rot] (cosines,
        then sines): the first rot channels of each map turn, in pairs (j, j + rot / 2) or, `interleaved`,
        (2 j, 2 j + 1); None: nothing turns."""
        rows = k.shape[0]
        qs = self._columns(q, "q", self.dtype, rows, q_heads * 2 * head_dim)
        ks = self._columns(k, "k", self.dtype, rows, kv_heads * 2 * head_dim)
        vs = self._columns(v, "v", self.dtype, rows, kv_heads * value_dim)
        self._check_diff_cache(k_pages, v_pages, kv_heads, head_dim, value_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        rot = 0
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            rot = rope.shape[1]
            _need(rot % 2 == 0 and 2 <= rot <= head_dim, "diff_qkv_prep: the rotation turns an even part of a map")
        fn = self._lib("diff_attention").mlr_diff_qkv_prep
        _ok(fn(_p(q), ctypes.c_long(qs), _p(k), ctypes.c_long(ks), _p(v), ctypes.c_long(vs), _p(k_pages), _p(v_pages),
               _p(block_table), _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(rope), _c_int(rot),
               _c_int(1 if interleaved else 0), _c_int(rows), _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim),
               _c_int(value_dim), _c_int(page_size), _c_int(1 if write_cache else 0), _stream()), "diff_qkv_prep")

    MASK_KINDS = {None: 0, "window": 1, "chunk": 2}

    @staticmethod
    def diff_partial_numel(rows, q_heads, value_dim, max_splits):
        return rows * q_heads * 2 * max(1, max_splits) * (value_dim + 2)

    @timed("attention")
    def diff_attention(self, q, k_pages, v_pages, block_table, slots, positions, gate, out, partial, q_heads, kv_heads,
                       head_dim, value_dim, page_size, scale, lam, out_scale, eps, softcap=None, temp_coef=0.0,
                       temp_every=1.0, split_keys=0, max_splits=1, mask=None, mask_size=0):
        """Differential attention of every token of the step over the cached keys at positions <= its own (the step's
        own keys are in the cache already): out [rows, q_heads * value_dim], normed, scaled and gated by
        sigmoid(gate) (gate None: no gate).  q: columns [rows, q_heads * 2 * head_dim].  `mask`: None, or "window"
        (the last mask_size positions) or "chunk" (the query's own block of mask_size positions)."""
        _need(mask in self.MASK_KINDS and (mask is None or mask_size >= 1), "diff_attention: mask rule")
        rows = q.shape[0]
        qs = self._columns(q, "q", self.dtype, rows, q_heads * 2 * head_dim)
        gs = self._columns(gate, "gate", self.dtype, rows, q_heads * value_dim) if gate is not None else 0
        self._check_diff_cache(k_pages, v_pages, kv_heads, head_dim, value_dim, page_size)
        _need(head_dim <= self.DIFF_MAX_HEAD_DIM and value_dim <= self.DIFF_MAX_VALUE_DIM,
              f"diff_attention: head sizes up to {self.DIFF_MAX_HEAD_DIM} (keys) and {self.DIFF_MAX_VALUE_DIM} (values)")
        _need(q_heads % kv_heads == 0, "diff_attention: q_heads must be a multiple of kv_heads")
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        _tensor(out, "out", self.dtype, (rows, q_heads * value_dim))
        _tensor(partial, "partial", torch.float32, ndim=1)
        max_splits = max(1, max_splits)
        _need(partial.numel() >= self.diff_partial_numel(rows, q_heads, value_dim, max_splits), "diff_attention: partial too small")
        _need(max_splits == 1 or (split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0 and max_splits <= MAX_KEY_SPLITS),
              "diff_attention: key ranges must be multiples of 64 keys, at most 1024 of them")
        _need(rows * 1 <= 2 ** 31 - 1 and q_heads * 2 <= 65535 and max_splits <= 65535, "diff_attention: grid too large")
        fn = self._lib("diff_attention").mlr_diff_attention
        _ok(fn(_p(q), ctypes.c_long(qs), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(gate), ctypes.c_long(gs), _p(out), _p(partial), _c_int(rows), _c_int(q_heads),
               _c_int(kv_heads), _c_int(head_dim), _c_int(value_dim), _c_int(page_size), _c_float(scale),
               _c_float(softcap or 0.0), _c_float(temp_coef), _c_float(temp_every), _c_float(lam), _c_float(out_scale),
               _c_float(eps), _c_int(split_keys), _c_int(max_splits), _ptr(0), _ptr(0), _c_int(0), _c_int(0),
               _c_int(self.MASK_KINDS[mask]), _c_int(mask_size), _stream()),
            "diff_attention")

    def diff_tiles_supported(self, q_heads, kv_heads, head_dim, value_dim, page_size, q_stride=0, gate_stride=0):
        """Whether the matrix-core kernel takes these sizes: the bfloat16 engine, head sizes in multiples of 16 up to
        128, pages in multiples of 8 tokens, operands aligned to its 16-byte accesses."""
        return (self.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 128 and value_dim % 16 == 0
                and value_dim <= 128 and page_size % 8 == 0 and q_heads % kv_heads == 0 and q_stride % 8 == 0
                and gate_stride % 4 == 0)

    DIFF_TILES_PAGES = 2048

    @classmethod
    def diff_tiles_reach(cls, page_size):
        """The most keys that one workgroup of the matrix-core kernel walks (it keeps their pages' ids in LDS)."""
        return (cls.DIFF_TILES_PAGES - 2) * page_size

    @staticmethod
    def diff_tiles_group_tokens(q_heads, kv_heads):
        """Tokens of a prompt portion that one workgroup of the matrix-core kernel takes: its four wavefronts serve
        16 tokens of one query head each, up to four heads of one kv head side by side."""
        return 16 * (4 // min(4, q_heads // kv_heads))

    @timed("attention")
    def diff_attention_tiles(self, q, k_pages, v_pages, block_table, slots, positions, gate, out, partial, group_row0,
                             group_ntok, groups, group_tokens, q_heads, kv_heads, head_dim, value_dim, page_size, scale, lam,
                             out_scale, eps, softcap=None, temp_coef=0.0, temp_every=1.0, split_keys=0, max_splits=1,
                             max_context=None, mask=None, mask_size=0):
        """As `diff_attention` for the rows of `groups` groups of consecutive tokens of one request each (first row,
        number of tokens: device int32 vectors; at most `group_tokens` tokens a group), on the matrix cores.
        `max_context`: a bound on the step's positions + 1 (default: what the block table can hold); the keys that one
        workgroup walks -- a key range, or all of them -- must lie in `DIFF_TILES_PAGES` pages at most."""
        rows = q.shape[0]
        qs = self._columns(q, "q", self.dtype, rows, q_heads * 2 * head_dim)
        gs = self._columns(gate, "gate", self.dtype, rows, q_heads * value_dim) if gate is not None else 0
        _need(self.diff_tiles_supported(q_heads, kv_heads, head_dim, value_dim, page_size, qs, gs),
              "diff_attention_tiles: sizes not taken (see diff_tiles_supported)")
        _need(q.data_ptr() % 16 == 0 and (gate is None or gate.data_ptr() % 8 == 0), "diff_attention_tiles: unaligned operands")
        self._check_diff_cache(k_pages, v_pages, kv_heads, head_dim, value_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        _tensor(out, "out", self.dtype, (rows, q_heads * value_dim))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(1 <= group_tokens <= self.diff_tiles_group_tokens(q_heads, kv_heads), "diff_attention_tiles: group too large")
        max_splits = max(1, max_splits)
        # partial results: with key ranges always; without them for groups of up to four tokens when `partial` is
        # given (the two maps then run in wavefronts of their own and the merge kernel finishes the head)
        through_partial = max_splits > 1 or (partial is not None and group_tokens <= 4)
        if through_partial:
            _tensor(partial, "partial", torch.float32, ndim=1)
            _need(partial.numel() >= self.diff_partial_numel(groups * group_tokens, q_heads, value_dim, max_splits),
                  "diff_attention_tiles: partial too small")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0 and max_splits <= MAX_KEY_SPLITS,
                  "diff_attention_tiles: key ranges must be multiples of 64 keys, at most 1024 of them")
        _need(kv_heads * 4 <= 65535 and max_splits <= 65535, "diff_attention_tiles: grid too large")
        if max_context is None:
            max_context = block_table.shape[1] * page_size
        _need(mask in self.MASK_KINDS and (mask is None or mask_size >= 1), "diff_attention_tiles: mask rule")
        walk = max_context if mask is None else min(max_context, mask_size + group_tokens + 2 * ATTENTION_TILE_KEYS)
        _need(self.diff_tiles_reach(page_size) >= (split_keys if max_splits > 1 else walk),
              "diff_attention_tiles: one workgroup would walk more pages than it keeps ids of; cut the keys into ranges")
        fn = self._lib("diff_attention").mlr_diff_attention_tiles
        _ok(fn(_p(q), ctypes.c_long(qs), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(gate), ctypes.c_long(gs), _p(out), _p(partial if through_partial else None), _p(group_row0),
               _p(group_ntok), _c_int(groups), _c_int(group_tokens), _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim),
               _c_int(value_dim), _c_int(page_size), _c_float(scale), _c_float(softcap or 0.0), _c_float(temp_coef),
               _c_float(temp_every), _c_float(lam), _c_float(out_scale), _c_float(eps), _c_int(split_keys),
               _c_int(max_splits), _c_int(max_context), _c_int(self.MASK_KINDS[mask]), _c_int(mask_size), _stream()),
            "diff_attention_tiles")

    # -- layer norm, plain activations ---------------------------------------------------------
    @timed("norm", _tensors_work())
    def layernorm_add(self, delta, weight, bias, h, cast=None, eps=1e-5):
        """h += layernorm(delta) * weight + bias, row by row (h the float residual stream, delta a sublayer's
        output); `cast`, when given, receives T(h): the stream as the next sublayer's input."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        if bias is not None:
            _tensor(bias, "bias", torch.float32, (width,))
        if cast is not None:
            _tensor(cast, "cast", self.dtype, (m, width))
        _ok(self._lib("elementwise").mlr_layernorm(_p(delta), _ptr(0), _p(weight), _p(bias), _ptr(0), _p(h), _p(cast),
                                                   _ptr(0), _c_int(m), _c_int(width), _c_float(eps), _c_float(1.0),
                                                   _stream()), "layernorm_add")

    @timed("norm", _tensors_work())
    def tanh_norm_rows(self, h, delta, weight, bias, alpha, out, rows=None, write_h=True):
        """x = h + delta (delta may be None; written back to h when write_h); out[r] = T(tanh(alpha x[rows[r] or r]) *
        weight + bias): a norm that takes no statistics, element by element in 32-bit."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        _tensor(bias, "bias", torch.float32, (width,))
        if rows is not None:
            _tensor(rows, "rows", torch.int32, ndim=1)
            _need(delta is None or not write_h, "tanh_norm_rows: a gathered norm does not write the stream")
        n_out = rows.numel() if rows is not None else m
        _tensor(out, "out", self.dtype, (n_out, width))
        _ok(self._lib("elementwise").mlr_tanh_norm_rows(_p(h), _p(delta), _p(weight), _p(bias), _c_float(alpha), _p(out),
                                                        _p(rows), _c_int(n_out), _c_int(width), _c_int(1 if write_h else 0),
                                                        _stream()), "tanh_norm_rows")

    @timed("norm", _tensors_work())
    def tanh_norm_add(self, delta, weight, bias, alpha, h, extra=None, then=None, out=None):
        """h += tanh(alpha delta) * weight + bias (+ extra, float like h): the norm of what a sublayer gave, added to the
        float residual stream; `then` = (weight, bias, alpha) of the norm in front of the next sublayer and `out` (the
        engine's element type): out = that norm of the new h, in the same pass."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        _tensor(bias, "bias", torch.float32, (width,))
        if extra is not None:
            _tensor(extra, "extra", torch.float32, (m, width))
        wn = bn = None
        an = 0.0
        if out is not None:
            _need(then is not None, "tanh_norm_add: an output needs the norm that makes it")
            wn, bn, an = then
            _tensor(wn, "then.weight", torch.float32, (width,))
            _tensor(bn, "then.bias", torch.float32, (width,))
            _tensor(out, "out", self.dtype, (m, width))
        _ok(self._lib("elementwise").mlr_tanh_norm_add(_p(delta), _p(weight), _p(bias), _c_float(alpha), _p(h), _p(extra),
                                                       _p(wn), _p(bn), _c_float(an), _p(out), _c_int(m), _c_int(width),
                                                       _stream()), "tanh_norm_add")

    @timed("norm", _tensors_work())
    def copy_float(self, src, dst):
        """dst = src (float tensors of one shape)."""
        _tensor(src, "src", torch.float32)
        _tensor(dst, "dst", torch.float32, tuple(src.shape))
        _ok(self._lib("elementwise").mlr_copy_float(_p(src), _p(dst), _c_size_t(src.numel()), _stream()), "copy_float")

    @timed("activation", _tensors_work())
    def tanh_cap(self, x, cap):
        """x <- cap * tanh(x / cap) on float values in place (a cap on logits)."""
        _tensor(x, "x", torch.float32)
        _need(cap > 0.0, "tanh_cap: the cap must be positive")
        _ok(self._lib("elementwise").mlr_tanh_cap(_p(x), _c_float(cap), _c_size_t(x.numel()), _stream()), "tanh_cap")

    @timed("activation", _tensors_work())
    def head_gate_mul(self, x, gate, out, heads):
        """out[m, head, :] = x[m, head, :] * sigmoid(gate[m, head]): x, out [rows, heads * part]; gate: columns
        [rows, heads] of a row-major matrix; out may be x."""
        _tensor(x, "x", self.dtype, ndim=2)
        m, width = x.shape
        _need(heads >= 1 and width % heads == 0, "head_gate_mul: the width is no multiple of the heads")
        stride = self._columns(gate, "gate", self.dtype, m, heads)
        _tensor(out, "out", self.dtype, (m, width))
        _ok(self._lib("elementwise").mlr_head_gate_mul(_p(x), _p(gate), ctypes.c_long(stride), _p(out), _c_int(m),
                                                       _c_int(width), _c_int(width // heads), _stream()), "head_gate_mul")

    @timed("norm", _tensors_work())
    def layernorm_rows(self, h, weight, bias, out, eps, rows=None, out_scale=1.0):
        """out[r] = T((layernorm(h[rows[r] or r]) * weight + bias) * out_scale), h float."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        _tensor(weight, "weight", torch.float32, (width,))
        if bias is not None:
            _tensor(bias, "bias", torch.float32, (width,))
        if rows is not None:
            _tensor(rows, "rows", torch.int32, ndim=1)
        n_out = rows.numel() if rows is not None else m
        _tensor(out, "out", self.dtype, (n_out, width))
        _ok(self._lib("elementwise").mlr_layernorm(_ptr(0), _p(h), _p(weight), _p(bias), _p(rows), _ptr(0), _ptr(0),
                                                   _p(out), _c_int(n_out), _c_int(width), _c_float(eps),
                                                   _c_float(out_scale), _stream()), "layernorm_rows")

    @timed("activation", _tensors_work())
    def relu_squared(self, x, out):
        """out = max(x, 0)^2 (x and out may be the same tensor)."""
        _tensor(x, "x", self.dtype)
        _tensor(out, "out", self.dtype, tuple(x.shape))
        _ok(self._lib("elementwise").mlr_relu_squared(_p(x), _p(out), _c_size_t(x.numel()), _stream()), "relu_squared")

    @timed("norm", _tensors_work())
    def cast_rows(self, h, out):
        """out = T(h), h float."""
        _tensor(h, "h", torch.float32)
        _tensor(out, "out", self.dtype, tuple(h.shape))
        _ok(self._lib("elementwise").mlr_cast_rows(_p(h), _p(out), _c_size_t(h.numel()), _stream()), "cast_rows")

    @timed("activation", _tensors_work())
    def scale_float(self, x, factor):
        """x *= factor, x float."""
        _tensor(x, "x", torch.float32)
        _ok(self._lib("elementwise").mlr_scale_float(_p(x), _c_float(factor), _c_size_t(x.numel()), _stream()),
            "scale_float")

    # -- attention with a sink and a mask rule -------------------------------------------------
    SINK_MASKS = {None: 0, "all": 0, "window": 1, "chunk": 2}
    SINK_MAX_KEY_DIM = 2048
    SINK_MAX_VALUE_DIM = 1024

    def _sink_pages(self, pages, name, kv_heads, page_size, least):
        """Row-major pages [pages, kv_heads, page, row]: the row's width (at least `least`)."""
        _tensor(pages, name, self.dtype, ndim=4)
        _need(pages.shape[1] == kv_heads and pages.shape[2] == page_size and pages.shape[3] >= least,
              lambda: f"{name}: expected [pages, {kv_heads}, {page_size}, >= {least}], got {tuple(pages.shape)}")
        return pages.shape[3]

    @timed("rope_kv", _rope_work)
    def sink_qkv_prep(self, proj, bias, q_out, k_pages, v_pages, block_table, slots, positions, q_norm_w, k_norm_w, eps,
                      rope, q_heads, kv_heads, key_dim, value_dim, page_size, write_cache=True, norm="auto",
                      interleaved=False):
        """From the stacked projection [rows, q_heads * key_dim + kv_heads * (key_dim + value_dim)] (further columns behind these are left alone): bias (float, may be
        None), per-head RMSNorm of q and k, rotation of a head's first rope.shape[1] channels in pairs (j, j + half)
        or, `interleaved`, (2 j, 2 j + 1) (rope float [positions, rot]: cosines | sines; may be None); q to q_out, k
        and v into their row-major pages.  `norm`: "before" the rotation, "after" it, None, or "auto" (before it when
        weights are given, else none); the weights may be None with any of them (a norm without a weight)."""
        total = q_heads * key_dim + kv_heads * (key_dim + value_dim)
        _tensor(proj, "proj", self.dtype, ndim=2)
        rows = proj.shape[0]
        _need(proj.shape[1] >= total, lambda: f"proj: expected a width of at least {total}, got {proj.shape[1]}")
        if bias is not None:
            _tensor(bias, "bias", torch.float32, (total,))
        _tensor(q_out, "q_out", self.dtype, (rows, q_heads * key_dim))
        _need(1 <= key_dim <= self.SINK_MAX_KEY_DIM, f"key_dim {key_dim}: up to {self.SINK_MAX_KEY_DIM}")
        k_row = self._sink_pages(k_pages, "k_pages", kv_heads, page_size, key_dim)
        v_row = self._sink_pages(v_pages, "v_pages", kv_heads, page_size, value_dim)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        if q_norm_w is not None:
            _tensor(q_norm_w, "q_norm_w", torch.float32, (key_dim,))
            _tensor(k_norm_w, "k_norm_w", torch.float32, (key_dim,))
        rot = 0
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            rot = rope.shape[1]
            _need(2 <= rot <= key_dim and rot % 2 == 0, f"rope: the table's width {rot} must be even and at most {key_dim}")
        if norm == "auto":
            norm = "before" if q_norm_w is not None else None
        _need(norm in (None, "before", "after"), f"sink_qkv_prep: norm {norm!r}")
        mode = {None: 0, "before": 1, "after": 2}[norm]
        _ok(self._lib("sink_attention").mlr_sink_qkv_prep(
            _p(proj), ctypes.c_long(proj.shape[1]), _p(bias), _p(q_out), _p(k_pages), ctypes.c_long(k_row), _p(v_pages),
            ctypes.c_long(v_row), _p(block_table), _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(q_norm_w),
            _p(k_norm_w), _c_float(eps), _p(rope), _c_int(rot), _c_int(rows), _c_int(q_heads), _c_int(kv_heads),
            _c_int(key_dim), _c_int(value_dim), _c_int(page_size), _c_int(1 if write_cache else 0), _c_int(mode),
            _c_int(1 if interleaved else 0), _stream()), "sink_qkv_prep")

    @timed("rope_kv", _rope_work)
    def latent_prep(self, proj, q_out, pages, block_table, slots, positions, norm_w, eps, rope, heads, dim, rot, rank,
                    page_size, write_cache=True, q_src=None, interleaved=False):
        """Latent attention's row work on proj [rows, heads * (dim + rot) + rank + rot]: every head's rotated query
        channels turned into q_out[:, head, rank:], the latent part normed and the shared rotated key part turned
        into the token's cache row [rank + rot] of pages [pages, 1, page, rank + rot].  With `q_src` (columns
        [rows, heads * (dim + rot)]) the queries come from there and proj holds [rows, rank + rot] only.  The rotated
        parts turn in pairs (j, j + rot / 2) or, `interleaved`, (2 j, 2 j + 1)."""
        rows = proj.shape[0]
        if q_src is None:
            _tensor(proj, "proj", self.dtype, ndim=2)
            _need(proj.shape[1] == heads * (dim + rot) + rank + rot, "proj: wrong width")
            q_ptr, q_ld = proj.data_ptr(), proj.shape[1]
            kv_ptr, kv_ld = proj.data_ptr() + heads * (dim + rot) * proj.element_size(), proj.shape[1]
        else:
            q_ld = self._columns(q_src, "q_src", self.dtype, rows, heads * (dim + rot))
            kv_ld = self._columns(proj, "proj", self.dtype, rows, rank + rot)
            q_ptr, kv_ptr = q_src.data_ptr(), proj.data_ptr()
        _tensor(q_out, "q_out", self.dtype, (rows, heads * (rank + rot)))
        _need(self._sink_pages(pages, "pages", 1, page_size, rank + rot) == rank + rot, "pages: rows of rank + rot")
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        _tensor(norm_w, "norm_w", torch.float32, (rank,))
        _tensor(rope, "rope", torch.float32, ndim=2)
        _need(rope.shape[1] == rot and rot % 2 == 0 and rot >= 2, "rope: as wide as the rotated part, which is even")
        _ok(self._lib("sink_attention").mlr_latent_prep(
            _ptr(q_ptr), ctypes.c_long(q_ld), _ptr(kv_ptr), ctypes.c_long(kv_ld), _p(q_out), _p(pages),
            ctypes.c_long(rank + rot), _p(block_table), _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(norm_w),
            _c_float(eps), _p(rope), _c_int(rows), _c_int(heads), _c_int(dim), _c_int(rot), _c_int(rank), _c_int(page_size),
            _c_int(1 if write_cache else 0), _c_int(1 if interleaved else 0), _stream()), "latent_prep")

    @timed("attention")
    def sink_attention(self, q, k_pages, v_pages, block_table, slots, positions, sink, out, q_heads, kv_heads, key_dim,
                       value_dim, page_size, scale, mask=None, mask_size=0):
        """out[m, h] = softmax (with one more summand exp(sink[h]) in the denominator; sink None: none) over the keys
        that token m sees of q.k * scale, times v.  mask: None/"all" (positions <= its own), "window" (the last
        mask_size positions), "chunk" (its own block of mask_size positions).  Keys are the first key_dim channels of
        k_pages' rows, values the first value_dim of v_pages' rows (which may be the same tensor)."""
        _tensor(q, "q", self.dtype, ndim=2)
        rows = q.shape[0]
        _need(q.shape[1] == q_heads * key_dim, "q: wrong width")
        _need(1 <= key_dim <= self.SINK_MAX_KEY_DIM and 1 <= value_dim <= self.SINK_MAX_VALUE_DIM,
              f"sink_attention: keys up to {self.SINK_MAX_KEY_DIM} channels, values up to {self.SINK_MAX_VALUE_DIM}")
        _need(q_heads % kv_heads == 0 and q_heads <= 65535, "q_heads must be a multiple of kv_heads")
        k_row = self._sink_pages(k_pages, "k_pages", kv_heads, page_size, key_dim)
        v_row = self._sink_pages(v_pages, "v_pages", kv_heads, page_size, value_dim)
        _need(mask in self.SINK_MASKS, f"mask {mask!r}: one of all, window, chunk")
        kind = self.SINK_MASKS[mask]
        _need(kind == 0 or mask_size >= 1, "a window or chunk needs a positive size")
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        if sink is not None:
            _tensor(sink, "sink", torch.float32, (q_heads,))
        _tensor(out, "out", self.dtype, (rows, q_heads * value_dim))
        _ok(self._lib("sink_attention").mlr_sink_attention(
            _p(q), ctypes.c_long(q.shape[1]), _p(k_pages), ctypes.c_long(k_row), _p(v_pages), ctypes.c_long(v_row),
            _p(block_table), _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(sink), _p(out),
            ctypes.c_long(out.shape[1]), _c_int(rows), _c_int(q_heads), _c_int(kv_heads), _c_int(key_dim),
            _c_int(value_dim), _c_int(page_size), _c_int(kind), _c_int(int(mask_size)), _c_float(scale), _stream()),
            "sink_attention")

    SINK_TILES_BLOCKS = 2048

    def sink_tiles_supported(self, key_dim, value_dim, k_row, v_row, page_size=16, mask=None, mask_size=0, max_context=0):
        """Whether the matrix-core kernel takes these sizes: the bfloat16 engine, keys in multiples of 8 channels up to
        576, values in multiples of 16 up to 512, cache rows that start at multiples of 16 bytes, and a key range of
        one workgroup (the window or chunk and its tokens; without a mask the step's longest context) whose page ids
        fit what the kernel keeps of them."""
        reach = max_context if self.SINK_MASKS.get(mask, 0) == 0 else mask_size + 64
        return (self.dtype == torch.bfloat16 and key_dim % 8 == 0 and value_dim % 16 == 0 and key_dim <= 576
                and value_dim <= 512 and k_row % 8 == 0 and v_row % 8 == 0
                and reach // page_size + 2 <= self.SINK_TILES_BLOCKS)

    @staticmethod
    def sink_tiles_layout(q_heads, kv_heads):
        """(heads side by side, tokens a group) of the matrix-core kernel's workgroups, for prompt portions (64 columns)
        and for single tokens and short portions (16 columns, `split_values`)."""
        per = q_heads // kv_heads
        p2 = 1
        while p2 < per:
            p2 *= 2
        big, small = min(p2, 64), min(p2, 16)
        return big, 64 // big, small, 16 // small

    @timed("attention")
    def sink_attention_tiles(self, q, k_pages, v_pages, block_table, slots, positions, sink, out, group_first, group_count,
                             groups, head_block, split_values, q_heads, kv_heads, key_dim, value_dim, page_size, scale,
                             mask=None, mask_size=0, max_context=0, partial=None, split_keys=0, splits=1):
        """`sink_attention` on the matrix cores for `groups` groups of consecutive tokens of one request each (device
        vectors group_first, group_count), at most 64 / head_block tokens a group (16 / head_block with
        `split_values`).  splits > 1: a group's keys in that many ranges of `split_keys` keys (a multiple of 32), one
        workgroup each, merged by a second launch through `partial` (float, `sink_partial_numel` elements)."""
        _tensor(q, "q", self.dtype, ndim=2)
        rows = q.shape[0]
        _need(q.shape[1] == q_heads * key_dim, "q: wrong width")
        k_row = self._sink_pages(k_pages, "k_pages", kv_heads, page_size, key_dim)
        v_row = self._sink_pages(v_pages, "v_pages", kv_heads, page_size, value_dim)
        _need(mask in self.SINK_MASKS, f"mask {mask!r}: one of all, window, chunk")
        _need(self.sink_tiles_supported(key_dim, value_dim, k_row, v_row, page_size, mask, mask_size, max_context)
              and q.shape[1] % 8 == 0, "sink_attention_tiles: sizes that the matrix-core kernel does not take")
        kind = self.SINK_MASKS[mask]
        _need(kind == 0 or mask_size >= 1, "a window or chunk needs a positive size")
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (rows,))
        _tensor(positions, "positions", torch.int32, (rows,))
        _tensor(group_first, "group_first", torch.int32, ndim=1)
        _tensor(group_count, "group_count", torch.int32, ndim=1)
        _need(group_first.numel() >= groups and group_count.numel() >= groups, "group vectors too short")
        if sink is not None:
            _tensor(sink, "sink", torch.float32, (q_heads,))
        _tensor(out, "out", self.dtype, (rows, q_heads * value_dim))
        if splits > 1:
            _tensor(partial, "partial", torch.float32, ndim=1)
            tokens = (16 if split_values else 64) // head_block
            _need(split_keys > 0 and split_keys % 32 == 0 and
                  partial.numel() >= self.sink_partial_numel(groups, tokens, q_heads, value_dim, splits),
                  "sink_attention_tiles: key ranges in multiples of 32 keys, and room for their shares")
        code = self._lib("sink_attention").mlr_sink_attention_tiles(
            _p(q), ctypes.c_long(q.shape[1]), _p(k_pages), ctypes.c_long(k_row), _p(v_pages), ctypes.c_long(v_row),
            _p(block_table), _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(sink), _p(out),
            ctypes.c_long(out.shape[1]), _p(group_first), _p(group_count), _c_int(groups), _c_int(head_block),
            _c_int(1 if split_values else 0), _c_int(q_heads), _c_int(kv_heads), _c_int(key_dim), _c_int(value_dim),
            _c_int(page_size), _c_int(kind), _c_int(int(mask_size)), _c_int(int(max_context)), _c_float(scale),
            _p(partial if splits > 1 else None), _c_int(int(split_keys)), _c_int(int(splits)), _stream())
        _ok(code, "sink_attention_tiles")

    @staticmethod
    def sink_partial_numel(groups, tokens, q_heads, value_dim, splits):
        """Floats that the shares of `splits` key ranges take for `groups` groups of up to `tokens` tokens."""
        return groups * tokens * q_heads * splits * (value_dim + 4)

    # -- many small products, routing ----------------------------------------------------------
    GROUPED_ACTS = {None: 0, "relu_squared": 1, "gated_silu": 2, "gated_gelu_tanh": 3}

    def experts_gated_fused(self, intermediate):
        """Whether `experts_gemm` takes the gated forms (act "gated_silu" / "gated_gelu_tanh": the weight's rows are a
        gate's and its up projection's in turn, 16 and 16; half as many columns leave): the bfloat16 engine, inner sizes
        in multiples of 16."""
        return self.dtype == torch.bfloat16 and intermediate % 16 == 0
    MAX_EXPERTS = 256

    @timed("gemm")
    def heads_gemm(self, a, w, out, act=None):
        """out[:, g, :] = act(a[:, g, :] . w[g]^T) for every group g: a [rows, groups, K] and out [rows, groups, N] may be
        views into wider rows (last stride 1, one stride per group), w [groups, N, K] contiguous."""
        for t, name in ((a, "a"), (out, "out")):
            _need(isinstance(t, torch.Tensor) and t.is_cuda and t.dtype is self.dtype and t.dim() == 3 and t.stride(2) == 1,
                  f"heads_gemm: {name} must be a [rows, groups, width] view of the engine's element type")
        _tensor(w, "w", self.dtype, ndim=3)
        rows, groups, k = a.shape
        _need(w.shape[0] == groups and w.shape[2] == k and tuple(out.shape) == (rows, groups, w.shape[1]),
              "heads_gemm: shapes do not fit")
        _need(act in self.GROUPED_ACTS, f"heads_gemm: activation {act!r}")
        n = w.shape[1]
        _ok(self._lib("grouped_gemm").mlr_grouped_gemm(
            _p(a), ctypes.c_long(a.stride(0)), ctypes.c_long(a.stride(1)), _p(w), ctypes.c_long(n * k), _p(out),
            ctypes.c_long(out.stride(0)), ctypes.c_long(out.stride(1)), _ptr(0), _ptr(0), _c_int(rows), _c_int(n), _c_int(k),
            _c_int(groups), _c_int(self.GROUPED_ACTS[act]), _c_int(0), _stream()), "heads_gemm")

    @timed("gemm")
    def experts_gemm(self, a, w, out, offsets, gather=None, act=None):
        """Rows sorted by expert: out[r] = act(a[gather[r] or r] . w[e]^T) for offsets[e] <= r < offsets[e + 1];
        a [*, K], w [experts, N, K], out [rows, N], offsets int32 [experts + 1] on the device."""
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=3)
        experts, n, k = w.shape
        _need(a.shape[1] == k, "experts_gemm: inner sizes differ")
        _tensor(out, "out", self.dtype, ndim=2)
        rows = out.shape[0]
        gated = act in ("gated_silu", "gated_gelu_tanh")
        _need(not gated or (n % 32 == 0 and self.dtype == torch.bfloat16), "experts_gemm: the gated forms take bfloat16 and blocks of 16")
        _need(out.shape[1] == (n // 2 if gated else n), "experts_gemm: out has the wrong width")
        _tensor(offsets, "offsets", torch.int32, (experts + 1,))
        if gather is not None:
            _tensor(gather, "gather", torch.int32, (rows,))
        else:
            _need(a.shape[0] == rows, "experts_gemm: without a gather list a has out's rows")
        _need(act in self.GROUPED_ACTS, f"experts_gemm: activation {act!r}")
        _ok(self._lib("grouped_gemm").mlr_grouped_gemm(
            _p(a), ctypes.c_long(k), ctypes.c_long(0), _p(w), ctypes.c_long(n * k), _p(out), ctypes.c_long(out.shape[1]),
            ctypes.c_long(0), _p(offsets), _p(gather), _c_int(rows), _c_int(n), _c_int(k), _c_int(experts),
            _c_int(self.GROUPED_ACTS[act]), _c_int(0), _stream()), "experts_gemm")

    @timed("activation", _tensors_work())
    def router_topk(self, logits, ids, weights, group_count=1, group_keep=1, correction=None, renormalize=False, scale=1.0):
        """Per row of the router logits [rows, experts] (float): s = sigmoid(z); of the group_count equal groups of
        neighbouring experts the group_keep with the largest sum of their two best s stay; ids [rows, top] int32 the
        experts with the largest s among those, weights [rows, top] float their s.  With `correction` (float
        [experts]) every choice goes by s + correction and the weights stay s; `renormalize`: the chosen weights over
        their sum (+ 1e-20); `scale` multiplies them."""
        if correction is not None:
            _tensor(correction, "correction", torch.float32, (logits.shape[1],))
        _tensor(logits, "logits", torch.float32, ndim=2)
        rows, experts = logits.shape
        _tensor(ids, "ids", torch.int32, ndim=2)
        top = ids.shape[1]
        _need(ids.shape[0] == rows, "ids: one row a token")
        _tensor(weights, "weights", torch.float32, (rows, top))
        _need(1 <= experts <= self.MAX_EXPERTS and group_count >= 1 and experts % group_count == 0
              and 1 <= group_keep <= group_count and 1 <= top <= group_keep * (experts // group_count),
              "router_topk: experts up to 256 in equal groups, and no more choices than the kept groups hold")
        _ok(self._lib("grouped_gemm").mlr_router_topk(_p(logits), _p(ids), _p(weights), _c_int(rows), _c_int(experts),
                                                      _c_int(top), _c_int(group_count), _c_int(group_keep), _p(correction),
                                                      _c_int(1 if renormalize else 0), _c_float(scale), _stream()),
            "router_topk")

    @timed("gemm")
    def route_sort(self, ids, experts, offsets, token_of, row_of):
        """The (token, choice) pairs of ids [rows, top] sorted by expert: offsets int32 [experts + 1], token_of
        [rows * top] the token of every sorted row, row_of [rows * top] the sorted row of every pair."""
        _tensor(ids, "ids", torch.int32, ndim=2)
        pairs = ids.numel()
        _tensor(offsets, "offsets", torch.int32, (experts + 1,))
        _tensor(token_of, "token_of", torch.int32, (pairs,))
        _tensor(row_of, "row_of", torch.int32, (pairs,))
        _need(1 <= experts <= self.MAX_EXPERTS, "route_sort: up to 256 experts")
        _ok(self._lib("grouped_gemm").mlr_route_sort(_p(ids), _c_int(pairs), _c_int(ids.shape[1]), _c_int(experts),
                                                     _p(offsets), _p(token_of), _p(row_of), _stream()), "route_sort")

    @timed("activation", _tensors_work())
    def route_combine(self, y, row_of, weights, out):
        """out[m] = sum_i weights[m, i] * y[row_of[m * top + i]] (32-bit sums, in the order of the choices)."""
        _tensor(weights, "weights", torch.float32, ndim=2)
        rows, top = weights.shape
        _tensor(y, "y", self.dtype, ndim=2)
        _need(y.shape[0] == rows * top, "route_combine: one row of y a pair")
        _tensor(row_of, "row_of", torch.int32, (rows * top,))
        _tensor(out, "out", self.dtype, (rows, y.shape[1]))
        _ok(self._lib("grouped_gemm").mlr_route_combine(_p(y), _p(row_of), _p(weights), _p(out), _c_int(rows),
                                                        _c_int(y.shape[1]), _c_int(top), _stream()), "route_combine")

    # -- sampling ----------------------------------------------------------------------------
    def sample_scratch(self, rows):
        """(floats, ints) of scratch memory that `sample` needs for this many rows."""
        lib = self._lib("sampling")
        return lib.mlr_sample_scratch_floats(_c_int(rows)), lib.mlr_sample_scratch_ints(_c_int(rows))

    @timed("sampler")
    def sample(self, logits, temperature, uniform, tokens, status, scratch_f, scratch_i, any_sampling=True):
        """tokens[r] = argmax (temperature <= 0) or the inverse-CDF draw at uniform[r]."""
        _tensor(logits, "logits", torch.float32, ndim=2)
        rows, vocab = logits.shape
        _tensor(temperature, "temperature", torch.float32, (rows,))
        _tensor(uniform, "uniform", torch.float32, (rows,))
        _tensor(tokens, "tokens", torch.int32, (rows,))
        _tensor(status, "status", torch.int32, (2,))
        need_f, need_i = self.sample_scratch(rows)
        _tensor(scratch_f, "scratch_f", torch.float32, ndim=1)
        _tensor(scratch_i, "scratch_i", torch.int32, ndim=1)
        _need(scratch_f.numel() >= need_f and scratch_i.numel() >= need_i, "sample: scratch buffers too small")
        _need(rows <= 65535, "sample: too many rows for the grid")
        fn = self._lib("sampling").mlr_sample
        _ok(fn(_p(logits), _c_int(rows), _c_int(vocab), _p(temperature), _p(uniform), _p(tokens),
               _p(status), _p(scratch_f), _p(scratch_i), _c_int(1 if any_sampling else 0), _stream()), "sample")
