"""The operations the parts are written against, bound to the gfx950 kernel library.

Every function checks shapes, dtypes, contiguity and device on the host before a
kernel is launched (a kernel never sees an operand it was not written for), then
calls the library's C entry point on the current stream.  There is no CPU path:
without the compiled library or without a GPU the first call raises.

Tests may install another backend with ``set_backend`` (an object with the same
functions) to exercise the engine's bookkeeping on the host; nothing in the
product does.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_F32, _BF16 = 0, 1
_backend = None


def set_backend(backend) -> None:
    """Install an object providing this module's functions (tests only); None restores the library."""
    global _backend
    _backend = backend


class KernelError(RuntimeError):
    pass


class _Library:
    """The compiled kernel library, loaded on first use."""

    _lib = None

    @classmethod
    def get(cls):
        if cls._lib is None:
            if not torch.cuda.is_available():
                raise KernelError("tempura_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
            from ..csrc.build import ensure_built
            path = ensure_built()
            try:
                lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelError(f"cannot load the kernel library {path}: {e}") from e
            lib.tp_last_error.restype = ctypes.c_char_p
            cls._lib = lib
            cls.path = path
        return cls._lib


def library():
    return _Library.get()


class KernelTimer:
    """Times every call into the kernel library made while it is active (``with KernelTimer() as t:``), with a pair
    of events on the current stream around each call: eager steps only (events cannot be recorded into a graph
    that is replayed), and the pairs serialise nothing, so a call's time includes what its kernels wait for.
    ``label`` (settable at any time) is stored with every call; ``table()`` waits for the device and returns
    rows (entry point, label, calls, total microseconds), largest first."""

    def __init__(self):
        self.label = ""
        self._events = []

    def __enter__(self):
        global _timer
        self._before, _timer = _timer, self
        return self

    def __exit__(self, *exc):
        global _timer
        _timer = self._before
        return False

    def table(self, by_label: bool = False):
        torch.cuda.synchronize()
        total = {}
        for name, label, e0, e1 in self._events:
            key = (name, label if by_label else "")
            calls, us = total.get(key, (0, 0.0))
            total[key] = (calls + 1, us + 1e3 * e0.elapsed_time(e1))
        return sorted(((k[0], k[1], c, us) for k, (c, us) in total.items()), key=lambda r: -r[3])


_timer: Optional[KernelTimer] = None


def _call(name: str, *args, tag: Optional[tuple] = None) -> None:
    """``tag``: what distinguishes this call in a ``KernelTimer``'s table (a product's sizes)."""
    lib = _Library.get()
    t = _timer
    if t is not None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(f"{name}: {lib.tp_last_error().decode()}")
    if t is not None:
        e1.record()
        t._events.append((name if tag is None else name + " " + "x".join(map(str, tag)), t.label, e0, e1))


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"unsupported dtype {t.dtype}")


def _dtcode(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"unsupported dtype {dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream():
    """The current stream's handle (of the current device).  Asked for at every launch: the direct call is
    some 8 us cheaper than ``torch.cuda.current_stream()``, a quarter of an eager launch's host time."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev_ok(*ts) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "operand is not on the GPU")
            _need(t.is_contiguous(), "operand is not contiguous")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    _need(t.dtype == torch.int32 and t.numel() >= n and t.dim() >= 1, f"{what}: need int32 with {n} elements")


# ---------------------------------------------------------------------------------
def embed(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """int32 [n] , [vocab, hidden] -> float32 [n, hidden]."""
    if _backend is not None:
        return _backend.embed(tokens, table)
    _dev_ok(tokens, table)
    n = tokens.numel()
    _i32(tokens, n, "embed tokens")
    _need(table.dim() == 2, "embed: table must be [vocab, hidden]")
    out = torch.empty((n, table.shape[1]), dtype=torch.float32, device=table.device)
    _call("tp_embed", _ptr(tokens), _ptr(table), _dt(table), _ptr(out), n, table.shape[1], _stream())
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [n, hidden] -> out_dtype [n or len(rows), hidden]."""
    if _backend is not None:
        return _backend.rmsnorm(h, weight, eps, out_dtype, rows)
    _dev_ok(h, weight, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2, "rmsnorm: input must be float32 [n, hidden]")
    _need(weight.dtype == torch.float32 and weight.numel() == h.shape[1], "rmsnorm: weight must be float32 [hidden]")
    n_out = h.shape[0]
    if rows is not None:
        n_out = rows.numel()
        _i32(rows, n_out, "rmsnorm rows") if n_out else None
    out = torch.empty((n_out, h.shape[1]), dtype=out_dtype, device=h.device)
    _call("tp_rmsnorm", _ptr(h), _ptr(weight), _ptr(rows), _ptr(out), _dtcode(out_dtype), n_out, h.shape[1],
          ctypes.c_float(eps), _stream())
    return out


#: bfloat16 products may use the matrix-core kernels (tests switch this off to grade the general kernel)
allow_mfma = True


def gated_layout_ok(n_rows: int, k: int) -> bool:
    """Whether ``linear_swiglu`` takes a weight of 2 * n_rows rows and k columns."""
    return n_rows % 8 == 0 and k % 32 == 0


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[i, k], [i, k] -> [2i, k] with eight gate rows and eight up rows in turn, the layout
    ``linear_swiglu`` reads."""
    i, k = gate.shape
    return torch.stack([gate.reshape(i // 8, 8, k), up.reshape(i // 8, 8, k)], dim=1).reshape(2 * i, k).contiguous()


class Prenormed:
    """Rows whose root-mean-square norm is finished by the product that consumes them: ``x`` is
    bfloat16(h * norm weight) [m, k]; ``ss`` [ceil(k / 16), 16] float32 holds, per block of 16 columns
    and row, the sum of squares of h; the consumer multiplies its float32 result rows by
    rsqrt(sum(ss) / k + eps).  Made by ``linear(..., residual=h, next_norm=(weight, eps))``."""
    __slots__ = ("x", "ss", "eps", "blocked")

    def __init__(self, x, ss, eps, blocked=None):
        self.x, self.ss, self.eps = x, ss, float(eps)
        #: None: ``x`` is row-major [m, k]; (m, k): ``x`` is stored k-blocked, [k / 8, m, 8] (see ``KBlocked``)
        self.blocked = blocked

    @property
    def shape(self):
        return self.x.shape if self.blocked is None else self.blocked

    def rows(self):
        """``x`` as a row-major [m, k] tensor (a copy when it is stored k-blocked)."""
        if self.blocked is None:
            return self.x
        m, k = self.blocked
        return self.x.permute(1, 0, 2).reshape(m, k)


class KBlocked:
    """bfloat16 activations of at most 16 rows stored k-blocked, ``data`` [k / 8, m, 8]: eight consecutive
    columns of all rows side by side.  A product of a few rows that reads its activations straight from
    global memory then fetches neighbouring bytes instead of short pieces of several rows.  Made by
    ``linear_swiglu(..., blocked_out=True)``, taken by ``linear``."""
    __slots__ = ("data", "rows", "width")

    def __init__(self, data, rows, width):
        self.data, self.rows, self.width = data, rows, width

    @property
    def shape(self):
        return (self.rows, self.width)

    def row_major(self) -> torch.Tensor:
        return self.data.permute(1, 0, 2).reshape(self.rows, self.width).contiguous()


class TiledWeight:
    """A bfloat16 weight [n, k] (n % 16 == 0, k % 64 == 0) stored tiled, ``data`` [n / 16, k / 32, 64, 8]: the block
    of rows 16 i.. and columns 32 j.. as 1,024 contiguous bytes in the matrix cores' operand order, lane l = (column
    group l / 16, row l % 16) holding eight consecutive columns.  The products read it with whole-cache-line loads
    where the row-major form makes a wave fetch 64-byte pieces of sixteen rows.  Made by ``tile_weight``; taken by
    ``linear``, ``linear_swiglu`` and ``linear_rope_kv``."""
    __slots__ = ("data", "n", "k")

    def __init__(self, data, n, k):
        self.data, self.n, self.k = data, n, k

    @property
    def shape(self):
        return (self.n, self.k)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def dim(self) -> int:
        return 2

    def rows(self, lo: int, hi: int) -> "TiledWeight":
        """Rows lo..hi (multiples of 16) as a weight of their own; no copy."""
        _need(lo % 16 == 0 and hi % 16 == 0 and 0 <= lo < hi <= self.n, f"tiled weight: rows {lo}..{hi} of {self.n}")
        return TiledWeight(self.data[lo // 16: hi // 16], hi - lo, self.k)

    def row_major(self) -> torch.Tensor:
        """The plain [n, k] tensor (a copy)."""
        return self.data.view(self.n // 16, self.k // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(self.n, self.k).contiguous()


#: weights that fit are stored tiled (False, or TEMPURA_TILE_WEIGHTS=0 in the environment: every weight stays row-major)
tile_weights = os.environ.get("TEMPURA_TILE_WEIGHTS", "1") != "0"


def tile_weight(w: torch.Tensor):
    """A weight [n, k] for the products: ``TiledWeight`` when it is bfloat16 on the GPU with n % 16 == 0 and
    k % 64 == 0 and the matrix-core kernels are in use, else ``w`` itself.  No value changes."""
    if not (tile_weights and _backend is None and allow_mfma and isinstance(w, torch.Tensor) and w.is_cuda
            and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 16 == 0 and w.shape[1] % 64 == 0):
        return w
    n, k = w.shape
    data = w.view(n // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(n // 16, k // 32, 64, 8)
    return TiledWeight(data, n, k)


def weight_rows(w, lo: int, hi: int):
    """Rows lo..hi of a weight, tiled or not, without a copy."""
    return w.rows(lo, hi) if isinstance(w, TiledWeight) else w[lo:hi]


def _w_args(w):
    """(tensor whose memory the kernel reads, layout bit) of a weight."""
    if isinstance(w, TiledWeight):
        return w.data, 4
    return w, 0


class Partials:
    """The float32 partial sums [splits, m, n] of a product whose K was split over blocks, not yet added:
    the kernel that consumes the rows adds them (in ascending order), which saves the reduction kernel.
    Made by ``linear(..., partial_ok=True)``, taken by ``rope_kv_write``."""
    __slots__ = ("data",)

    def __init__(self, data):
        self.data = data

    @property
    def shape(self):
        return tuple(self.data.shape[1:])


def split_norm_ok(m: int, width: int, dtype: torch.dtype) -> bool:
    """Whether the product before a norm over ``width`` columns of ``m`` rows can carry it (``linear`` with
    ``next_norm``): up to 16 rows the two products around the norm share it; with more rows the kernel that
    adds the product's partial sums into the residual stream also norms the rows, where the product splits K
    (``linear`` says whether it did)."""
    if _backend is not None:
        return _backend.split_norm_ok(m, width, dtype)
    return allow_mfma and dtype == torch.bfloat16 and 0 < m and width % 32 == 0


def _pre_args(x):
    """(the tensor a product reads, the arguments of its row scale, its rows and columns, layout bit 1 when the
    tensor is k-blocked) of plain rows or of ``Prenormed`` rows."""
    if isinstance(x, Prenormed):
        _dev_ok(x.x, x.ss)
        m, k = x.shape
        _need(x.x.dtype == torch.bfloat16 and x.ss.dtype == torch.float32 and x.x.numel() == m * k and
              tuple(x.ss.shape) == ((k + 15) // 16, 16), "linear: malformed handed-over rows")
        return x.x, (_ptr(x.ss), x.ss.shape[0], ctypes.c_float(x.eps)), (m, k), (1 if x.blocked is not None else 0)
    return x, (_ptr(None), 0, ctypes.c_float(0.0)), (tuple(x.shape) if x.dim() == 2 else None), 0


def linear_swiglu(x, w: torch.Tensor, blocked_out: bool = False):
    """bfloat16 x [m, k] (or ``Prenormed``), interleaved gate/up weight [2i, k] -> bfloat16 [m, i] =
    silu(x g^T) * (x u^T), the gate applied to the float32 accumulators (no rounding in between).
    With ``blocked_out`` the result comes as ``KBlocked`` when there are at most 16 rows and i % 32 == 0 (else as a tensor)."""
    if _backend is not None:
        return _backend.linear_swiglu(x, w, blocked_out) if blocked_out else _backend.linear_swiglu(x, w)
    x, pre, mk, xl = _pre_args(x)
    wd, wl = _w_args(w)
    _dev_ok(x, wd)
    _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear_swiglu: shapes {mk} x {tuple(w.shape)}")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "linear_swiglu: operands must be bfloat16")
    m, k = mk
    n = w.shape[0]
    _need(n % 16 == 0 and k % 32 == 0, "linear_swiglu: needs 2i % 16 == 0 and k % 32 == 0")
    # (the product that takes such rows is an MFMA kernel over K in steps of 32)
    blocked_out = blocked_out and allow_mfma and 0 < m <= 16 and (n // 2) % 32 == 0
    if blocked_out:
        out = KBlocked(torch.empty((n // 16, m, 8), dtype=torch.bfloat16, device=x.device), m, n // 2)
    else:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    scratch, nscratch = _splitk_scratch(x, m, n)
    _call("tp_linear_fused", _ptr(x), _ptr(wd), _BF16, _ptr(out.data if blocked_out else out), _BF16, 2, m, n, k, 1,
          _ptr(scratch), ctypes.c_size_t(nscratch), *pre, _ptr(None), _ptr(None), _ptr(None), (2 if blocked_out else 0) | wl | xl,
          0, _ptr(None), _stream(), tag=(m, n, k))
    return out


def _splitk_scratch(x: torch.Tensor, m: int, n: int):
    """Room for the partial sums of a bfloat16 product whose K is split over blocks: products of 17..128
    rows (64-row blocks up to 64 rows, 128-row blocks above), and larger ones with too few result tiles (256 x 128)
    to give every CU work."""
    if x.dtype != torch.bfloat16 or m <= 16:
        return None, 0
    if m <= 128:
        splits = min(16, max(1, -(-512 // (-(-n // 128) * -(-m // 64)))))
    else:
        tiles = -(-m // 256) * -(-n // 128)
        if tiles >= 128:
            return None, 0
        splits = min(16, 2 * -(-256 // tiles))      # (room for the library to choose: it prices the candidates)
    count = splits * m * n
    return torch.empty((count,), dtype=torch.float32, device=x.device), count


def linear(x, w: torch.Tensor, out_dtype: torch.dtype, residual: Optional[torch.Tensor] = None, next_norm=None,
           partial_ok: bool = False):
    """x [m, k] (or ``Prenormed`` / ``KBlocked``) @ w[n, k]^T -> out_dtype [m, n]; with ``residual`` (float32
    [m, n]) the product is added into it in place and it is returned.
    With ``next_norm`` = (float32 weight [n], eps) (needs ``residual``) the result is the pair (residual, rows
    for the part behind that norm): ``Prenormed`` rows up to 16 rows of bfloat16, the normed rows themselves
    from 17 rows on when the product's K was split (one kernel adds the partial sums into the residual and norms
    it), or None when the norm has to run on its own.
    With ``partial_ok`` (float32 output, no residual) the result may be ``Partials``."""
    if _backend is not None:
        if next_norm is not None:
            return _backend.linear(x, w, out_dtype, residual, next_norm)
        return _backend.linear(x, w, out_dtype, residual)
    layout = 0
    wd, wl = _w_args(w)
    if isinstance(x, KBlocked):
        _need(allow_mfma and x.data.dtype == torch.bfloat16 and tuple(x.data.shape) == (x.width // 8, x.rows, 8)
              and x.width % 32 == 0, "linear: malformed k-blocked rows")
        kb, layout = x, 1
        x, pre = x.data, (_ptr(None), 0, ctypes.c_float(0.0))
        m, k = kb.rows, kb.width
        _dev_ok(x, wd, residual)
        _need(w.dim() == 2 and w.shape[1] == k and w.dtype == torch.bfloat16, f"linear: shapes {(m, k)} x {tuple(w.shape)}")
    else:
        x, pre, mk, layout = _pre_args(x)
        _dev_ok(x, wd, residual)
        _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear: shapes {mk} x {tuple(w.shape)}")
        _need(x.dtype == w.dtype, f"linear: operand dtypes differ ({x.dtype}, {w.dtype})")
        m, k = mk
    n = w.shape[0]
    if residual is not None:
        _need(residual.dtype == torch.float32 and tuple(residual.shape) == (m, n), "linear: residual must be float32 [m, n]")
        out, acc = residual, 1
    else:
        out, acc = torch.empty((m, n), dtype=out_dtype, device=x.device), 0
    post, handed = (_ptr(None), _ptr(None), _ptr(None)), None
    if next_norm is not None and split_norm_ok(m, n, x.dtype) and k % 32 == 0 and m <= 16:
        weight, eps = next_norm
        _dev_ok(weight)
        _need(residual is not None, "linear: next_norm needs a residual")
        _need(weight.dtype == torch.float32 and weight.numel() == n, "linear: norm weight must be float32 [n]")
        # (the rows go on k-blocked where the consumer can read them so: a product of a few rows then takes its
        # activations straight from memory as operands instead of staging them through LDS)
        hand_blocked = handoff_blocked and n % 32 == 0
        handed = Prenormed(torch.empty((n // 8, m, 8) if hand_blocked else (m, n), dtype=torch.bfloat16, device=x.device),
                           torch.empty(((n + 15) // 16, 16), dtype=torch.float32, device=x.device), eps,
                           (m, n) if hand_blocked else None)
        post = (_ptr(weight), _ptr(handed.x), _ptr(handed.ss))
        if hand_blocked:
            layout |= 8
    scratch, nscratch = _splitk_scratch(x, m, n) if allow_mfma else (None, 0)
    # from 17 rows on: the partial sums of a split K may stay unadded for the kernel that consumes the rows
    layout |= wl
    defer = scratch is not None and 16 < m and (layout & 3) == 0 and \
        ((next_norm is not None and residual is not None and split_norm_ok(m, n, x.dtype) and n % 4 == 0 and n <= 16384) or
         (partial_ok and residual is None and out_dtype == torch.float32))
    splits = ctypes.c_int(1)
    _call("tp_linear_fused", _ptr(x), _ptr(wd), _dt(x), _ptr(out), _dt(out), acc, m, n, k, int(allow_mfma), _ptr(scratch),
          ctypes.c_size_t(nscratch), *pre, *post, layout, int(defer), ctypes.byref(splits), _stream(), tag=(m, n, k))
    if defer and splits.value > 1:
        if next_norm is None:
            return Partials(scratch[: splits.value * m * n].view(splits.value, m, n))
        weight, eps = next_norm
        _dev_ok(weight)
        _need(weight.dtype == torch.float32 and weight.numel() == n, "linear: norm weight must be float32 [n]")
        normed = torch.empty((m, n), dtype=x.dtype, device=x.device)
        _call("tp_splitk_add_rmsnorm", _ptr(scratch), splits.value, _ptr(residual), _ptr(weight), ctypes.c_float(eps),
              _ptr(normed), _dt(normed), m, n, _stream())
        return out, normed
    return out if next_norm is None else (out, handed)


#: rows handed from one product to the next with a norm between them travel k-blocked (up to 16 rows)
handoff_blocked = True
#: long steps may rotate and store in the projection's epilogue too (False: only the few rows of decoding)
rope_in_long_products = True


def linear_rope_ok(m: int, n: int, k: int, head_dim: int, rotary_dim: int, page_size: int, x_dtype: torch.dtype,
                   cache_dtype: torch.dtype, prenormed: bool = False) -> bool:
    """Whether ``linear_rope_kv`` takes a projection of m rows onto n columns: a few rows (decoding), or a long
    step with enough result tiles (128 x 128) to give half the CUs work without splitting K, heads of a multiple of 64."""
    if not (_backend is None and allow_mfma and x_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16):
        return False
    if 0 < m <= 16:
        return k % 32 == 0 and head_dim % 16 == 0
    tiles = -(-m // 128) * -(-n // 128)      # (of 128 x 128, the smallest blocks of the pipelined products)
    return (rope_in_long_products and m > 128 and tiles >= 128 and k % 64 == 0 and 255 * k * 2 + 128 < 2 ** 31 and head_dim % 64 == 0
            and rotary_dim % 8 == 0 and page_size % 8 == 0 and not prenormed)


def linear_rope_kv(x, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, inv_freq: Optional[torch.Tensor],
                   rotary_dim: int, factor: float, num_heads: int, num_kv_heads: int, head_dim: int,
                   k_cache: torch.Tensor, v_cache: torch.Tensor, cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The q/k/v projection of bfloat16 rows (at most 16, also ``Prenormed``; or a long step, see
    ``linear_rope_ok``) with the rotation and the cache write in its epilogue: the same result as ``linear``
    to float32 followed by ``rope_kv_write`` (w's q and k heads in paired order), without the kernel and the
    rows in between.  Returns q as bfloat16 [m, heads, head_dim]."""
    x, pre, mk, xl = _pre_args(x)
    wd, wl = _w_args(w)
    _dev_ok(x, wd, positions, slots, inv_freq, k_cache, v_cache)
    _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear_rope_kv: shapes {mk} x {tuple(w.shape)}")
    m, k = mk
    n = w.shape[0]
    _need(linear_rope_ok(m, n, k, head_dim, rotary_dim, k_cache.shape[2] if k_cache.dim() == 4 else 0, x.dtype, k_cache.dtype,
                         pre[1] != 0) and w.dtype == torch.bfloat16,
          "linear_rope_kv: sizes or dtypes that the fused projection does not take (see linear_rope_ok)")
    _need(m <= 16 or cos_sin is not None, "linear_rope_kv: a long step needs the table of cosines and sines")
    _need(n == (num_heads + 2 * num_kv_heads) * head_dim, f"linear_rope_kv: {n} weight rows for {num_heads} + 2 x {num_kv_heads} heads of {head_dim}")
    _i32(positions, m, "positions")
    _i32(slots, m, "slots")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim
          and tuple(v_cache.shape) == (k_cache.shape[0], k_cache.shape[1], k_cache.shape[3], k_cache.shape[2])
          and v_cache.dtype == torch.bfloat16,
          "linear_rope_kv: caches must be k [pages, kv_heads, page_size, head_dim], v [pages, kv_heads, head_dim, page_size]")
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
              "linear_rope_kv: inv_freq must be float64 [rotary_dim / 2]")
    if cos_sin is not None:
        _dev_ok(cos_sin)
        _need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and tuple(cos_sin.shape) == (m, rotary_dim // 2, 2),
              "linear_rope_kv: table must be float32 [m, rotary_dim / 2, 2]")
    q = torch.empty((m, num_heads, head_dim), dtype=torch.bfloat16, device=x.device)
    _call("tp_linear_rope", _ptr(x), _ptr(wd), int(wl != 0) | (2 if xl else 0), m, n, k, *pre, _ptr(positions), _ptr(slots), _ptr(inv_freq), rotary_dim,
          ctypes.c_float(factor), num_heads, num_kv_heads, head_dim, _ptr(q), _ptr(k_cache), _ptr(v_cache),
          k_cache.shape[2], _ptr(cos_sin), _stream(), tag=(m, n, k))
    return q


def rope_kv_write(qkv, positions: torch.Tensor, slots: Optional[torch.Tensor],
                  inv_freq: Optional[torch.Tensor], rotary_dim: int, factor: float, num_heads: int,
                  num_kv_heads: int, head_dim: int, k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor], q_dtype: torch.dtype,
                  cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate q and k of float32 rows [n, (heads + 2 kv_heads) * head_dim] (or the ``Partials`` of the
    projection that makes them), store k and v into the cache rows ``slots`` and return q as q_dtype
    [n, heads, head_dim].  With ``slots`` None the rows hold q only and nothing is stored.
    The q and k heads are in PAIRED order: elements (2 d, 2 d + 1) of a head rotate together by the angle
    of pair d (they are elements (d, d + rotary_dim / 2) of the split-half order).
    ``cos_sin``: this step's table from ``rope_table`` (the same values, computed once for all layers)."""
    if _backend is not None:
        return _backend.rope_kv_write(qkv, positions, slots, inv_freq, rotary_dim, factor, num_heads,
                                      num_kv_heads, head_dim, k_cache, v_cache, q_dtype)
    splits = 1
    if isinstance(qkv, Partials):
        splits, qkv = qkv.data.shape[0], qkv.data.view(-1, qkv.data.shape[2])[: qkv.data.shape[1]]
        _need(qkv.is_contiguous() or splits == 1, "rope_kv_write: malformed partial sums")
    _dev_ok(positions, slots, inv_freq, k_cache, v_cache)
    _need(qkv.is_cuda, "operand is not on the GPU")
    _need(qkv.dtype == torch.float32 and qkv.dim() == 2, "rope_kv_write: rows must be float32 [n, width]")
    n = qkv.shape[0]
    width = (num_heads + (2 * num_kv_heads if slots is not None else 0)) * head_dim
    _need(qkv.shape[1] == width, f"rope_kv_write: row width {qkv.shape[1]} != {width}")
    _i32(positions, n, "positions") if n else None
    page_size, cache_dt = 1, _F32
    if slots is not None:
        _i32(slots, n, "slots") if n else None
        _need(k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4
              and tuple(v_cache.shape) == (k_cache.shape[0], k_cache.shape[1], k_cache.shape[3], k_cache.shape[2]),
              "rope_kv_write: caches must be k [pages, kv_heads, page_size, head_dim], v [pages, kv_heads, head_dim, page_size]")
        _need(k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim, "rope_kv_write: cache layout mismatch")
        _need(k_cache.dtype == v_cache.dtype, "rope_kv_write: cache dtypes differ")
        page_size, cache_dt = k_cache.shape[2], _dt(k_cache)
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
              "rope_kv_write: inv_freq must be float64 [rotary_dim / 2]")
    if cos_sin is not None:
        _need(cos_sin.is_cuda and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and tuple(cos_sin.shape) == (n, rotary_dim // 2, 2), "rope_kv_write: table must be float32 [n, rotary_dim / 2, 2]")
    q = torch.empty((n, num_heads, head_dim), dtype=q_dtype, device=qkv.device)
    _call("tp_rope_kv_write", _ptr(qkv), qkv.shape[1], _ptr(positions), _ptr(slots), _ptr(inv_freq), rotary_dim,
          ctypes.c_float(factor), n, num_heads, num_kv_heads, head_dim, _ptr(q), _dtcode(q_dtype),
          _ptr(k_cache), _ptr(v_cache), cache_dt, page_size, splits, _ptr(cos_sin), _stream())
    return q


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, rotary_dim: int, factor: float) -> torch.Tensor:
    """float32 [n, rotary_dim / 2, 2]: cosine and sine (times factor) of every token's angles, as
    ``rope_kv_write`` would compute them itself."""
    if _backend is not None:
        return None
    _dev_ok(positions, inv_freq)
    n = positions.numel()
    _i32(positions, n, "positions") if n else None
    _need(rotary_dim > 0 and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
          "rope_table: inv_freq must be float64 [rotary_dim / 2]")
    table = torch.empty((n, rotary_dim // 2, 2), dtype=torch.float32, device=positions.device)
    _call("tp_rope_table", _ptr(positions), _ptr(inv_freq), rotary_dim, ctypes.c_float(factor), n, _ptr(table), _stream())
    return table


#: bfloat16 attention may use the matrix-core kernels
allow_fast_attention = True
#: the split decode kernel aims at this many blocks (of four waves) in flight
decode_target_blocks = 256


def decode_rows_padded(rows: int) -> int:
    """The number of rows a decode step of `rows` requests is sized for: the next power of two up to 128, beyond
    that the next multiple of 128.  A captured step has that many rows and an eager one chooses its kernels and
    splits as if it had, so the two give the same bits."""
    if rows > 128:
        return (rows + 127) // 128 * 128
    padded = 1
    while padded < rows:
        padded *= 2
    return padded
#: and at least this many splits while a split has at most 64 blocks
decode_min_splits = 8
#: measurements: this many splits whatever the batch (0: chosen by the rules below)
decode_force_splits = 0
#: portions of prompts with fewer query blocks than this have their keys split over blocks (1: never)
portion_target_blocks = 1024
#: in parts of at least this many keys
portion_min_keys = 1024
#: and only while the partial results stay below this many bytes
portion_scratch_limit = 256 << 20


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    cu_seqlens: torch.Tensor, context_lens: torch.Tensor, token_req: torch.Tensor,
                    scale: float, window: int, max_q_len: int, max_context_len: int,
                    num_single: Optional[int] = None) -> torch.Tensor:
    """q [n, heads, head_dim] over k [pages, kv_heads, page_size, head_dim] and transposed
    v [pages, kv_heads, head_dim, page_size] -> [n, heads * head_dim]."""
    if _backend is not None:
        return _backend.paged_attention(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens,
                                        token_req, scale, window, max_q_len, max_context_len)
    # num_single: requests that bring exactly one token (None: all of them iff max_q_len == 1, else unknown
    # and every request is treated as a portion).
    _dev_ok(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens, token_req)
    _need(q.dim() == 3 and k_cache.dim() == 4 and v_cache.dim() == 4, "paged_attention: bad operand ranks")
    n, heads, d = q.shape
    pages, kvh, page_size, d2 = k_cache.shape
    _need(tuple(v_cache.shape) == (pages, kvh, d2, page_size), "paged_attention: v cache must be [pages, kv_heads, head_dim, page_size]")
    _need(d == d2, "paged_attention: head_dim of q and cache differ")
    _need(q.dtype == k_cache.dtype == v_cache.dtype, "paged_attention: q and cache dtypes differ")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32, "paged_attention: block_tables must be int32 [r, width]")
    r, width = block_tables.shape
    _i32(cu_seqlens, r + 1, "cu_seqlens")
    _i32(context_lens, r, "context_lens")
    _i32(token_req, n, "token_req") if n else None
    _need(pages * kvh * page_size < 2 ** 31, "paged_attention: cache pool too large for 32-bit row indices")
    _need(max_context_len <= width * page_size, "paged_attention: block table narrower than the longest context")
    out = torch.empty((n, heads * d), dtype=q.dtype, device=q.device)
    if num_single is None:
        num_single = r if max_q_len == 1 else 0
    _need(0 <= num_single <= r, "paged_attention: num_single out of range")
    fast = allow_fast_attention and q.dtype == torch.bfloat16 and d % 32 == 0 and d <= 128 and page_size % 8 == 0
    splits, scratch = 1, None
    if fast and num_single > 0:
        # enough blocks to fill 256 CUs, but at least 128 keys per block
        blocks_per_split = decode_rows_padded(num_single) * kvh * ((heads // kvh + 15) // 16)
        # (two blocks fit a CU, 512 the chip.  From 65 to 256 blocks per split, as many splits as fill it once: measured
        # alone at 2,100 keys, 16 requests 35.8 -> 33.5 us, 20 requests 47.2 -> 38.5, 32 requests 54.3 -> 52.7, and more
        # for contexts that differ; through the engine 16 requests of the 8B shape 4.33 -> 4.25 ms a step, 32 requests
        # 5.27 -> 5.20; 12 requests in five splits against three 4.11 / 4.27, 20 in three against two 4.77 / 4.92, 24 in
        # two against three 4.97 / 5.21.)
        if blocks_per_split <= 64:
            want = -(-decode_target_blocks // blocks_per_split)
        elif blocks_per_split <= decode_target_blocks:
            want = max(1, 2 * decode_target_blocks // blocks_per_split)
        else:
            # (more blocks than half the chip's places: no split.  Through the engine, requests of 2,048+ keys of the 8B
            # shape, one split against two: 36 requests 6.06 / 5.97 ms a step, 40: 6.14 / 6.04, 48: 6.27 / 6.49,
            # 56: 6.42 / 6.68, 64: 6.62 / 6.89; three splits at 36 and 40 requests, which the kernel timed alone
            # prefers, 6.07 and 6.13)
            want = 1
        if blocks_per_split <= 64:
            want = max(want, decode_min_splits)     # (batch 8 of the 8B shape: eight splits 3.87 ms a step, four 3.94)
        if decode_force_splits > 0:
            want = decode_force_splits
        # (at least 128 keys a split, by the longest context rounded up to a power of two from 256: a step captured
        # for a bound on the context and an eager step at the actual length then cut alike and give the same bits)
        bound = 256
        while bound < max_context_len:
            bound *= 2
        splits = max(1, min(64, want, bound // 128))
        if splits > 1:
            scratch = torch.empty((r * heads * splits * (d + 2),), dtype=torch.float32, device=q.device)
    parts, part_scratch = 1, None
    if fast and num_single < r and d in (32, 64, 128) and page_size & (page_size - 1) == 0 and page_size >= max(8, 512 // d):
        # Few query blocks under a long context (a portion of a prompt behind a long cached prefix): the keys of
        # every portion are split over blocks until the chip is full (T = 512 behind 7,680 keys: 219 -> 137 us).
        q_blocks = -(-(n - num_single) // 32) + (r - num_single)
        blocks = q_blocks * kvh * ((heads // kvh + 3) // 4)
        # (a query block is split into at most as many parts as it has portion_min_keys keys: the short blocks
        # of a prompt from an empty cache stay whole)
        parts = max(1, min(16, portion_target_blocks // blocks, max_context_len // portion_min_keys, 65535 // r))
        if parts > 1 and n * heads * parts * (d + 4) * 4 > portion_scratch_limit:
            parts = 1
        if parts > 1:
            part_scratch = torch.empty((n * heads * parts * (d + 4),), dtype=torch.float32, device=q.device)
    _call("tp_paged_attention", _ptr(q), _dt(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables), width,
          _ptr(cu_seqlens), _ptr(context_lens), _ptr(token_req), _ptr(out), n, r, heads, kvh, d, page_size,
          ctypes.c_float(scale), int(window), int(max_q_len), int(max_context_len), int(fast),
          int(num_single), int(splits), _ptr(scratch), int(parts), max(1, portion_min_keys // 32), _ptr(part_scratch), _stream())
    return out


def swiglu(gu: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[m, 2i] (gate columns then up columns) -> out_dtype [m, i]."""
    if _backend is not None:
        return _backend.swiglu(gu, out_dtype)
    _dev_ok(gu)
    _need(gu.dim() == 2 and gu.shape[1] % 2 == 0, "swiglu: input must be [m, 2i]")
    m, i2 = gu.shape
    out = torch.empty((m, i2 // 2), dtype=out_dtype, device=gu.device)
    _call("tp_swiglu", _ptr(gu), _dt(gu), _ptr(out), _dtcode(out_dtype), m, i2 // 2, _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """float32 [m, vocab] -> int32 [m]; the last maximum wins on exact ties."""
    if _backend is not None:
        return _backend.argmax(logits)
    _dev_ok(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits must be float32 [m, vocab]")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    part = torch.empty((logits.shape[0] * 128,), dtype=torch.float32, device=logits.device)
    _call("tp_argmax", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _ptr(part), _stream())
    return out


class HostCopy:
    """A small device tensor on its way to the host: the copy into pinned memory is queued when the object is
    made, ``result()`` waits for that copy alone (not for work queued behind it) and returns a list.  The pinned
    buffers are taken in turn from a ring, so at most ``RING`` copies may be outstanding."""
    RING = 8
    _ring: list = []
    _next = 0

    def __init__(self, t: torch.Tensor):
        cls = HostCopy
        n = t.numel()
        if not cls._ring:
            cls._ring = [None] * cls.RING
        slot = cls._ring[cls._next]
        if slot is None or slot[0].numel() < n or slot[0].dtype != t.dtype:
            slot = (torch.empty(max(n, 256), dtype=t.dtype, pin_memory=True), torch.cuda.Event())
            cls._ring[cls._next] = slot
        cls._next = (cls._next + 1) % cls.RING
        self._buf, self._event, self._n = slot[0], slot[1], n
        self._buf[:n].copy_(t.reshape(-1), non_blocking=True)
        self._event.record()

    def result(self) -> list:
        self._event.synchronize()
        return self._buf[: self._n].tolist()


class _Staging:
    """Small per-call option arrays on their way to the device through pinned memory: the copy is queued behind
    the work in flight instead of making the host wait for it (a pageable copy would).  Buffers are taken in
    turn from a ring and reused once their copy has run."""
    RING = 8
    _ring: list = []
    _next = 0

    @classmethod
    def send(cls, arrays, device) -> list:
        """``arrays``: numpy arrays of 4-byte elements, each [rows..]; returns device tensors of the same shapes
        and dtypes (views of one packed transfer)."""
        import numpy as np
        total = sum(a.size for a in arrays)
        if not cls._ring:
            cls._ring = [None] * cls.RING
        slot = cls._ring[cls._next]
        if slot is None or slot[0].numel() < total:
            slot = (torch.empty(max(total, 1024), dtype=torch.int32, pin_memory=True), torch.cuda.Event())
            cls._ring[cls._next] = slot
        cls._next = (cls._next + 1) % cls.RING
        host, event = slot
        event.synchronize()                       # the copy that last used this buffer has run
        flat = host.numpy()
        views, off = [], 0
        for a in arrays:
            flat[off: off + a.size] = np.ascontiguousarray(a).reshape(-1).view(np.int32)
            off += a.size
        dev = host[:total].to(device, non_blocking=True)
        event.record()
        off = 0
        for a in arrays:
            t = dev[off: off + a.size]
            views.append((t.view(torch.float32) if a.dtype == np.float32 else t).view(a.shape))
            off += a.size
        return views


def apply_penalties(logits: torch.Tensor, rows, tokens, counts, in_window, presence, frequency, repeat) -> None:
    """In place on float32 [m, vocab]: for entry i, logits[rows[i], tokens[i]] gets the presence/frequency
    penalty when counts[i] > 0 and the repetition penalty when in_window[i]; penalties are per row."""
    if _backend is not None:
        return _backend.apply_penalties(logits, rows, tokens, counts, in_window, presence, frequency, repeat)
    import numpy as np
    _dev_ok(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "apply_penalties: logits must be float32 [m, vocab]")
    m, vocab = logits.shape
    n = len(rows)
    _need(len(tokens) == n and len(counts) == n and len(in_window) == n, "apply_penalties: entry lists differ in length")
    _need(len(presence) == m and len(frequency) == m and len(repeat) == m, "apply_penalties: one penalty per row")
    _need(all(0 <= r < m for r in rows), "apply_penalties: row out of range")
    dev = logits.device
    ints, fl = _Staging.send([np.asarray([rows, tokens, counts, in_window], dtype=np.int32),
                              np.asarray([presence, frequency, repeat], dtype=np.float32)], dev)
    _call("tp_apply_penalties", _ptr(logits), vocab, _ptr(ints[0]), _ptr(ints[1]), _ptr(ints[2]), _ptr(ints[3]),
          _ptr(fl[0]), _ptr(fl[1]), _ptr(fl[2]), n, _stream())


_SAMPLE_LIMITS: Optional[tuple] = None


def _sample_limits() -> tuple:
    """(pieces of a row, candidates per piece, largest top_k settled from candidates, most elements of a piece,
    bins of a counting pass) as the sampling kernels were compiled; ``sample`` sizes their scratch by these."""
    global _SAMPLE_LIMITS
    if _SAMPLE_LIMITS is None:
        buf = (ctypes.c_int * 5)()
        lib = _Library.get()
        if lib.tp_sample_limits(buf) != 0:
            raise KernelError(f"tp_sample_limits: {lib.tp_last_error().decode()}")
        _SAMPLE_LIMITS = tuple(int(v) for v in buf)
    return _SAMPLE_LIMITS


def sample(logits: torch.Tensor, work: torch.Tensor, temperature, top_k, top_p, min_p, rnd, typical_p=None,
           info: Optional[torch.Tensor] = None, settled: Optional[list] = None) -> torch.Tensor:
    """float32 [m, vocab] and per-row options (host arrays) -> int32 [m] chosen tokens.
    ``work`` is float32 scratch of at least [m, vocab].  temperature 0 rows return the argmax.
    ``typical_p`` None leaves that filter off (1.0) in every row.
    ``info``: float32 [m, 4] that receives, per row, what log-probabilities of the filtered distribution need
    (maximum, ln of the normaliser, smallest surviving value) and the chosen token's log-probability in column 3;
    ``work`` then holds the filtered, scaled logits for ``top_logprobs``.
    ``settled``: a list that receives, per row, 1 when the row was settled from the candidates of its pieces (a
    small top_k, or top_p alone on a row whose kept prefix is short) and 0 when the one block per row did it; for tests."""
    if typical_p is None:
        typical_p = [1.0] * len(temperature)
    if _backend is not None:
        if settled is not None:
            settled[:] = [0] * len(temperature)
        return _backend.sample(logits, work, temperature, top_k, top_p, min_p, rnd, typical_p, info)
    import numpy as np
    _dev_ok(logits, work)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample: logits must be float32 [m, vocab]")
    m, vocab = logits.shape
    _need(work.dtype == torch.float32 and work.numel() >= m * vocab, "sample: work buffer too small")
    for a in (temperature, top_k, top_p, min_p, rnd, typical_p):
        _need(len(a) == m, "sample: one option per row")
    dev = logits.device
    fl, tk = _Staging.send([np.asarray([temperature, top_p, min_p, rnd, typical_p], dtype=np.float32),
                            np.asarray(top_k, dtype=np.int32)], dev)
    out = torch.empty((m,), dtype=torch.int32, device=dev)
    # (the scratch buffers are laid out by the library's own sizes, asked of it once: pieces of a row, candidates a
    # piece may hand over, the largest top_k settled from candidates, the most elements of a piece, bins of a pass)
    pieces, ccap, kmax, per_max, bins = _sample_limits()
    part_max = torch.empty((m * pieces,), dtype=torch.float32, device=dev)    # (maxima of the pieces of each row)
    # rows that are only scaled (and cut by min_p) before the draw get the masses of their pieces from a kernel
    # of many blocks; worth it when there is such a row
    plain_rows = any(t > 0 and not (0 < k < vocab) and not (0.0 < p < 1.0) and not (ty < 1.0)
                     for t, k, p, ty in zip(temperature, top_k, top_p, typical_p))
    # rows cut by top_p alone are settled from the candidates of their pieces against the mass of the whole row
    piece_ok = -(-vocab // pieces) <= per_max and info is None
    topp_rows = piece_ok and vocab > kmax and any(
        t > 0 and not (0 < k < vocab) and 0.0 < p < 1.0 and not (ty < 1.0)
        for t, k, p, ty in zip(temperature, top_k, top_p, typical_p))
    part_mass = torch.empty((m * pieces,), dtype=torch.int64, device=dev) if (plain_rows or topp_rows) and info is None else None
    # rows cut by top_k have the first pass of their selection counted by the kernel of many blocks that scales the row
    # ... unless top_k is small: such a row is settled from the few candidates that each piece of it hands over
    small = lambda k, ty: 0 < k <= kmax and not (ty < 1.0) and piece_ok
    topk_rows = [(k, ty) for t, k, ty in zip(temperature, top_k, typical_p) if t > 0 and 0 < k < vocab]
    part_cnt = None
    if any(not small(k, ty) for k, ty in topk_rows):
        part_cnt = torch.empty((m * pieces * bins,), dtype=torch.int32, device=dev)
    cand_val = cand_idx = cand_cnt = cand_thr = done = None
    if topp_rows or any(small(k, ty) for k, ty in topk_rows):
        cand_val = torch.empty((m * pieces * ccap,), dtype=torch.float32, device=dev)
        cand_idx = torch.empty((m * pieces * ccap,), dtype=torch.int32, device=dev)
        cand_cnt = torch.empty((m * pieces,), dtype=torch.int32, device=dev)
        cand_thr = torch.empty((m * pieces,), dtype=torch.int32, device=dev)
        done = torch.empty((m,), dtype=torch.int32, device=dev)
    if info is not None:
        _dev_ok(info)
        _need(info.dtype == torch.float32 and info.is_contiguous() and tuple(info.shape) == (m, 4), "sample: info must be float32 [m, 4]")
    _call("tp_sample", _ptr(logits), _ptr(work), m, vocab, _ptr(fl[0]), _ptr(tk), _ptr(fl[1]), _ptr(fl[2]),
          _ptr(fl[4]), _ptr(fl[3]), _ptr(out), _ptr(info), _ptr(part_max), _ptr(part_mass), _ptr(part_cnt),
          _ptr(cand_val), _ptr(cand_idx), _ptr(cand_cnt), _ptr(cand_thr), _ptr(done), _stream())
    if settled is not None:
        settled[:] = [0] * m if done is None else done.tolist()
    return out


def top_logprobs(work: torch.Tensor, info: torch.Tensor, vocab: int, n: int):
    """After ``sample(..., info=info)``: the ``n`` most probable tokens of each row's filtered distribution,
    most probable first (ties by index), as (int32 [m, n] ids, float32 [m, n] log-probabilities); id -1 where a
    row has fewer survivors."""
    if _backend is not None:
        return _backend.top_logprobs(work, info, vocab, n)
    _dev_ok(work, info)
    m = info.shape[0]
    _need(info.dtype == torch.float32 and info.is_contiguous() and tuple(info.shape) == (m, 4), "top_logprobs: info must be float32 [m, 4]")
    _need(work.dtype == torch.float32 and work.is_contiguous() and work.numel() >= m * vocab, "top_logprobs: work buffer too small")
    _need(0 <= n <= vocab, "top_logprobs: n out of range")
    ids = torch.empty((m, n), dtype=torch.int32, device=info.device)
    lps = torch.empty((m, n), dtype=torch.float32, device=info.device)
    _call("tp_top_logprobs", _ptr(work), _ptr(info), m, vocab, n, _ptr(ids), _ptr(lps), _stream())
    return ids, lps


def take_rows(t: torch.Tensor, rows=None) -> torch.Tensor:
    """A new tensor holding rows ``rows`` (a list of indices; None: all of them, a plain copy) of a float32 or
    int32 tensor [n] or [n, width], by the library's own copy kernel."""
    if _backend is not None:
        return _backend.take_rows(t, rows)
    import numpy as np
    _dev_ok(t)
    _need(t.dtype in (torch.float32, torch.int32) and t.dim() in (1, 2), "take_rows: needs float32 or int32 [n] or [n, width]")
    n_in = t.shape[0]
    width = 1 if t.dim() == 1 else t.shape[1]
    if rows is None:
        n, idx = n_in, None
    else:
        n = len(rows)
        _need(all(0 <= int(r) < n_in for r in rows), "take_rows: row out of range")
        idx = _Staging.send([np.asarray(rows, dtype=np.int32)], t.device)[0] if n else None
    out = torch.empty((n,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
    if n and width:
        _call("tp_copy_rows4", _ptr(t), _ptr(idx), _ptr(out), n, width, _stream())
    return out


def zero_rows(t: torch.Tensor, rows) -> None:
    """t[rows] = 0 in place for a float32 or int32 tensor [n, ...] (rows: a list of indices)."""
    if _backend is not None:
        return _backend.zero_rows(t, rows)
    import numpy as np
    _dev_ok(t)
    _need(t.dtype in (torch.float32, torch.int32) and t.dim() >= 1, "zero_rows: needs a float32 or int32 tensor")
    n_in = t.shape[0]
    width = t[0].numel() if n_in else 0
    _need(all(0 <= int(r) < n_in for r in rows), "zero_rows: row out of range")
    if len(rows) and width:
        idx = _Staging.send([np.asarray(rows, dtype=np.int32)], t.device)[0]
        _call("tp_zero_rows4", _ptr(t), _ptr(idx), len(rows), width, _stream())


def fill_normal(out: torch.Tensor, seed: int, mean: float, std: float) -> torch.Tensor:
    """Fill a device tensor with mean + std * N(0, 1); element i depends only on (seed, i) and has the bits
    that ``weights.random_init.fill_normal_host`` gives it on the host."""
    if _backend is not None:
        return _backend.fill_normal(out, seed, mean, std)
    _dev_ok(out)
    _call("tp_fill_normal", _ptr(out), _dt(out), ctypes.c_size_t(out.numel()), ctypes.c_ulonglong(seed & (2 ** 64 - 1)),
          ctypes.c_double(mean), ctypes.c_double(std), _stream())
    return out
