"""The operations the parts are made of, each one a hand-written gfx950 kernel.

Every function checks on the host that operand shapes, dtypes and devices are
what its kernel and grid assume, then calls the kernel library.  There is no
other implementation behind them: without the built library they raise
`KernelLibraryMissing`.  Activations are float32 or bfloat16 ("T" below); the
residual stream, norm weights, rotation frequencies and logits are float32
always.

`use_backend` swaps the object the calls go to.  The engine never does; it is
the seam through which tests check the engine's bookkeeping against a plain
emulation of each kernel's contract.
"""
from __future__ import annotations

import contextlib
from typing import Optional

import torch

_ACT = (torch.float32, torch.bfloat16)
HEAD_DIM_STEP, MAX_HEAD_DIM = 4, 256      # what `paged_attention` takes: multiples of 4 up to 256
_backend = None


class KernelShapeError(ValueError):
    """An operand does not have the shape, dtype or layout the kernel needs."""


def backend():
    global _backend
    if _backend is None:
        from wllm_amd.kernels.hip_backend import HipBackend
        _backend = HipBackend()
    return _backend


@contextlib.contextmanager
def use_backend(obj):
    global _backend
    old, _backend = _backend, obj
    try:
        yield obj
    finally:
        _backend = old


def _need(cond: bool, msg) -> None:
    """`msg` is the message or a function that makes it (so that it is made only on failure)."""
    if not cond:
        raise KernelShapeError(msg() if callable(msg) else msg)


def _dense(t: torch.Tensor, name: str, dtype, shape=None) -> None:
    # the messages are made only when a check fails: this runs for every operand of every launch
    if not isinstance(t, torch.Tensor):
        raise KernelShapeError(f"{name}: expected a tensor")
    if isinstance(dtype, tuple):
        if t.dtype not in dtype:
            raise KernelShapeError(f"{name}: dtype {t.dtype}, expected one of {dtype}")
    elif t.dtype != dtype:
        raise KernelShapeError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if not t.is_contiguous():
        raise KernelShapeError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelShapeError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


# ---- operations that parts bring with them ------------------------------------------------------
class RegisteredOp:
    """An operation added by `register_op`: a kernel of a library of its own (or of the framework's)
    with its host-side check, its launch and, for tests without a GPU, its plain emulation."""

    def __init__(self, name, entry_point, argtypes, launch, check, emulate, library):
        self.name, self.entry_point, self.argtypes = name, entry_point, list(argtypes)
        self.launch, self.check, self.emulate, self.library = launch, check, emulate, library


_REGISTERED: dict = {}


def register_op(name: str, *, entry_point: str, argtypes, launch, check=None, emulate=None, library=None,
                replace: bool = False) -> RegisteredOp:
    """Adds an operation without a change to this package: a new part's kernel is a `.hip` file and a
    Python file of the part's own.

    entry_point, argtypes: the `extern "C"` function (returning 0, a HIP error code, or -1 for sizes it
        does not take) and its ctypes signature, the stream last.
    library: a function that returns the loaded library holding it (`library.load(source_dir=...)` of a
        folder of kernels), or None for the framework's own library.
    check(*args, **kwargs): raises `KernelShapeError` unless shapes, dtypes and layouts are what the kernel
        and its grid assume; it runs on the host before every launch.
    launch(fn, stream, *args, **kwargs) -> int: calls `fn` with raw pointers (`ops.pointer(tensor)`) and the stream.
    emulate(*args, **kwargs): the same contract in plain torch, for the tests that run the engine's
        bookkeeping without a GPU; never used by the engine.

    `ops.call(name, ...)` then checks the operands and launches on the stream of the step."""
    if name in _REGISTERED and not replace:
        raise ValueError(f"operation {name!r} is already registered")
    op = RegisteredOp(name, entry_point, argtypes, launch, check, emulate, library)
    _REGISTERED[name] = op
    return op


def call(name: str, *args, **kwargs) -> None:
    """Runs a registered operation on the current backend."""
    op = _REGISTERED.get(name)
    if op is None:
        raise KeyError(f"operation {name!r} is not registered; known: {sorted(_REGISTERED)}")
    if op.check is not None:
        op.check(*args, **kwargs)
    backend().run_registered(op, args, kwargs)


def pointer(t: Optional[torch.Tensor]):
    """A tensor's address as a ctypes argument (None: a null pointer)."""
    import ctypes
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def embed_lookup(ids: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> None:
    """out[i] = float32(table[ids[i]]) * scale.  ids int32 [n], table T [V, H], out float32 [n, H]."""
    _dense(ids, "ids", torch.int32)
    _need(ids.dim() == 1, "ids: expected one axis")
    _dense(table, "table", _ACT)
    _need(table.dim() == 2, "table: expected [vocab, hidden]")
    _dense(out, "out", torch.float32, (ids.shape[0], table.shape[1]))
    if ids.shape[0]:
        call("embed_lookup", ids, table, float(scale), out)


def feed_tokens(ids: torch.Tensor, dst: torch.Tensor, src: torch.Tensor, source: torch.Tensor) -> None:
    """ids[dst[j]] = source[src[j]] for every j with dst[j] >= 0 (entries out of range are skipped).
    All int32 and one axis; dst and src of equal length.  It feeds a step the tokens that the step
    before it sampled on the device."""
    for t, name in ((ids, "ids"), (dst, "dst"), (src, "src"), (source, "source")):
        _dense(t, name, torch.int32)
        _need(t.dim() == 1, lambda: f"{name}: expected one axis")
    _need(dst.shape == src.shape, "dst and src: expected equal lengths")
    if dst.shape[0]:
        call("feed_tokens", ids, dst, src, source)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             delta_bias: Optional[torch.Tensor] = None) -> None:
    """out = x * rsqrt(mean(x^2) + eps) * (offset + weight), all in float32, cast to out's dtype.

    x float32 [n, H]; weight float32 [H]; out T [m, H].  With `delta` (T [n, H], or a stack
    float32 [S, n, H] of partial sums that are added in order) the row normalised is
    x + delta; `delta_bias` (float32 [H]) is a row added to every row with it (the bias of the
    projection that made delta).  Without `rows`, m = n and the sum is written back
    to x (the residual stream moves on).  With `rows` (int32 [m]) only those rows are
    read, x is left alone and out[i] belongs to row rows[i].
    """
    _dense(x, "x", torch.float32)
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    n, h = x.shape
    _dense(weight, "weight", torch.float32, (h,))
    if delta is not None:
        if delta.dim() == 3:
            _dense(delta, "delta", torch.float32, (delta.shape[0], n, h))
            _need(delta.shape[0] >= 1, "delta: an empty stack")
        else:
            _dense(delta, "delta", _ACT, (n, h))
    m = n
    if rows is not None:
        _dense(rows, "rows", torch.int32)
        _need(rows.dim() == 1, "rows: expected one axis")
        m = rows.shape[0]
    _dense(out, "out", _ACT, (m, h))
    if delta_bias is not None:
        _dense(delta_bias, "delta_bias", torch.float32, (h,))
    if m:
        if delta_bias is not None:
            backend().rms_norm(x, weight, float(eps), float(offset), out, delta, rows, delta_bias)
        else:
            backend().rms_norm(x, weight, float(eps), float(offset), out, delta, rows)


def rope_and_cache_write(qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                         inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                         cache: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int,
                         head_dim: int, page_size: int, parts: Optional[torch.Tensor] = None) -> None:
    """Adds `bias`, rotates queries and keys in place and stores keys and values in pages.

    qkv T [n, (num_heads + 2*num_kv_heads) * head_dim]: queries, then keys, then values.
    bias float32 of a row's width, or None.  positions int32 [n].  inv_freq float32
    [rotary_dim/2] (None: no rotation): element j of a head is paired with j + rotary_dim/2
    and the pair is turned by position * inv_freq[j], the angle and its sine and cosine in
    float32.  slots int32 [n]: page * page_size + offset for each token; cache
    T [pages, 2, num_kv_heads, page_size*head_dim] holds a page's keys as [page_size,
    head_dim] and its values as [head_dim, page_size].  slots and cache None: nothing is
    stored (the layer reads another layer's cache).  `parts` (float32 [S, n, width]): the
    projection arrives as a stack of partial sums; their sum in order replaces what qkv holds
    on entry.
    """
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(qkv, "qkv", _ACT)
    _need(qkv.dim() == 2 and qkv.shape[1] == width, lambda: f"qkv: shape {tuple(qkv.shape)}, expected [n, {width}]")
    n = qkv.shape[0]
    if bias is not None:
        _dense(bias, "bias", torch.float32, (width,))
    if parts is not None:
        _need(parts.dim() == 3 and parts.shape[0] >= 1, "parts: expected [S, n, width]")
        _dense(parts, "parts", torch.float32, (parts.shape[0], n, width))
    _dense(positions, "positions", torch.int32, (n,))
    rotary_dim = 0
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1, "inv_freq: expected one axis")
        rotary_dim = 2 * inv_freq.shape[0]
        _need(0 < rotary_dim <= head_dim, lambda: f"rotary_dim {rotary_dim} does not fit head_dim {head_dim}")
    _need((slots is None) == (cache is None), "slots and cache go together")
    if cache is not None:
        _dense(slots, "slots", torch.int32, (n,))
        _dense(cache, "cache", qkv.dtype)
        _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
              lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    if n:
        backend().rope_and_cache_write(qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                                       head_dim, rotary_dim, page_size, parts)


def linear_residual_takes(rows: int, dtype: torch.dtype, out_features: int, in_features: int) -> bool:
    """Whether `linear_residual` has a kernel for these sizes."""
    return bool(backend().linear_residual_takes(rows, dtype, out_features, in_features))


SUMSQ_BAND = 16      # columns whose squares `linear_residual` adds into one entry of `sumsq`


def linear_residual_sumsq_shape(rows: int, out_features: int) -> tuple:
    """The shape of the `sumsq` operand of `linear_residual` for a residual of [rows, out_features]."""
    return (rows, out_features // SUMSQ_BAND)


def linear_residual(x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, sumsq: torch.Tensor,
                    tiles: Optional[torch.Tensor] = None) -> None:
    """residual += x @ weight^T in float32, and sumsq[m, b] = the sum of squares of the new
    residual[m, 16b : 16b + 16].  x T [m, k]; weight T [n, k] (`tiles`: its tile-major copy);
    residual float32 [m, n]; sumsq float32 [m, n / 16].  A row's mean square is then the sum of
    its row of `sumsq` over n: what a norm needs, without a pass over the residual.  Only for sizes
    that `linear_residual_takes`."""
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    m, k = x.shape
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == k, lambda: f"weight: shape {tuple(weight.shape)}, expected [out, {k}]")
    n = weight.shape[0]
    _check_tiles(tiles, weight, 1)
    _need(linear_residual_takes(m, x.dtype, n, k), "linear_residual: no kernel for these sizes")
    _dense(residual, "residual", torch.float32, (m, n))
    _dense(sumsq, "sumsq", torch.float32, linear_residual_sumsq_shape(m, n))
    if m:
        backend().linear_residual(x, weight, tiles, residual, sumsq)


def qkv_rope_takes(rows: int, dtype: torch.dtype, in_features: int, head_dim: int, rotary_dim: int) -> bool:
    """Whether `qkv_rope` has a kernel for these sizes (else the caller runs `linear` and
    `rope_and_cache_write`)."""
    return bool(backend().qkv_rope_takes(rows, dtype, in_features, head_dim, rotary_dim))


def qkv_rope(x: torch.Tensor, weight: torch.Tensor, qkv: torch.Tensor, bias: Optional[torch.Tensor],
             positions: torch.Tensor, inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
             cache: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
             tiles: Optional[torch.Tensor] = None) -> None:
    """qkv = x @ weight^T, then everything `rope_and_cache_write` does, in one kernel: the
    projection of a decode step never leaves the registers between the product and the rotation.
    x T [n, k]; weight T [(num_heads + 2*num_kv_heads) * head_dim, k], the stacked query, key and
    value matrices (`tiles`: its tile-major copy); the other operands as in `rope_and_cache_write`,
    with inv_freq of head_dim/2 entries or None.  Only for sizes that `qkv_rope_takes`."""
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    n = x.shape[0]
    _dense(weight, "weight", x.dtype, (width, x.shape[1]))
    _check_tiles(tiles, weight, 1)
    _dense(qkv, "qkv", x.dtype, (n, width))
    rotary_dim = 0
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1, "inv_freq: expected one axis")
        rotary_dim = 2 * inv_freq.shape[0]
    _need(qkv_rope_takes(n, x.dtype, x.shape[1], head_dim, rotary_dim or head_dim),
          "qkv_rope: no kernel for these sizes; run linear and rope_and_cache_write")
    if bias is not None:
        _dense(bias, "bias", torch.float32, (width,))
    _dense(positions, "positions", torch.int32, (n,))
    _need((slots is None) == (cache is None), "slots and cache go together")
    if cache is not None:
        _dense(slots, "slots", torch.int32, (n,))
        _dense(cache, "cache", x.dtype)
        _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
              lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    if n:
        backend().qkv_rope(x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                           head_dim, page_size)


def paged_attention(qkv: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                    token_segment: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor,
                    seg_ctx_len: torch.Tensor, out: torch.Tensor, *, num_heads: int, num_kv_heads: int,
                    head_dim: int, page_size: int, scale: float, window: int = 0,
                    max_q_len: int = 0, max_ctx_len: int = 0, plan=None, softcap: float = 0.0,
                    exact_weights: bool = False, chunk: int = 0, sinks: Optional[torch.Tensor] = None) -> None:
    """Softmax attention of every query over the keys of its own request in the paged cache.

    The batch is a row of segments; segment s holds tokens seg_q_start[s] .. +seg_q_len[s],
    the last seg_q_len[s] positions of a request that is seg_ctx_len[s] long after this
    step.  Token i of it is at position p = ctx_len - q_len + i and sees keys
    max(0, p - window + 1) .. p (window 0: from key 0); with `chunk` c > 0 instead, the keys of its
    own chunk of c positions counted from 0, (p // c) * c .. p.  With `sinks` (float32 [num_heads]) the
    softmax's denominator holds exp(sinks[h]) once more: a term with no key and no value, not scaled.
    Query head h uses key/value head
    h // (num_heads // num_kv_heads).  Scores are scaled by `scale` and then, with `softcap` c > 0,
    bent to c * tanh(score / c); scores, softmax and the weighted sum accumulate in float32.
    The bfloat16 matrix-core kernels round a softmax weight to bfloat16 before they multiply it with the
    values; with `exact_weights` they carry what the rounding left out through a second product, so the
    weights count with 16 bits (2^-17 of a weight, where float32 leaves 2^-24 and the values' own
    rounding 2^-9).  The other kernels weigh in float32 either way.
    qkv T [n, width]: a row begins with the num_heads query heads, which is all that is read of it
    (the row of `rope_and_cache_write`, or any wider one); block_tables int32 [S, max_pages];
    out T [n, num_heads*head_dim].
    max_q_len / max_ctx_len are host-side bounds of the segment arrays (0: unknown).
    `plan`: what `plan_paged_attention` returned for these segments and sizes, or None.
    """
    width = num_heads * head_dim
    _dense(qkv, "qkv", _ACT)
    _need(qkv.dim() == 2 and qkv.shape[1] >= width,
          lambda: f"qkv: shape {tuple(qkv.shape)}, expected [n, at least {width}]")
    n = qkv.shape[0]
    _need(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    _need(softcap >= 0.0, "softcap must not be negative (0: none)")
    _dense(cache, "cache", qkv.dtype)
    _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
          lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    _dense(block_tables, "block_tables", torch.int32)
    _need(block_tables.dim() == 2, "block_tables: expected [segments, pages]")
    s = block_tables.shape[0]
    _dense(token_segment, "token_segment", torch.int32, (n,))
    for name, t in (("seg_q_start", seg_q_start), ("seg_q_len", seg_q_len), ("seg_ctx_len", seg_ctx_len)):
        _dense(t, name, torch.int32, (s,))
    _dense(out, "out", qkv.dtype, (n, num_heads * head_dim))
    _need(window >= 0, "window must not be negative")
    _need(chunk >= 0 and not (chunk and window), "chunk must not be negative, and excludes a window")
    if sinks is not None:
        _dense(sinks, "sinks", torch.float32, (num_heads,))
    if n:
        backend().paged_attention(qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len,
                                  out, num_heads, num_kv_heads, head_dim, page_size, float(scale), int(window),
                                  int(max_q_len), int(max_ctx_len), plan,
                                  **({"softcap": float(softcap)} if softcap else {}),
                                  **({"exact_weights": True} if exact_weights else {}),
                                  **({"chunk": int(chunk)} if chunk else {}),
                                  **({"sinks": sinks} if sinks is not None else {}))


def head_prepare(rows: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                 inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor], cache: Optional[torch.Tensor], *,
                 num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, interleaved: bool = False,
                 norm_eps: Optional[float] = None, values_are_keys: bool = False,
                 parts: Optional[torch.Tensor] = None, norm_dim: Optional[int] = None,
                 head_norm: Optional[tuple] = None, rot_scale: float = 1.0) -> None:
    """What `rope_and_cache_write` does, for attention blocks that do more between projection and
    attention.  rows T [n, width]: num_heads query heads, num_kv_heads key heads, num_kv_heads value
    heads unless `values_are_keys`, then any further columns.  In this order, in float32: every
    element takes its bias (float32 [w] with w <= width: the row's first w columns have one; or None)
    and, with `parts` (float32 [S, n, width]), is
    the sum of the stack in order instead of what the row held; with `values_are_keys` a key head
    as it is now is stored as the value head; the first 2 * len(inv_freq) elements of every query
    and key head turn by position * inv_freq[j], pair j being elements (2j, 2j + 1) if
    `interleaved`, else (j, j + len(inv_freq)); with `norm_eps` every query and key head is
    divided by sqrt(sum of its squares / norm_dim + norm_eps) (norm_dim: head_dim unless given; less where
    the last elements of every head are padding that is always zero); the heads are written back and the
    key heads stored.  slots, cache as in `rope_and_cache_write` (both None: nothing is stored).
    `head_norm` = (w_q, w_k, eps), float32 [head_dim] each: before the rotation every query head is divided by
    sqrt(sum of its squares / norm_dim + eps) and multiplied by w_q, every key head likewise by w_k (an RMS
    norm with a weight over each head).  `rot_scale`: sine and cosine are multiplied by it."""
    heads = num_heads + (1 if values_are_keys else 2) * num_kv_heads
    _dense(rows, "rows", _ACT)
    _need(rows.dim() == 2 and rows.shape[1] >= heads * head_dim,
          lambda: f"rows: shape {tuple(rows.shape)}, expected [n, at least {heads * head_dim}]")
    n, width = rows.shape
    _need(0 < head_dim <= 256, "head_dim: at most 256")
    if bias is not None:
        _dense(bias, "bias", torch.float32)
        _need(bias.dim() == 1 and 0 < bias.shape[0] <= width, lambda: f"bias: shape {tuple(bias.shape)}, expected at most [{width}]")
    if parts is not None:
        _need(parts.dim() == 3 and parts.shape[0] >= 1, "parts: expected [S, n, width]")
        _dense(parts, "parts", torch.float32, (parts.shape[0], n, width))
    _dense(positions, "positions", torch.int32, (n,))
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1 and 0 < 2 * inv_freq.shape[0] <= head_dim,
              lambda: f"inv_freq: {tuple(inv_freq.shape)} does not fit head_dim {head_dim}")
    _need(norm_eps is None or norm_eps >= 0.0, "norm_eps must not be negative")
    norm_dim = head_dim if norm_dim is None else int(norm_dim)
    _need(0 < norm_dim <= head_dim, "norm_dim: from 1 to head_dim")
    _need((slots is None) == (cache is None), "slots and cache go together")
    if cache is not None:
        _dense(slots, "slots", torch.int32, (n,))
        _dense(cache, "cache", rows.dtype)
        _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
              lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    extra = {}
    if head_norm is not None:
        w_q, w_k, pre_eps = head_norm
        _dense(w_q, "head_norm[0]", torch.float32, (head_dim,))
        _dense(w_k, "head_norm[1]", torch.float32, (head_dim,))
        _need(pre_eps >= 0.0, "head_norm: eps must not be negative")
        extra["head_norm"] = (w_q, w_k, float(pre_eps))
    if rot_scale != 1.0:
        extra["rot_scale"] = float(rot_scale)
    if n:
        call("head_prepare", rows, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim,
             page_size, bool(interleaved), norm_eps, bool(values_are_keys), parts, norm_dim, **extra)


def _band(t: torch.Tensor, name: str, dtype, rows: int, cols: int) -> None:
    """A tensor [rows, cols] or a band of columns of a wider contiguous one."""
    if not isinstance(t, torch.Tensor) or t.dtype != dtype:
        raise KernelShapeError(f"{name}: expected a tensor of {dtype}")
    _need(t.dim() == 2 and tuple(t.shape) == (rows, cols), lambda: f"{name}: shape {tuple(t.shape)}, expected {(rows, cols)}")
    _need(rows == 0 or cols == 0 or (t.stride(1) == 1 and t.stride(0) >= cols),
          lambda: f"{name}: strides {t.stride()}: rows must be runs of consecutive elements")


def sigmoid_gate(a: torch.Tensor, gate: torch.Tensor, out: torch.Tensor, per: int = 1) -> None:
    """out = a * sigmoid(gate), in float32, cast to T.  a and out T [n, c]; gate T [n, c / per]: one
    gate for every `per` consecutive columns (per = the head size: a number a head).  Each operand may
    be a band of columns of a wider tensor (a view whose rows are runs of consecutive elements); out
    may be a."""
    _need(a.dim() == 2 and a.dtype in _ACT, "a: expected T [n, c]")
    n, c = a.shape
    _need(per >= 1 and c % per == 0, "per: a positive divisor of the columns")
    for t, name in ((a, "a"), (out, "out")):
        _band(t, name, a.dtype, n, c)
    _band(gate, "gate", a.dtype, n, c // per)
    if n and c:
        if per > 1:
            call("sigmoid_gate", a, gate, out, per)
        else:
            call("sigmoid_gate", a, gate, out)


def copy_columns(src: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out = src * scale (in float32, cast to T; scale 1: the same bits); both T [n, c], each possibly a
    band of columns of a wider tensor; out may be src."""
    _need(src.dim() == 2 and src.dtype in _ACT, "src: expected T [n, c]")
    n, c = src.shape
    _band(src, "src", src.dtype, n, c)
    _band(out, "out", src.dtype, n, c)
    if n and c:
        if scale != 1.0:
            call("copy_columns", src, out, float(scale))
        else:
            call("copy_columns", src, out)


def stream_add(x: torch.Tensor, addend: Optional[torch.Tensor] = None, delta: Optional[torch.Tensor] = None,
               delta_bias: Optional[torch.Tensor] = None) -> None:
    """x = ((x + delta) + delta_bias) + addend in float32, in place.  x float32 [n, H]; delta T [n, H]
    or a stack float32 [S, n, H] added in order; delta_bias float32 [H]; addend float32 [n, H]; any
    of the three may be None."""
    _dense(x, "x", torch.float32)
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    n, h = x.shape
    if delta is not None:
        if delta.dim() == 3:
            _dense(delta, "delta", torch.float32, (delta.shape[0], n, h))
            _need(delta.shape[0] >= 1, "delta: an empty stack")
        else:
            _dense(delta, "delta", _ACT, (n, h))
    if delta_bias is not None:
        _dense(delta_bias, "delta_bias", torch.float32, (h,))
    if addend is not None:
        _dense(addend, "addend", torch.float32, (n, h))
    if n and (delta is not None or delta_bias is not None or addend is not None):
        call("stream_add", x, addend, delta, delta_bias)


def plan_paged_attention(host_q_len, host_ctx_len, *, num_heads: int, num_kv_heads: int, head_dim: int,
                         page_size: int, window: int, dtype: torch.dtype, device):
    """Cuts a step's attention into work items for the kernels that want them, once per step
    and attention shape (all layers of that shape share it).  Returns an opaque plan, or None
    when the kernel that will run needs none.  host_q_len / host_ctx_len: the segment arrays
    on the host."""
    return backend().plan_paged_attention(host_q_len, host_ctx_len, num_heads, num_kv_heads, head_dim, page_size,
                                          int(window), dtype, device)


def static_attention_plan(segments: int, *, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                          window: int, dtype: torch.dtype, device, max_context: int, max_total_keys: int):
    """The same for a captured graph of `segments` requests of one token each: a plan of fixed shape in
    device memory, with room for contexts of up to `max_context` keys and `max_total_keys` keys of all
    requests together, whose `update(host_q_len, host_ctx_len)` rewrites it in place before a replay.
    None when the kernel that will run needs no plan."""
    make = getattr(backend(), "static_attention_plan", None)
    if make is None:
        return None
    return make(int(segments), num_heads, num_kv_heads, head_dim, page_size, int(window), dtype, device,
                int(max_context), int(max_total_keys))


def linear_splits(rows: int, out_features: int, in_features: int, dtype: torch.dtype) -> int:
    """Into how many partial sums over the input axis the product kernel for these sizes splits
    its work (1: it does not).  A caller that can take the sum later (the next norm, the rotation)
    hands `linear` an output of shape [S, rows, out_features] and saves the pass that adds them."""
    return int(backend().linear_splits(rows, out_features, in_features, dtype))


def tiled_size(rows: int, in_features: int, dtype: torch.dtype = torch.bfloat16) -> int:
    """Elements of the tile-major copy of a [rows, in_features] weight (`tile_weight`)."""
    if dtype == torch.float32:
        return -(-rows // 16) * 16 * -(-in_features // 16) * 16
    return -(-rows // 16) * 16 * in_features


def tile_weight(weight: torch.Tensor, halves: int = 1) -> Optional[torch.Tensor]:
    """The tile-major copy of a weight [n, k] that the few-row product kernels stream: a wavefront's
    load is one contiguous KiB of it, and its walk along k one contiguous run.
    bfloat16 (k a multiple of 32): for each band of 16 rows (the last padded with zero rows) and each
    step of 32 keys, a tile of 1 KiB in which lane l = 16g + i of a wavefront finds
    w[16 * band + i][32 * step + 8g .. +8].  With halves = 2 (a stacked gate and up matrix) each half
    is tiled by itself, the gate's bands first.
    float32 (k a multiple of 4): for each band of 16 rows and each chunk of 16 keys (rows and keys
    beyond the weight are zeros) a tile of 1 KiB in which lane l = 16g + i finds
    w[16 * band + i][16 * chunk + 4g .. +4]; a stacked matrix is tiled as the one matrix it is.
    Returns a flat tensor, or None for weights the few-row kernels do not take."""
    _dense(weight, "weight", _ACT)
    _need(weight.dim() == 2 and halves in (1, 2) and weight.shape[0] % halves == 0, "weight: expected [out, in]")
    if weight.dtype == torch.float32:
        n, k = weight.shape
        if k % 4 != 0 or n == 0 or k < 4:
            return None
        tiles = torch.empty(tiled_size(n, k, torch.float32), dtype=weight.dtype, device=weight.device)
        backend().tile_weight(weight, tiles)
        return tiles
    n, k = weight.shape[0] // halves, weight.shape[1]
    if k % 32 != 0 or n == 0:
        return None
    size = tiled_size(n, k)
    tiles = torch.empty(halves * size, dtype=weight.dtype, device=weight.device)
    for h in range(halves):
        backend().tile_weight(weight[h * n:(h + 1) * n], tiles[h * size:(h + 1) * size])
    return tiles


def _check_tiles(tiles, weight, halves: int) -> None:
    if tiles is None:
        return
    if weight.dtype == torch.float32:
        _need(weight.shape[1] % 4 == 0, "tiles: float32 weights have them only with in_features % 4 == 0")
        _dense(tiles, "tiles", weight.dtype, (tiled_size(weight.shape[0], weight.shape[1], torch.float32),))
        return
    n, k = weight.shape[0] // halves, weight.shape[1]
    _dense(tiles, "tiles", weight.dtype, (halves * tiled_size(n, k),))
    _need(k % 32 == 0, "tiles: bfloat16 weights have them only with in_features % 32 == 0")


def linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, tiles: Optional[torch.Tensor] = None) -> None:
    """out = x @ weight^T.  x T [m, k]; weight T [n, k]; out T or float32 [m, n], or float32
    [S, m, n] with S = linear_splits(m, n, k, T): then the S slices are partial sums whose sum in
    order is the product.  Products of bfloat16 accumulate in float32; float32 stays float32.
    `tiles` is `tile_weight(weight)`, the same numbers in the order the few-row kernels read
    fastest; with it they read that copy instead."""
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == x.shape[1],
          lambda: f"weight: shape {tuple(weight.shape)}, expected [out, {x.shape[1]}]")
    _check_tiles(tiles, weight, 1)
    if out.dim() == 3:
        s = linear_splits(x.shape[0], weight.shape[0], x.shape[1], x.dtype)
        _dense(out, "out", torch.float32, (s, x.shape[0], weight.shape[0]))
        _need(s > 1, "out: a stack of partial sums where the product is not split")
    else:
        _dense(out, "out", (x.dtype, torch.float32), (x.shape[0], weight.shape[0]))
    if x.shape[0]:
        backend().linear(x, weight, out, tiles)


# the activations of a gated feed-forward and the numbers the kernels know them by (`common.h` holds
# the same table): a new one is a line here, a line and a case there
ACTIVATIONS = {"gelu_tanh": 0, "silu": 1}


def gated_activation(gate_up: torch.Tensor, out: torch.Tensor, activation: str) -> None:
    """out = act(gate_up[:, :I]) * gate_up[:, I:], in float32, cast to T.  gate_up T [n, 2I]; out T [n, I],
    possibly a band of columns of a wider tensor."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    _dense(gate_up, "gate_up", _ACT)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gate_up: expected [n, 2*intermediate]")
    _band(out, "out", gate_up.dtype, gate_up.shape[0], gate_up.shape[1] // 2)
    if gate_up.shape[0]:
        call("gated_activation", gate_up, out, activation)


class NormOnLoad:
    """The input of a product as something the product kernel computes while it reads it:
    rms_norm(residual) with the rows' sums of squares already known.  residual float32 [m, k];
    sumsq float32 [m, c] whose rows add up to the rows' sums of squares (`linear_residual` leaves
    it); weight float32 [k]; the result is what `rms_norm(residual, weight, eps, offset)` gives in
    dtype T."""

    def __init__(self, residual: torch.Tensor, sumsq: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
                 dtype: torch.dtype):
        _dense(residual, "residual", torch.float32)
        _need(residual.dim() == 2, "residual: expected [rows, hidden]")
        _dense(sumsq, "sumsq", torch.float32)
        _need(sumsq.dim() == 2 and sumsq.shape[0] == residual.shape[0] and sumsq.shape[1] >= 1,
              "sumsq: expected [rows, columns]")
        _dense(weight, "weight", torch.float32, (residual.shape[1],))
        self.residual, self.sumsq, self.weight = residual, sumsq, weight
        self.eps, self.offset, self.dtype = float(eps), float(offset), dtype

    @property
    def shape(self):
        return self.residual.shape


def gated_linear_norm_takes(rows: int, dtype: torch.dtype, in_features: int) -> bool:
    """Whether `gated_linear` can take its input as a `NormOnLoad` at these sizes."""
    return bool(backend().gated_linear_norm_takes(rows, dtype, in_features))


def gated_linear_writes_band(rows: int, dtype: torch.dtype, in_features: int) -> bool:
    """Whether `gated_linear` at these sizes can write `out` as a band of columns of a wider tensor whose
    rows begin at multiples of 16 bytes."""
    return bool(getattr(backend(), "gated_linear_writes_band", lambda *a: False)(rows, dtype, in_features))


def gated_linear(x, weight: torch.Tensor, out: torch.Tensor, activation: str,
                 scratch: Optional[torch.Tensor], tiles: Optional[torch.Tensor] = None) -> None:
    """out = act(x @ Wg^T) * (x @ Wu^T) with weight = [Wg; Wu] stacked, T [2I, k]; x T [m, k];
    out T [m, I] (a band of a wider tensor where `gated_linear_writes_band`); scratch T [m, 2I] may be
    used for the unfused product.  `tiles` is
    `tile_weight(weight, halves=2)`.  x may be a `NormOnLoad` where `gated_linear_norm_takes` says so:
    the norm is then applied as the kernel reads the residual stream (scratch is not used)."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    if isinstance(x, NormOnLoad):
        _need(gated_linear_norm_takes(x.shape[0], x.dtype, x.shape[1]), "gated_linear: no kernel with the norm on load for these sizes")
        _dense(weight, "weight", x.dtype)
        _need(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.shape[0] % 2 == 0,
              lambda: f"weight: shape {tuple(weight.shape)}, expected [2*intermediate, {x.shape[1]}]")
        _dense(out, "out", x.dtype, (x.shape[0], weight.shape[0] // 2))
        _check_tiles(tiles, weight, 2)
        if x.shape[0]:
            backend().gated_linear_norm(x, weight, out, activation, tiles)
        return
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.shape[0] % 2 == 0,
          lambda: f"weight: shape {tuple(weight.shape)}, expected [2*intermediate, {x.shape[1]}]")
    inter = weight.shape[0] // 2
    if out.is_contiguous():
        _dense(out, "out", x.dtype, (x.shape[0], inter))
    else:
        _band(out, "out", x.dtype, x.shape[0], inter)
        _need(gated_linear_writes_band(x.shape[0], x.dtype, x.shape[1]), "out: a band of columns at sizes whose kernel writes whole rows")
    _dense(scratch, "scratch", x.dtype, (x.shape[0], 2 * inter))
    _check_tiles(tiles, weight, 2)
    if x.shape[0]:
        backend().gated_linear(x, weight, out, activation, scratch, tiles)


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = index of the largest value of row i, the lowest index among equals.
    logits float32 [m, V]; out int32 [m]."""
    _dense(logits, "logits", torch.float32)
    _need(logits.dim() == 2 and logits.shape[1] > 0, "logits: expected [rows, vocab]")
    _dense(out, "out", torch.int32, (logits.shape[0],))
    if logits.shape[0]:
        backend().argmax_rows(logits, out)


def sample_rows(logits: torch.Tensor, params: torch.Tensor, seeds: torch.Tensor,
                penalty_ids: Optional[torch.Tensor], penalty_offsets: Optional[torch.Tensor],
                out_tokens: torch.Tensor, out_logprobs: torch.Tensor, truncations: bool = True) -> None:
    """Samples one token per row.

    logits float32 [m, V].  params float32 [m, 5]: temperature (0: greedy), top_k (0: off),
    top_p (1: off), min_p (0: off), repetition_penalty (1: off).  seeds int64 [m, 2]: the
    key and counter of the row's uniform draw.  penalty_ids int32 [P] with penalty_offsets
    int32 [m+1]: the ids the repetition penalty applies to, row by row (None: no row has
    any).  out_tokens int32 [m]; out_logprobs float32 [m]: log-probability of the token
    under the penalised, temperature-scaled distribution before truncation (temperature 1
    for greedy rows).  `truncations` may be False only if no row has top_k or top_p on: the
    kernels then skip the passes that find their thresholds.
    """
    _dense(logits, "logits", torch.float32)
    _need(logits.dim() == 2 and logits.shape[1] > 0, "logits: expected [rows, vocab]")
    m = logits.shape[0]
    _dense(params, "params", torch.float32, (m, 5))
    _dense(seeds, "seeds", torch.int64, (m, 2))
    _need((penalty_ids is None) == (penalty_offsets is None), "penalty_ids and penalty_offsets go together")
    if penalty_ids is not None:
        _dense(penalty_ids, "penalty_ids", torch.int32)
        _dense(penalty_offsets, "penalty_offsets", torch.int32, (m + 1,))
    _dense(out_tokens, "out_tokens", torch.int32, (m,))
    _dense(out_logprobs, "out_logprobs", torch.float32, (m,))
    if m:
        backend().sample_rows(logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                              truncations)



# ---- norms around the residual stream, general form ---------------------------------------------------
NORM_KINDS = {"none": 0, "rms": 1, "layer": 2}


class NormRecipe:
    """A norm as the kernels take it: `kind` "rms" (v / sqrt(mean(v^2) + eps)) or "layer" ((v - mean) /
    sqrt(mean((v - mean)^2) + eps), no bias), times (offset + weight); weight float32 [H]."""

    def __init__(self, kind: str, weight: torch.Tensor, eps: float, offset: float = 0.0):
        _need(kind in ("rms", "layer"), lambda: f"norm kind {kind!r}: expected rms or layer")
        _dense(weight, "weight", torch.float32)
        _need(weight.dim() == 1, "weight: expected one axis")
        self.kind, self.weight, self.eps, self.offset = kind, weight, float(eps), float(offset)


def norm_add(x: torch.Tensor, *, delta: Optional[torch.Tensor] = None, delta_norm: Optional[NormRecipe] = None,
             out: Optional[torch.Tensor] = None, out_norm: Optional[NormRecipe] = None,
             rows: Optional[torch.Tensor] = None, conv: Optional[tuple] = None) -> None:
    """x += delta_norm(delta); out = out_norm(x), all in float32.

    x float32 [n, H], the residual stream.  delta T [n, H] or a stack float32 [S, n, H] of partial sums
    added in order; with `delta_norm` it is normalised before it is added (a norm behind a sublayer).
    out T or float32 [m, H] (optional): the new x under `out_norm` (None: as it is, cast).  Without
    `rows`, m = n and the sum is written back to x.  With `rows` (int32 [m]) only those rows are read,
    x is left alone and out[i] belongs to row rows[i].
    `conv` = (weight, state, carried_offset, state_slots), for a step in which every row is its request's one new
    token: out is then the new x through `stream_conv` with `single_tokens` (weight float32 [taps, H]; the carried rows
    of row i lie in row state_slots[i] of state), in the same launch; neither `out_norm` nor `rows` goes with it."""
    _dense(x, "x", torch.float32)
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    n, h = x.shape
    _need(h <= 16384, "hidden: at most 16384")
    if delta is not None:
        if delta.dim() == 3:
            _dense(delta, "delta", torch.float32, (delta.shape[0], n, h))
            _need(delta.shape[0] >= 1, "delta: an empty stack")
        else:
            _dense(delta, "delta", _ACT, (n, h))
    else:
        _need(delta_norm is None, "delta_norm without delta")
    for recipe, name in ((delta_norm, "delta_norm"), (out_norm, "out_norm")):
        if recipe is not None:
            _need(tuple(recipe.weight.shape) == (h,), lambda: f"{name}: weight of {tuple(recipe.weight.shape)}, expected [{h}]")
    m = n
    if rows is not None:
        _dense(rows, "rows", torch.int32)
        _need(rows.dim() == 1, "rows: expected one axis")
        _need(out is not None, "rows without out")
        m = rows.shape[0]
    if out is not None:
        _dense(out, "out", _ACT, (m, h))
    else:
        _need(out_norm is None, "out_norm without out")
    extra = {}
    if conv is not None:
        weight, state, carried_offset, state_slots = conv
        _need(out is not None and out_norm is None and rows is None, "conv: with out, without out_norm and rows")
        _dense(weight, "conv weight", torch.float32)
        _need(weight.dim() == 2 and weight.shape[1] == h and 1 <= weight.shape[0] <= 64, "conv weight: expected [taps <= 64, hidden]")
        _dense(state, "conv state", torch.float32)
        _need(state.dim() == 2 and 0 <= carried_offset and carried_offset + (weight.shape[0] - 1) * h <= state.shape[1],
              "conv state: a row holds the carried rows from carried_offset")
        _dense(state_slots, "conv state_slots", torch.int32, (n,))
        extra["conv"] = (weight, state, int(carried_offset), state_slots)
    if m and (delta is not None or out is not None):
        call("norm_add", x, delta, delta_norm, out, out_norm, rows, **extra)


def band_norm(bands: list, eps: float) -> None:
    """RMS norm with a weight over bands of columns: for each (src, weight, count, out[, bias]) of `bands`
    (one or two), out[r] = v / sqrt(sum(v^2) / count + eps) * weight with v = src[r] (+ bias, float32 [c]
    or None: a projection's bias that belongs in front of its norm).  src T [n, c] and out T
    [n, c'] with c' >= c may be bands of wider tensors and may be the same band; columns of out beyond c
    become zero.  weight float32 [c].  `count` is the number of elements the mean is taken over (less
    than c where the band carries padding that is always zero)."""
    _need(1 <= len(bands) <= 2, "bands: one or two")
    n, dtype = bands[0][0].shape[0], bands[0][0].dtype
    _need(dtype in _ACT, "src: expected T")
    bands = [tuple(b) + (None,) * (5 - len(b)) for b in bands]
    for src, weight, count, out, bias in bands:
        if bias is not None:
            _dense(bias, "bias", torch.float32, (src.shape[1],))
        _need(src.dim() == 2 and out.dim() == 2 and out.shape[1] >= src.shape[1], "out: at least as wide as src")
        _band(src, "src", dtype, n, src.shape[1])
        _band(out, "out", dtype, n, out.shape[1])
        _dense(weight, "weight", torch.float32, (src.shape[1],))
        _need(0 < count <= src.shape[1], "count: from 1 to the band's width")
    if n:
        call("band_norm", bands, float(eps))


def gated_lookup(gate: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int, out: torch.Tensor,
                 activation: str) -> None:
    """out[r, c] = act(gate[r, c]) * table[ids[r], col0 + c].  gate, out T [n, d]; ids int32 [n];
    table T [V, D] with col0 + d <= D."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    _dense(gate, "gate", _ACT)
    _need(gate.dim() == 2, "gate: expected [n, d]")
    n, d = gate.shape
    _dense(ids, "ids", torch.int32, (n,))
    _dense(table, "table", gate.dtype)
    _need(table.dim() == 2 and 0 <= col0 and col0 + d <= table.shape[1], "table: expected [V, at least col0 + d]")
    _dense(out, "out", gate.dtype, (n, d))
    if n and d:
        call("gated_lookup", gate, ids, table, int(col0), out, activation)


def head_linear(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor) -> None:
    """A product head by head: y[r, h*O + o] = sum_k x[r, h*K + k] * w[h, o, k], float32 sums in ascending
    order of k.  x T [n, heads*K] and y T [n, heads*O] may be bands of wider tensors; w T [heads, O, K]."""
    _dense(w, "w", _ACT)
    _need(w.dim() == 3, "w: expected [heads, out, in]")
    heads, o, k = w.shape
    _need(x.dim() == 2 and y.dim() == 2, "x, y: expected two axes")
    n = x.shape[0]
    _band(x, "x", w.dtype, n, heads * k)
    _band(y, "y", w.dtype, n, heads * o)
    if n:
        call("head_linear", x, w, y)


def causal_conv(inp: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor, carried_offset: int,
                token_segment: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor,
                state_slots: torch.Tensor, out: torch.Tensor) -> None:
    """A short causal convolution per channel over each segment, with silu, and the inputs it carries
    from step to step.  inp T [n, C] (may be a band of a wider row); weight float32 [C, taps], the last
    column the current token's; bias float32 [C]; out T [n, C] = silu(bias + sum_k weight[:, k] *
    inp[t - (taps-1) + k]), where inputs before a segment's first token are the request's carried
    rows: state float32 [slots, W] holds, from column `carried_offset` of row state_slots[segment],
    [taps-1, C], the oldest first (zeros for a fresh request).  Afterwards the carried rows are the
    segment's last taps-1 inputs (older carried rows move up where the segment is shorter)."""
    _need(inp.dim() == 2 and inp.dtype in _ACT, "inp: expected T [n, C]")
    n, c = inp.shape
    _band(inp, "inp", inp.dtype, n, c)
    _dense(weight, "weight", torch.float32)
    _need(weight.dim() == 2 and weight.shape[0] == c and 1 <= weight.shape[1] <= 64, "weight: expected [C, taps]")
    taps = weight.shape[1]
    _dense(bias, "bias", torch.float32, (c,))
    _dense(state, "state", torch.float32)
    _need(state.dim() == 2 and 0 <= carried_offset and carried_offset + (taps - 1) * c <= state.shape[1],
          "state: expected [slots, at least carried_offset + (taps-1)*C]")
    _dense(token_segment, "token_segment", torch.int32, (n,))
    s = seg_q_start.shape[0]
    for t, name in ((seg_q_start, "seg_q_start"), (seg_q_len, "seg_q_len"), (state_slots, "state_slots")):
        _dense(t, name, torch.int32, (s,))
    _dense(out, "out", inp.dtype, (n, c))
    if n:
        call("causal_conv", inp, weight, bias, state, int(carried_offset), token_segment, seg_q_start, seg_q_len,
             state_slots, out)


def stream_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, carried_offset: int, token_segment: torch.Tensor,
                seg_q_start: torch.Tensor, seg_q_len: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                single_tokens: bool = False) -> None:
    """A short causal convolution over time on each channel of the residual stream, added to the stream's own value:
    out[t, c] = x[t, c] + sum_k weight[k, c] * x[t - (taps - 1) + k, c], the rows before a segment's first token taken
    from the request's carried rows (zeros for a fresh request), which afterwards hold the segment's last taps - 1 rows.
    x float32 [n, C]; weight float32 [taps, C] (a row a tap, the last the current token's); state float32 [slots, W] with the carried rows [taps - 1, C] from column
    `carried_offset` of row state_slots[segment]; out T [n, C].  float32 sums in the order written.
    `single_tokens`: the caller knows that every segment is one token (a decode step); the carried rows are then moved
    by the launch that reads them (the same results, one launch less)."""
    _dense(x, "x", torch.float32)
    _need(x.dim() == 2, "x: expected [n, channels]")
    n, channels = x.shape
    _dense(weight, "weight", torch.float32)
    _need(weight.dim() == 2 and weight.shape[1] == channels and 1 <= weight.shape[0] <= 64, "weight: expected [taps <= 64, channels]")
    taps = weight.shape[0]
    _dense(state, "state", torch.float32)
    _need(state.dim() == 2 and 0 <= carried_offset and carried_offset + (taps - 1) * channels <= state.shape[1],
          "state: a row holds the carried rows from carried_offset")
    _dense(token_segment, "token_segment", torch.int32, (n,))
    _segments(seg_q_start, seg_q_len, state_slots)
    _dense(out, "out", _ACT, (n, channels))
    _need(not single_tokens or seg_q_start.shape[0] == n, "single_tokens: as many segments as tokens")
    if n:
        call("stream_conv", x, weight, state, int(carried_offset), token_segment, seg_q_start, seg_q_len, state_slots, out,
             **({"single_tokens": True} if single_tokens else {}))


def ssm_scan(xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
             state: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor, state_slots: torch.Tensor,
             y: torch.Tensor, *, heads: int, groups: int, state_size: int, head_dim: int,
             steps: Optional[torch.Tensor] = None) -> None:
    """The selective state-space recurrence over each segment's tokens in order, from and into the
    request's carried state.  Per head h (group h // (heads // groups)) and token:
        step = softplus(dt + dt_bias[h]);  S = exp(-exp(a_log[h]) * step) * S + step * B x^T;
        y = S^T C + d_skip[h] * x
    xbc T [n, heads*P + 2*groups*N]: x, then B, then C; dt T [n, heads] (may be a band of a wider row);
    dt_bias, a_log, d_skip float32 [heads]; state float32 [slots, W], whose row state_slots[segment]
    begins with S as [heads, N, P]; y float32 [n, heads*P].  All of the recurrence is float32.
    `steps`: float32 [2, n, heads] of scratch for the step sizes and decays (made here if not given; a
    caller whose step may be captured in a graph gives its own)."""
    _dense(xbc, "xbc", _ACT)
    inner = heads * head_dim
    _need(heads > 0 and groups > 0 and heads % groups == 0, "heads must be a multiple of groups")
    _need(0 < state_size <= 256, "state_size: from 1 to 256")
    _need(xbc.dim() == 2 and xbc.shape[1] == inner + 2 * groups * state_size,
          lambda: f"xbc: shape {tuple(xbc.shape)}, expected [n, {inner + 2 * groups * state_size}]")
    n = xbc.shape[0]
    _band(dt, "dt", xbc.dtype, n, heads)
    for t, name in ((dt_bias, "dt_bias"), (a_log, "a_log"), (d_skip, "d_skip")):
        _dense(t, name, torch.float32, (heads,))
    _dense(state, "state", torch.float32)
    _need(state.dim() == 2 and state.shape[1] >= heads * state_size * head_dim, "state: a row holds at least [heads, N, P]")
    s = seg_q_start.shape[0]
    for t, name in ((seg_q_start, "seg_q_start"), (seg_q_len, "seg_q_len"), (state_slots, "state_slots")):
        _dense(t, name, torch.int32, (s,))
    _dense(y, "y", torch.float32, (n, inner))
    if steps is None:
        steps = torch.empty((2, n, heads), dtype=torch.float32, device=xbc.device)
    _dense(steps, "steps", torch.float32, (2, n, heads))
    if n:
        call("ssm_scan", xbc, dt, dt_bias, a_log, d_skip, state, seg_q_start, seg_q_len, state_slots, y, heads, groups,
             state_size, head_dim, steps)


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, groups: int,
                     eps: float) -> None:
    """out = v / sqrt(mean over the part (v^2) + eps) * weight with v = y * silu(z), the row cut into
    `groups` equal parts that are each divided by their own root mean square.  y float32 [n, W]; z T
    [n, W] (may be a band of a wider row); weight float32 [W]; out T [n, W]."""
    _dense(y, "y", torch.float32)
    _need(y.dim() == 2, "y: expected [n, W]")
    n, w = y.shape
    _need(groups > 0 and w % groups == 0, "groups must divide the width")
    _need(z.dtype in _ACT, "z: expected T")
    _band(z, "z", z.dtype, n, w)
    _dense(weight, "weight", torch.float32, (w,))
    _dense(out, "out", z.dtype, (n, w))
    if n:
        call("gated_group_norm", y, z, weight, out, int(groups), float(eps))


# ---- a matrix memory a head (linear attention in its recurrent form) ------------------------------------
GATE_KINDS = {"sigmoid": 0, "silu": 1, "none": 2}
QUERY_ACTIVATIONS = {"none": 0, "silu": 1}


def _segments(seg_q_start, seg_q_len, state_slots) -> int:
    s = seg_q_start.shape[0]
    for t, name in ((seg_q_start, "seg_q_start"), (seg_q_len, "seg_q_len"), (state_slots, "state_slots")):
        _dense(t, name, torch.int32, (s,))
    return s


def memory_inputs(row: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], qk: torch.Tensor, *,
                  heads: int, head_dim: int, q_scale: float = 1.0, k_scale: float = 1.0) -> None:
    """Queries and keys as a matrix memory's recurrence takes them, in float32: qk[0] = q_scale * rot(q),
    qk[1] = k_scale * rot(k).  row T [n, at least 2 * heads * head_dim] (may be a band of a wider row)
    begins with the query heads, then the key heads; rot turns the first 2 * len(inv_freq) elements of
    every head by position * inv_freq[j], element j paired with j + len(inv_freq) (inv_freq None: nothing
    turns); qk float32 [2, n, heads * head_dim]."""
    _need(row.dim() == 2 and row.dtype in _ACT, "row: expected T [n, w]")
    n, width = row.shape[0], heads * head_dim
    _band(row, "row", row.dtype, n, row.shape[1])
    _need(heads > 0 and head_dim > 0 and row.shape[1] >= 2 * width, lambda: f"row: at least {2 * width} columns")
    _dense(positions, "positions", torch.int32, (n,))
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1 and 0 < 2 * inv_freq.shape[0] <= head_dim,
              lambda: f"inv_freq: {tuple(inv_freq.shape)} does not fit head_dim {head_dim}")
    _dense(qk, "qk", torch.float32, (2, n, width))
    if n:
        call("memory_inputs", row, positions, inv_freq, qk, heads, head_dim, float(q_scale), float(k_scale))


def memory_forget_inputs(row: torch.Tensor, bias: Optional[torch.Tensor], lower: Optional[torch.Tensor], qkf: torch.Tensor, *,
                         width: int, q_activation: str = "none") -> None:
    """The inputs of a recurrence whose forget gate a channel also decides what is written.  row T [n, >= 2 * width]
    (may be a band) begins with the queries and then the gate's projection z; bias, lower float32 [width] or None.
    f = lower + (1 - lower) * sigmoid(z + bias);  qkf[0] = act(q) ("none" or "silu"), qkf[1] = 1 - f, qkf[2] = f, all
    float32 [3, n, width]: what `memory_scan(row_decays=True)` takes."""
    _need(q_activation in QUERY_ACTIVATIONS, lambda: f"q_activation {q_activation!r}: one of {sorted(QUERY_ACTIVATIONS)}")
    _need(row.dim() == 2 and row.dtype in _ACT, "row: expected T [n, >= 2 * width]")
    n = row.shape[0]
    _band(row[:, :2 * width], "row", row.dtype, n, 2 * width)
    for t, name in ((bias, "bias"), (lower, "lower")):
        if t is not None:
            _dense(t, name, torch.float32, (width,))
    _dense(qkf, "qkf", torch.float32, (3, n, width))
    if n:
        call("memory_forget_inputs", row, bias, lower, qkf, width, q_activation)


def memory_gates(gates: torch.Tensor, i_bias: Optional[torch.Tensor], f_bias: Optional[torch.Tensor], state: torch.Tensor,
                 m_offset: int, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor, state_slots: torch.Tensor,
                 steps: torch.Tensor, *, heads: int, cap: Optional[float] = None) -> None:
    """Exponential gates held in range by a running maximum, over each segment's tokens in order.  Per head:
        i = cap tanh((z_i + i_bias) / cap);  f = logsigmoid(cap tanh((z_f + f_bias) / cap))   (cap None: no cap)
        m_t = max(f + m_(t-1), i);  a = exp(f + m_(t-1) - m_t);  b = exp(i - m_t);  floor = exp(-m_t)
    gates T [n, 2 * heads] (may be a band): z_i of all heads, then z_f; biases float32 [heads] or None;
    state float32 [slots, W] holds m as [heads] from column `m_offset` of row state_slots[segment]
    (zeros for a fresh request); steps float32 [3, n, heads] takes a, b and floor.  All float32."""
    _need(gates.dim() == 2 and gates.dtype in _ACT, "gates: expected T [n, 2 * heads]")
    n = gates.shape[0]
    _band(gates, "gates", gates.dtype, n, 2 * heads)
    for t, name in ((i_bias, "i_bias"), (f_bias, "f_bias")):
        if t is not None:
            _dense(t, name, torch.float32, (heads,))
    _dense(state, "state", torch.float32)
    _need(state.dim() == 2 and 0 <= m_offset and m_offset + heads <= state.shape[1], "state: a row holds m from m_offset")
    _segments(seg_q_start, seg_q_len, state_slots)
    _dense(steps, "steps", torch.float32, (3, n, heads))
    _need(cap is None or cap > 0, "cap must be positive or None")
    if n:
        call("memory_gates", gates, i_bias, f_bias, state, int(m_offset), seg_q_start, seg_q_len, state_slots, steps, heads, cap)


def memory_scan(qk: torch.Tensor, v: torch.Tensor, steps: Optional[torch.Tensor], decays: Optional[torch.Tensor],
                state: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor, state_slots: torch.Tensor,
                y: torch.Tensor, *, heads: int, head_dim: int, value_dim: int, nq: Optional[torch.Tensor] = None,
                n_offset: int = 0, row_decays: bool = False) -> None:
    """The matrix memory's recurrence over each segment's tokens in order, from and into the request's
    carried state.  Per head:  S = a S + b k v^T;  y = S^T q  with (a, b) of the token from `steps` (float32
    [3, n, heads], of which the first two are read) or, with `decays` (float32 [heads]) instead, (decays[h], 1).
    With `steps` the normaliser n = a n + b k is carried too, as [heads, head_dim] from column `n_offset` of the
    request's row, and nq (float32 [n, heads]) takes n . q.  qk float32 [2, n, heads * head_dim]: queries, then
    keys; v T [n, heads * value_dim] (may be a band); state float32 [slots, W], whose row state_slots[segment]
    begins with S as [heads, head_dim, value_dim]; y float32 [n, heads * value_dim].  All of the recurrence is float32.
    `row_decays` (then neither `steps` nor `decays`): qk has a third plane, float32 [3, n, heads * head_dim], of decays a
    row of S and token: S[i, :] = qk[2][i] S[i, :] + k[i] v^T."""
    if row_decays:
        _need(steps is None and decays is None, "row_decays: neither steps nor decays")
    else:
        _need((steps is None) != (decays is None), "steps or decays, one of the two")
    _need(v.dim() == 2 and v.dtype in _ACT, "v: expected T [n, heads * value_dim]")
    n = v.shape[0]
    _band(v, "v", v.dtype, n, heads * value_dim)
    _need(0 < head_dim <= 256 and value_dim > 0, "head_dim: from 1 to 256")
    _dense(qk, "qk", torch.float32, (3 if row_decays else 2, n, heads * head_dim))
    _dense(state, "state", torch.float32)
    memory = heads * head_dim * value_dim
    _need(state.dim() == 2 and state.shape[1] >= memory, "state: a row holds at least [heads, D, P]")
    if steps is not None:
        _dense(steps, "steps", torch.float32, (3, n, heads))
        _need(nq is not None, "nq: the normaliser's sums go with steps")
        _dense(nq, "nq", torch.float32, (n, heads))
        _need(memory <= n_offset and n_offset + heads * head_dim <= state.shape[1], "state: the normaliser lies behind S")
    else:
        if not row_decays:
            _dense(decays, "decays", torch.float32, (heads,))
        _need(nq is None, "nq: only with steps")
    _segments(seg_q_start, seg_q_len, state_slots)
    _dense(y, "y", torch.float32, (n, heads * value_dim))
    if n:
        call("memory_scan", qk, v, steps, decays, state, seg_q_start, seg_q_len, state_slots, y, heads, head_dim, value_dim, nq,
             int(n_offset), **({"row_decays": True} if row_decays else {}))


def head_norm_gate(y: torch.Tensor, gate: Optional[torch.Tensor], weight: Optional[torch.Tensor], out: torch.Tensor, *, heads: int,
                   eps: float, activation: str = "sigmoid", scale: float = 1.0, nq: Optional[torch.Tensor] = None,
                   floor: Optional[torch.Tensor] = None, den_eps: float = 0.0) -> None:
    """out = o / rms_of_its_head(o) * weight * act(gate) * scale with o = y / den: every one of `heads` equal parts
    of a row of y is divided by its denominator den = max(|nq|, floor) + den_eps (nq, floor float32 [n, heads]; without
    them den = 1) and then by sqrt(mean of its squares + eps).  y float32 [n, W]; gate T [n, W] and out T [n, W]
    may be bands of wider tensors; weight float32 [W] or None; activation "sigmoid" or "silu", or "none" with gate None."""
    _need(activation in GATE_KINDS, lambda: f"activation {activation!r}: expected one of {sorted(GATE_KINDS)}")
    _dense(y, "y", torch.float32)
    _need(y.dim() == 2 and heads > 0 and y.shape[1] % heads == 0, "y: expected [n, heads * P]")
    n, w = y.shape
    _need((gate is None) == (activation == "none"), "gate: None goes with the activation 'none'")
    if gate is not None:
        _need(gate.dtype in _ACT, "gate: expected T")
        _band(gate, "gate", gate.dtype, n, w)
    _need(out.dtype in _ACT and (gate is None or out.dtype == gate.dtype), "out: expected T")
    _band(out, "out", out.dtype, n, w)
    if weight is not None:
        _dense(weight, "weight", torch.float32, (w,))
    _need((nq is None) == (floor is None), "nq and floor go together")
    if nq is not None:
        _dense(nq, "nq", torch.float32, (n, heads))
        _dense(floor, "floor", torch.float32, (n, heads))
    if n:
        call("head_norm_gate", y, gate, weight, out, heads, float(eps), activation, float(scale), nq, floor, float(den_eps))


# ---- a mixture of experts ------------------------------------------------------------------------------
MOE_TILE_ROWS = 16           # rows of a tile of the kernels that stream an expert's weights past a few rows: 16, 32 or 64
MOE_STREAM_TILE_ROWS = (16, 32, 64)
MOE_BIG_TILE_ROWS = 128      # rows of a tile of the kernel that tiles many rows an expert through shared memory
MOE_MAX_EXPERTS = 256


def moe_tile_rows(assignments: int, experts: int, dtype, *inner_sizes: int) -> int:
    """The tile a step's plan should have: tiles of 128 rows where the experts get some tens of rows each on average
    (a prompt's portion) and the tiled kernel takes the sizes (bfloat16, inner sizes in multiples of 64); else tiles of
    16, 32 or 64 rows for the kernels that stream the weights (a fragment of the weights feeds a product for every 16
    rows of the tile): the smallest that most experts fill no more than once, so that their weights are read once."""
    big = dtype == torch.bfloat16 and assignments >= 32 * experts and all(k % 64 == 0 and k >= 64 for k in inner_sizes)
    if big:
        return MOE_BIG_TILE_ROWS
    mean = assignments / experts
    return 16 if mean <= 6 else 32 if mean <= 16 else 64


def moe_max_tiles(assignments: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    """The most tiles of `tile_rows` rows that `assignments` (token, expert) pairs can fill when the
    pairs of an expert lie together and every expert's last tile may be partly empty."""
    return assignments // tile_rows + experts


def moe_plan_size(assignments: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    """int32 elements of the plan `moe_plan` writes: the number of tiles in use, a tile's expert for
    every tile there is room for, and the rows of every tile."""
    return 1 + moe_max_tiles(assignments, experts, tile_rows) * (1 + tile_rows)


MOE_SCORINGS = {"softmax": 0, "sigmoid": 1}


def moe_route(x: torch.Tensor, router: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, *, groups: int = 1,
              keep: int = 1, eps: float = 1e-20, scoring: str = "softmax", normalize: bool = True) -> None:
    """Which experts each token uses.  z = x router^T in float32; s = softmax(z) over all experts; the
    experts form `groups` equal groups of neighbours, a group's score is its largest s, and only experts of
    the `keep` best groups may be chosen; the `top` = ids.shape[1] allowed experts with the largest s are
    chosen (of equal scores the lower index first), weights = their s / (sum of the chosen + eps).
    `scoring` "sigmoid": s = sigmoid(z), every expert by itself.  `normalize` False: weights = the chosen s themselves.
    x T [n, width]; router float32 [experts, width]; ids int32 [n, top]; weights float32 [n, top]."""
    _need(scoring in MOE_SCORINGS, lambda: f"scoring {scoring!r}: one of {sorted(MOE_SCORINGS)}")
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [n, width]")
    n, width = x.shape
    _dense(router, "router", torch.float32)
    _need(router.dim() == 2 and router.shape[1] == width and 0 < router.shape[0] <= MOE_MAX_EXPERTS,
          lambda: f"router: expected [at most {MOE_MAX_EXPERTS} experts, {width}]")
    experts = router.shape[0]
    _dense(ids, "ids", torch.int32)
    _need(ids.dim() == 2 and ids.shape[0] == n, "ids: expected [n, top]")
    top = ids.shape[1]
    _dense(weights, "weights", torch.float32, (n, top))
    _need(groups > 0 and experts % groups == 0 and 0 < keep <= groups, "groups must divide the experts; keep from 1 to groups")
    _need(0 < top <= keep * (experts // groups), "top: at most the experts of the kept groups")
    if n:
        extra = {} if scoring == "softmax" and normalize else {"scoring": scoring, "normalize": bool(normalize)}
        call("moe_route", x, router, ids, weights, int(groups), int(keep), float(eps), **extra)


def moe_plan(ids: torch.Tensor, plan: torch.Tensor, experts: int, tile_rows: int = MOE_TILE_ROWS) -> None:
    """Sorts a step's assignments (a = token * top + slot, expert ids.flat[a]) by expert, in tiles of
    `tile_rows` rows (R): plan[0] = tiles in use; plan[1 + t] = expert of tile t; plan[1 + T + R t + r] =
    the assignment in row r of tile t, or -1, with T = moe_max_tiles(ids.numel(), experts, R).  An expert's
    assignments lie together in any order.  ids int32 [n, top]; plan int32 [moe_plan_size(...)]."""
    _dense(ids, "ids", torch.int32)
    _need(ids.dim() == 2, "ids: expected [n, top]")
    _need(0 < experts <= MOE_MAX_EXPERTS, f"experts: from 1 to {MOE_MAX_EXPERTS}")
    _need(tile_rows in MOE_STREAM_TILE_ROWS or tile_rows == MOE_BIG_TILE_ROWS, "tile_rows: 16, 32, 64 or 128")
    _dense(plan, "plan", torch.int32, (moe_plan_size(ids.numel(), experts, tile_rows),))
    if ids.numel():
        call("moe_plan", ids, plan, int(experts), int(tile_rows))


def _big_tiles(tile_rows: int, dtype, inner: int) -> bool:
    _need(tile_rows in MOE_STREAM_TILE_ROWS or tile_rows == MOE_BIG_TILE_ROWS, "tile_rows: 16, 32, 64 or 128")
    if tile_rows == MOE_BIG_TILE_ROWS:
        _need(dtype == torch.bfloat16 and inner % 64 == 0 and inner >= 64,
              "tiles of 128 rows: bfloat16 and an inner size that is a multiple of 64")
        return True
    return False


def _expert_tiles(tiles: Optional[torch.Tensor], w: torch.Tensor) -> None:
    if tiles is not None:
        _need(w.dtype == torch.bfloat16 and w.shape[1] % 16 == 0 and w.shape[2] % 32 == 0,
              "tiles: bfloat16 experts of a multiple of 16 rows and of 32 keys")
        _dense(tiles, "tiles", w.dtype, (w.numel(),))


def moe_experts_up(x: torch.Tensor, w: torch.Tensor, plan: torch.Tensor, act: torch.Tensor, top: int,
                   activation: str, tile_rows: int = MOE_TILE_ROWS, tiles: Optional[torch.Tensor] = None,
                   in_weights: Optional[torch.Tensor] = None) -> None:
    """act[a] = activation(x[a // top] Wg_e^T) * (x[a // top] Wu_e^T) for every assignment a of the plan (of tiles of
    `tile_rows` rows), e its expert.  x T [n, width]; w T [experts, 2 * ff, width]: an expert's gate rows, then its
    up rows; act T [n * top, ff]; float32 sums.  `tiles`: `tile_weight` of w as one matrix [experts * 2 * ff, width]
    (ff a multiple of 16), which the kernel for tiles of 16 rows streams instead of w.  `in_weights` (float32
    [n, top]): the expert's input is in_weights.flat[a] * x[a // top]; the factor is taken out of both sums and
    multiplied in, in float32, before the activation."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [n, width]")
    n, width = x.shape
    _dense(w, "w", x.dtype)
    _need(w.dim() == 3 and w.shape[2] == width and w.shape[1] % 2 == 0, "w: expected [experts, 2 * ff, width]")
    experts, ff = w.shape[0], w.shape[1] // 2
    _dense(act, "act", x.dtype, (n * top, ff))
    _dense(plan, "plan", torch.int32, (moe_plan_size(n * top, experts, tile_rows),))
    _need(tiles is None or ff % 16 == 0, "tiles: ff must be a multiple of 16")
    _expert_tiles(tiles, w)
    extra = {}
    if in_weights is not None:
        _dense(in_weights, "in_weights", torch.float32, (n, top))
        extra["in_weights"] = in_weights
    if n:
        if _big_tiles(tile_rows, x.dtype, width):
            call("moe_experts_up_tiled", x, w, plan, act, int(top), activation, **extra)
        else:
            call("moe_experts_up", x, w, plan, act, int(top), activation, tiles, int(tile_rows), **extra)


def moe_experts_down(act: torch.Tensor, w: torch.Tensor, plan: torch.Tensor, weights: torch.Tensor,
                     out: torch.Tensor, tile_rows: int = MOE_TILE_ROWS, tiles: Optional[torch.Tensor] = None,
                     weighted: bool = True) -> None:
    """out[a % top][a // top] = weights.flat[a] * (act[a] Wd_e^T) for every assignment a of the plan: the
    experts' weighted results as a stack of `top` float32 partial sums over the tokens.  act T [n * top, ff];
    w T [experts, width, ff]; weights float32 [n, top]; out float32 [top, n, width] (or the first `top` slices of a
    taller stack).  `weighted` False: the factor is 1 (the weights entered elsewhere)."""
    _dense(act, "act", _ACT)
    _need(act.dim() == 2, "act: expected [n * top, ff]")
    _dense(weights, "weights", torch.float32)
    _need(weights.dim() == 2 and weights.numel() == act.shape[0], "weights: expected [n, top]")
    n, top = weights.shape
    _dense(w, "w", act.dtype)
    _need(w.dim() == 3 and w.shape[2] == act.shape[1], "w: expected [experts, width, ff]")
    _dense(out, "out", torch.float32, (top, n, w.shape[1]))
    _dense(plan, "plan", torch.int32, (moe_plan_size(n * top, w.shape[0], tile_rows),))
    _expert_tiles(tiles, w)
    extra = {} if weighted else {"weighted": False}
    if n:
        if _big_tiles(tile_rows, act.dtype, act.shape[1]):
            call("moe_experts_down_tiled", act, w, plan, weights, out, **extra)
        else:
            call("moe_experts_down", act, w, plan, weights, out, tiles, int(tile_rows), **extra)


# ---- the framework's own operations that go through the same door as a part's ------------------
def _register_own() -> None:
    from ctypes import c_float, c_int, c_longlong, c_void_p
    p = pointer
    register_op("embed_lookup", entry_point="wllm_embed_lookup",
                argtypes=[c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, ids, table, scale, out: fn(
                    p(ids), p(table), int(table.dtype == torch.bfloat16), scale, p(out), ids.shape[0], table.shape[1],
                    table.shape[0], stream))
    register_op("feed_tokens", entry_point="wllm_feed_tokens",
                argtypes=[c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, ids, dst, src, source: fn(
                    p(ids), p(dst), p(src), p(source), dst.shape[0], ids.shape[0], source.shape[0], stream))
    register_op("gated_activation", entry_point="wllm_gated_activation",
                argtypes=[c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_longlong, c_void_p],
                launch=lambda fn, stream, gate_up, out, activation: fn(
                    p(gate_up), p(out), int(gate_up.dtype == torch.bfloat16), ACTIVATIONS[activation], gate_up.shape[0],
                    out.shape[1], out.stride(0) if out.shape[0] > 1 else out.shape[1], stream))


    def prepare(fn, stream, rows, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim,
                page_size, interleaved, norm_eps, values_are_keys, parts, norm_dim, head_norm=None, rot_scale=1.0):
        w_q, w_k, pre_eps = head_norm if head_norm is not None else (None, None, -1.0)
        splits, stride = (parts.shape[0], parts.shape[1] * parts.shape[2]) if parts is not None else (0, 0)
        return fn(p(rows), int(rows.dtype == torch.bfloat16), rows.shape[1], p(parts), splits, stride, p(bias),
                  bias.shape[0] if bias is not None else 0, p(positions), p(inv_freq), p(slots), p(cache), cache.shape[0] if cache is not None else 0,
                  rows.shape[0], num_heads, num_kv_heads, head_dim,
                  2 * inv_freq.shape[0] if inv_freq is not None else 0, int(interleaved),
                  float(norm_eps) if norm_eps is not None else -1.0, norm_dim, int(values_are_keys), page_size,
                  p(w_q), p(w_k), pre_eps, rot_scale, stream)

    register_op("head_prepare", entry_point="wllm_head_prepare",
                argtypes=[c_void_p, c_int, c_int, c_void_p, c_int, c_longlong, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_longlong, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p,
                          c_void_p, c_float, c_float, c_void_p],
                launch=prepare)
    register_op("sigmoid_gate", entry_point="wllm_sigmoid_gate",
                argtypes=[c_void_p, c_longlong, c_void_p, c_longlong, c_void_p, c_longlong, c_int, c_int, c_int, c_int,
                          c_void_p],
                launch=lambda fn, stream, a, gate, out, per=1: fn(
                    p(a), a.stride(0), p(gate), gate.stride(0), p(out), out.stride(0), int(a.dtype == torch.bfloat16),
                    a.shape[0], a.shape[1], per, stream))
    register_op("copy_columns", entry_point="wllm_copy_columns",
                argtypes=[c_void_p, c_longlong, c_void_p, c_longlong, c_int, c_int, c_int, c_float, c_void_p],
                launch=lambda fn, stream, src, out, scale=1.0: fn(
                    p(src), src.stride(0), p(out), out.stride(0), int(src.dtype == torch.bfloat16), src.shape[0],
                    src.shape[1], scale, stream))

    def add(fn, stream, x, addend, delta, delta_bias):
        splits, stride = 1, 0
        if delta is not None and delta.dim() == 3:
            splits, stride = delta.shape[0], delta.shape[1] * delta.shape[2]
        return fn(p(x), p(delta), int(delta is not None and delta.dtype == torch.bfloat16), splits, stride,
                  p(delta_bias), p(addend), x.shape[0], x.shape[1], stream)

    register_op("stream_add", entry_point="wllm_stream_add",
                argtypes=[c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_int, c_int, c_void_p],
                launch=add)


    def norm_add_launch(fn, stream, x, delta, delta_norm, out, out_norm, rows, conv=None):
        splits, stride = 1, 0
        if delta is not None and delta.dim() == 3:
            splits, stride = delta.shape[0], delta.shape[1] * delta.shape[2]

        def recipe(r):
            return (NORM_KINDS[r.kind], p(r.weight), r.eps, r.offset) if r is not None else (0, p(None), 0.0, 0.0)

        return fn(p(x), p(delta), int(delta is not None and delta.dtype == torch.bfloat16), splits, stride,
                  *recipe(delta_norm), p(rows), p(out), int(out is not None and out.dtype == torch.bfloat16),
                  *recipe(out_norm), out.shape[0] if out is not None else x.shape[0], x.shape[1],
                  *((p(conv[0]), conv[0].shape[0], p(conv[1]), conv[1].stride(0), conv[2], p(conv[3])) if conv is not None
                    else (p(None), 0, p(None), 0, 0, p(None))), stream)

    register_op("norm_add", entry_point="wllm_norm_add",
                argtypes=[c_void_p, c_void_p, c_int, c_int, c_longlong, c_int, c_void_p, c_float, c_float, c_void_p, c_void_p,
                          c_int, c_int, c_void_p, c_float, c_float, c_int, c_int, c_void_p, c_int, c_void_p, c_longlong,
                          c_longlong, c_void_p, c_void_p],
                launch=norm_add_launch)

    def band_norm_launch(fn, stream, bands, eps):
        args = []
        for src, weight, count, out, bias in bands:
            args += [p(src), src.stride(0), src.shape[1], p(weight), float(count), p(out), out.stride(0), out.shape[1],
                     p(bias)]
        if len(bands) == 1:
            args += [p(None), 0, 0, p(None), 1.0, p(None), 0, 0, p(None)]
        first = bands[0][0]
        return fn(*args, eps, int(first.dtype == torch.bfloat16), first.shape[0], stream)

    one_band = [c_void_p, c_longlong, c_int, c_void_p, c_float, c_void_p, c_longlong, c_int, c_void_p]
    register_op("band_norm", entry_point="wllm_band_norm", argtypes=one_band + one_band + [c_float, c_int, c_int, c_void_p],
                launch=band_norm_launch)
    register_op("gated_lookup", entry_point="wllm_gated_lookup",
                argtypes=[c_void_p, c_void_p, c_void_p, c_longlong, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, gate, ids, table, col0, out, activation: fn(
                    p(gate), p(ids), p(table), table.shape[1], col0, p(out), int(gate.dtype == torch.bfloat16),
                    ACTIVATIONS[activation], gate.shape[0], gate.shape[1], stream))
    register_op("head_linear", entry_point="wllm_head_linear",
                argtypes=[c_void_p, c_longlong, c_void_p, c_void_p, c_longlong, c_int, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, x, w, y: fn(
                    p(x), x.stride(0), p(w), p(y), y.stride(0), int(w.dtype == torch.bfloat16), x.shape[0], w.shape[0],
                    w.shape[1], w.shape[2], stream))
    register_op("causal_conv", entry_point="wllm_causal_conv",
                argtypes=[c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_longlong, c_longlong, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, inp, weight, bias, state, carried_offset, token_segment, seg_q_start, seg_q_len,
                state_slots, out: fn(
                    p(inp), inp.stride(0), p(weight), p(bias), p(state), state.stride(0), carried_offset, p(token_segment),
                    p(seg_q_start), p(seg_q_len), p(state_slots), p(out), int(inp.dtype == torch.bfloat16), inp.shape[0],
                    seg_q_start.shape[0], inp.shape[1], weight.shape[1], stream))
    register_op("stream_conv", entry_point="wllm_stream_conv",
                argtypes=[c_void_p, c_void_p, c_void_p, c_longlong, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, x, weight, state, carried_offset, token_segment, seg_q_start, seg_q_len, state_slots,
                out, single_tokens=False: fn(
                    p(x), p(weight), p(state), state.stride(0), carried_offset, p(token_segment), p(seg_q_start), p(seg_q_len),
                    p(state_slots), p(out), int(out.dtype == torch.bfloat16), x.shape[0], seg_q_start.shape[0], x.shape[1],
                    weight.shape[0], int(single_tokens), stream))
    register_op("ssm_scan", entry_point="wllm_ssm_scan",
                argtypes=[c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, xbc, dt, dt_bias, a_log, d_skip, state, seg_q_start, seg_q_len, state_slots, y,
                heads, groups, state_size, head_dim, steps: fn(
                    p(xbc), p(dt), dt.stride(0), p(dt_bias), p(a_log), p(d_skip), p(state), state.stride(0), p(seg_q_start),
                    p(seg_q_len), p(state_slots), p(y), p(steps), int(xbc.dtype == torch.bfloat16), xbc.shape[0],
                    seg_q_start.shape[0], heads, groups, state_size, head_dim, stream))
    register_op("gated_group_norm", entry_point="wllm_gated_group_norm",
                argtypes=[c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p],
                launch=lambda fn, stream, y, z, weight, out, groups, eps: fn(
                    p(y), p(z), z.stride(0), p(weight), p(out), int(z.dtype == torch.bfloat16), y.shape[0], y.shape[1],
                    groups, eps, stream))

    bf = lambda t: int(t.dtype == torch.bfloat16)
    register_op("memory_inputs", entry_point="wllm_memory_inputs",
                argtypes=[c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                          c_float, c_void_p],
                launch=lambda fn, stream, row, positions, inv_freq, qk, heads, head_dim, q_scale, k_scale: fn(
                    p(row), row.stride(0), p(positions), p(inv_freq), p(qk), bf(row), row.shape[0], heads, head_dim,
                    2 * inv_freq.shape[0] if inv_freq is not None else 0, q_scale, k_scale, stream))
    register_op("memory_forget_inputs", entry_point="wllm_memory_forget_inputs",
                argtypes=[c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, row, bias, lower, qkf, width, q_activation: fn(
                    p(row), row.stride(0), p(bias), p(lower), p(qkf), bf(row), row.shape[0], width,
                    QUERY_ACTIVATIONS[q_activation], stream))
    register_op("memory_gates", entry_point="wllm_memory_gates",
                argtypes=[c_void_p, c_longlong, c_void_p, c_void_p, c_float, c_void_p, c_longlong, c_longlong, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, gates, i_bias, f_bias, state, m_offset, seg_q_start, seg_q_len, state_slots, steps,
                heads, cap: fn(
                    p(gates), gates.stride(0), p(i_bias), p(f_bias), float(cap) if cap else 0.0, p(state), state.stride(0),
                    m_offset, p(seg_q_start), p(seg_q_len), p(state_slots), p(steps), bf(gates), gates.shape[0],
                    seg_q_start.shape[0], heads, stream))
    register_op("memory_scan", entry_point="wllm_memory_scan",
                argtypes=[c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_longlong, c_longlong, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, qk, v, steps, decays, state, seg_q_start, seg_q_len, state_slots, y, heads,
                head_dim, value_dim, nq=None, n_offset=0, row_decays=False: fn(
                    p(qk), p(v), v.stride(0), p(steps), p(decays), p(state), state.stride(0), n_offset, p(seg_q_start),
                    p(seg_q_len), p(state_slots), p(y), p(nq), bf(v), v.shape[0], seg_q_start.shape[0], heads, head_dim,
                    value_dim, int(row_decays), stream))
    register_op("head_norm_gate", entry_point="wllm_head_norm_gate",
                argtypes=[c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_float, c_int,
                          c_int, c_int, c_int, c_int, c_float, c_float, c_void_p],
                launch=lambda fn, stream, y, gate, weight, out, heads, eps, activation, scale, nq=None, floor=None,
                den_eps=0.0: fn(
                    p(y), p(gate), gate.stride(0) if gate is not None else 0, p(weight), p(out), out.stride(0), p(nq), p(floor),
                    den_eps, bf(out), GATE_KINDS[activation], y.shape[0], heads, y.shape[1] // heads, eps, scale, stream))
    register_op("moe_route", entry_point="wllm_moe_route",
                argtypes=[c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                          c_int, c_int, c_void_p],
                launch=lambda fn, stream, x, router, ids, weights, groups, keep, eps, scoring="softmax", normalize=True: fn(
                    p(x), p(router), p(ids), p(weights), bf(x), x.shape[0], x.shape[1], router.shape[0], ids.shape[1], groups,
                    keep, eps, MOE_SCORINGS[scoring], int(normalize), stream))
    register_op("moe_plan", entry_point="wllm_moe_plan", argtypes=[c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, ids, plan, experts, tile_rows=MOE_TILE_ROWS: fn(
                    p(ids), p(plan), ids.numel(), experts, moe_max_tiles(ids.numel(), experts, tile_rows), tile_rows, stream))
    register_op("moe_experts_up", entry_point="wllm_moe_up",
                argtypes=[c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
                          c_void_p, c_void_p],
                launch=lambda fn, stream, x, w, plan, act, top, activation, tiles=None, tile_rows=MOE_TILE_ROWS,
                in_weights=None: fn(
                    p(x), p(w), p(tiles), p(plan), moe_max_tiles(act.shape[0], w.shape[0], tile_rows), tile_rows, p(act), bf(x),
                    ACTIVATIONS[activation], x.shape[1], act.shape[1], top, p(in_weights), stream))
    register_op("moe_experts_down", entry_point="wllm_moe_down",
                argtypes=[c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_int, c_void_p],
                launch=lambda fn, stream, act, w, plan, weights, out, tiles=None, tile_rows=MOE_TILE_ROWS, weighted=True: fn(
                    p(act), p(w), p(tiles), p(plan), moe_max_tiles(act.shape[0], w.shape[0], tile_rows), tile_rows,
                    p(weights if weighted else None), p(out), bf(act), weights.shape[0], act.shape[1], w.shape[1], weights.shape[1], stream))
    tiles = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
             c_void_p]
    register_op("moe_experts_up_tiled", entry_point="wllm_moe_tiles", argtypes=tiles,
                launch=lambda fn, stream, x, w, plan, act, top, activation, in_weights=None: fn(
                    p(x), p(w), p(plan), moe_max_tiles(act.shape[0], w.shape[0], MOE_BIG_TILE_ROWS), p(act), p(None), p(in_weights),
                    ACTIVATIONS[activation], x.shape[0], act.shape[1], x.shape[1], top, x.shape[0], stream))
    register_op("moe_experts_down_tiled", entry_point="wllm_moe_tiles", argtypes=tiles,
                launch=lambda fn, stream, act, w, plan, weights, out, weighted=True: fn(
                    p(act), p(w), p(plan), moe_max_tiles(act.shape[0], w.shape[0], MOE_BIG_TILE_ROWS), p(None), p(out),
                    p(weights if weighted else None), -1, act.shape[0], w.shape[1], act.shape[1], weights.shape[1], weights.shape[0], stream))

_register_own()
