"""Python face of the HIP library: one function per kernel entry point.

Each function checks on the host what its kernel assumes (device, dtype,
contiguity, shapes, index ranges where cheap), passes raw device pointers and
the current HIP stream, and raises `KernelError` with the library's message when
a launch is refused.  There is no fallback: without a GPU and the built library
these functions fail.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def lib():
    return _build.load()


def _dt(t: torch.Tensor) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not float32 or bfloat16") from None


# The entry points' argument types are set when the library is loaded (csrc/build.py `signatures`), so the
# helpers below hand over plain Python values: an address or None for a pointer, ints and floats for numbers.
def _ptr(t: Optional[torch.Tensor]):
    if t is None:
        return None
    if t.is_contiguous() and t.is_cuda:
        return t.data_ptr()
    raise KernelError("kernel operands must live on the GPU (no CPU path exists)" if not t.is_cuda
                      else "kernel operands must be contiguous")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current HIP stream of the current device (what torch launches on, also under graph capture)."""
    if _raw_stream is not None and _raw_device is not None:
        # the same value as below, without building a Stream object (17 us a call) or the checks of
        # torch.cuda.current_device (1 us)
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


_i64 = int
_i32 = int
_f32 = float
_functions = {}


def _call(name: str, *args):
    fn = _functions.get(name)
    if fn is None:
        fn = _functions[name] = getattr(lib(), name)
    if fn(*args) != 0:
        raise KernelError(lib().ix_last_error().decode("utf-8", "replace"))


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _is_i32(t, n=None):
    _need(t.dtype == torch.int32, "index arrays must be int32")
    if n is not None:
        _need(t.numel() >= n, f"index array holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------
def embed(h: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """h[t] = table[ids[t]] * scale; h float32 [T, H]."""
    T, H = h.shape
    _need(h.dtype == torch.float32, "the residual stream is float32")
    _need(table.dim() == 2 and table.shape[1] == H, "table width differs from h")
    _is_i32(ids, T)
    _call("ix_embed", _ptr(h), _ptr(table), _i32(_dt(table)), _ptr(ids), _i64(T), _i64(H), _i64(table.shape[0]),
          _f32(scale), _stream())


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, out: torch.Tensor, eps: float,
                rows: Optional[torch.Tensor] = None, groups: int = 1) -> None:
    """out = rmsnorm(h + delta) * weight; h += delta in place when `rows` is None.
    With `rows`, out[r] is computed from row rows[r] and h is not changed.  `groups`: the width is cut into that
    many equal runs, each divided by its own root mean square."""
    H = h.shape[1]
    _need(groups >= 1 and H % groups == 0, "the groups must divide the width")
    _need(h.dtype == torch.float32, "the residual stream is float32")
    _need(weight.numel() == H and out.shape[1] == H, "width mismatch")
    n_out = out.shape[0]
    if rows is None:
        _need(n_out == h.shape[0], "out must have a row per row of h")
    else:
        _is_i32(rows, n_out)
    if delta is not None:
        _need(delta.shape == h.shape, "delta must have the shape of h")
    _call("ix_add_rmsnorm", _ptr(h), _ptr(delta), _i32(_dt(delta) if delta is not None else F32), _ptr(weight),
          _i32(_dt(weight)), _ptr(out), _i32(_dt(out)), _ptr(rows), _i64(n_out), _i64(H), _i32(groups), _f32(eps), _stream())


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, W + i]."""
    T, W2 = gate_up.shape
    _need(W2 % 2 == 0 and out.shape == (T, W2 // 2) and out.dtype == gate_up.dtype, "shape or dtype mismatch")
    _call("ix_silu_mul", _ptr(gate_up), _ptr(out), _i32(_dt(out)), _i64(T), _i64(W2 // 2), _stream())


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y [T, N] += bias [N], in place (summed in float32, rounded to y's type)."""
    _need(y.dim() == 2 and y.is_contiguous() and bias.numel() == y.shape[1], "bias must hold one number per column")
    _call("ix_add_bias", _ptr(y), _i32(_dt(y)), _ptr(bias), _i32(_dt(bias)), _i64(y.shape[0]), _i64(y.shape[1]),
          _stream())


def rope_table(cos_sin: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, gain: float = 1.0) -> None:
    """cos_sin[t, j] = (cos, sin)(positions[t] * inv_freq[j]) * gain; float32 [T, half, 2]."""
    T, half, two = cos_sin.shape
    _need(two == 2 and cos_sin.dtype == torch.float32 and inv_freq.dtype == torch.float32, "float32 tables needed")
    _need(inv_freq.numel() == half, "inv_freq length differs")
    _is_i32(positions, T)
    _call("ix_rope_table", _ptr(cos_sin), _ptr(positions), _ptr(inv_freq), _i64(T), _i32(half), _f32(gain), _stream())


def polynorm(z: torch.Tensor, coef: torch.Tensor, out: torch.Tensor, eps: float) -> None:
    """out = a N(z) + b N(z^2) + c N(z^3) + e row by row, N(v) = v / sqrt(mean(v^2) + eps), coef = (a, b, c, e)."""
    _need(z.dim() == 2 and z.is_contiguous() and out.shape == z.shape and out.dtype == z.dtype and out.is_contiguous(),
          "z and out must be dense rows of one type")
    _need(coef.numel() == 4 and coef.is_contiguous(), "four coefficients")
    _call("ix_polynorm", _ptr(z), _ptr(coef), _i32(_dt(coef)), _ptr(out), _i32(_dt(z)), _i64(z.shape[0]), _i64(z.shape[1]),
          _f32(eps), _stream())


def weighted_sum(a: torch.Tensor, fa: float, b: Optional[torch.Tensor], fb: float, out: torch.Tensor) -> None:
    """out = fa * a + fb * b, float32 (b may be None)."""
    _need(a.is_contiguous() and out.dtype == torch.float32 and out.shape == a.shape and out.is_contiguous(), "dense operands")
    _need(b is None or (b.shape == a.shape and b.dtype == a.dtype and b.is_contiguous()), "b must be like a")
    _call("ix_weighted_sum", _ptr(a), _f32(fa), _ptr(b), _f32(fb), _i32(_dt(a)), _ptr(out), _i64(a.numel()), _stream())


def sigmoid_gate(y: torch.Tensor, gate: torch.Tensor) -> None:
    """y[t, c] *= sigmoid(gate[t, c]) in place; gate's rows may be strided."""
    _need(y.dim() == 2 and y.is_contiguous() and gate.shape == y.shape and gate.dtype == y.dtype and gate.stride(1) == 1
          and gate.is_cuda, "y dense, gate rows of y's type and width")
    _call("ix_sigmoid_gate", _ptr(y), gate.data_ptr(), _i64(gate.stride(0)), _i32(_dt(y)), _i64(y.shape[0]), _i64(y.shape[1]),
          _stream())


def qkv_rope_append(qkv: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                    slots: Optional[torch.Tensor], q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                    rotated: Optional[Tuple[int, int]] = None) -> None:
    """Bias, rotation and cache append after the fused q/k/v product.
    qkv [T, (heads + 2 kv_heads) * d]; key cache [pages, kv_heads, page_size, d], value cache
    [pages, kv_heads, d, page_size].  `rotated` = (first element, number of elements) of every head that the
    table rotates (the whole head if not given); the table is [T, elements / 2, 2]."""
    T = qkv.shape[0]
    rot_begin, rot_dim = rotated if rotated is not None else (0, head_dim)
    _need(0 <= rot_begin and rot_dim >= 0 and rot_dim % 2 == 0 and rot_begin + rot_dim <= head_dim,
          "the rotated part must be an even number of elements within the head")
    width = (heads + 2 * kv_heads) * head_dim
    _need(qkv.shape == (T, width), f"qkv must be [T, {width}]")
    _need(q_out.dtype == qkv.dtype and q_out.numel() == T * heads * head_dim, "q_out mismatch")
    if bias is not None:
        _need(bias.numel() == width, "bias length differs")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.shape == (T, rot_dim // 2, 2), "rotary table mismatch")
    page_size, total = 1, 0
    if k_cache is not None:
        _need(v_cache is not None and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "cache mismatch")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == kv_heads and k_cache.shape[3] == head_dim, "cache layout")
        _need(v_cache.shape == (k_cache.shape[0], kv_heads, head_dim, k_cache.shape[2]), "value cache layout")
        page_size = k_cache.shape[2]
        total = k_cache.shape[0] * page_size
        _need(slots is not None, "slots needed to write the cache")
        _is_i32(slots, T)
    _call("ix_qkv_rope_append", _ptr(qkv), _i32(_dt(qkv)), _ptr(bias), _i32(_dt(bias) if bias is not None else F32),
          _ptr(cos_sin), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _i64(T), _i32(heads),
          _i32(kv_heads), _i32(head_dim), _i32(page_size), _i64(total), _i32(rot_begin), _i32(rot_dim), _stream())


def qkv_rope_skinny(x: torch.Tensor, w_qkv: torch.Tensor, bias: Optional[torch.Tensor],
                    cos_sin: Optional[torch.Tensor], slots: Optional[torch.Tensor], q_out: torch.Tensor,
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], heads: int, kv_heads: int,
                    head_dim: int) -> None:
    """For at most 32 tokens (bfloat16): the q/k/v product, bias, rotation and cache append in one launch."""
    T, K = x.shape
    width = (heads + 2 * kv_heads) * head_dim
    _need(x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and q_out.dtype == torch.bfloat16,
          "the fused q/k/v kernel is bfloat16 only")
    _need(w_qkv.shape == (width, K), f"q/k/v weight must be [{width}, {K}]")
    _need(q_out.numel() == T * heads * head_dim, "q_out mismatch")
    if bias is not None:
        _need(bias.numel() == width, "bias length differs")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.shape == (T, head_dim // 2, 2), "rotary table mismatch")
    page_size, total = 1, 0
    if k_cache is not None:
        _need(v_cache is not None and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16,
              "cache mismatch")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == kv_heads and k_cache.shape[3] == head_dim, "cache layout")
        _need(v_cache.shape == (k_cache.shape[0], kv_heads, head_dim, k_cache.shape[2]), "value cache layout")
        page_size = k_cache.shape[2]
        total = k_cache.shape[0] * page_size
        _need(slots is not None, "slots needed to write the cache")
        _is_i32(slots, T)
    _call("ix_qkv_rope_skinny", _ptr(x), _ptr(w_qkv), _ptr(bias), _i32(_dt(bias) if bias is not None else F32),
          _ptr(cos_sin), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _i32(T), _i64(K), _i32(heads),
          _i32(kv_heads), _i32(head_dim), _i32(page_size), _i64(total), _stream())


def _check_caches(q, k_cache, v_cache):
    d = q.shape[2]
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache dtype differs from q")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == d, "key cache must be [pages, kv_heads, page_size, d]")
    _need(v_cache.shape == (k_cache.shape[0], k_cache.shape[1], d, k_cache.shape[2]),
          "value cache must be [pages, kv_heads, d, page_size]")


def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float,
                    window: int, sink: Optional[torch.Tensor] = None, turn_back: Optional[torch.Tensor] = None) -> None:
    """Paged attention, one workgroup per (token, head).  q [T, heads, d], out [T, heads, value size] (the value
    cache's).  `sink` float32 [heads]: exp(sink) joins every softmax's denominator, with no key and no value.
    `turn_back` float32 [T, value size / 2, 2]: every head's result is rotated by minus these angles (halves paired)."""
    T, heads, d = q.shape
    vd = v_cache.shape[2]
    _need(out.shape == (T, heads, vd) and out.dtype == q.dtype, "out mismatch")
    _check_kv(q.dtype, k_cache, v_cache, k_cache.shape[1], d, vd)
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == heads), "one float32 sink per head")
    _need(turn_back is None or (turn_back.dtype == torch.float32 and turn_back.shape == (T, vd // 2, 2) and vd % 2 == 0
                                and turn_back.is_contiguous()), "turn_back must be float32 [T, value size / 2, 2]")
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    _call("ix_attention_plain", _ptr(q), _ptr(k_cache), _ptr(v_cache), _i32(_dt(q)), _ptr(block_table),
          _ptr(seq_of_token), _ptr(positions), _ptr(out), _i64(T), _i32(heads), _i32(kv_heads), _i32(d), _i32(vd),
          _i32(page_size), _i32(block_table.shape[1]), _f32(scale), _i32(window), _ptr(sink), _ptr(turn_back), _stream())


def qkv_norm_rope_append(qkv: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float,
                         cos_sin: Optional[torch.Tensor], rot_begin: int, v_cos_sin: Optional[torch.Tensor],
                         slots: Optional[torch.Tensor], q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                         v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                         value_dim: int) -> None:
    """After the q|k|v product, per token and head: an RMS norm over the head with a weight per element (q and k,
    where `q_norm`, `k_norm` [head_dim] are given), the rotation of the 2 * cos_sin.shape[1] elements from `rot_begin`
    on (pairs (i, i + half) within them; float32 table [T, half, 2]), the rotation of ALL of a value head by its own
    table `v_cos_sin` [T, value_dim / 2, 2]; q goes to q_out [T, heads, head_dim], k and v to the token's slot of the
    paged caches (keys [pages, kv_heads, page_size, head_dim], values [pages, kv_heads, value_dim, page_size])."""
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.is_cuda
          and qkv.shape[1] >= (heads + kv_heads) * head_dim + kv_heads * value_dim, "qkv rows too short")
    _need(q_out.shape == (T, heads, head_dim) and q_out.dtype == qkv.dtype and q_out.is_contiguous(), "q_out mismatch")
    for w in (q_norm, k_norm):
        _need(w is None or (w.numel() == head_dim and w.is_contiguous()), "a norm weight per element of a head")
    half = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[0] == T and cos_sin.shape[2] == 2
              and cos_sin.is_contiguous(), "the rotation table must be float32 [T, half, 2]")
        half = cos_sin.shape[1]
        _need(rot_begin >= 0 and rot_begin + 2 * half <= head_dim, "the rotated part must lie within the head")
    if v_cos_sin is not None:
        _need(v_cos_sin.dtype == torch.float32 and v_cos_sin.shape == (T, value_dim // 2, 2) and value_dim % 2 == 0
              and v_cos_sin.is_contiguous(), "the values' rotation table must be float32 [T, value_dim / 2, 2]")
    page_size = 1
    if slots is not None:
        _check_kv(qkv.dtype, k_cache, v_cache, kv_heads, head_dim, value_dim)
        _need(k_cache.is_contiguous() and v_cache.is_contiguous(), "the caches must be contiguous")
        page_size = k_cache.shape[2]
        _is_i32(slots, T)
    wq, wk = q_norm, k_norm
    _call("ix_qkv_norm_rope_append", qkv.data_ptr(), _i32(_dt(qkv)), _i64(qkv.stride(0)), _ptr(wq),
          _i32(_dt(wq) if wq is not None else F32), _ptr(wk), _i32(_dt(wk) if wk is not None else F32), _f32(eps),
          _ptr(cos_sin), _i32(rot_begin), _i32(half), _ptr(v_cos_sin), _ptr(slots), _ptr(q_out),
          _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, _i64(T), _i32(heads),
          _i32(kv_heads), _i32(head_dim), _i32(value_dim), _i32(page_size),
          _i64(k_cache.shape[0] * page_size if slots is not None else 0), _stream())


def rotate_heads(x: torch.Tensor, cos_sin: torch.Tensor, inverse: bool = False) -> None:
    """x [T, heads, d] in place: every head's pair (i, i + d / 2) turned by the token's angle i of `cos_sin` (float32
    [T, d / 2, 2]); `inverse` turns the other way."""
    T, heads, d = x.shape
    _need(x.is_contiguous() and d % 2 == 0, "x must be dense [T, heads, d] with an even d")
    _need(cos_sin.dtype == torch.float32 and cos_sin.shape == (T, d // 2, 2) and cos_sin.is_contiguous(),
          "the rotation table must be float32 [T, d / 2, 2]")
    _call("ix_rotate_heads", _ptr(x), _i32(_dt(x)), _ptr(cos_sin), _i64(T), _i32(heads), _i32(d), _i32(1 if inverse else 0),
          _stream())


def attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                   tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, n_splits: int,
                   workspace: Optional[torch.Tensor], scale: float, window: int, tile_queries: int = 16,
                   prefetch: bool = False, grouped: bool = False, sink: Optional[torch.Tensor] = None,
                   turn_back: Optional[torch.Tensor] = None) -> None:
    """Paged attention on the matrix cores (bfloat16).  `tiles` int32 [3, n_tiles]: request, first token row and
    number of rows (<= tile_queries, which is 16 or 32) of each query tile.  `workspace` float32 with T * heads * n_splits * (d + 2) entries
    when n_splits > 1.  `grouped`: every tile is ONE token, and the query heads of a key/value head (at most 16)
    are served together, so that its keys and values are read once for all of them."""
    T, heads, d = q.shape
    _need(q.dtype == torch.bfloat16, "the matrix-core attention kernel is bfloat16 only")
    _need(out.shape == q.shape and out.dtype == q.dtype, "out mismatch")
    _check_caches(q, k_cache, v_cache)
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(positions, T)
    _is_i32(tiles)
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    n_tiles = tiles.shape[1]
    _need(not grouped or (tile_queries == 16 and heads // kv_heads <= 16 and n_tiles <= T),
          "grouped queries: one token per tile, tiles of 16, at most 16 query heads per key/value head")
    part_o = part_ml = None
    if n_splits > 1:
        need = T * heads * n_splits * (d + 2)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"workspace of {need} float32 needed")
        part_o = workspace
        part_ml = workspace[T * heads * n_splits * d:]
    args = (_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
            _ptr(tiles[1]), _ptr(tiles[2]), _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml), _i64(T),
            _i32(n_tiles), _i32(tile_queries), _i32(n_splits), _i32(heads), _i32(kv_heads), _i32(d), _i32(page_size),
            _i32(block_table.shape[1]), _f32(scale), _i32(window), _i32(1 if prefetch else 0),
            _i32(1 if grouped else 0))
    if sink is None and turn_back is None:
        _call("ix_attention_mfma", *args, _stream())
        return
    # `sink` float32 [heads]: exp(sink) joins every softmax's denominator; `turn_back` float32 [T, d / 2, 2]: the
    # result of every (token, head) is rotated by minus these angles, halves paired (d a multiple of 32)
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == heads), "one float32 sink per head")
    _need(turn_back is None or (turn_back.dtype == torch.float32 and turn_back.shape == (T, d // 2, 2) and d % 32 == 0
                                and turn_back.is_contiguous()), "turn_back must be float32 [T, d / 2, 2], d a multiple of 32")
    _call("ix_attention_mfma_sink", *args, _ptr(sink), _ptr(turn_back), _stream())


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float, window: int,
                      tile_queries: int = 64, pairs: Optional[torch.Tensor] = None, n_splits: int = 1,
                      workspace: Optional[torch.Tensor] = None) -> None:
    """Paged attention for prompt portions (bfloat16, head_dim <= 128): tiles of up to 64 queries of one
    request, keys and values shared through LDS; or, with `tile_queries` 128 (head_dim a multiple of 32), tiles of
    up to 128 queries, 32 per wavefront, with wavefronts of their own for the loads.  `tiles` as for attention_mfma.  `pairs` int32 [2, n]: the two
    units that workgroup i takes one after the other (second -1: none); every unit is to be named exactly once
    (a tile left out stays unwritten).  Without `pairs` every unit gets a workgroup of its own.

    A unit is a tile, or with n_splits > 1 slice `unit % n_splits` of the keys of tile `unit // n_splits`; then
    `workspace` (float32, T * heads * n_splits * (d + 2) entries) takes the slices' parts, and ALL T rows of `out`
    are written from it: rows that no tile covers get no meaningful values and are for the caller to fill."""
    T, heads, d = q.shape
    _need(q.dtype == torch.bfloat16, "the matrix-core attention kernel is bfloat16 only")
    _need(out.shape == q.shape and out.dtype == q.dtype, "out mismatch")
    _check_caches(q, k_cache, v_cache)
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(positions, T)
    _is_i32(tiles)
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    n_units = tiles.shape[1] * n_splits
    if pairs is None:
        pairs = torch.stack([torch.arange(n_units, dtype=torch.int32), torch.full((n_units,), -1, dtype=torch.int32)])
        pairs = pairs.to(q.device)
    _is_i32(pairs)
    _need(pairs.dim() == 2 and pairs.shape[0] == 2 and pairs.is_contiguous(), "pairs must be int32 [2, n_pairs]")
    _need(pairs.shape[1] <= n_units <= 2 * pairs.shape[1], "pairs must name every unit once")
    _need(page_size & (page_size - 1) == 0, "this kernel takes pages of a power of two of keys")
    part_o = part_ml = None
    if n_splits > 1:
        need = T * heads * n_splits * (d + 2)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"workspace of {need} float32 needed")
        part_o = workspace
        part_ml = workspace[T * heads * n_splits * d:]
    if tile_queries == 128:
        _need(d % 32 == 0, "tiles of 128 queries take head sizes in steps of 32")
        _call("ix_attention_prefill128", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
              _ptr(tiles[1]), _ptr(tiles[2]), _ptr(pairs[0]), _ptr(pairs[1]), _i32(pairs.shape[1]), _ptr(positions),
              _ptr(out), _ptr(part_o), _ptr(part_ml), _i32(n_splits), _i64(T), _i32(tiles.shape[1]), _i32(heads),
              _i32(kv_heads), _i32(d), _i32(page_size), _i32(block_table.shape[1]), _f32(scale), _i32(window),
              _stream())
        return
    _call("ix_attention_prefill", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
          _ptr(tiles[1]), _ptr(tiles[2]), _ptr(pairs[0]), _ptr(pairs[1]), _i32(pairs.shape[1]), _ptr(positions),
          _ptr(out), _ptr(part_o), _ptr(part_ml), _i32(n_splits), _i64(T), _i32(tiles.shape[1]), _i32(tile_queries),
          _i32(heads), _i32(kv_heads), _i32(d), _i32(page_size), _i32(block_table.shape[1]), _f32(scale),
          _i32(window), _stream())


ROUTE_SMALL_TOKENS = 128


def route_mode(renormalize: bool, sigmoid: bool = False, group_top2: bool = False) -> int:
    """The bits that tell a router's selection what to do (IX_ROUTE_* of the kernels)."""
    return (1 if renormalize else 0) | (2 if sigmoid else 0) | (4 if group_top2 else 0)


def moe_route(x: torch.Tensor, router_w: torch.Tensor, shared_gate_w: Optional[torch.Tensor], topk_w: torch.Tensor,
              topk_e: torch.Tensor, shared_gate: Optional[torch.Tensor], renormalize: bool, scale: float,
              always: int = 0, groups: int = 1, groups_keep: int = 1, sigmoid: bool = False,
              group_top2: bool = False) -> None:
    """Router product, softmax and top-k in float32; optional sigmoid gate of the shared expert.
    `sigmoid`: an expert's score is sigmoid(z) of its own logit instead of the softmax over all; `group_top2`: a
    group's score is the sum of its two largest scores instead of its largest.
    `always`: that many further slots per token after the chosen ones (topk_w and topk_e are [T, k + always]), naming
    the experts E .. E + always - 1 with the shared gate's value (or 1) as their weight: experts that every token uses.
    `groups`, `groups_keep`: the experts form that many equal groups of neighbours, and only experts of the
    `groups_keep` groups with the largest best score can be chosen (1, 1: every expert can)."""
    T, H = x.shape
    E = router_w.shape[0]
    k = topk_w.shape[1] - always
    _need(router_w.shape == (E, H), "router weight must be [experts, hidden]")
    _need(k > 0 and always >= 0, "at least one chosen slot")
    _need(1 <= groups <= 64 and E % groups == 0 and 1 <= groups_keep <= groups and k <= groups_keep * (E // groups),
          "the experts must split into at most 64 equal groups, and the kept groups must hold top_k experts")
    _need(topk_w.shape == (T, k + always) and topk_w.dtype == torch.float32, "topk_w must be float32 [T, k + always]")
    _need(topk_e.shape == (T, k + always) and topk_e.dtype == torch.int32, "topk_e must be int32 [T, k + always]")
    if shared_gate_w is not None:
        _need(shared_gate_w.numel() == H, "shared gate weight must hold `hidden` numbers")
        _need(shared_gate is not None and shared_gate.dtype == torch.float32 and shared_gate.numel() >= T,
              "shared_gate must be float32 [T]")
    scratch = None
    all_bf16 = (x.dtype == torch.bfloat16 and router_w.dtype == torch.bfloat16
                and (shared_gate_w is None or shared_gate_w.dtype == torch.bfloat16))
    if T <= ROUTE_SMALL_TOKENS or all_bf16:
        # few tokens: scores go through a scratch so that many workgroups share the rows; many tokens in
        # bfloat16: the scores are a product on the matrix cores
        scratch = torch.empty((T, E + 1), dtype=torch.float32, device=x.device)
    _call("ix_moe_route", _ptr(x), _i32(_dt(x)), _ptr(router_w), _i32(_dt(router_w)), _ptr(shared_gate_w),
          _i32(_dt(shared_gate_w) if shared_gate_w is not None else F32), _ptr(topk_w), _ptr(topk_e),
          _ptr(shared_gate if shared_gate_w is not None else None), _ptr(scratch), _i64(T), _i64(H), _i32(E), _i32(k),
          _i32(route_mode(renormalize, sigmoid, group_top2)), _f32(scale), _i32(always), _i32(groups),
          _i32(groups_keep), _stream())


# the one-launch router: at most this many tokens, experts and bytes of one token as float32
ROUTE_ONE_LAUNCH_EXPERTS, ROUTE_ONE_LAUNCH_ROW_BYTES = 256, 40 * 1024
ROUTE_ONE_LAUNCH_TOKENS = 16
_arrival_counters: dict = {}


def _arrival_counter(device: torch.device) -> torch.Tensor:
    """Counters (one for the launch and one per token) per device that the one-launch router's workgroups count
    themselves off on; every launch leaves them zero.  Launches on one device follow one another on a stream, so
    they can share them."""
    c = _arrival_counters.get(device)
    if c is None:
        c = _arrival_counters[device] = torch.zeros(1 + ROUTE_ONE_LAUNCH_TOKENS, dtype=torch.int32, device=device)
    return c


def route_one_launch_fits(tokens: int, width: int, experts: int) -> bool:
    """Whether `moe_route_dispatch` takes these sizes.  Beyond 16 tokens `moe_route` and `moe_dispatch` are as
    fast (12.4 us both at 16 tokens of 4 experts each out of 60, 11.2 against 12.3 us at 8)."""
    return (0 < tokens <= ROUTE_ONE_LAUNCH_TOKENS and experts <= ROUTE_ONE_LAUNCH_EXPERTS
            and width * 4 <= ROUTE_ONE_LAUNCH_ROW_BYTES)


def moe_route_dispatch(x: Optional[torch.Tensor], router_w: torch.Tensor, shared_gate_w: Optional[torch.Tensor],
                       topk_w: torch.Tensor, topk_e: torch.Tensor, shared_gate: Optional[torch.Tensor],
                       renormalize: bool, scale: float, offsets: torch.Tensor, rows: torch.Tensor,
                       dest: torch.Tensor, tile_rows: int = 0, tile_map: Optional[torch.Tensor] = None,
                       norm: Optional[tuple] = None, groups: int = 1, groups_keep: int = 1, sigmoid: bool = False,
                       group_top2: bool = False) -> None:
    """`moe_route` and `moe_dispatch` for up to 16 tokens in one launch: the router scores are spread over many
    workgroups, and the last one to finish its scores selects and groups (`route_one_launch_fits`).

    With `norm` = (h, delta, weight, eps, x_out) the norm before the feed-forward is part of the launch too
    (`x` is None then): x_out = rmsnorm(h + delta) * weight is written and routed, and h += delta."""
    if norm is not None:
        h, delta, gamma, eps, x_out = norm
        _need(x is None, "x is made by the norm")
        _need(h.dtype == torch.float32 and h.dim() == 2, "the residual stream is float32 [T, H]")
        _need(delta.shape == h.shape and x_out.shape == h.shape and delta.dtype == x_out.dtype,
              "delta and x_out must have the shape of h and one type")
        _need(gamma.numel() == h.shape[1], "the norm weight must hold `hidden` numbers")
        x = x_out
    T, H = x.shape
    E = router_w.shape[0]
    k = topk_w.shape[1]
    A = T * k
    _need(route_one_launch_fits(T, H, E), "too many tokens or experts, or too wide, for the one-launch router")
    _need(1 <= groups <= 64 and E % groups == 0 and 1 <= groups_keep <= groups and k <= groups_keep * (E // groups),
          "the experts must split into at most 64 equal groups, and the kept groups must hold top_k experts")
    _need(router_w.shape == (E, H), "router weight must be [experts, hidden]")
    _need(topk_w.shape == (T, k) and topk_w.dtype == torch.float32, "topk_w must be float32 [T, k]")
    _need(topk_e.shape == (T, k) and topk_e.dtype == torch.int32, "topk_e must be int32 [T, k]")
    if shared_gate_w is not None:
        _need(shared_gate_w.numel() == H, "shared gate weight must hold `hidden` numbers")
        _need(shared_gate is not None and shared_gate.dtype == torch.float32 and shared_gate.numel() >= T,
              "shared_gate must be float32 [T]")
    _is_i32(offsets, E + 1)
    _is_i32(rows, A)
    _is_i32(dest, A)
    te = tr = ti = None
    if tile_rows > 0:
        mt = moe_max_tiles(A, E, tile_rows)
        _need(tile_map is not None, "tile_map needed")
        _is_i32(tile_map, 2 * mt + 1)
        te, tr, ti = tile_map[:mt], tile_map[mt:2 * mt], tile_map[2 * mt:]
    logits = torch.empty((T, E + 1), dtype=torch.float32, device=x.device)
    router = (_ptr(router_w), _i32(_dt(router_w)), _ptr(shared_gate_w),
              _i32(_dt(shared_gate_w) if shared_gate_w is not None else F32), _ptr(logits),
              _ptr(_arrival_counter(x.device)), _i64(H), _ptr(topk_w), _ptr(topk_e),
              _ptr(shared_gate if shared_gate_w is not None else None), _ptr(offsets), _ptr(rows), _ptr(dest),
              _i32(T), _i32(E), _i32(k), _i32(route_mode(renormalize, sigmoid, group_top2)), _f32(scale), _i32(groups),
              _i32(groups_keep),
              _i32(tile_rows), _ptr(te), _ptr(tr), _ptr(ti), _stream())
    if norm is not None:
        _call("ix_moe_norm_route_dispatch_small", _ptr(h), _ptr(delta), _i32(_dt(x_out)), _ptr(gamma),
              _i32(_dt(gamma)), _f32(eps), _ptr(x_out), *router)
    else:
        _call("ix_moe_route_dispatch_small", _ptr(x), _i32(_dt(x)), *router)


def moe_dispatch(topk_e: torch.Tensor, offsets: torch.Tensor, rows: torch.Tensor, dest: torch.Tensor,
                 experts: int, tile_rows: int = 0, tile_map: Optional[torch.Tensor] = None) -> None:
    """Group assignments by expert: offsets [E+1], rows [A] (grouped row -> token), dest [A].
    With tile_rows > 0 also the row-tile map for the matrix-core product: `tile_map` int32
    [2 * max_tiles + 1] = tile_expert | tile_row0 | number of tiles, max_tiles = moe_max_tiles(A, E, tile_rows)."""
    T, k = topk_e.shape
    A = T * k
    _is_i32(topk_e)
    _is_i32(offsets, experts + 1)
    _is_i32(rows, A)
    _is_i32(dest, A)
    te = tr = ti = None
    if tile_rows > 0:
        mt = moe_max_tiles(A, experts, tile_rows)
        _need(tile_map is not None, "tile_map needed")
        _is_i32(tile_map, 2 * mt + 1)
        te, tr, ti = tile_map[:mt], tile_map[mt:2 * mt], tile_map[2 * mt:]
    _call("ix_moe_dispatch", _ptr(topk_e), _ptr(offsets), _ptr(rows), _ptr(dest), _i64(A), _i32(experts), _i32(k),
          _i32(tile_rows), _ptr(te), _ptr(tr), _ptr(ti), _stream())


PLAIN_PRODUCT, GATE_UP_SWIGLU, RELU_SQUARED = 0, 1, 2


def _epilogue(gate_up) -> int:
    """What a grouped product does with its sums: False / 0 nothing, True / 1 the weights hold gate rows then up rows
    and the result is silu(gate) * up, 2 the square of relu of a plain product."""
    code = int(gate_up)
    _need(code in (PLAIN_PRODUCT, GATE_UP_SWIGLU, RELU_SQUARED), "unknown epilogue of a grouped product")
    return code


def moe_max_tiles(assignments: int, experts: int, tile_rows: int) -> int:
    """Upper bound of the number of row tiles: every expert may end with a partial tile."""
    return max(1, min(assignments, -(-assignments // tile_rows) + experts))


def moe_grouped_mfma(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                     rows: Optional[torch.Tensor], tile_map: torch.Tensor, tile_rows: int, gate_up: bool,
                     k_split: int, glu_limit: float = 0.0) -> None:
    """Grouped product on the matrix cores (bfloat16), shapes as `moe_grouped_plain`; `tile_map` from `moe_dispatch`."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if _epilogue(gate_up) == GATE_UP_SWIGLU else n_out),
          "expert weight shape does not fit")
    _need(K % 8 == 0, "the reduction width must be a multiple of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, tile_rows)
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_mfma", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i32(tile_rows), _i64(n_out), _i64(K),
          _i32(_epilogue(gate_up)), _i32(k_split), _f32(glu_limit), _stream())


def moe_grouped_dual(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                     rows: Optional[torch.Tensor], tile_map: torch.Tensor, tile_rows: int, a_s: torch.Tensor,
                     w_s: torch.Tensor, out_s: torch.Tensor, gate_up: bool, glu_limit: float = 0.0,
                     glu_limit_s: float = 0.0) -> None:
    """`moe_grouped_mfma` (split reduction) for the routed experts and, in the same launch, the shared expert:
    out_s = a_s . w_s^T (with SwiGLU when gate_up; `glu_limit`, `glu_limit_s`: the clamped form, for the routed
    experts and for the shared one)."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    T, n_out_s = out_s.shape
    K_s = a_s.shape[1]
    for t in (a, w, out, a_s, w_s, out_s):
        _need(t.dtype == torch.bfloat16, "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if _epilogue(gate_up) == GATE_UP_SWIGLU else n_out),
          "expert weight shape does not fit")
    _need(w_s.shape == ((2 * n_out_s if gate_up else n_out_s), K_s) and a_s.shape[0] == T,
          "shared weight shape does not fit")
    _need(K % 8 == 0 and K_s % 8 == 0, "the reduction widths must be multiples of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, tile_rows)
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_dual", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i32(tile_rows), _i64(n_out), _i64(K),
          _ptr(a_s), _ptr(w_s), _ptr(out_s), _i32(T), _i64(n_out_s), _i64(K_s), _i32(1 if gate_up else 0),
          _f32(glu_limit), _f32(glu_limit_s), _stream())


_no_library_kernel = set()  # shapes that the vendor's library has no kernel for


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """out [T, N] = x [T, K] . w[N, K]^T, bfloat16 operands, 32-bit accumulation, out bfloat16 or float32, through the
    vendor library's C interface.  False if that library has no kernel for the shape: nothing was queued then."""
    T, K = x.shape
    N = w.shape[0]
    key = (T, N, K, out.dtype)
    if key in _no_library_kernel:
        return False
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32),
          "bfloat16 operands and a bfloat16 or float32 result")
    _need(w.dim() == 2 and w.shape[1] == K and out.shape == (T, N), "shapes do not fit")
    fn = _functions.get("ix_gemm_bf16")
    if fn is None:
        fn = _functions["ix_gemm_bf16"] = lib().ix_gemm_bf16
    rc = fn(_ptr(x), _ptr(w), _ptr(out), T, N, K, 1 if out.dtype == torch.float32 else 0, _stream())
    if rc == 2:
        _no_library_kernel.add(key)
        return False
    if rc != 0:
        raise KernelError(lib().ix_last_error().decode("utf-8", "replace"))
    return True


def linear_skinny_f32(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out float32 [T, N] = x [T, K] . w[N, K]^T for at most 64 rows, bfloat16 operands (the head of a decode step)."""
    T, K = x.shape
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.float32,
          "bfloat16 operands and a float32 result")
    _need(w.dim() == 2 and w.shape[1] == K and out.shape == (T, w.shape[0]), "shapes do not fit")
    _need(0 < T <= 64 and K % 8 == 0, "between 1 and 64 rows and a reduction width that is a multiple of 8")
    _call("ix_linear_skinny_f32", _ptr(x), _ptr(w), _ptr(out), _i32(T), _i64(w.shape[0]), _i64(K), _stream())


MOE_TILED_ROWS = 160  # rows per tile of the LDS-staged grouped product
MOE_TILED_ROWS_WIDE = 192  # ... of its wide form


def moe_tiled_rows(wide: bool) -> int:
    return MOE_TILED_ROWS_WIDE if wide else MOE_TILED_ROWS


def moe_grouped_tiled(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                      rows: Optional[torch.Tensor], tile_map: torch.Tensor, gate_up: bool, wide: bool = False,
                      glu_limit: float = 0.0) -> None:
    """Grouped product staged through LDS (bfloat16, many rows per expert); `tile_map` made for tiles of
    `moe_tiled_rows(wide)` rows.  `wide`: 256 instead of 128 weight rows per workgroup (the same sums in the same
    order; which rows share a tile, and with it where a row's sum starts, differs)."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if _epilogue(gate_up) == GATE_UP_SWIGLU else n_out),
          "expert weight shape does not fit")
    _need(K % 8 == 0, "the reduction width must be a multiple of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, moe_tiled_rows(wide))
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_tiled", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i64(a.shape[0]), _i64(n_out), _i64(K),
          _i32(_epilogue(gate_up)), _i32(1 if wide else 0), _f32(glu_limit), _stream())


def moe_grouped_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                      rows: Optional[torch.Tensor], gate_up: bool, glu_limit: float = 0.0) -> None:
    """Grouped product over device offsets.  gate_up: a [T, H] gathered through `rows`,
    w [E, 2n, H], out [A, n] = silu(gate) * up (with `glu_limit` > 0 the clamped form: gate = min(gate, limit),
    up = clamp(up, -limit, limit), gate * sigmoid(1.702 gate) * (up + 1)).  Otherwise a [A, K], w [E, n, K],
    out [A, n]."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if _epilogue(gate_up) == GATE_UP_SWIGLU else n_out),
          "expert weight shape does not fit")
    _need(out.dtype == a.dtype, "out must have the activations' dtype")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    _call("ix_moe_grouped_plain", _ptr(a), _i32(_dt(a)), _ptr(w), _i32(_dt(w)), _ptr(out), _ptr(offsets), _ptr(rows),
          _i64(A), _i32(E), _i64(n_out), _i64(K), _i32(_epilogue(gate_up)), _f32(glu_limit), _stream())


def moe_combine(y: torch.Tensor, dest: torch.Tensor, topk_w: torch.Tensor, shared: Optional[torch.Tensor],
                shared_gate: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[t] = sum_s topk_w[t, s] * y[dest[t, s]] (+ shared_gate[t] * shared[t])."""
    T, k = topk_w.shape
    H = y.shape[1]
    _need(out.shape == (T, H) and out.dtype == y.dtype, "out mismatch")
    _need(y.shape[0] >= T * k, "y has too few rows")
    _is_i32(dest, T * k)
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == y.dtype, "shared mismatch")
    _call("ix_moe_combine", _ptr(y), _i32(_dt(y)), _ptr(dest), _ptr(topk_w), _ptr(shared),
          _ptr(shared_gate if shared is not None else None), _ptr(out), _i64(T), _i64(H), _i32(k), _stream())


def moe_combine_add_rmsnorm(h: torch.Tensor, y: torch.Tensor, dest: torch.Tensor, topk_w: torch.Tensor,
                            shared: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor], weight: torch.Tensor,
                            out: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
                            sum_weight: Optional[torch.Tensor] = None, sum_eps: float = 0.0, groups: int = 1) -> None:
    """`moe_combine` followed by `add_rmsnorm` in one pass: h += sum; out = rmsnorm(h) * weight.  With `sum_weight`
    the sum passes an RMS norm of its own first: h += rmsnorm(sum, sum_eps) * sum_weight.  `groups`: the last norm
    runs over that many equal runs of the width, each with its own root mean square."""
    T, k = topk_w.shape
    H = h.shape[1]
    _need(h.dtype == torch.float32 and h.shape[0] == T, "the residual stream is float32 [T, H]")
    _need(y.shape[1] == H and y.shape[0] >= T * k and out.dtype == y.dtype and out.shape[1] == H, "shape mismatch")
    _need(weight.numel() == H and (sum_weight is None or sum_weight.numel() == H), "norm weight length differs")
    _is_i32(dest, T * k)
    n_out = out.shape[0]
    if rows is None:
        _need(n_out == T, "out must have a row per token")
    else:
        _is_i32(rows, n_out)
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == y.dtype, "shared mismatch")
    _call("ix_moe_combine_add_rmsnorm", _ptr(h), _ptr(y), _i32(_dt(y)), _ptr(dest), _ptr(topk_w), _ptr(shared),
          _ptr(shared_gate if shared is not None else None), _ptr(weight), _i32(_dt(weight)), _ptr(out), _ptr(rows),
          _i64(n_out), _i64(H), _i32(k), _f32(eps), _ptr(sum_weight),
          _i32(_dt(sum_weight) if sum_weight is not None else F32), _f32(sum_eps), _i32(groups), _stream())


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(out, R)
    if V > 4 * 4096 and R < 256:  # few long rows: two stages, so that they still fill the machine
        chunks = -(-V // 4096)
        part_v = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        part_i = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
        _call("ix_argmax_two_stage", _ptr(logits), _ptr(out), _ptr(part_v), _ptr(part_i), _i64(R), _i64(V), _stream())
        return
    _call("ix_argmax", _ptr(logits), _ptr(out), _i64(R), _i64(V), _stream())


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           top_k: torch.Tensor, min_p: torch.Tensor, rng_key: torch.Tensor, rng_counter: torch.Tensor,
           advance: bool = False) -> None:
    """Row r's draw is number rng_counter[r] of the stream rng_key[r]; with `advance` the kernel leaves
    rng_counter[r] + 1 there."""
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(out, R)
    _is_i32(top_k, R)
    for t in (temperature, top_p, min_p):
        _need(t.dtype == torch.float32 and t.numel() >= R, "sampling parameters must be float32 [rows]")
    for t in (rng_key, rng_counter):
        _need(t.dtype == torch.int64 and t.numel() >= R, "rng key and counter must be int64 [rows]")
    _call("ix_sample", _ptr(logits), _ptr(out), _ptr(temperature), _ptr(top_p), _ptr(top_k), _ptr(min_p),
          _ptr(rng_key), _ptr(rng_counter), _i32(1 if advance else 0), _i64(R), _i64(V), _stream())


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, chosen_lp: torch.Tensor, top_ids: torch.Tensor,
             top_lp: torch.Tensor) -> None:
    """Log-probability of each row's chosen token and of its n_top most probable tokens (n_top = top_ids.shape[1])."""
    R, V = logits.shape
    n_top = top_ids.shape[1]
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(chosen, R)
    _need(chosen_lp.dtype == torch.float32 and chosen_lp.numel() >= R, "chosen_lp must be float32 [rows]")
    _need(top_ids.shape == (R, n_top) and top_ids.dtype == torch.int32, "top_ids must be int32 [rows, n_top]")
    _need(top_lp.shape == (R, n_top) and top_lp.dtype == torch.float32, "top_lp must be float32 [rows, n_top]")
    _call("ix_logprobs", _ptr(logits), _ptr(chosen), _ptr(chosen_lp), _ptr(top_ids), _ptr(top_lp), _i64(R), _i64(V),
          _i32(n_top), _stream())


def apply_penalties(logits: torch.Tensor, hist_begin: torch.Tensor, hist_ids: torch.Tensor,
                    hist_counts: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor,
                    repetition: torch.Tensor, mask_begin: torch.Tensor, mask_ids: torch.Tensor) -> None:
    """In place on float32 logits [R, V]; histories and masks in CSR form (begin arrays hold R + 1 entries)."""
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    for t in (hist_begin, mask_begin):
        _is_i32(t, R + 1)
    for t in (hist_ids, hist_counts, mask_ids):
        _is_i32(t)
    for t in (presence, frequency, repetition):
        _need(t.dtype == torch.float32 and t.numel() >= R, "penalties must be float32 [rows]")
    _call("ix_apply_penalties", _ptr(logits), _ptr(hist_begin), _ptr(hist_ids), _ptr(hist_counts), _ptr(presence),
          _ptr(frequency), _ptr(repetition), _ptr(mask_begin), _ptr(mask_ids), _i64(R), _i64(V), _stream())


def measured_ceilings(device=None, read_bytes: int = 4 << 30) -> dict:
    """What this machine gives a kernel that only reads memory (GB/s, over a buffer far larger than any cache)
    and one that only issues bfloat16 matrix-core products (TFLOP/s): the measured ceilings that results are
    priced against beside the published peaks.  Takes a few tens of milliseconds and `read_bytes` of memory."""
    device = torch.device(device or "cuda:0")
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    buf = torch.empty(read_bytes // 4, dtype=torch.int32, device=device)
    buf.fill_(1)
    out = torch.zeros(1024, dtype=torch.int32, device=device)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = 0.0
    for blocks in (cus * 8, cus * 16, cus * 32):
        _call("ix_probe_read", _ptr(buf), _i64(read_bytes), _ptr(out), _i32(blocks), _i32(1), _stream())  # warm
        start.record()
        _call("ix_probe_read", _ptr(buf), _i64(read_bytes), _ptr(out), _i32(blocks), _i32(4), _stream())
        stop.record()
        stop.synchronize()
        best_read = max(best_read, 4 * read_bytes / (start.elapsed_time(stop) * 1e-3) / 1e9)
    del buf
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    flops = ctypes.c_double(0.0)
    best_mfma = 0.0
    for waves_per_simd in (2, 4):
        blocks, iters = cus * waves_per_simd, 100000
        _call("ix_probe_mfma", _i32(blocks), _i32(200), _ptr(sink), ctypes.byref(flops), _stream())  # warm
        start.record()
        _call("ix_probe_mfma", _i32(blocks), _i32(iters), _ptr(sink), ctypes.byref(flops), _stream())
        stop.record()
        stop.synchronize()
        best_mfma = max(best_mfma, flops.value / (start.elapsed_time(stop) * 1e-3) / 1e12)
    return {"hbm_read_gbs": round(best_read, 1), "mfma_bf16_tflops": round(best_mfma, 1)}


# ---------------------------------------------------------------------------
def _f32_vec(t: Optional[torch.Tensor], n: int, what: str):
    if t is None:
        return None
    _need(t.dtype == torch.float32 and t.numel() == n, f"{what} must hold {n} float32 numbers")
    return _ptr(t)


class ShiftOperands:
    """What a token shift needs of a step: the blend per channel (float32 [width]), the state [slots, width] and the
    step's index arrays on the device."""

    def __init__(self, mix, state, seq_of_token, q_start, state_slots, positions):
        self.mix, self.state = mix, state
        self.seq_of_token, self.q_start, self.state_slots, self.positions = seq_of_token, q_start, state_slots, positions

    def check(self, tokens: int, width: int) -> None:
        _need(self.mix.dtype == torch.float32 and self.mix.numel() == width, "the blend must be float32 [width]")
        _need(self.state.dtype == torch.float32 and self.state.dim() == 2 and self.state.shape[1] == width
              and self.state.is_contiguous(), "the state must be float32 [slots, width]")
        _is_i32(self.seq_of_token, tokens)
        _is_i32(self.positions, tokens)
        _is_i32(self.q_start)
        _is_i32(self.state_slots)
        _need(self.q_start.numel() == self.state_slots.numel() + 1, "q_start must hold one entry more than there are requests")


def add_dyt(h: torch.Tensor, delta: Optional[torch.Tensor], gain: Optional[torch.Tensor], weight: torch.Tensor,
            bias: Optional[torch.Tensor], alpha: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
            h_out: Optional[torch.Tensor] = None, shift: Optional[ShiftOperands] = None) -> None:
    """out = tanh(alpha * v) * weight + bias with v = h + gain * delta, optionally blended with the row before
    (`shift`).  v is written to `h_out` (h itself if not given) unless `rows` picks rows out; a shifted call needs
    an `h_out` that is not h."""
    H = h.shape[1]
    _need(h.dtype == torch.float32 and h.dim() == 2, "the residual stream is float32 [T, width]")
    _need(out.shape[1] == H, "width mismatch")
    n_out = out.shape[0]
    if rows is None:
        _need(n_out == h.shape[0], "out must have a row per row of h")
    else:
        _is_i32(rows, n_out)
    if delta is not None:
        _need(delta.shape == h.shape, "delta must have the shape of h")
    target = h if h_out is None else h_out
    _need(target.dtype == torch.float32 and target.shape == h.shape, "h_out must be float32 of the shape of h")
    if shift is not None:
        _need(rows is None, "a shifted call takes all rows")
        _need(target.data_ptr() != h.data_ptr(), "a shifted call cannot update the stream in place")
        shift.check(h.shape[0], H)
    write = delta is not None or target.data_ptr() != h.data_ptr()
    s = shift
    _call("ix_add_dyt", _ptr(h), _ptr(target) if (write and rows is None) else None, _ptr(delta),
          _i32(_dt(delta) if delta is not None else F32), _f32_vec(gain, H, "the gain"), _f32_vec(weight, H, "the weight"),
          _f32_vec(bias, H, "the bias"), _f32(alpha), _ptr(out), _i32(_dt(out)), _ptr(rows), _i64(n_out), _i64(H),
          _ptr(s.mix) if s else None, _ptr(s.state) if s else None, _ptr(s.seq_of_token) if s else None,
          _ptr(s.q_start) if s else None, _ptr(s.state_slots) if s else None, _ptr(s.positions) if s else None, _stream())


def token_shift(x: torch.Tensor, out: torch.Tensor, shift: ShiftOperands) -> None:
    """out[t] = x[t] + (x[t-1] - x[t]) * blend; the row before a request's first row comes from its state slot
    (zero at position 0), which is left holding the request's last row."""
    T, W = x.shape
    _need(out.shape == x.shape and out.dtype == x.dtype and out.data_ptr() != x.data_ptr(), "out must be another tensor like x")
    shift.check(T, W)
    _call("ix_token_shift", _ptr(x), _ptr(out), _i32(_dt(x)), _ptr(shift.mix), _ptr(shift.state), _ptr(shift.seq_of_token),
          _ptr(shift.q_start), _ptr(shift.state_slots), _ptr(shift.positions), _i64(T), _i64(W), _stream())


def scale_columns(x: torch.Tensor, gain: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = x[t, i] * gain[i]."""
    T, W = x.shape
    _need(out.shape == x.shape and out.dtype == x.dtype, "out must be like x")
    _call("ix_scale_columns", _ptr(x), _ptr(out), _i32(_dt(x)), _f32_vec(gain, W, "the gain"), _i64(T), _i64(W), _stream())


def _check_kv(q_dtype, k_cache, v_cache, kv_heads, head_dim, value_dim):
    _need(k_cache.dtype == q_dtype and v_cache.dtype == q_dtype, "cache dtype differs from the activations'")
    _need(k_cache.dim() == 4 and k_cache.shape[1] == kv_heads and k_cache.shape[3] == head_dim,
          "key cache must be [pages, kv_heads, page_size, head_dim]")
    _need(v_cache.shape == (k_cache.shape[0], kv_heads, value_dim, k_cache.shape[2]),
          "value cache must be [pages, kv_heads, value_dim, page_size]")


def qk_norm_append(qkv: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float,
                   v_first: Optional[torch.Tensor], blend: float, v_out: Optional[torch.Tensor],
                   slots: Optional[torch.Tensor], q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int, value_dim: int) -> None:
    """After the q|k|v product (rows of `qkv`, which may be longer than the three): RMS norm over all of a token's
    query numbers (`q_norm` float32 [heads * head_dim]) and over all of its key numbers, values blended with
    `v_first` (v = (1 - blend) v + blend v_first), written to `v_out` if given, queries to `q_out`, keys and
    values to the cache."""
    T, stride = qkv.shape
    qd, kd, vd = heads * head_dim, kv_heads * head_dim, kv_heads * value_dim
    _need(stride >= qd + kd + vd and qkv.is_contiguous(), "a row of the product is shorter than q, k and v together")
    _need(q_out.dtype == qkv.dtype and q_out.numel() == T * qd, "q_out mismatch")
    for t in (v_first, v_out):
        if t is not None:
            _need(t.dtype == qkv.dtype and t.numel() == T * vd and t.is_contiguous(), "values of another layer mismatch")
    page_size = 1
    if slots is not None:
        _need(k_cache is not None and v_cache is not None, "the cache is needed where slots are given")
        _check_kv(qkv.dtype, k_cache, v_cache, kv_heads, head_dim, value_dim)
        page_size = k_cache.shape[2]
        _is_i32(slots, T)
    _call("ix_qk_norm_append", _ptr(qkv), _i32(_dt(qkv)), _i64(stride), _f32_vec(q_norm, qd, "the query norm's weight"),
          _f32_vec(k_norm, kd, "the key norm's weight"), _f32(eps), _ptr(v_first), _f32(blend), _ptr(v_out), _ptr(slots),
          _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _i64(T), _i32(heads), _i32(kv_heads), _i32(head_dim),
          _i32(value_dim), _i32(page_size), _stream())


def attention_talk_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                         seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor,
                         talk: Optional[torch.Tensor], sink: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                         scale: float, window: int = 0) -> None:
    """Paged attention whose heads' scores are mixed before the softmax (`talk` float32 [heads, heads]), with a
    sink per head in the softmax (`sink` float32 [heads]) and a sigmoid gate per head on the result (`gate`
    [T, heads] in the activations' type, rows may be strided).  q [T, heads, head_dim], out [T, heads, value_dim]."""
    T, heads, d = q.shape
    kv_heads, vd = k_cache.shape[1], v_cache.shape[2]
    _need(out.shape == (T, heads, vd) and out.dtype == q.dtype, "out must be [T, heads, value_dim]")
    _check_kv(q.dtype, k_cache, v_cache, kv_heads, d, vd)
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        _need(gate.dtype == q.dtype and gate.shape == (T, heads) and gate.stride(1) == 1 and gate.is_cuda,
              "the gate must be [T, heads] in the activations' type")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _call("ix_attention_talk_plain", _ptr(q), _ptr(k_cache), _ptr(v_cache), _i32(_dt(q)), _ptr(block_table),
          _ptr(seq_of_token), _ptr(positions), _ptr(out),
          None if talk is None else _f32_vec(talk, heads * heads, "the mixing matrix"),
          None if sink is None else _f32_vec(sink, heads, "the sinks"), gate_ptr, _i64(gate_stride), _i64(T),
          _i32(heads), _i32(kv_heads), _i32(d), _i32(vd), _i32(k_cache.shape[2]), _i32(block_table.shape[1]),
          _f32(scale), _i32(window), _stream())


def attention_talk_mfma_heads_per_wave(heads: int, kv_heads: int, head_dim: int, value_dim: int, page_size: int) -> int:
    """How many heads a wavefront of `attention_talk_mfma` takes for these sizes; 0 if the kernel does not take them."""
    fn = _functions.get("ix_attention_talk_mfma_heads_per_wave")
    if fn is None:
        fn = _functions["ix_attention_talk_mfma_heads_per_wave"] = lib().ix_attention_talk_mfma_heads_per_wave
    return int(fn(heads, kv_heads, head_dim, value_dim, page_size))


def attention_talk_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                        tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, n_splits: int,
                        workspace: Optional[torch.Tensor], talk: Optional[torch.Tensor], sink: Optional[torch.Tensor],
                        gate: Optional[torch.Tensor], scale: float, heads_per_wave: int = 0) -> None:
    """`attention_talk_plain` on the matrix cores (bfloat16, no window).  `tiles` int32 [3, n_tiles]: request, first
    row and rows (at most 16) of each query tile; the keys of a tile are cut into `n_splits` slices, whose parts go
    through `workspace` (float32, T * heads * n_splits * (value_dim + 2) entries) when there are several."""
    T, heads, d = q.shape
    _need(q.dtype == torch.bfloat16, "the matrix-core attention kernel is bfloat16 only")
    kv_heads, vd = k_cache.shape[1], v_cache.shape[2]
    _need(out.shape == (T, heads, vd) and out.dtype == q.dtype, "out must be [T, heads, value_dim]")
    _check_kv(q.dtype, k_cache, v_cache, kv_heads, d, vd)
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(positions, T)
    _is_i32(tiles)
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    part_o = part_ml = None
    if n_splits > 1:
        need = T * heads * n_splits * (vd + 2)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"workspace of {need} float32 needed")
        part_o = workspace
        part_ml = workspace[T * heads * n_splits * vd:]
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        _need(gate.dtype == q.dtype and gate.shape == (T, heads) and gate.stride(1) == 1 and gate.is_cuda,
              "the gate must be [T, heads] in the activations' type")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _call("ix_attention_talk_mfma", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
          _ptr(tiles[1]), _ptr(tiles[2]), _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml),
          None if talk is None else _f32_vec(talk, heads * heads, "the mixing matrix"),
          None if sink is None else _f32_vec(sink, heads, "the sinks"), gate_ptr, _i64(gate_stride), _i64(T),
          _i32(tiles.shape[1]), _i32(n_splits), _i32(heads), _i32(kv_heads), _i32(d), _i32(vd), _i32(k_cache.shape[2]),
          _i32(block_table.shape[1]), _f32(scale), _i32(heads_per_wave), _stream())


# ---- layers that norm a branch's result as well, short convolutions, the delta rule, differential attention ------
def add_normed_rmsnorm(h: torch.Tensor, delta: torch.Tensor, delta_weight: torch.Tensor, delta_eps: float,
                       weight: Optional[torch.Tensor], out: Optional[torch.Tensor], eps: float,
                       rows: Optional[torch.Tensor] = None) -> None:
    """h += rmsnorm(delta) * delta_weight; out = rmsnorm(h) * weight, one pass.  With `rows`, out[r] comes from row
    rows[r] and h stays as it was.  `weight` and `out` None: only the sum."""
    H = h.shape[1]
    _need(h.dtype == torch.float32, "the residual stream is float32")
    _need(delta.shape == h.shape and delta_weight.numel() == H, "the branch's result must have the shape of h")
    _need((weight is None) == (out is None), "a following norm and its output come together")
    if out is not None:
        _need(weight.numel() == H and out.shape[1] == H, "width mismatch")
    n_out = h.shape[0] if out is None else out.shape[0]
    if rows is None:
        _need(n_out == h.shape[0], "out must have a row per row of h")
    else:
        _is_i32(rows, n_out)
    _call("ix_add_normed_rmsnorm", _ptr(h), _ptr(delta), _i32(_dt(delta)), _ptr(delta_weight), _i32(_dt(delta_weight)),
          _f32(delta_eps), _ptr(weight), _i32(_dt(weight) if weight is not None else F32), _f32(eps), _ptr(out),
          _i32(_dt(out) if out is not None else F32), _ptr(rows), _i64(n_out), _i64(H), _stream())


class StepRows:
    """Where the rows of a step belong: what a kernel that carries something from a request's last step needs."""

    def __init__(self, seq_of_token, q_start, state_slots):
        self.seq_of_token, self.q_start, self.state_slots = seq_of_token, q_start, state_slots

    def check(self, tokens: int) -> None:
        _is_i32(self.seq_of_token, tokens)
        _is_i32(self.q_start, 2)
        _is_i32(self.state_slots, self.q_start.numel() - 1)


def short_conv(x: torch.Tensor, bias: Optional[torch.Tensor], weight: torch.Tensor, state: torch.Tensor,
               rows: StepRows, sizes: Tuple[int, int, int, int, int], out_q: torch.Tensor,
               out_k: torch.Tensor, out_v: torch.Tensor, slots: Optional[torch.Tensor] = None,
               cos_sin: Optional[torch.Tensor] = None, silu: bool = False, weight_t: Optional[torch.Tensor] = None,
               bias_f32: Optional[torch.Tensor] = None) -> None:
    """A causal convolution of `taps` = weight.shape[1] taps over time on the first q + k + v channels of x
    [T, >= channels] (a bias added first), continued from `state` (a float32 view [slots, >= (taps - 1) * channels]
    of each request's last inputs, brought up to date), then silu and / or the rotation of the first
    2 * cos_sin.shape[1] elements of every q and k head.  `sizes` = (q channels, k channels, v channels, head_dim,
    value_dim).  With `slots` k and v go into the paged caches out_k [pages, k heads, page, head_dim] and out_v
    [pages, v heads, value_dim, page]; else to rows [T, k channels], [T, v channels].  q goes to out_q [T, q channels].
    `weight_t` float32 [taps, channels] and `bias_f32` float32 [channels]: the same numbers as `weight` and `bias`, laid
    out for the kernel's 16-byte form (used where the sizes come in eights)."""
    cq, ck, cv, d, vd = sizes
    T = x.shape[0]
    C = cq + ck + cv
    taps = weight.shape[1]
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= C and x.is_cuda, "x must be rows of at least q + k + v channels")
    _need(weight.shape == (C, taps) and (bias is None or bias.numel() == C), "one row of taps (and one bias) per channel")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= (taps - 1) * C, "the state must be float32 [slots, >= (taps - 1) * channels]")
    rows.check(T)
    _need(out_q.dtype == x.dtype and out_k.dtype == x.dtype and out_v.dtype == x.dtype, "results have the type of x")
    _need(out_q.numel() >= T * cq, "out_q too small")
    page_size = 0
    if slots is not None:
        _is_i32(slots, T)
        page_size = out_k.shape[2]
        _need(out_k.dim() == 4 and out_k.shape[1] * d == ck and out_k.shape[3] == d, "key cache must be [pages, k heads, page, head_dim]")
        _need(out_v.shape == (out_k.shape[0], cv // vd, vd, page_size), "value cache must be [pages, v heads, value_dim, page]")
    else:
        _need(out_k.numel() >= T * ck and out_v.numel() >= T * cv, "out_k or out_v too small")
    rot = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[0] == T and cos_sin.shape[2] == 2,
              "the rotation table must be float32 [T, pairs, 2]")
        rot = 2 * cos_sin.shape[1]
    if weight_t is not None:
        _need(weight_t.dtype == torch.float32 and weight_t.shape == (taps, C) and weight_t.is_contiguous(), "weight_t shape")
    if bias_f32 is not None:
        _need(bias_f32.dtype == torch.float32 and bias_f32.numel() == C and bias_f32.is_contiguous(), "bias_f32 shape")
    _call("ix_short_conv", x.data_ptr(), _i32(_dt(x)), _i64(x.stride(0)), _ptr(bias),
          _i32(_dt(bias) if bias is not None else F32), _ptr(weight), _i32(_dt(weight)), _i32(taps), state.data_ptr(),
          _i64(state.stride(0)), _ptr(rows.seq_of_token), _ptr(rows.q_start), _ptr(rows.state_slots), _ptr(cos_sin),
          _i32(rot), _i32(1 if silu else 0), _ptr(slots), _i32(page_size), _ptr(out_q), _ptr(out_k), _ptr(out_v),
          _i64(T), _i32(cq), _i32(ck), _i32(cv), _i32(d), _i32(vd), _ptr(weight_t), _ptr(bias_f32), _stream())


def delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, ab: torch.Tensor, a_log: torch.Tensor,
               dt_bias: torch.Tensor, state: torch.Tensor, rows: StepRows, out: torch.Tensor, heads: int,
               kv_heads: int, dim: int, vdim: int, channel_decays: Optional[torch.Tensor] = None) -> None:
    """The gated delta rule over the rows of a step, request by request, from and to `state` (a float32 view
    [slots, >= heads * dim * vdim]).  q, k [T, kv_heads * dim], v [T, heads * vdim] (rows may be strided);
    ab float32 [T, 2 heads]: the decay's and the step size's logits; out float32 [T, heads, vdim].
    `channel_decays` float32 [T, heads * dim]: a decay per key channel (the decays themselves, see
    `channel_decays`); ab is then float32 [T, heads], the step size's logits alone, and dt_bias is not read."""
    T = q.shape[0]
    channel_logits = channel_decays
    for t, n in ((q, kv_heads * dim), (k, kv_heads * dim), (v, heads * vdim)):
        _need(t.dim() == 2 and t.shape == (T, n) and t.stride(1) == 1 and t.dtype == q.dtype and t.is_cuda, "q, k or v shape")
    if channel_logits is None:
        _need(ab.dtype == torch.float32 and ab.shape == (T, 2 * heads) and ab.is_contiguous(), "ab must be float32 [T, 2 heads]")
    else:
        _need(ab.dtype == torch.float32 and ab.shape == (T, heads) and ab.is_contiguous(), "ab must be float32 [T, heads]")
        _need(channel_logits.dtype == torch.float32 and channel_logits.shape == (T, heads * dim)
              and channel_logits.is_contiguous(), "the decays must be float32 [T, heads * dim]")
    _need(a_log.dtype == torch.float32 and a_log.numel() == heads and dt_bias.dtype == torch.float32
          and (channel_logits is not None or dt_bias.numel() == heads) and dt_bias.is_contiguous(),
          "a_log and dt_bias must be float32 [heads]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= heads * dim * vdim, "the state must be float32 [slots, >= heads * dim * vdim]")
    _need(out.dtype == torch.float32 and out.shape == (T, heads, vdim), "out must be float32 [T, heads, vdim]")
    rows.check(T)
    S = rows.q_start.numel() - 1
    _call("ix_delta_rule", q.data_ptr(), k.data_ptr(), v.data_ptr(), _i32(_dt(q)), _i64(q.stride(0)), _i64(k.stride(0)),
          _i64(v.stride(0)), _ptr(ab), _ptr(channel_logits), _ptr(a_log), _ptr(dt_bias), state.data_ptr(), _i64(state.stride(0)),
          _ptr(rows.q_start), _ptr(rows.state_slots), _ptr(out), _i64(T), _i32(S), _i32(heads), _i32(kv_heads),
          _i32(dim), _i32(vdim), _stream())


def channel_decays(logits: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, heads: int, dim: int) -> None:
    """logits float32 [T, heads * dim] in place: exp(-exp(a_log[h]) softplus(logit + dt_bias[h, i])), the decay of
    every head's every key channel."""
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[1] == heads * dim and logits.is_contiguous(),
          "the logits must be float32 [T, heads * dim]")
    _need(a_log.dtype == torch.float32 and a_log.numel() == heads and dt_bias.dtype == torch.float32
          and dt_bias.numel() == heads * dim and dt_bias.is_contiguous(), "a_log float32 [heads], dt_bias float32 [heads * dim]")
    _call("ix_channel_decays", _ptr(logits), _ptr(a_log), _ptr(dt_bias), _i64(logits.shape[0]), _i32(heads), _i32(dim), _stream())


def matrix_memory_state_floats(heads: int, dim: int, vdim: int) -> int:
    """Floats of a request's state for `matrix_memory`: the matrices with n as one more column, then the maxima."""
    return heads * dim * (vdim + 1) + heads


def matrix_memory(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gates: torch.Tensor, gate_bias: torch.Tensor,
                  cap: float, state: torch.Tensor, rows: StepRows, out: torch.Tensor, nq: torch.Tensor,
                  work: torch.Tensor, heads: int, dim: int, vdim: int) -> None:
    """The matrix memory with exponential gates over the rows of a step, request by request, from and to `state` (a
    float32 view [slots, >= matrix_memory_state_floats(...)]: per head [vdim + 1, dim] with n as the last column, then
    the running maxima).  q, k [T, heads * dim], v [T, heads * vdim] (rows may be strided); gates float32 [T, 2 heads]
    (input gate's logits, then forget gate's), gate_bias float32 [2 heads].  Leaves out float32 [T, heads, vdim] =
    S^T q', nq float32 [T, heads] = n . q' and work float32 [T, heads, 3] = (keep, take, exp(-m')): the read-out is
    out / (max(|nq|, work[..., 2]) + 1e-6), which `head_norm_gate` forms on its way (`den_a`, `den_b`)."""
    T = q.shape[0]
    for t, n in ((q, heads * dim), (k, heads * dim), (v, heads * vdim)):
        _need(t.dim() == 2 and t.shape == (T, n) and t.stride(1) == 1 and t.dtype == q.dtype and t.is_cuda, "q, k or v shape")
    _need(gates.dtype == torch.float32 and gates.shape == (T, 2 * heads) and gates.is_contiguous(),
          "gates must be float32 [T, 2 heads]")
    _need(gate_bias.dtype == torch.float32 and gate_bias.numel() == 2 * heads and gate_bias.is_contiguous(),
          "gate_bias must be float32 [2 heads]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= matrix_memory_state_floats(heads, dim, vdim), "the state must be float32 [slots, >= matrices + maxima]")
    _need(out.dtype == torch.float32 and out.shape == (T, heads, vdim) and out.is_contiguous(), "out must be float32 [T, heads, vdim]")
    _need(nq.dtype == torch.float32 and nq.shape == (T, heads) and nq.is_contiguous(), "nq must be float32 [T, heads]")
    _need(work.dtype == torch.float32 and work.shape == (T, heads, 3) and work.is_contiguous(), "work must be float32 [T, heads, 3]")
    rows.check(T)
    S = rows.q_start.numel() - 1
    _call("ix_matrix_memory", q.data_ptr(), k.data_ptr(), v.data_ptr(), _i32(_dt(q)), _i64(q.stride(0)), _i64(k.stride(0)),
          _i64(v.stride(0)), _ptr(gates), _ptr(gate_bias), _f32(cap), state.data_ptr(), _i64(state.stride(0)),
          _ptr(rows.q_start), _ptr(rows.state_slots), _ptr(work), _ptr(out), _ptr(nq), _i64(T), _i32(S), _i32(heads),
          _i32(dim), _i32(vdim), _stream())


def head_norm_gate(x: torch.Tensor, out: torch.Tensor, eps: float, weight: Optional[torch.Tensor] = None,
                   gate: Optional[torch.Tensor] = None, x2: Optional[torch.Tensor] = None, lam: float = 0.0,
                   mult: float = 1.0, weight_per_head: bool = False, gate_sigmoid: bool = False,
                   den_a: Optional[torch.Tensor] = None, den_b: Optional[torch.Tensor] = None) -> None:
    """Per (token, head): o = x - lam * x2 (x2 optional); out = o / sqrt(mean(o^2) + eps) * weight * silu(gate) * mult.
    x, x2 float32 [T, heads, vdim]; weight [vdim] (`weight_per_head`: [heads, vdim]); `gate_sigmoid`: sigmoid(gate)
    instead of silu(gate); gate [T, >= heads * vdim] (rows may be strided) and out
    [T, heads * vdim] of the run's type.  `den_a` float32 [T, heads] with `den_b` float32 [T, heads] (a view with any
    stride between its numbers): x is first divided by max(|den_a|, den_b) + 1e-6."""
    T, heads, vdim = x.shape
    stride_b = 0
    if den_a is not None:
        _need(den_a.dtype == torch.float32 and den_a.shape == (T, heads) and den_a.is_contiguous(), "den_a must be float32 [T, heads]")
        _need(den_b is not None and den_b.dtype == torch.float32 and den_b.shape == (T, heads) and den_b.is_cuda
              and (T == 0 or den_b.stride(0) == heads * den_b.stride(1)), "den_b must be float32 [T, heads], evenly strided")
        stride_b = den_b.stride(1)
    _need(x.dtype == torch.float32 and (x2 is None or (x2.dtype == torch.float32 and x2.shape == x.shape)), "x, x2 float32")
    _need(out.shape == (T, heads * vdim), "out must be [T, heads * vdim]")
    _need(weight is None or weight.numel() == (heads * vdim if weight_per_head else vdim),
          "one weight per value column (of every head, with weight_per_head)")
    stride = 0
    if gate is not None:
        _need(gate.dim() == 2 and gate.shape == (T, heads * vdim) and gate.stride(1) == 1 and gate.dtype == out.dtype
              and gate.is_cuda, "gate must be rows of heads * vdim of out's type")
        stride = gate.stride(0)
    _call("ix_head_norm_gate", _ptr(x), _ptr(x2), _f32(lam), _ptr(weight), _i32(_dt(weight) if weight is not None else F32),
          gate.data_ptr() if gate is not None else None, _i64(stride), _ptr(out), _i32(_dt(out)), _i64(T), _i32(heads),
          _i32(vdim), _f32(eps), _f32(mult), _i32(1 if weight_per_head else 0), _i32(1 if gate_sigmoid else 0),
          _ptr(den_a), den_b.data_ptr() if den_a is not None else None, _i32(stride_b), _stream())


def attention_diff_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                         seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float,
                         window: int, keep_first: int, lam: float, eps: float, mult: float) -> None:
    """Differential attention, one workgroup per (token, head): q [T, heads, 2, d], keys [pages, 2 kv_heads, page, d],
    values [pages, kv_heads, vd, page], out [T, heads, vd] = rmsnorm(a_0 - lam a_1) * mult."""
    T, heads, two, d = q.shape
    _need(two == 2 and q.is_contiguous(), "q must be [T, heads, 2, d]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and out.dtype == q.dtype, "dtype mismatch")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == d and k_cache.shape[1] % 2 == 0, "key cache must be [pages, 2 kv_heads, page, d]")
    kv_heads, page_size = k_cache.shape[1] // 2, k_cache.shape[2]
    _need(v_cache.dim() == 4 and v_cache.shape[0] == k_cache.shape[0] and v_cache.shape[1] == kv_heads
          and v_cache.shape[3] == page_size, "value cache must be [pages, kv_heads, vd, page]")
    vd = v_cache.shape[2]
    _need(out.shape == (T, heads, vd), "out must be [T, heads, vd]")
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    _call("ix_attention_diff_plain", _ptr(q), _ptr(k_cache), _ptr(v_cache), _i32(_dt(q)), _ptr(block_table),
          _ptr(seq_of_token), _ptr(positions), _ptr(out), _i64(T), _i32(heads), _i32(kv_heads), _i32(d), _i32(vd),
          _i32(page_size), _i32(block_table.shape[1]), _f32(scale), _i32(window), _i32(keep_first), _f32(lam),
          _f32(eps), _f32(mult), _stream())


def attention_diff_mfma_fits(head_dim: int, value_dim: int, page_size: int) -> bool:
    """Whether the matrix-core kernel of differential attention is built for these sizes."""
    return bool(lib().ix_attention_diff_mfma_fits(int(head_dim), int(value_dim), int(page_size)))


def attention_diff_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                        tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, n_splits: int,
                        workspace: torch.Tensor, scale: float, window: int, keep_first: int, lam: float, eps: float,
                        mult: float, grouped: bool = False) -> None:
    """Differential attention on the matrix cores (bfloat16), shapes as `attention_diff_plain`.  `tiles` int32
    [3, n_tiles]: request, first token row and rows (at most 16) of every tile; the keys that a tile reads are cut into
    `n_splits` slices; `workspace` float32 of T * heads * 2 * n_splits * (vd + 2) numbers.  `grouped`: every tile is
    one token, and the query heads of a key/value head (at most 16) are served side by side."""
    T, heads, two, d = q.shape
    _need(two == 2 and q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "bfloat16 q [T, heads, 2, d]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache dtype differs from q")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == d and k_cache.shape[1] % 2 == 0, "key cache must be [pages, 2 kv_heads, page, d]")
    kv_heads, page_size = k_cache.shape[1] // 2, k_cache.shape[2]
    _need(v_cache.dim() == 4 and v_cache.shape[0] == k_cache.shape[0] and v_cache.shape[1] == kv_heads
          and v_cache.shape[3] == page_size, "value cache must be [pages, kv_heads, vd, page]")
    vd = v_cache.shape[2]
    _need(out.shape == (T, heads, vd), "out must be [T, heads, vd]")
    _need(attention_diff_mfma_fits(d, vd, page_size), "sizes that the matrix-core kernel is not built for")
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    _is_i32(tiles)
    _is_i32(block_table)
    _is_i32(positions, T)
    n_tiles = tiles.shape[1]
    parts = T * heads * 2 * n_splits
    _need(workspace.dtype == torch.float32 and workspace.numel() >= parts * (vd + 2), "workspace too small")
    _call("ix_attention_diff_mfma", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]), _ptr(tiles[1]),
          _ptr(tiles[2]), _ptr(positions), _ptr(out), workspace.data_ptr(), workspace.data_ptr() + 4 * parts * vd,
          _i64(T), _i32(n_tiles), _i32(n_splits), _i32(heads), _i32(kv_heads), _i32(d), _i32(vd), _i32(page_size),
          _i32(block_table.shape[1]), _f32(scale), _i32(window), _i32(keep_first), _f32(lam), _f32(eps), _f32(mult),
          _i32(1 if grouped else 0), _stream())


# ---- a gated product's activation with biases and limits; two branches added to the stream ---------------------
def glu_bias(gate_up: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, limit: float = 0.0) -> None:
    """out[t, i] = glu(gate_up[t, i] + bias[i], gate_up[t, W + i] + bias[W + i]); glu(g, u) = silu(g) * u, or with
    `limit` > 0 the clamped form g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit)."""
    T, W2 = gate_up.shape
    _need(W2 % 2 == 0 and out.shape == (T, W2 // 2) and out.dtype == gate_up.dtype, "shape or dtype mismatch")
    _need(bias is None or bias.numel() == W2, "the bias holds the gate's numbers, then the up's")
    _call("ix_glu_bias", _ptr(gate_up), _ptr(bias), _i32(_dt(bias) if bias is not None else F32), _ptr(out),
          _i32(_dt(out)), _i64(T), _i64(W2 // 2), _f32(limit), _stream())


def add_branches(h: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None) -> None:
    """h [T, W] float32 += a + b + bias (b and bias optional), summed in float32."""
    _need(h.dtype == torch.float32 and h.dim() == 2, "the residual stream is float32 [T, W]")
    _need(a.shape == h.shape and (b is None or (b.shape == h.shape and b.dtype == a.dtype)), "the branches have h's shape")
    _need(bias is None or bias.numel() == h.shape[1], "one bias per column")
    _call("ix_add_branches", _ptr(h), _ptr(a), _ptr(b), _i32(_dt(a)), _ptr(bias),
          _i32(_dt(bias) if bias is not None else F32), _i64(h.shape[0]), _i64(h.shape[1]), _stream())


# ---- recurrent mixers with a matrix of state per head ---------------------------------------------------------------
def linear_state(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, rows: StepRows,
                 out: torch.Tensor, heads: int, dim: int, vdim: int, w_rows: Optional[torch.Tensor] = None,
                 w_head: Optional[torch.Tensor] = None, a_rows: Optional[torch.Tensor] = None,
                 b_rows: Optional[torch.Tensor] = None, silu: bool = False) -> None:
    """S <- diag(w) S - a (b^T S) + k v^T;  o = S^T r, over the rows of a step, request by request, from and to
    `state` (a float32 view [slots, >= heads * vdim * dim], a head's matrix kept [vdim][dim]).  r, k [T, heads * dim],
    v [T, heads * vdim] of the run's type (rows may be strided), through silu first if `silu`.  The decay w comes per
    row and key channel (`w_rows` float32 [T, heads * dim]) or per head (`w_head` float32 [heads]); the correction's
    vectors `a_rows`, `b_rows` (float32 [T, heads * dim]) come together or not at all.  out float32 [T, heads, vdim]."""
    T = r.shape[0]
    for t, n in ((r, heads * dim), (k, heads * dim), (v, heads * vdim)):
        _need(t.dim() == 2 and t.shape == (T, n) and t.stride(1) == 1 and t.dtype == r.dtype and t.is_cuda, "r, k or v shape")
    for t in (w_rows, a_rows, b_rows):
        _need(t is None or (t.dtype == torch.float32 and t.shape == (T, heads * dim) and t.is_contiguous()),
              "the rows of decays and corrections must be float32 [T, heads * dim]")
    _need((w_rows is None) != (w_head is None), "the decay comes per row and channel or per head")
    _need(w_head is None or (w_head.dtype == torch.float32 and w_head.numel() == heads), "w_head must be float32 [heads]")
    _need((a_rows is None) == (b_rows is None), "the correction's two vectors come together")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= heads * dim * vdim, "the state must be float32 [slots, >= heads * dim * vdim]")
    _need(out.dtype == torch.float32 and out.shape == (T, heads, vdim) and out.is_contiguous(), "out must be float32 [T, heads, vdim]")
    rows.check(T)
    S = rows.q_start.numel() - 1
    _call("ix_linear_state", r.data_ptr(), k.data_ptr(), v.data_ptr(), _i32(_dt(r)), _i64(r.stride(0)), _i64(k.stride(0)),
          _i64(v.stride(0)), _ptr(w_rows), _ptr(w_head), _ptr(a_rows), _ptr(b_rows), state.data_ptr(),
          _i64(state.stride(0)), _ptr(rows.q_start), _ptr(rows.state_slots), _ptr(out), _i64(T), _i32(S), _i32(heads),
          _i32(dim), _i32(vdim), _i32(1 if silu else 0), _stream())


def delta_operands(w_logit: torch.Tensor, w_bias: torch.Tensor, a_logit: torch.Tensor, a_bias: torch.Tensor,
                   k: torch.Tensor, w: torch.Tensor, a: torch.Tensor, u: torch.Tensor, heads: int, dim: int,
                   decay_scale: float, unit_eps: float) -> None:
    """Per token, head and key channel, float32 [T, heads * dim]: w = exp(-decay_scale sigmoid(w_logit + w_bias)),
    u = k / sqrt(sum over the head of k^2 + unit_eps), a = sigmoid(a_logit + a_bias) u.  w_logit float32; a_logit and
    k of the run's type (rows may be strided)."""
    T, C = w_logit.shape
    _need(C == heads * dim and w_logit.dtype == torch.float32 and w_logit.is_contiguous(), "w_logit must be float32 [T, heads * dim]")
    for t in (a_logit, k):
        _need(t.dim() == 2 and t.shape == (T, C) and t.stride(1) == 1 and t.dtype == k.dtype and t.is_cuda, "a_logit or k shape")
    _need(w_bias.numel() == C and a_bias.numel() == C, "one bias per channel")
    for t in (w, a, u):
        _need(t.dtype == torch.float32 and t.shape == (T, C) and t.is_contiguous(), "results are float32 [T, heads * dim]")
    _call("ix_delta_operands", _ptr(w_logit), _ptr(w_bias), _i32(_dt(w_bias)), a_logit.data_ptr(), _i64(a_logit.stride(0)),
          _ptr(a_bias), _i32(_dt(a_bias)), k.data_ptr(), _i64(k.stride(0)), _i32(_dt(k)), _ptr(w), _ptr(a), _ptr(u),
          _i64(T), _i32(heads), _i32(dim), _f32(decay_scale), _f32(unit_eps), _stream())


def tanh_(x: torch.Tensor) -> None:
    """x = tanh(x) in place, float32."""
    _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be float32")
    _call("ix_tanh_inplace", _ptr(x), _i64(x.numel()), _stream())


# ---- attention over a compressed cache ------------------------------------------------------------------------------
def latent_prepare(q: torch.Tensor, dkv: torch.Tensor, norm_w: torch.Tensor, eps: float,
                   cos_sin: Optional[torch.Tensor], slots: Optional[torch.Tensor], cache: torch.Tensor, heads: int,
                   rot_dim: int, rank: int, halves: bool = False) -> None:
    """Per token: the last `rot_dim` numbers of every head of q [T, heads * q_dim] are rotated in place (pairs
    (2i, 2i + 1), i < cos_sin.shape[1]; float32 table [T, pairs, 2]; with `halves` the pairs (i, i + pairs)); the first `rank` numbers of the dkv row pass an
    RMS norm with `norm_w` (float32 sums), its last rot_dim are rotated likewise, and [c | kr] goes to row slots[t] of
    `cache` [pages, 1, page_size, rank + rot_dim]."""
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.is_cuda and q.shape[1] % heads == 0, "q must be rows of heads * q_dim")
    q_dim = q.shape[1] // heads
    _need(dkv.dim() == 2 and dkv.shape[0] == T and dkv.shape[1] >= rank + rot_dim and dkv.stride(1) == 1
          and dkv.dtype == q.dtype and dkv.is_cuda, "dkv must be rows of at least rank + rot_dim numbers of q's type")
    _need(norm_w.numel() == rank, "one norm weight per latent number")
    pairs = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[0] == T and cos_sin.shape[2] == 2
              and cos_sin.is_contiguous(), "the rotation table must be float32 [T, pairs, 2]")
        pairs = cos_sin.shape[1]
    _need(2 * pairs <= rot_dim <= q_dim, "the rotated pairs must fit into the rotated part")
    _need(cache.dtype == q.dtype and cache.dim() == 4 and cache.shape[1] == 1 and cache.shape[3] == rank + rot_dim
          and cache.is_contiguous(), "the cache must be [pages, 1, page_size, rank + rot_dim] of q's type")
    if slots is not None:
        _is_i32(slots, T)
    _call("ix_latent_prepare", q.data_ptr(), _i64(q.stride(0)), dkv.data_ptr(), _i64(dkv.stride(0)), _i32(_dt(q)), _ptr(norm_w),
          _i32(_dt(norm_w)), _f32(eps), _ptr(cos_sin), _i32(pairs), _ptr(slots), _ptr(cache), _i64(T), _i32(heads),
          _i32(q_dim), _i32(rot_dim), _i32(rank), _i32(1 if halves else 0), _stream())


def _head_rows(t: torch.Tensor, tokens: int, heads: int, n: int, what: str):
    """(token stride, head stride) of a tensor indexed [token, head, i] whose last dimension is dense."""
    _need(t.dim() == 3 and t.shape[0] == tokens and t.shape[1] == heads and t.shape[2] >= n and t.stride(2) == 1
          and t.is_cuda, f"{what} must be indexed [token, head, i] with a dense last dimension")
    return t.stride(0), t.stride(1)


def latent_attention_plain(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                           seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, rank: int,
                           rot_dim: int, scale: float, window: int = 0) -> None:
    """Causal attention of queries [token, head] over cached rows [c | kr]: score = (q_lat . c + q_rot . kr) * scale,
    softmax in float32, out = sum of weights * c.  `window` W > 0: a query reads its own and the W - 1 rows before.  q_lat, out [token, head, rank] and q_rot [token, head, rot_dim] are
    views with any token and head strides; cache [pages, 1, page_size, rank + rot_dim]."""
    T, heads = q_lat.shape[0], q_lat.shape[1]
    ql_t, ql_h = _head_rows(q_lat, T, heads, rank, "q_lat")
    qr_t, qr_h = _head_rows(q_rot, T, heads, rot_dim, "q_rot")
    o_t, o_h = _head_rows(out, T, heads, rank, "out")
    _need(q_rot.dtype == q_lat.dtype and out.dtype == q_lat.dtype and cache.dtype == q_lat.dtype, "one element type")
    _need(cache.dim() == 4 and cache.shape[1] == 1 and cache.shape[3] == rank + rot_dim and cache.is_contiguous(),
          "the cache must be [pages, 1, page_size, rank + rot_dim]")
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    _call("ix_latent_attention_plain", q_lat.data_ptr(), _i64(ql_t), _i64(ql_h), q_rot.data_ptr(), _i64(qr_t), _i64(qr_h),
          _ptr(cache), _i32(_dt(q_lat)), _ptr(block_table), _ptr(seq_of_token), _ptr(positions), out.data_ptr(),
          _i64(o_t), _i64(o_h), _i64(T), _i32(heads), _i32(rank), _i32(rot_dim), _i32(cache.shape[2]),
          _i32(block_table.shape[1]), _f32(scale), _i32(window), _stream())


LATENT_MFMA_MAX_SPLITS = 32


def latent_mfma_fits(q_lat: torch.Tensor, q_rot: torch.Tensor, out: torch.Tensor, rank: int, rot_dim: int) -> bool:
    """Whether the matrix-core kernel takes these operands: bfloat16, rank + rot_dim a multiple of 32 up to 576, rank a
    multiple of 16 up to 512, queries on 16-byte and results on 8-byte boundaries."""
    width = rank + rot_dim
    if q_lat.dtype != torch.bfloat16 or width % 32 or rank % 16 or width > 576 or rank > 512:
        return False
    if q_lat.stride(2) != 1 or out.stride(2) != 1 or (rot_dim and q_rot.stride(2) != 1):
        return False
    if (q_lat.data_ptr() | q_rot.data_ptr()) % 16 or out.data_ptr() % 8:
        return False
    return not ((q_lat.stride(0) | q_lat.stride(1) | q_rot.stride(0) | q_rot.stride(1)) % 8
                or (out.stride(0) | out.stride(1)) % 4)


def latent_mfma_splits(tokens: int, heads: int) -> int:
    """Into how many slices a step of one token per request cuts every request's keys: enough workgroups for the
    compute units, whatever the contexts (a captured step keeps its number)."""
    return max(1, min(LATENT_MFMA_MAX_SPLITS, 256 // (tokens * (-(-heads // 64)))))


def latent_attention_mfma(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                          seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, rank: int,
                          rot_dim: int, scale: float, one_token_each: bool = False, n_splits: int = 1,
                          work: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, window: int = 0) -> None:
    """`latent_attention_plain` on the matrix cores (see `latent_mfma_fits`).  `one_token_each`: every request brings
    one token; its keys may then be cut into `n_splits` slices, with `work` = float32 ([T * heads * n_splits, rank],
    [T * heads * n_splits, 2]) and a contiguous `out` [T, heads, rank]."""
    T, heads = q_lat.shape[0], q_lat.shape[1]
    ql_t, ql_h = _head_rows(q_lat, T, heads, rank, "q_lat")
    qr_t, qr_h = _head_rows(q_rot, T, heads, rot_dim, "q_rot")
    o_t, o_h = _head_rows(out, T, heads, rank, "out")
    _need(latent_mfma_fits(q_lat, q_rot, out, rank, rot_dim), "sizes or alignment that the matrix-core kernel does not take")
    _need(q_rot.dtype == q_lat.dtype and out.dtype == q_lat.dtype and cache.dtype == q_lat.dtype, "one element type")
    _need(cache.dim() == 4 and cache.shape[1] == 1 and cache.shape[3] == rank + rot_dim and cache.is_contiguous(),
          "the cache must be [pages, 1, page_size, rank + rot_dim]")
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    _need(n_splits == 1 or one_token_each, "keys are cut into slices for single tokens only")
    part_o = part_ml = None
    if n_splits > 1:
        part_o, part_ml = work
        _need(part_o.dtype == torch.float32 and part_o.numel() >= T * heads * n_splits * rank and part_o.is_contiguous()
              and part_ml.dtype == torch.float32 and part_ml.numel() >= T * heads * n_splits * 2
              and part_ml.is_contiguous() and out.is_contiguous(), "the slices' workspace or a result that is not contiguous")
    _call("ix_latent_attention_mfma", q_lat.data_ptr(), _i64(ql_t), _i64(ql_h), q_rot.data_ptr(), _i64(qr_t), _i64(qr_h),
          _ptr(cache), _ptr(block_table), _ptr(seq_of_token), _ptr(positions), out.data_ptr(), _i64(o_t), _i64(o_h),
          _ptr(part_o), _ptr(part_ml), _i32(n_splits), _i64(T), _i32(heads), _i32(rank), _i32(rot_dim),
          _i32(cache.shape[2]), _i32(block_table.shape[1]), _f32(scale), _i32(1 if one_token_each else 0), _i32(window),
          _stream())
