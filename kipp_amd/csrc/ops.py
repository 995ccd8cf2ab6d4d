"""Python bindings of the HIP kernels: shape and type checks on the host, then
one launch on torch's current stream.  Every function fails loudly when its
library cannot be built or loaded, or when there is no GPU; there is no CPU
path behind any of them.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from . import build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_c_int, _c_float, _c_size, _c_ptr = ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_void_p


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


# The helpers below run a few hundred times in a step that is not replayed as a graph, so they
# are kept cheap: plain integers for pointers, the raw stream handle, one dictionary lookup for a
# kernel's entry point.

def _ptr(t: Optional[torch.Tensor]):
    return t.data_ptr() if t is not None else None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """torch's current stream of the current device (also the one a graph is recorded on)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise KernelError("kernel operand is not on the GPU (there is no CPU path)" if not t.is_cuda
                              else "kernel operand is not contiguous")


def _i32(t: torch.Tensor, name: str) -> None:
    _need(t.dtype == torch.int32, f"{name} must be int32, got {t.dtype}")


_entry_points = {}


def _fn(lib_name: str, fn_name: str, argtypes, defines=None):
    key = (lib_name, fn_name, tuple(sorted(defines.items())) if defines else None)
    fn = _entry_points.get(key)
    if fn is None:
        fn = getattr(build.library(lib_name, defines), fn_name)
        fn.argtypes = argtypes
        fn.restype = _c_int
        _entry_points[key] = fn
    return fn


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise KernelError(f"{what}: launch failed or arguments refused (code {rc})")


# --------------------------------------------------------------------------- elementwise

def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(table, tokens, out)
    _i32(tokens, "tokens")
    n, hidden = out.shape
    _need(table.dim() == 2 and table.shape[1] == hidden, "embed: table width differs from output width")
    _need(tokens.numel() == n and out.dtype == torch.float32, "embed: one float32 output row per token")
    fn = _fn("elementwise", "kipp_embed", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(table), _code(table), _ptr(tokens), _ptr(out), n, hidden, _stream()), "embed")
    return out


def embed_scaled(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float) -> torch.Tensor:
    """out[t] = table[tokens[t]] * scale, in float32."""
    _dev(table, tokens, out)
    _i32(tokens, "tokens")
    n, hidden = out.shape
    _need(table.dim() == 2 and table.shape[1] == hidden, "embed: table width differs from output width")
    _need(tokens.numel() == n and out.dtype == torch.float32, "embed: one float32 output row per token")
    fn = _fn("elementwise", "kipp_embed_scaled", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_ptr])
    _check(fn(_ptr(table), _code(table), _ptr(tokens), _ptr(out), n, hidden, float(scale), _stream()), "embed_scaled")
    return out


def scaled_add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], alpha: float, weight: torch.Tensor, eps: float,
                       rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x <- rmsnorm(alpha * x + delta) * weight in place (float32); `rows`, if given, receives the same rows in its
    own type.  `delta` is [rows, width], or slabs [parts, rows, width] that are added in order, or None."""
    _dev(x, weight, delta, rows)
    n, width = x.shape
    _need(x.dtype == torch.float32 and weight.dtype == torch.float32, "scaled_add_rmsnorm: x and weight are float32")
    _need(weight.numel() == width and (rows is None or rows.shape == x.shape), "scaled_add_rmsnorm: shapes differ")
    parts = 0
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == tuple(x.shape) and delta.dim() in (2, 3), "scaled_add_rmsnorm: delta shape differs from x")
        parts = delta.shape[0] if delta.dim() == 3 else 1
    fn = _fn("elementwise", "kipp_scaled_add_rmsnorm",
             [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_float, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), _code(delta) if delta is not None else F32, parts, _ptr(weight), _ptr(rows),
              _code(rows) if rows is not None else F32, n, width, float(eps), float(alpha), _stream()), "scaled_add_rmsnorm")
    return x


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = rmsnorm(x [+ delta]) * weight; with `delta`, x += delta in place.
    `delta` is [rows, width] or, in slabs that are added in order, [parts, rows, width]."""
    _dev(x, weight, out, delta)
    rows, width = x.shape
    _need(x.dtype == torch.float32 and weight.dtype == torch.float32, "rmsnorm: x and weight are float32")
    _need(weight.numel() == width and out.shape == x.shape, "rmsnorm: shapes differ")
    parts = 1
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == tuple(x.shape) and delta.dim() in (2, 3), "rmsnorm: delta shape differs from x")
        parts = delta.shape[0] if delta.dim() == 3 else 1
    fn = _fn("elementwise", "kipp_rmsnorm",
             [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), _code(delta) if delta is not None else F32, parts, _ptr(weight), _ptr(out),
              _code(out), rows, width, float(eps), _stream()), "rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(x, delta)
    _need(x.dtype == torch.float32 and tuple(delta.shape[-2:]) == tuple(x.shape) and delta.dim() in (2, 3),
          "residual_add: float32 x and a delta of its shape (or slabs of it)")
    parts = delta.shape[0] if delta.dim() == 3 else 1
    fn = _fn("elementwise", "kipp_residual_add", [_c_ptr, _c_ptr, _c_int, _c_int, _c_size, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), _code(delta), parts, x.numel(), _stream()), "residual_add")
    return x


def residual_add_scaled(x: torch.Tensor, delta: torch.Tensor, scale: float = 1.0, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += scale * (delta + bias): `delta` float32 of x's shape or slabs of it (added in order), `bias` float32 [width] or none."""
    _dev(x, delta, bias)
    _need(x.dtype == delta.dtype == torch.float32 and x.dim() == 2 and tuple(delta.shape[-2:]) == tuple(x.shape) and delta.dim() in (2, 3),
          "residual_add_scaled: float32 x [rows, width] and a float32 delta of its shape (or slabs of it)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == x.shape[1]), "residual_add_scaled: float32 bias [width]")
    parts = delta.shape[0] if delta.dim() == 3 else 1
    fn = _fn("elementwise", "kipp_residual_add_scaled", [_c_ptr, _c_ptr, _c_int, _c_size, _c_float, _c_ptr, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), parts, x.numel(), float(scale), _ptr(bias), x.shape[1], _stream()), "residual_add_scaled")
    return x


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, pairs: bool = False) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, inner + i]; `gate_up` is
    [rows, 2 inner] or slabs [parts, rows, 2 inner] that are added in order.
    `pairs`: the columns come in tiles of 16, 8 gates over the 8 matching ups
    (a product from `tile_weight_pairs`), 16 ceil(inner / 8) of them a row."""
    _dev(gate_up, out)
    rows, inner = out.shape
    width = 16 * ((inner + 7) // 8) if pairs else 2 * inner
    _need(tuple(gate_up.shape[-2:]) == (rows, width) and gate_up.dim() in (2, 3), "swiglu: input must be [rows, 2 * inner]")
    parts = gate_up.shape[0] if gate_up.dim() == 3 else 1
    fn = _fn("elementwise", "kipp_swiglu", [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(gate_up), _code(gate_up), parts, _ptr(out), _code(out), rows, inner, int(pairs), _stream()), "swiglu")
    return out


def scale_values(x: torch.Tensor, scale: float) -> torch.Tensor:
    """x *= scale in place (float32)."""
    _dev(x)
    _need(x.dtype == torch.float32, "scale_values: float32")
    fn = _fn("elementwise", "kipp_scale_values", [_c_ptr, _c_float, _c_size, _c_ptr])
    _check(fn(_ptr(x), float(scale), x.numel(), _stream()), "scale_values")
    return x


def cast(src: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(src, out)
    _need(src.numel() == out.numel(), "cast: sizes differ")
    fn = _fn("elementwise", "kipp_cast", [_c_ptr, _c_int, _c_ptr, _c_int, _c_size, _c_ptr])
    _check(fn(_ptr(src), _code(src), _ptr(out), _code(out), src.numel(), _stream()), "cast")
    return out


def gather_rows(x: torch.Tensor, index: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[i] = x[index[i]] for rows of float32 or int32 [n, width], copied bit for bit."""
    _dev(x, index, out)
    _i32(index, "index")
    _need(x.dtype == out.dtype and x.dtype in (torch.float32, torch.int32) and x.dim() == 2, "gather_rows: rows of float32 or int32")
    _need(out.shape == (index.numel(), x.shape[1]), "gather_rows: output shape")
    fn = _fn("elementwise", "kipp_gather_rows", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(index), _ptr(out), index.numel(), x.shape[1], _stream()), "gather_rows")
    return out


def copy(src: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = src, bit for bit, for contiguous tensors of one type and size whose bytes are whole 4-byte words."""
    _dev(src, out)
    nbytes = src.numel() * src.element_size()
    _need(src.dtype == out.dtype and src.numel() == out.numel() and nbytes % 4 == 0, "copy: same type and size, whole words")
    fn = _fn("elementwise", "kipp_copy_words", [_c_ptr, _c_ptr, _c_size, _c_ptr])
    _check(fn(_ptr(src), _ptr(out), nbytes // 4, _stream()), "copy")
    return out


def fill_zero(out: torch.Tensor) -> torch.Tensor:
    """out[...] = 0 by a kernel (no memset node when a graph records it)."""
    _dev(out)
    nbytes = out.numel() * out.element_size()
    _need(nbytes % 4 == 0, "fill_zero: whole 4-byte words")
    fn = _fn("elementwise", "kipp_fill_zero", [_c_ptr, _c_size, _c_ptr])
    _check(fn(_ptr(out), nbytes // 4, _stream()), "fill_zero")
    return out


# --------------------------------------------------------------------------- attention

def _angles_ok(angles, n_tokens: int, rotary_dim: int, what: str) -> None:
    if angles is not None:
        _need(angles.dtype == torch.float32 and angles.is_contiguous() and tuple(angles.shape) == (n_tokens, rotary_dim),
              f"{what}: angles are float32 [tokens, rotary_dim]")


def rotary_angles(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = [cos(float32(pos_t) * inv_freq[i]) for i | sin(...) for i], float32 [tokens, 2 * len(inv_freq)]:
    the angles of a step, made once for every layer that rotates with these frequencies."""
    _dev(positions, inv_freq, out)
    _i32(positions, "positions")
    half = inv_freq.numel()
    _need(inv_freq.dtype == torch.float32 and out.dtype == torch.float32 and out.is_contiguous()
          and tuple(out.shape) == (positions.numel(), 2 * half), "rotary_angles: out is float32 [tokens, 2 * len(inv_freq)]")
    fn = _fn("rope_kv", "kipp_rotary_angles", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(positions), _ptr(inv_freq), _ptr(out), positions.numel(), half, _stream()), "rotary_angles")
    return out


def qk_norm_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                          positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                          n_q: int, n_kv: int, head_dim: int,
                          q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], eps: float,
                          inv_freq: Optional[torch.Tensor], rotary_dim: int, write_kv: bool = True,
                          angles: Optional[torch.Tensor] = None, pairing: str = "half") -> torch.Tensor:
    """Per-head norm of q and k, rotation at each token's position, q to `q_out`
    and k, v into their pages.  Caches are [pages, n_kv, page, head_dim].  With
    `angles` (rotary_angles) the cosines and sines are read, not computed.
    `pairing`: "half" rotates dim i with dim i + rotary_dim / 2, "interleaved" dim 2i with dim 2i + 1."""
    _need(pairing in ("half", "interleaved"), f"qk_norm_rope: pairing {pairing!r} is not one of half, interleaved")
    _dev(qkv, q_out, k_cache, v_cache, positions, seq_of_token, block_table, q_norm_w, k_norm_w, inv_freq, angles)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    n = qkv.shape[-2]
    parts = qkv.shape[0] if qkv.dim() == 3 else 1
    _need(tuple(qkv.shape[-2:]) == (n, (n_q + 2 * n_kv) * head_dim) and qkv.dim() in (2, 3),
          "qk_norm_rope: qkv must be [tokens, (n_q + 2 n_kv) d], or slabs of it")
    _need(q_out.shape == (n, n_q * head_dim), "qk_norm_rope: q_out must be [tokens, n_q d]")
    _need(k_cache.shape == v_cache.shape and k_cache.dim() == 4 and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == head_dim and k_cache.dtype == v_cache.dtype,
          "qk_norm_rope: caches must be [pages, n_kv, page, d] of one type")
    _need(positions.numel() == n and seq_of_token.numel() == n, "qk_norm_rope: one position and sequence per token")
    _need(block_table.dim() == 2, "qk_norm_rope: block_table is [sequences, blocks]")
    for w in (q_norm_w, k_norm_w):
        if w is not None:
            _need(w.dtype == torch.float32 and w.numel() == head_dim, "qk_norm_rope: norm weight is float32 [d]")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2 and rotary_dim % 2 == 0
              and 0 < rotary_dim <= head_dim, "qk_norm_rope: inv_freq is float32 [rotary_dim / 2]")
    _angles_ok(angles, n, rotary_dim, "qk_norm_rope")
    fn = _fn("rope_kv", "kipp_qk_norm_rope_kv",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(qkv), _code(qkv), _ptr(q_out), _code(q_out), _ptr(k_cache), _ptr(v_cache), _code(k_cache),
              _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1],
              _ptr(q_norm_w), _ptr(k_norm_w), float(eps), _ptr(inv_freq), _ptr(angles), int(rotary_dim),
              1 if pairing == "interleaved" else 0, n, n_q, n_kv, head_dim, k_cache.shape[2], 1 if write_kv else 0, parts, _stream()), "qk_norm_rope_kv_write")
    return q_out


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                            positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                            n_q: int, n_kv: int, head_dim: int, scale: float, window: int = 0) -> torch.Tensor:
    _dev(q, k_cache, v_cache, out, positions, seq_of_token, block_table)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    n = q.shape[0]
    _need(q.shape == (n, n_q * head_dim) and out.shape == q.shape, "attention: q and out are [tokens, n_q d]")
    _need(k_cache.shape == v_cache.shape and k_cache.dim() == 4 and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == head_dim and k_cache.dtype == v_cache.dtype,
          "attention: caches must be [pages, n_kv, page, d] of one type")
    _need(positions.numel() == n and seq_of_token.numel() == n and block_table.dim() == 2,
          "attention: one position and sequence per token, block_table [sequences, blocks]")
    fn = _fn("attention_generic", "kipp_paged_attention_generic",
             [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr])
    _check(fn(_ptr(q), _code(q), _ptr(k_cache), _ptr(v_cache), _code(k_cache), _ptr(out), _code(out),
              _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1],
              n, n_q, n_kv, head_dim, k_cache.shape[2], float(scale), int(window), _stream()),
           "paged_attention_generic")
    return out


def _attn_common(q, k_cache, v_cache, out, n_q, n_kv, head_dim, what):
    n = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16
          and v_cache.dtype == torch.bfloat16, f"{what}: bfloat16 queries, caches and output")
    _need(q.shape == (n, n_q * head_dim) and out.shape == q.shape, f"{what}: q and out are [tokens, n_q d]")
    _need(k_cache.shape == v_cache.shape and k_cache.dim() == 4 and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == head_dim, f"{what}: caches must be [pages, n_kv, page, d]")
    _need(head_dim % 16 == 0 and 0 < head_dim <= 256 and n_q % n_kv == 0, f"{what}: head size or head counts refused")
    page = k_cache.shape[2]
    _need(page > 0 and page & (page - 1) == 0, f"{what}: the page size must be a power of two (the generic kernel takes any)")


# --------------------------------------------------------------------------- several residual streams

STREAMS_MAX = 8


def streams_open(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out [tokens, R, width] (float32): every one of the R rows of a token is table[token]."""
    _dev(table, tokens, out)
    _i32(tokens, "tokens")
    _need(out.dim() == 3 and out.dtype == torch.float32 and table.dim() == 2 and table.shape[1] == out.shape[2]
          and tokens.numel() == out.shape[0] and 0 < out.shape[1] <= STREAMS_MAX, "streams_open: out is float32 [tokens, R <= 8, width]")
    fn = _fn("streams", "kipp_streams_open", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(table), _code(table), _ptr(tokens), _ptr(out), out.shape[0], out.shape[1], out.shape[2], _stream()), "streams_open")
    return out


def _streams_write_args(x, delta, mix, outw, what):
    n, r, width = x.shape
    parts = 0
    if delta is not None:
        _need(delta.dtype == torch.float32 and delta.dim() in (2, 3) and tuple(delta.shape[-2:]) == (n, width),
              f"{what}: delta is float32 [tokens, width] or slabs of it")
        parts = delta.shape[0] if delta.dim() == 3 else 1
        _need(mix is not None and outw is not None and mix.dtype == outw.dtype == torch.float32 and mix.numel() == r * r
              and outw.numel() == r, f"{what}: float32 coefficients [R, R] and [R]")
    else:
        _need(mix is None and outw is None, f"{what}: coefficients without a delta")
    return parts


def streams_step(x: torch.Tensor, delta: Optional[torch.Tensor], mix: Optional[torch.Tensor], outw: Optional[torch.Tensor],
                 inw: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], eps: float, h: Optional[torch.Tensor],
                 which: Optional[torch.Tensor] = None, store: bool = True):
    """One pass over the R rows of every token of x [tokens, R, width] (float32): with `delta` (a sublayer's result,
    maybe in slabs) the rows become X_t <- sum_r mix[r, t] X_r + outw[t] delta; with `inw` the weighted sum
    sum_r inw[r] X_r is RMS-normed with `norm_w` into `h` [tokens, width].  `which` (int32 token numbers) with `store`
    False: only those tokens are read, into `h` [len(which), width], and the written rows are not stored (the last read
    of a forward pass, when only some rows go on)."""
    _dev(x, delta, mix, outw, inw, norm_w, h)
    _need(x.dim() == 3 and x.dtype == torch.float32 and 0 < x.shape[1] <= STREAMS_MAX, "streams_step: x is float32 [tokens, R <= 8, width]")
    n, r, width = x.shape
    parts = _streams_write_args(x, delta, mix, outw, "streams_step")
    if inw is not None:
        _need(inw.dtype == torch.float32 and inw.numel() == r and norm_w is not None and norm_w.dtype == torch.float32
              and norm_w.numel() == width and h is not None and h.shape == (n if which is None else which.numel(), width),
              "streams_step: float32 [R] and [width], h [rows, width]")
    _need(delta is not None or inw is not None, "streams_step: nothing to do")
    if which is not None:
        _dev(which)
        _i32(which, "which")
        _need(not store and inw is not None, "streams_step: named rows are read only, and nothing is stored")
    fn = _fn("streams", "kipp_streams_step", [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int,
                                              _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), parts, _ptr(mix), _ptr(outw), _ptr(inw), _ptr(norm_w), float(eps),
              _ptr(h) if inw is not None else None, _code(h) if inw is not None else F32, n, r, width, _ptr(which),
              which.numel() if which is not None else n, int(bool(store)), _stream()), "streams_step")
    return h


def streams_close(x: torch.Tensor, delta: Optional[torch.Tensor], mix: Optional[torch.Tensor], outw: Optional[torch.Tensor],
                  which: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """out [rows, width] (float32) = the sum of a token's R rows after the last write (which is not stored), for the
    tokens that `which` names (None: all, in order)."""
    _dev(x, delta, mix, outw, which, out)
    _need(x.dim() == 3 and x.dtype == torch.float32 and 0 < x.shape[1] <= STREAMS_MAX, "streams_close: x is float32 [tokens, R <= 8, width]")
    n, r, width = x.shape
    parts = _streams_write_args(x, delta, mix, outw, "streams_close")
    if which is not None:
        _i32(which, "which")
    rows = which.numel() if which is not None else n
    _need(out.dtype == torch.float32 and out.shape == (rows, width), "streams_close: out is float32 [rows, width]")
    fn = _fn("streams", "kipp_streams_close", [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), parts, _ptr(mix), _ptr(outw), _ptr(which), _ptr(out), n, rows, r, width, _stream()), "streams_close")
    return out


# --------------------------------------------------------------------------- heads made ready without a rotation

def head_prepare(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                 n_q: int, n_kv: int, d: int, dv: int, bias: Optional[torch.Tensor], norm: str, eps: float,
                 q_norm_w: Optional[torch.Tensor] = None, k_norm_w: Optional[torch.Tensor] = None,
                 temp_coef: float = 0.0, temp_every: int = 0, write_kv: bool = True,
                 q_head_scale: Optional[torch.Tensor] = None, v_norm_eps: Optional[float] = None,
                 angles: Optional[torch.Tensor] = None, rotary_dim: int = 0, v_first_in: Optional[torch.Tensor] = None,
                 v_first_out: Optional[torch.Tensor] = None, v_lambda: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From a step's input product `proj` (float32 [tokens, >= n_q d + n_kv d + n_kv dv], columns q | k | v | ..., or slabs
    of it): `bias` added (float32 over the q | k | v columns), every head of q and k RMS-normed (`norm`: "none", "plain"
    or "weighted" with `q_norm_w` / `k_norm_w` [d]), queries at position p times 1 + temp_coef ln(floor((p + 1) /
    temp_every) + 1) (temp_every 0: none), queries of head h times `q_head_scale[h]` (float32 [n_q]), every value head over
    its root mean square with `v_norm_eps` inside the root (None: values as they are), q kept in `q_out`, k and v written
    into the pages of their positions.  `angles` (`rotary_angles`, float32 [tokens, rotary_dim]): after the norm the first
    `rotary_dim` numbers of every q and k head are turned, number i with number i + rotary_dim / 2.  `v_first_out` (float32
    [tokens, n_kv dv]) receives the values as they are; with `v_first_in` (another layer's, of the same tokens) and `v_lambda`
    (float32, one number on the device) the value that is cached is (1 - lambda) v + lambda v_first."""
    _dev(proj, q_out, k_cache, v_cache, positions, seq_of_token, block_table, bias, q_norm_w, k_norm_w, q_head_scale, angles,
         v_first_in, v_first_out, v_lambda)
    if angles is not None:
        _need(0 < rotary_dim <= d and rotary_dim % 2 == 0, "head_prepare: rotary_dim is even and at most d")
        _angles_ok(angles, proj.shape[-2], rotary_dim, "head_prepare")
    for vf in (v_first_in, v_first_out):
        if vf is not None:
            _need(write_kv and vf.dtype == torch.float32 and tuple(vf.shape) == (proj.shape[-2], n_kv * dv), "head_prepare: first values are float32 [tokens, n_kv dv]")
    if v_first_in is not None:
        _need(v_lambda is not None and v_lambda.dtype == torch.float32 and v_lambda.numel() == 1 and v_first_in is not v_first_out,
              "head_prepare: mixing values needs a float32 lambda on the device")
    if q_head_scale is not None:
        _need(q_head_scale.dtype == torch.float32 and q_head_scale.numel() == n_q, "head_prepare: float32 q_head_scale [n_q]")
    _need(v_norm_eps is None or v_norm_eps >= 0, "head_prepare: v_norm_eps must not be negative")
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    parts, n, stride = _slabs(proj, "head_prepare")
    _need(norm in ("none", "plain", "weighted"), "head_prepare: norm is one of none, plain, weighted")
    _need(stride >= n_q * d + (n_kv * d + n_kv * dv if write_kv else 0), "head_prepare: the projections are narrower than q, k and v")
    _need(0 < d <= 256 and 0 < dv <= 256, "head_prepare: head sizes from 1 to 256")
    _need(q_out.shape == (n, n_q * d) and positions.numel() == n and seq_of_token.numel() == n, "head_prepare: one row a token")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n_q * d + n_kv * d + n_kv * dv, "head_prepare: float32 bias over q | k | v")
    if norm == "weighted":
        _need(q_norm_w is not None and k_norm_w is not None and q_norm_w.dtype == k_norm_w.dtype == torch.float32
              and q_norm_w.numel() == d and k_norm_w.numel() == d, "head_prepare: float32 norm weights [d]")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[:3] == v_cache.shape[:3] and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == d and dv <= v_cache.shape[3] <= 256 and k_cache.dtype == v_cache.dtype,
          "head_prepare: caches must be [pages, n_kv, page, d] and [pages, n_kv, page, >= dv] (the rest of a value's row is written as zeros)")
    _need(block_table.dim() == 2 and int(temp_every) >= 0, "head_prepare: block_table is [sequences, blocks]")
    fn = _fn("head_prepare", "kipp_head_prepare_rotated",
             [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_int, _c_ptr, _c_ptr, _c_float, _c_float, _c_int] + [_c_int] * 7 + [_c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr])
    _check(fn(_ptr(proj), parts, stride, _ptr(bias), _ptr(q_out), _code(q_out), _ptr(k_cache), _ptr(v_cache), _code(k_cache),
              _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1],
              {"none": 0, "plain": 1, "weighted": 2}[norm], _ptr(q_norm_w), _ptr(k_norm_w), float(eps), float(temp_coef),
              int(temp_every), n, n_q, n_kv, d, dv, k_cache.shape[2], int(write_kv), _ptr(q_head_scale),
              -1.0 if v_norm_eps is None else float(v_norm_eps), _ptr(angles), int(rotary_dim) if angles is not None else 0,
              _ptr(v_first_in), _ptr(v_first_out), _ptr(v_lambda), v_cache.shape[3], _stream()), "head_prepare")
    return q_out


def paged_attention_wide(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                         positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                         n_q: int, n_kv: int, d: int, dv: int, scale: float, window: int = 0, softcap: float = 0.0,
                         chunk: int = 0, sink: bool = False) -> torch.Tensor:
    """The generic attention kernel with values of their own width: keys of up to 1,024 numbers, values of `dv`.
    `v_cache` may be `k_cache` itself: a value is then the first dv numbers of its key's row.  `softcap` c > 0: a
    scaled score s becomes c tanh(s / c).  `chunk` c > 0 (instead of a window): position p sees the keys from p - p % c
    on.  `sink`: one is added to the softmax's denominator (a key of score 0 that has no value)."""
    _need(chunk >= 0 and not (chunk and window), "attention: a chunk or a window, not both")
    _dev(q, k_cache, v_cache, out, positions, seq_of_token, block_table)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    n = q.shape[0]
    _need(q.shape == (n, n_q * d) and out.shape == (n, n_q * dv), "attention: q is [tokens, n_q d] and out [tokens, n_q dv]")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[:3] == v_cache.shape[:3] and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == d and v_cache.shape[3] >= dv and k_cache.dtype == v_cache.dtype and 0 < d <= 1024 and 0 < dv <= 1024,
          "attention: caches must be [pages, n_kv, page, d] and [pages, n_kv, page, >= dv] of one type")
    _need(positions.numel() == n and seq_of_token.numel() == n and block_table.dim() == 2,
          "attention: one position and sequence per token, block_table [sequences, blocks]")
    _need(softcap >= 0, "attention: softcap must not be negative")
    fn = _fn("attention_generic", "kipp_paged_attention_generic_masked",
             [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_float, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(q), _code(q), _ptr(k_cache), _ptr(v_cache), _code(k_cache), _ptr(out), _code(out),
              _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1],
              n, n_q, n_kv, d, dv, v_cache.shape[3], k_cache.shape[2], float(scale), int(window), float(softcap), int(chunk),
              int(bool(sink)), _stream()),
           "paged_attention_wide")
    return out


# --------------------------------------------------------------------------- attention through a latent

def latent_prepare(proj: torch.Tensor, cq_out: torch.Tensor, cache: torch.Tensor, positions: torch.Tensor,
                   seq_of_token: torch.Tensor, block_table: torch.Tensor, q_rank: int, rank: int, dr: int,
                   q_norm_w: torch.Tensor, c_norm_w: torch.Tensor, eps: float, freq: torch.Tensor, rot_dims: int,
                   magnitude: float, write_kv: bool = True) -> torch.Tensor:
    """From the input product `proj` (float32 [tokens, >= q_rank + rank + dr], columns query latent | key/value latent |
    rotated key part | ..., or slabs of it): the query latent RMS-normed with `q_norm_w` into `cq_out`; the key/value latent
    RMS-normed with `c_norm_w` and the key part rotated at the token's position, both written as one row of rank + dr
    numbers into the token's page of `cache` [pages, 1, page, rank + dr]."""
    _dev(proj, cq_out, cache, positions, seq_of_token, block_table, q_norm_w, c_norm_w, freq)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    parts, n, stride = _slabs(proj, "latent_prepare")
    _need(stride >= q_rank + rank + dr and cq_out.shape == (n, q_rank) and positions.numel() == n and seq_of_token.numel() == n,
          "latent_prepare: one row a token, projections [query latent | latent | rotated part]")
    _need(cache.dim() == 4 and cache.shape[1] == 1 and cache.shape[3] == rank + dr and block_table.dim() == 2,
          "latent_prepare: the cache is [pages, 1, page, rank + dr]")
    _need(q_norm_w.dtype == c_norm_w.dtype == torch.float32 and q_norm_w.numel() == q_rank and c_norm_w.numel() == rank,
          "latent_prepare: float32 norm weights")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= dr and freq.dtype == torch.float32 and freq.numel() >= rot_dims // 2,
          "latent_prepare: float32 frequencies for rot_dims / 2 pairs")
    fn = _fn("latent", "kipp_latent_prepare",
             [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_ptr, _c_int, _c_float] + [_c_int] * 6 + [_c_ptr])
    _check(fn(_ptr(proj), parts, stride, _ptr(q_norm_w), _ptr(c_norm_w), float(eps), _ptr(cq_out), _code(cq_out), _ptr(cache),
              _code(cache), _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], _ptr(freq), int(rot_dims),
              float(magnitude), n, q_rank, rank, dr, cache.shape[2], int(write_kv), _stream()), "latent_prepare")
    return cq_out


def latent_absorb(q: torch.Tensor, w_uk: torch.Tensor, out: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor,
                  rot_dims: int, magnitude: float, heads: int, d: int, dr: int, rank: int) -> torch.Tensor:
    """out [tokens, heads (rank + dr)]: every head's unrotated query part carried into the latent's space by
    `w_uk` [heads d, rank] (q_h W_uk_h), its rotated part turned at the token's position."""
    _dev(q, w_uk, out, positions, freq)
    _i32(positions, "positions")
    parts, n, stride = _slabs(q, "latent_absorb")
    _need(stride == heads * (d + dr) and out.shape == (n, heads * (rank + dr)) and positions.numel() == n,
          "latent_absorb: q is [tokens, heads (d + dr)], out [tokens, heads (rank + dr)]")
    _need(w_uk.shape == (heads * d, rank) and _code(w_uk) == _code(out), "latent_absorb: w_uk is [heads d, rank] in the output's type")
    _need(d * 32 + 8192 <= 64 * 1024, "latent_absorb: unrotated head size too large")
    fn = _fn("latent", "kipp_latent_absorb", [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_float]
             + [_c_int] * 5 + [_c_ptr])
    _check(fn(_ptr(q), parts, _ptr(w_uk), _code(w_uk), _ptr(out), _code(out), _ptr(positions), _ptr(freq), int(rot_dims),
              float(magnitude), n, heads, d, dr, rank, _stream()), "latent_absorb")
    return out


def latent_expand(lat: torch.Tensor, w_uv_t: torch.Tensor, out: torch.Tensor, heads: int, rank: int, dv: int,
                  gate: Optional[torch.Tensor] = None, gate_at: int = 0) -> torch.Tensor:
    """out [tokens, heads dv]: head h's latent result (the first `rank` numbers of its row of `lat` [tokens, heads row])
    carried back by `w_uv_t` [heads, rank, dv], times sigmoid(gate[t, gate_at + h]) where `gate` (the float32 input
    product, maybe in slabs) is given."""
    _dev(lat, w_uv_t, out, gate)
    n = lat.shape[0]
    _need(lat.dim() == 2 and lat.shape[1] % heads == 0 and lat.shape[1] // heads >= rank, "latent_expand: lat is [tokens, heads row]")
    _need(w_uv_t.shape == (heads, rank, dv) and out.shape == (n, heads * dv) and _code(lat) == _code(w_uv_t) == _code(out),
          "latent_expand: w_uv_t is [heads, rank, dv]; one type")
    _need(rank * 32 + 8192 <= 64 * 1024, "latent_expand: latent too wide")
    g_parts, g_stride, g_ptr = 0, 0, None
    if gate is not None:
        g_parts, g_n, g_stride = _slabs(gate, "latent_expand")
        _need(g_n == n and gate_at + heads <= g_stride, "latent_expand: the gate's columns lie outside the product")
        g_ptr = gate.data_ptr() + 4 * gate_at
    fn = _fn("latent", "kipp_latent_expand", [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_int]
             + [_c_int] * 4 + [_c_ptr])
    _check(fn(_ptr(lat), _code(lat), lat.shape[1] // heads, _ptr(w_uv_t), _code(w_uv_t), g_ptr, g_parts, g_stride, _ptr(out),
              _code(out), n, heads, rank, dv, _stream()), "latent_expand")
    return out


# --------------------------------------------------------------------------- matrix memory (mLSTM)

def mlstm_columns(d: int) -> int:
    """Columns of the memory that a workgroup of the scan takes (fewer where a column's rows need more lanes)."""
    return 256 // (4 if d <= 32 else (16 if d <= 256 else 64))


def mlstm_state_size(heads: int, d: int, dv: int) -> int:
    """float32 numbers of a request's state: S [heads, dv, d], then a copy of n [heads, d] and m [heads] for every
    workgroup's columns."""
    size = heads * d * dv + -(-dv // mlstm_columns(d)) * (heads * d + heads)
    return -(-size // 4) * 4       # slots begin at multiples of 16 bytes


def mlstm_scan(proj: torch.Tensor, bias_i: torch.Tensor, bias_f: torch.Tensor, cap: float, state: torch.Tensor,
               q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor, o_raw: torch.Tensor,
               heads: int, d: int, dv: int, few: bool = False) -> torch.Tensor:
    """The recurrence over every entry's tokens, in order, from and into the entry's slot of `state` [slots, size]
    (float32).  `few`: every entry brings few tokens (single decoded tokens): fewer, larger workgroups; the same bits.  `proj`: float32 [tokens, >= 2 heads d + 2 heads dv + 2 heads], columns q | k | v | gate | zi | zf;
    `o_raw` float32 [tokens, heads dv] receives S^T q over its denominator."""
    _dev(proj, bias_i, bias_f, state, q_start, q_len, slots, o_raw)
    for t, name in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _i32(t, name)
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.shape[1] >= 2 * heads * d + 2 * heads * dv + 2 * heads,
          "mlstm_scan: proj is float32 [tokens, q | k | v | gate | zi | zf]")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.shape[1] >= mlstm_state_size(heads, d, dv),
          "mlstm_scan: state is float32 [slots, size]")
    _need(bias_i.dtype == bias_f.dtype == torch.float32 and bias_i.numel() == heads and bias_f.numel() == heads, "mlstm_scan: float32 gate biases [heads]")
    _need(o_raw.dtype == torch.float32 and o_raw.shape == (proj.shape[0], heads * dv) and 0 < d <= 1024 and cap > 0,
          "mlstm_scan: o_raw is float32 [tokens, heads dv]; key size up to 1,024")
    _need(q_start.numel() == q_len.numel() == slots.numel(), "mlstm_scan: one start, length and slot an entry")
    fn = _fn("mlstm", "kipp_mlstm_scan", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_size, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(proj), proj.shape[1], _ptr(bias_i), _ptr(bias_f), float(cap), _ptr(state), state.shape[1], _ptr(q_start),
              _ptr(q_len), _ptr(slots), _ptr(o_raw), q_start.numel(), heads, d, dv, int(bool(few)), _stream()), "mlstm_scan")
    return o_raw


def mlstm_finish(o_raw: torch.Tensor, proj: torch.Tensor, gate_at: int, norm_w: torch.Tensor, eps: float, out: torch.Tensor,
                 heads: int, dv: int) -> torch.Tensor:
    """out [tokens, heads dv] = every head of `o_raw` over its root mean square, times `norm_w`, times
    sigmoid(proj[:, gate_at:gate_at + heads dv])."""
    _dev(o_raw, proj, norm_w, out)
    n = o_raw.shape[0]
    _need(o_raw.dtype == proj.dtype == norm_w.dtype == torch.float32 and o_raw.shape == (n, heads * dv) and out.shape == o_raw.shape
          and proj.dim() == 2 and proj.shape[0] == n and proj.shape[1] >= gate_at + heads * dv and norm_w.numel() == heads * dv,
          "mlstm_finish: float32 [tokens, heads dv] rows, gate columns inside proj")
    fn = _fn("mlstm", "kipp_mlstm_finish", [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(o_raw), _ptr(proj), proj.shape[1], int(gate_at), _ptr(norm_w), float(eps), _ptr(out), _code(out), n, heads, dv,
              _stream()), "mlstm_finish")
    return out


# --------------------------------------------------------------------------- layer norm and the sandwich step

LAYER_NORM_MAX_WIDTH = 8192


def layer_norm(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out = scale * ((u - mean) / sqrt(var + eps) * weight + bias) over rows; `u` is float32 [rows, width] or slabs
    [parts, rows, width] that are added in order."""
    _dev(u, weight, bias, out)
    parts, rows, width = _slabs(u, "layer_norm")
    _need(weight.dtype == bias.dtype == torch.float32 and weight.numel() == bias.numel() == width, "layer_norm: float32 weight and bias [width]")
    _need(out.shape == (rows, width) and width <= LAYER_NORM_MAX_WIDTH, "layer_norm: out is [rows, width], width up to 8,192")
    fn = _fn("layer_norm", "kipp_layer_norm", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_float, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(u), parts, _ptr(weight), _ptr(bias), float(eps), float(scale), _ptr(out), _code(out), rows, width, _stream()), "layer_norm")
    return out


def sandwich_step(x: torch.Tensor, delta: torch.Tensor, post_w: torch.Tensor, post_b: torch.Tensor, post_eps: float, mult: float,
                  extra: Optional[torch.Tensor] = None, next_w: Optional[torch.Tensor] = None, next_b: Optional[torch.Tensor] = None,
                  next_eps: float = 0.0, out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x += mult * LN_post(delta) [+ extra] in place (float32 [rows, width]; `delta` may come in slabs), and, with `out`,
    out = LN_next(x) in out's type: the end of one normed sublayer and the beginning of the next in one pass over a row."""
    _dev(x, delta, post_w, post_b, extra, next_w, next_b, out)
    parts, rows, width = _slabs(delta, "sandwich_step")
    _need(x.dtype == torch.float32 and x.shape == (rows, width) and width <= LAYER_NORM_MAX_WIDTH, "sandwich_step: x is float32 [rows, width], width up to 8,192")
    for t in (post_w, post_b, next_w, next_b):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == width), "sandwich_step: float32 weights and biases [width]")
    _need(extra is None or (extra.dtype == torch.float32 and extra.shape == x.shape), "sandwich_step: extra is float32 of x's shape")
    _need(out is None or (out.shape == x.shape and next_w is not None and next_b is not None), "sandwich_step: out needs the next norm")
    fn = _fn("layer_norm", "kipp_sandwich_step", [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_float,
                                                  _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(delta), parts, _ptr(post_w), _ptr(post_b), float(post_eps), float(mult), _ptr(extra), _ptr(next_w), _ptr(next_b),
              float(next_eps), _ptr(out), _code(out) if out is not None else F32, rows, width, _stream()), "sandwich_step")
    return out


# --------------------------------------------------------------------------- matrix memories: fixed decay, gated delta rule

def _scan_args(state, q_start, q_len, slots, o_raw, tokens, heads, d, dv, what):
    for t, name in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _i32(t, name)
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.shape[1] >= heads * d * dv, f"{what}: state is float32 [slots, >= heads d dv]")
    _need(o_raw.dtype == torch.float32 and o_raw.shape == (tokens, heads * dv) and 0 < d <= 1024, f"{what}: o_raw is float32 [tokens, heads dv]; key size up to 1,024")
    _need(q_start.numel() == q_len.numel() == slots.numel(), f"{what}: one start, length and slot an entry")


def decay_scan(proj: torch.Tensor, decays: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
               slots: torch.Tensor, o_raw: torch.Tensor, heads: int, d: int, dv: int, longest: int = 0) -> torch.Tensor:
    """Linear attention with a fixed decay a head over every entry's tokens, in order, from and into the entry's slot of
    `state` [slots, size] (float32, S as [head][column][row]).  `proj`: float32 [tokens, >= 2 heads d + heads dv], columns
    q | k | v before their silu; `o_raw` float32 [tokens, heads dv] receives S^T q.  `longest`: the most tokens an entry
    brings, if known (it sizes the kernel's chunks and changes no result)."""
    _dev(proj, decays, state, q_start, q_len, slots, o_raw)
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.shape[1] >= 2 * heads * d + heads * dv, "decay_scan: proj is float32 [tokens, q | k | v ...]")
    _need(decays.dtype == torch.float32 and decays.numel() == heads, "decay_scan: float32 decays [heads]")
    _scan_args(state, q_start, q_len, slots, o_raw, proj.shape[0], heads, d, dv, "decay_scan")
    fn = _fn("linear_scan", "kipp_decay_scan", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_size, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(proj), proj.shape[1], _ptr(decays), _ptr(state), state.shape[1], _ptr(q_start), _ptr(q_len), _ptr(slots), _ptr(o_raw),
              q_start.numel(), heads, d, dv, max(0, int(longest)), _stream()), "decay_scan")
    return o_raw


def delta_state_size(heads: int, kv_heads: int, d: int, dv: int, taps: int) -> int:
    """float32 numbers of a request's state: S [heads, dv, d], then the last taps - 1 inputs of the q | k | v channels."""
    size = heads * d * dv + (taps - 1) * (2 * kv_heads * d + heads * dv)
    return -(-size // 4) * 4


def delta_prepare(proj: torch.Tensor, conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor,
                  seq_of_token: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor, prep: torch.Tensor,
                  heads: int, kv_heads: int, d: int, dv: int, beta_col: int, a_col: int, unit_eps: float) -> torch.Tensor:
    """The gated delta rule's inputs from its input product `proj` (float32 [tokens, >= channels], columns q | k | v first,
    the beta and decay pre-activations at `beta_col` and `a_col`): `prep` [tokens, channels + 2 heads] receives q | k | v
    behind their short convolutions (`conv_w` [channels, taps], the slot's kept inputs in front of a portion) and silu, every
    q and k head a unit vector (q also over sqrt(d)), then beta = sigmoid and g = exp(-exp(a_log) softplus(. + dt_bias)) a
    head.  The slot's kept inputs are then moved on by the portion."""
    _dev(proj, conv_w, a_log, dt_bias, state, seq_of_token, q_start, q_len, slots, prep)
    for t, name in ((seq_of_token, "seq_of_token"), (q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _i32(t, name)
    channels = 2 * kv_heads * d + heads * dv
    n = proj.shape[0]
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.shape[1] >= max(channels, beta_col + heads, a_col + heads), "delta_prepare: proj is float32 [tokens, q | k | v | ...]")
    _need(conv_w.dtype == torch.float32 and conv_w.dim() == 2 and conv_w.shape[0] == channels and 1 <= conv_w.shape[1] <= 16, "delta_prepare: float32 filters [channels, taps], up to 16 taps")
    taps = conv_w.shape[1]
    _need(a_log.dtype == dt_bias.dtype == torch.float32 and a_log.numel() == dt_bias.numel() == heads, "delta_prepare: float32 a_log and dt_bias [heads]")
    _need(prep.dtype == torch.float32 and prep.shape == (n, channels + 2 * heads) and seq_of_token.numel() == n, "delta_prepare: prep is float32 [tokens, channels + 2 heads]")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.shape[1] >= delta_state_size(heads, kv_heads, d, dv, taps), "delta_prepare: state is float32 [slots, size]")
    _need(q_start.numel() == q_len.numel() == slots.numel(), "delta_prepare: one start, length and slot an entry")
    fn = _fn("linear_scan", "kipp_delta_prepare", [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_size, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                                   _c_ptr, _c_int] + [_c_int] * 8 + [_c_float, _c_ptr])
    _check(fn(_ptr(proj), proj.shape[1], _ptr(conv_w), taps, _ptr(a_log), _ptr(dt_bias), _ptr(state), state.shape[1], heads * d * dv,
              _ptr(seq_of_token), _ptr(q_start), _ptr(q_len), _ptr(slots), _ptr(prep), prep.shape[1], n, q_start.numel(), heads, kv_heads, d, dv,
              int(beta_col), int(a_col), float(unit_eps), _stream()), "delta_prepare")
    return prep


def delta_scan(prep: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
               o_raw: torch.Tensor, heads: int, kv_heads: int, d: int, dv: int, longest: int = 0) -> torch.Tensor:
    """The gated delta rule over every entry's tokens, in order, from and into the entry's slot: S <- g S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q, with `prep` as `delta_prepare` leaves it.  `longest` as for `decay_scan`."""
    _dev(prep, state, q_start, q_len, slots, o_raw)
    _need(prep.dim() == 2 and prep.dtype == torch.float32 and prep.shape[1] >= 2 * kv_heads * d + heads * dv + 2 * heads and heads % kv_heads == 0,
          "delta_scan: prep is float32 [tokens, q | k | v | beta | g]")
    _scan_args(state, q_start, q_len, slots, o_raw, prep.shape[0], heads, d, dv, "delta_scan")
    fn = _fn("linear_scan", "kipp_delta_scan", [_c_ptr, _c_int, _c_ptr, _c_size, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(prep), prep.shape[1], _ptr(state), state.shape[1], _ptr(q_start), _ptr(q_len), _ptr(slots), _ptr(o_raw), q_start.numel(),
              heads, kv_heads, d, dv, max(0, int(longest)), _stream()), "delta_scan")
    return o_raw


def ssd_state_size(heads: int, groups: int, n: int, p: int, taps: int) -> int:
    """float32 numbers of a request's state: S [heads, p, n], then the last taps - 1 inputs of the x | B | C channels."""
    size = heads * n * p + (taps - 1) * (heads * p + 2 * groups * n)
    return -(-size // 4) * 4


def ssd_prep_width(heads: int, groups: int, n: int, p: int) -> int:
    """Columns of what `ssd_prepare` writes: C | B | dt x | x | g."""
    return 2 * groups * n + 2 * heads * p + heads


def ssd_prepare(proj: torch.Tensor, conv_w: torch.Tensor, conv_b: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                state: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
                prep: torch.Tensor, heads: int, groups: int, n: int, p: int) -> torch.Tensor:
    """The state space recurrence's inputs from its input product `proj` (float32 [tokens, z | x | B | C | dt], z and x of
    heads p columns, B and C of groups n, dt of heads): x, B and C behind their short causal filter (`conv_w` [channels,
    taps], `conv_b` [channels], the slot's kept inputs ahead of a portion) and silu; dt = softplus(dt + dt_bias);
    `prep` [tokens, `ssd_prep_width`] receives C | B | dt x | x | g with g = exp(-exp(a_log) dt) a head.  The slot's kept
    inputs are then moved on by the portion."""
    _dev(proj, conv_w, conv_b, a_log, dt_bias, state, seq_of_token, q_start, q_len, slots, prep)
    for t, name in ((seq_of_token, "seq_of_token"), (q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _i32(t, name)
    inner, channels = heads * p, heads * p + 2 * groups * n
    tokens = proj.shape[0]
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.shape[1] >= inner + channels + heads, "ssd_prepare: proj is float32 [tokens, z | x | B | C | dt]")
    _need(conv_w.dtype == conv_b.dtype == torch.float32 and conv_w.dim() == 2 and conv_w.shape[0] == channels and conv_b.numel() == channels
          and 1 <= conv_w.shape[1] <= 16, "ssd_prepare: float32 filters [channels, taps] with a bias a channel, up to 16 taps")
    taps = conv_w.shape[1]
    _need(a_log.dtype == dt_bias.dtype == torch.float32 and a_log.numel() == dt_bias.numel() == heads and 0 < heads <= 1024 and heads % groups == 0,
          "ssd_prepare: float32 a_log and dt_bias [heads], up to 1,024 heads in equal groups")
    _need(prep.dtype == torch.float32 and prep.shape == (tokens, ssd_prep_width(heads, groups, n, p)) and seq_of_token.numel() == tokens,
          "ssd_prepare: prep is float32 [tokens, 2 groups n + 2 heads p + heads]")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.shape[1] >= ssd_state_size(heads, groups, n, p, taps), "ssd_prepare: state is float32 [slots, size]")
    _need(q_start.numel() == q_len.numel() == slots.numel(), "ssd_prepare: one start, length and slot an entry")
    fn = _fn("linear_scan", "kipp_ssd_prepare", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_size, _c_ptr, _c_ptr, _c_ptr,
                                                 _c_ptr, _c_ptr, _c_int] + [_c_int] * 6 + [_c_ptr])
    _check(fn(_ptr(proj), proj.shape[1], _ptr(conv_w), _ptr(conv_b), taps, _ptr(a_log), _ptr(dt_bias), _ptr(state), state.shape[1], heads * n * p,
              _ptr(seq_of_token), _ptr(q_start), _ptr(q_len), _ptr(slots), _ptr(prep), prep.shape[1], tokens, q_start.numel(), heads, groups, n, p,
              _stream()), "ssd_prepare")
    return prep


def gated_scan(prep: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
               o_raw: torch.Tensor, heads: int, groups: int, n: int, p: int, longest: int = 0) -> torch.Tensor:
    """The recurrence with a decay a token and head over every entry's tokens, in order, from and into the entry's slot:
    S <- g S + k v^T; o = S^T q, with `prep` as `ssd_prepare` leaves it (q = C, k = B shared by the heads of a group, v = dt x).
    `longest` as for `decay_scan`."""
    _dev(prep, state, q_start, q_len, slots, o_raw)
    _need(prep.dim() == 2 and prep.dtype == torch.float32 and prep.shape[1] >= ssd_prep_width(heads, groups, n, p) and heads % groups == 0,
          "gated_scan: prep is float32 [tokens, C | B | dt x | x | g]")
    _scan_args(state, q_start, q_len, slots, o_raw, prep.shape[0], heads, n, p, "gated_scan")
    fn = _fn("linear_scan", "kipp_gated_scan", [_c_ptr, _c_int, _c_ptr, _c_size, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(prep), prep.shape[1], _ptr(state), state.shape[1], _ptr(q_start), _ptr(q_len), _ptr(slots), _ptr(o_raw), q_start.numel(),
              heads, groups, n, p, max(0, int(longest)), _stream()), "gated_scan")
    return o_raw


def ssd_finish(o_raw: torch.Tensor, prep: torch.Tensor, x_at: int, proj: torch.Tensor, z_at: int, skip: torch.Tensor, p: int,
               norm_w: torch.Tensor, eps: float, span: int, out: torch.Tensor) -> torch.Tensor:
    """out [tokens, width]: y = (o_raw + skip[column // p] x) silu(z), x at column `x_at` of `prep` and z at column `z_at` of
    `proj`; then every run of `span` columns of y over its root mean square, times norm_w[column] (the gate before the norm)."""
    _dev(o_raw, prep, proj, skip, norm_w, out)
    tokens, width = o_raw.shape
    _need(o_raw.dtype == prep.dtype == proj.dtype == skip.dtype == norm_w.dtype == torch.float32 and out.shape == o_raw.shape
          and prep.dim() == proj.dim() == 2 and prep.shape[0] == proj.shape[0] == tokens and prep.shape[1] >= x_at + width
          and proj.shape[1] >= z_at + width and width % span == 0 and width % p == 0 and skip.numel() == width // p and norm_w.numel() == width,
          "ssd_finish: float32 rows, x and z columns inside their rows, one skip a head, a weight a column")
    fn = _fn("linear_scan", "kipp_ssd_finish", [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int,
                                                _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(o_raw), _ptr(prep), prep.shape[1], int(x_at), _ptr(proj), proj.shape[1], int(z_at), _ptr(skip), int(p), _ptr(norm_w), float(eps),
              _ptr(out), _code(out), tokens, width, int(span), _stream()), "ssd_finish")
    return out


def scan_finish(o_raw: torch.Tensor, gates: torch.Tensor, gate_at: int, norm_w: torch.Tensor, eps: float, gate: str, span: int,
                out: torch.Tensor) -> torch.Tensor:
    """out [tokens, width] = every run of `span` columns of `o_raw` over its root mean square, times norm_w[column % len(norm_w)],
    times gate(gates[:, gate_at + column]), gate "sigmoid" or "silu"."""
    _dev(o_raw, gates, norm_w, out)
    n, width = o_raw.shape
    _need(o_raw.dtype == gates.dtype == norm_w.dtype == torch.float32 and out.shape == o_raw.shape and gates.dim() == 2 and gates.shape[0] == n
          and gates.shape[1] >= gate_at + width and width % span == 0 and gate in ("sigmoid", "silu"), "scan_finish: float32 rows, gate columns inside `gates`")
    fn = _fn("linear_scan", "kipp_scan_finish", [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(o_raw), _ptr(gates), gates.shape[1], int(gate_at), _ptr(norm_w), norm_w.numel(), float(eps), 0 if gate == "sigmoid" else 1,
              _ptr(out), _code(out), n, width, int(span), _stream()), "scan_finish")
    return out


# --------------------------------------------------------------------------- routed feed-forward

ACTIVATIONS = {"silu": 0, "relu": 1, "gelu": 2, "gelu_tanh": 3, "relu2": 4}     # relu2: the square of relu
MOE_TILE_ROWS = 16
MOE_MFMA_ROWS = 128    # rows of a tile of the experts' products on the matrix cores


def moe_tile_rows(dtype: torch.dtype, *contractions: int) -> int:
    """Rows of the tiles that the experts' products take: 128 on the matrix cores (bfloat16, every contraction a multiple of
    32), else 16."""
    return MOE_MFMA_ROWS if dtype == torch.bfloat16 and all(k % 32 == 0 for k in contractions) else MOE_TILE_ROWS


def moe_max_tiles(tokens: int, experts: int, top: int, tile_rows: int = 16) -> int:
    """Tiles of up to `tile_rows` rows that the sorted pairs of a step can need at most (every expert may end in a partial one)."""
    pairs = tokens * top
    return -(-pairs // tile_rows) + min(experts, pairs)


def moe_route(z: torch.Tensor, experts: int, top: int, eps: float, chosen: torch.Tensor, weight: torch.Tensor,
              pair_token: torch.Tensor, place_of_pair: torch.Tensor, tiles: torch.Tensor, tile_rows: int = 16,
              router: str = "softmax", correction: Optional[torch.Tensor] = None, groups: Optional[tuple] = None, scale: float = 1.0):
    """From router logits `z` (float32 [tokens, >= experts] or slabs): softmax over the experts, the `top` largest a token
    (`chosen`, int32 [tokens, top]) with weights p / (sum of the chosen p + eps) (`weight`, float32 [tokens, top]); then the
    pairs sorted by expert: `pair_token` [pairs] the token of every sorted row, `place_of_pair` [pairs] the row of pair
    (token, choice), `tiles` int32 [max_tiles, 3] = (expert, first row, rows) of up to `tile_rows` rows, unused tiles with 0 rows."""
    _dev(z, chosen, weight, pair_token, place_of_pair, tiles)
    parts, n, stride = _slabs(z, "moe_route")
    for t, name in ((chosen, "chosen"), (pair_token, "pair_token"), (place_of_pair, "place_of_pair"), (tiles, "tiles")):
        _i32(t, name)
    _need(0 < top <= experts <= 1024 and top <= 32 and stride >= experts, "moe_route: up to 1,024 experts, up to 32 a token")
    _need(chosen.shape == (n, top) and weight.shape == (n, top) and weight.dtype == torch.float32 and pair_token.numel() == n * top
          and place_of_pair.numel() == n * top and tiles.dim() == 2 and tiles.shape[1] == 3 and tiles.shape[0] >= moe_max_tiles(n, experts, top, tile_rows),
          "moe_route: output shapes")
    _need(router in ("softmax", "sigmoid"), "moe_route: router is softmax or sigmoid")
    if router == "sigmoid":
        _dev(correction)
        count, keep = groups if groups is not None else (1, 1)
        _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == experts), "moe_route: float32 correction [experts]")
        _need(count > 0 and experts % count == 0 and 0 < keep <= count and top <= keep * (experts // count),
              "moe_route: equal groups, of which at least one stays, with experts enough for a token's choice")
        fn = _fn("moe", "kipp_moe_route_grouped", [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_float,
                                                   _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
        _check(fn(_ptr(z), parts, stride, _ptr(correction), _ptr(chosen), _ptr(weight), n, experts, top, float(eps), int(count), int(keep), float(scale),
                  _ptr(pair_token), _ptr(place_of_pair), _ptr(tiles), tiles.shape[0], int(tile_rows), _stream()), "moe_route")
        return chosen, weight
    _need(correction is None and groups is None and scale == 1.0, "moe_route: correction, groups and scale belong to the sigmoid router")
    fn = _fn("moe", "kipp_moe_route", [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(z), parts, stride, _ptr(chosen), _ptr(weight), n, experts, top, float(eps), _ptr(pair_token), _ptr(place_of_pair), _ptr(tiles),
              tiles.shape[0], int(tile_rows), _stream()), "moe_route")
    return chosen, weight


def moe_expert(x: torch.Tensor, gather: Optional[torch.Tensor], w: torch.Tensor, tiles: torch.Tensor, out: torch.Tensor,
               activation: Optional[str] = None, tile_rows: int = 16) -> torch.Tensor:
    """Every tile's rows against its expert's matrix: out[row] = act(w[expert] x_row), x_row = x[gather[row]] (or x[row]);
    `w` [experts, n_out, k], `out` [sorted rows, n_out].  `tile_rows`: what `moe_route` was given (128: the matrix cores)."""
    _dev(x, gather, w, tiles, out)
    _i32(tiles, "tiles")
    if gather is not None:
        _i32(gather, "gather")
    _need(w.dim() == 3 and x.dim() == 2 and x.shape[1] == w.shape[2] and out.dim() == 2 and out.shape[1] == w.shape[1] and x.dtype == w.dtype,
          "moe_expert: x [rows, k], w [experts, n_out, k] of one type, out [rows, n_out]")
    _need(out.shape[0] == (gather.numel() if gather is not None else x.shape[0]), "moe_expert: one output row a sorted row")
    _need(activation is None or activation in ACTIVATIONS, f"moe_expert: activation is one of {sorted(ACTIVATIONS)}")
    _need(tile_rows == MOE_TILE_ROWS or (tile_rows == MOE_MFMA_ROWS and x.dtype == torch.bfloat16 and w.shape[2] % 32 == 0),
          "moe_expert: tiles of 16 rows, or of 128 for bfloat16 with K a multiple of 32")
    fn = _fn("moe", "kipp_moe_expert", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _code(x), _ptr(gather), _ptr(w), _code(w), _ptr(tiles), tiles.shape[0], _ptr(out), _code(out), w.shape[1], w.shape[2],
              -1 if activation is None else ACTIVATIONS[activation], int(tile_rows), _stream()), "moe_expert")
    return out


def moe_combine(y: torch.Tensor, place_of_pair: torch.Tensor, weight: torch.Tensor, shared: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """out[t] = sum_j weight[t, j] y[place_of_pair[t top + j]] + shared[t] (float32; `shared` may come in slabs or be None)."""
    _dev(y, place_of_pair, weight, shared, out)
    _i32(place_of_pair, "place_of_pair")
    n, width = out.shape
    top = weight.shape[1]
    _need(y.dtype == weight.dtype == out.dtype == torch.float32 and y.shape == (n * top, width) and place_of_pair.numel() == n * top,
          "moe_combine: float32 y [tokens top, width], weight [tokens, top], out [tokens, width]")
    parts = 0
    if shared is not None:
        parts, rows, w2 = _slabs(shared, "moe_combine")
        _need((rows, w2) == (n, width), "moe_combine: shared is [tokens, width] or slabs of it")
    fn = _fn("moe", "kipp_moe_combine", [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(y), _ptr(place_of_pair), _ptr(weight), _ptr(shared), parts, _ptr(out), n, width, top, _stream()), "moe_combine")
    return out


def activate(u: torch.Tensor, out: torch.Tensor, activation: str, glu: bool = False, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(u), or with `glu` out[r, i] = act(u[r, i]) * u[r, inner + i]; `u` float32 [rows, width] or slabs of it;
    `bias` (float32 [width]) is added to u's columns first."""
    _dev(u, out, bias)
    parts, rows, width = _slabs(u, "activate")
    inner = out.shape[1]
    _need(out.shape[0] == rows and width == (2 * inner if glu else inner) and activation in ACTIVATIONS, "activate: shapes or activation")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == width), "activate: float32 bias over u's columns")
    fn = _fn("moe", "kipp_activate_biased", [_c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr])
    _check(fn(_ptr(u), parts, _ptr(out), _code(out), rows, inner, int(glu), ACTIVATIONS[activation], _ptr(bias), _stream()), "activate")
    return out


# --------------------------------------------------------------------------- attention with mixed heads

def _slabs(t: torch.Tensor, what: str):
    """(parts, rows, width) of a float32 product that may come in slabs [parts, rows, width]."""
    _need(t.dtype == torch.float32 and t.dim() in (2, 3), f"{what}: a float32 product [rows, width] or its slabs")
    return (1,) + tuple(t.shape) if t.dim() == 2 else tuple(t.shape)


def mixed_prepare(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                  n_q: int, n_kv: int, d: int, dv: int, q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float,
                  write_kv: bool = True) -> torch.Tensor:
    """From a step's projections `proj` (float32 [tokens, >= n_q d + n_kv d + n_kv dv], columns q | k | v | ..., or
    slabs of it): q and k RMS-normed over their whole width with plain weights, q kept in `q_out`, k and v
    written into the pages of their positions."""
    _dev(proj, q_out, k_cache, v_cache, positions, seq_of_token, block_table, q_weight, k_weight)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    parts, n, stride = _slabs(proj, "mixed_prepare")
    _need(stride >= n_q * d + n_kv * d + n_kv * dv, "mixed_prepare: the projections are narrower than q, k and v")
    _need(q_out.shape == (n, n_q * d) and positions.numel() == n and seq_of_token.numel() == n, "mixed_prepare: one row a token")
    _need(q_weight.dtype == torch.float32 and k_weight.dtype == torch.float32 and q_weight.numel() == n_q * d
          and k_weight.numel() == n_kv * d, "mixed_prepare: float32 norm weights over the whole projections")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[:3] == v_cache.shape[:3] and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == d and v_cache.shape[3] == dv and k_cache.dtype == v_cache.dtype,
          "mixed_prepare: caches must be [pages, n_kv, page, d] and [pages, n_kv, page, dv]")
    _need(block_table.dim() == 2, "mixed_prepare: block_table is [sequences, blocks]")
    fn = _fn("attention_mixed", "kipp_mixed_prepare",
             [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int,
              _c_ptr, _c_ptr, _c_ptr, _c_int] + [_c_int] * 7 + [_c_ptr])
    _check(fn(_ptr(proj), parts, stride, n_q * d, n_q * d + n_kv * d, _ptr(q_weight), _ptr(k_weight), float(eps),
              _ptr(q_out), _code(q_out), _ptr(k_cache), _ptr(v_cache), _code(k_cache), _ptr(positions), _ptr(seq_of_token),
              _ptr(block_table), block_table.shape[1], n, n_q, n_kv, d, dv, k_cache.shape[2], int(write_kv), _stream()),
           "mixed_prepare")
    return q_out


def _mixed_common(q, k_cache, v_cache, out, gate, gate_at, n_q, n_kv, d, dv, r1, r2, sink, mix, what):
    n = q.shape[0]
    _need(q.shape == (n, n_q * d) and out.shape == (n, n_q * dv), f"{what}: q is [tokens, n_q d], out [tokens, n_q dv]")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[:3] == v_cache.shape[:3] and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == d and v_cache.shape[3] == dv, f"{what}: caches must be [pages, n_kv, page, d] and [pages, n_kv, page, dv]")
    _need(n_kv > 0 and n_q % n_kv == 0, f"{what}: query heads must be a multiple of key/value heads")
    for t, size, name in ((r1, n_q, "r1"), (r2, n_q, "r2"), (sink, n_q, "sink"), (mix, n_q * n_q, "mix")):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == size), f"{what}: {name} must be float32 with {size} numbers")
    _need((r1 is None) == (r2 is None), f"{what}: the distance bias needs both of its numbers a head")
    gate_parts, gate_stride = 0, 0
    if gate is not None:
        gate_parts, rows, gate_stride = _slabs(gate, what)
        _need(rows == n and 0 <= gate_at and gate_at + n_q * dv <= gate_stride, f"{what}: the gate's columns lie outside its rows")
    return n, gate_parts, gate_stride


def mixed_attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                          positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                          n_q: int, n_kv: int, d: int, dv: int, scale: float, window: int, keep_first: int,
                          r1: Optional[torch.Tensor], r2: Optional[torch.Tensor], sink: Optional[torch.Tensor],
                          mix: Optional[torch.Tensor], gate: Optional[torch.Tensor] = None, gate_at: int = 0) -> torch.Tensor:
    """Attention with a distance bias, kept first keys beside a window, a sink in the softmax, heads mixed after the
    softmax and an output gate, for every token of a step (one workgroup a token; float32 or bfloat16 storage, float32
    arithmetic).  `gate`: a float32 product (or its slabs) whose columns from `gate_at` on hold the gate's logits."""
    _dev(q, k_cache, v_cache, out, positions, seq_of_token, block_table, r1, r2, sink, mix, gate)
    for t, name in ((positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    n, gate_parts, gate_stride = _mixed_common(q, k_cache, v_cache, out, gate, gate_at, n_q, n_kv, d, dv, r1, r2, sink, mix,
                                               "mixed_attention_plain")
    _need(0 < d <= 256 and 0 < dv <= 256 and n_q <= 64, "mixed_attention_plain: head sizes up to 256, up to 64 heads")
    lib = "attention_mixed"
    lds = _fn(lib, "kipp_mixed_attention_lds_bytes", [_c_int, _c_int])(n_q, d)
    _need(lds <= 64 * 1024, f"mixed_attention_plain: {n_q} heads of {d} need {lds} bytes of LDS, more than 65,536")
    fn = _fn(lib, "kipp_mixed_attention",
             [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
              _c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_int] * 6 + [_c_float, _c_int, _c_int, _c_ptr])
    gate_ptr = gate.data_ptr() + 4 * gate_at if gate is not None else None
    _check(fn(_ptr(q), _code(q), _ptr(k_cache), _ptr(v_cache), _code(k_cache), _ptr(out), _code(out), gate_ptr, gate_stride,
              gate_parts, _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1],
              _ptr(r1), _ptr(r2), _ptr(sink), _ptr(mix), n, n_q, n_kv, d, dv, k_cache.shape[2], float(scale),
              int(window), int(keep_first), _stream()), "mixed_attention_plain")
    return out


MIXED_ROWS = 16         # query rows of a tile of the matrix-core form
MIXED_KEYS = 32         # keys it takes at a time
MIXED_WAVES = 8


def mixed_attention_defines(n_q: int, n_kv: int, d: int, dv: int, sliced: bool = False) -> dict:
    """The build of attention_mixed_mfma.hip that takes these sizes.  `sliced`: the build in which several workgroups
    share an item, each with a part of the value columns (and all of the weights, computed again): twice the workgroups
    for a step that leaves compute units idle, and a wave's sums within 64 registers."""
    hpw = -(-n_q // MIXED_WAVES)
    blocks = dv // 16
    while sliced and hpw * blocks > 16 and blocks % 2 == 0:
        blocks //= 2
    return {"HEAD_DIM": d, "V_DIM": dv, "HPW": hpw, "SHARED_KV": int(hpw == 1 or (n_q // n_kv) % hpw == 0), "V_SLICE": 16 * blocks}


def mixed_attention_builds(n_q: int, n_kv: int, d: int, dv: int) -> list:
    """Both builds (one where slicing changes nothing)."""
    whole, sliced = mixed_attention_defines(n_q, n_kv, d, dv), mixed_attention_defines(n_q, n_kv, d, dv, sliced=True)
    return [whole] if whole == sliced else [whole, sliced]


def mixed_attention_fast_ok(n_q: int, d: int, dv: int, page: int) -> bool:
    """Whether the matrix-core form takes this geometry: key size a multiple of 32, value size a multiple of 16,
    up to 32 heads whose sums fit a wave's registers, pages of a multiple of 16 keys."""
    hpw = -(-n_q // MIXED_WAVES)
    return d % 32 == 0 and 0 < d <= 256 and dv % 16 == 0 and 0 < dv <= 256 and 0 < n_q <= 32 and hpw * (dv // 16) <= 32 \
        and page > 0 and page % 16 == 0


def mixed_attention_workspace(n_items: int, n_rows: int, n_q: int, dv: int, max_splits: int, device) -> tuple:
    """(statistics of every item, partial sums of the rows whose keys are cut into runs or None)."""
    stats = torch.empty((n_items, n_q, MIXED_ROWS, 2), dtype=torch.float32, device=device)
    partial = torch.empty((max_splits, n_rows, n_q * dv), dtype=torch.float32, device=device) if max_splits > 1 else None
    return stats, partial


def mixed_attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                         items: tuple, n_items: int, row_splits: Optional[torch.Tensor], max_splits: int,
                         q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor, block_table: torch.Tensor,
                         n_q: int, n_kv: int, d: int, dv: int, scale: float, window: int, keep_first: int,
                         r1: Optional[torch.Tensor], r2: Optional[torch.Tensor], sink: Optional[torch.Tensor],
                         mix: Optional[torch.Tensor], workspace: tuple, gate: Optional[torch.Tensor] = None,
                         gate_at: int = 0) -> torch.Tensor:
    """The same attention on the matrix cores (bfloat16).  `items`: four int32 tensors [n_items] (entry, first row of
    the tile within the entry, which run of the tile's keys, runs of the tile; a tile's items are consecutive);
    `row_splits` [rows]: the runs of each row's tile (needed when `max_splits` > 1); `workspace` from
    `mixed_attention_workspace`.  The kernels take every length from the device (`q_len`, `ctx_len`), so an item
    list made for longer contexts than the step's stays valid."""
    stats, partial = workspace
    _dev(q, k_cache, v_cache, out, *items, row_splits, q_start, q_len, ctx_len, block_table, r1, r2, sink, mix, gate, stats, partial)
    for t, name in ((q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len"), (block_table, "block_table")) \
            + tuple((t, "items") for t in items) + (((row_splits, "row_splits"),) if row_splits is not None else ()):
        _i32(t, name)
    n, gate_parts, gate_stride = _mixed_common(q, k_cache, v_cache, out, gate, gate_at, n_q, n_kv, d, dv, r1, r2, sink, mix,
                                               "mixed_attention_mfma")
    _need(all(t.dtype == torch.bfloat16 for t in (q, k_cache, v_cache, out)), "mixed_attention_mfma: bfloat16 queries, caches and output")
    _need(mixed_attention_fast_ok(n_q, d, dv, k_cache.shape[2]), "mixed_attention_mfma: sizes refused (the plain form takes them)")
    _need(len(items) == 4 and all(t.numel() >= n_items for t in items) and n_items > 0, "mixed_attention_mfma: four lists of n_items")
    _need(stats.numel() >= n_items * n_q * MIXED_ROWS * 2, "mixed_attention_mfma: the statistics' workspace is too small")
    _need(max_splits == 1 or (partial is not None and partial.numel() >= max_splits * n * n_q * dv and row_splits is not None
                              and row_splits.numel() >= n), "mixed_attention_mfma: cut keys need partial sums and the rows' runs")
    entries = q_start.numel()
    _need(q_len.numel() == entries and ctx_len.numel() == entries and block_table.dim() == 2 and block_table.shape[0] >= entries,
          "mixed_attention_mfma: one q_start, q_len, ctx_len and table row an entry")
    fn = _fn("attention_mixed_mfma", "kipp_mixed_attention_mfma",
             [_c_ptr] * 5 + [_c_int, _c_int] + [_c_ptr] * 4 + [_c_int, _c_ptr, _c_int] + [_c_ptr] * 4 + [_c_int] + [_c_ptr] * 6
             + [_c_int] * 6 + [_c_float, _c_int, _c_int, _c_ptr],
             # fewer items than compute units: the value columns are shared out over more workgroups
             mixed_attention_defines(n_q, n_kv, d, dv, sliced=n_items < COMPUTE_UNITS))
    gate_ptr = gate.data_ptr() + 4 * gate_at if gate is not None else None
    _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), gate_ptr, gate_stride, gate_parts,
              _ptr(items[0]), _ptr(items[1]), _ptr(items[2]), _ptr(items[3]), n_items, _ptr(row_splits), max_splits,
              _ptr(q_start), _ptr(q_len), _ptr(ctx_len), _ptr(block_table), block_table.shape[1],
              _ptr(r1), _ptr(r2), _ptr(sink), _ptr(mix), _ptr(stats), _ptr(partial),
              n, n_q, n_kv, d, dv, k_cache.shape[2], float(scale), int(window), int(keep_first), _stream()), "mixed_attention_mfma")
    return out


PREFILL_MAX_BLOCKS = 4096   # table entries of one sequence the prefill kernel stages in LDS


def attention_fast_ok(n_q: int, n_kv: int, page: int, max_blocks: int = 0) -> bool:
    """Whether the matrix-core attention kernels take this geometry."""
    return n_q // n_kv <= 16 and page > 0 and page & (page - 1) == 0 and max_blocks <= PREFILL_MAX_BLOCKS


DECODE_SPLIT = 256      # keys per workgroup of the decode kernel (checked against the library at load)
DECODE_SPLIT_MIN = 192  # ... and of its shortest splits (few sequences), which size the workspace
PREFILL_ROWS = 128      # query rows per workgroup of the prefill kernel (64 or 32 where that fills the GPU better)
COMPUTE_UNITS = 256     # of the MI355X (what the kernels' own plans assume); `compute_units()` asks the device
PREFILL_MIN_CUT = 512   # fewest keys of a cut of the prefill kernel's keys (below, the merge costs more than the cut gains)


def compute_units(device=None) -> int:
    """Compute units of the device at hand (the MI355X has 256), for host-side plans that fill the GPU."""
    if torch.cuda.is_available():
        return int(torch.cuda.get_device_properties(device if device is not None else torch.cuda.current_device()).multi_processor_count)
    return COMPUTE_UNITS


def attention_build_defines(head_dim: int, group: Optional[int] = None, capped: bool = False, chunked: bool = False, sink: bool = False) -> dict:
    """The constants of a build of the matrix-core attention kernels (`group` None: the kernel for prompt portions)."""
    defines = {"HEAD_DIM": head_dim}
    if group is not None:
        defines["GROUP"] = group
    if capped:
        defines["SOFTCAP"] = 1
    if chunked:
        defines["CHUNKED"] = 1
    if sink:
        defines["SINK"] = 1
    return defines


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     rows: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                     n_q: int, n_kv: int, head_dim: int, scale: float, window: int, max_context: int,
                     workspace: tuple, grid_splits: Optional[int] = None, capped: bool = False, chunked: bool = False,
                     sink: bool = False) -> torch.Tensor:
    """Attention of single query tokens (batch rows `rows`) over their pages.
    `chunked`: the build in which `window` is the length of a chunk: position p sees the keys from p - p % window on.
    `sink`: the build that adds one to the softmax's denominator (a key of score 0 that has no value).
    `capped`: the build whose scores pass tanh: `scale` is then the cap c, and q comes multiplied by (the score's
    scale / c), so that a weight is exp(c tanh(q . k scale / c) - maximum).
    `max_context`: the longest context among them (sizes the grid); `workspace`:
    (part_acc, part_ml, arrivals) from `attention_decode_workspace` (without `arrivals`, or with None for it,
    the splits are merged by a launch of its own instead of by the last workgroup of every head)."""
    _dev(q, k_cache, v_cache, out, rows, positions, seq_of_token, block_table, *workspace)
    for t, name in ((rows, "rows"), (positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    _attn_common(q, k_cache, v_cache, out, n_q, n_kv, head_dim, "attention_decode")
    group = n_q // n_kv
    _need(group <= 16, "attention_decode: more than 16 query heads per key/value head are refused")
    n_items = rows.numel()
    part_acc, part_ml, arrivals = _decode_workspace(workspace, n_items, n_kv, "attention_decode")
    max_splits = part_ml.numel() // max(1, n_items * n_q * 2)
    span = min(max_context, window) if window else max_context
    need = (span + DECODE_SPLIT - 1) // DECODE_SPLIT + (1 if window else 0)
    grid = grid_splits if grid_splits is not None else max(1, min(need, max_splits))
    _need(part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32
          and part_acc.numel() >= n_items * n_q * max_splits * head_dim and need <= max_splits,
          "attention_decode: workspace too small for this context")
    _need(not chunked or window > 0, "attention_decode: a chunk's length must be positive")
    defines = attention_build_defines(head_dim, group, capped, chunked, sink)
    fn = _fn("attention_decode", "kipp_attention_decode",
             [_c_ptr] * 10 + [_c_int] * 6 + [_c_float, _c_int, _c_int, _c_int, _c_ptr, _c_ptr], defines)
    _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(part_acc), _ptr(part_ml), _ptr(rows),
              _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], n_items, n_q, n_kv,
              head_dim, k_cache.shape[2], float(scale), int(window), grid, max_splits, _ptr(arrivals), _stream()),
           "attention_decode")
    return out


def _decode_workspace(workspace, n_items: int, n_kv: int, what: str):
    part_acc, part_ml = workspace[0], workspace[1]
    arrivals = workspace[2] if len(workspace) > 2 else None
    if arrivals is not None:
        _i32(arrivals, "arrivals")
        _need(arrivals.numel() >= n_items * n_kv, f"{what}: one count per token and key/value head")
    return part_acc, part_ml, arrivals


DECODE_FUSED_SLABS = 4


@functools.lru_cache(maxsize=None)
def attention_decode_streams(n_items: int, n_kv: int, head_dim: int, group: int, page: int, max_context: int,
                             window: int = 0) -> bool:
    """Does a decode launch of this shape go to the kernel that streams keys and values
    through LDS (many sequences: a workgroup a whole context; few sequences with long
    contexts: long ranges)?  Its fused form takes any number of rows and any context."""
    if head_dim % 16 or group > 16:
        return False
    span = min(max_context, window) if window else max_context
    splits = (span + DECODE_SPLIT - 1) // DECODE_SPLIT + (1 if window else 0)
    lib = build.library("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group})
    return bool(lib.kipp_attention_decode_ring_takes(int(n_items), int(n_kv), int(page), int(max(1, splits))))


def attention_decode_fused_ok(head_dim: int, rotary_dim: int, rotates: bool, slabs: int = 1) -> bool:
    """Can decode attention start from the QKV projection's output?  Head sizes that
    are multiples of 128, rotated over their whole width (or not at all), a
    projection in at most 4 slabs."""
    return head_dim % 128 == 0 and head_dim <= 256 and (not rotates or rotary_dim == head_dim) and slabs <= DECODE_FUSED_SLABS


def attention_decode_fused(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                           rows: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                           block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int,
                           q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], eps: float,
                           inv_freq: Optional[torch.Tensor], rotary_dim: int, write_kv: bool, scale: float, window: int,
                           max_context: int, workspace: tuple, grid_splits: Optional[int] = None,
                           angles: Optional[torch.Tensor] = None, out_steps_major: bool = False) -> torch.Tensor:
    """Decode attention straight from the QKV projection: per-head q/k RMSNorm,
    rotation, the write of the token's key and value into its page and the
    attention over the pages in one kernel (plus the merge of the splits).
    `qkv`: float32 [tokens, width] or slabs [parts, tokens, width].  `out_steps_major`: `out` is written in the
    order of `steps_major` (for the few-rows product that reads it next)."""
    _dev(qkv, k_cache, v_cache, out, rows, positions, seq_of_token, block_table, angles, *workspace)
    for t, name in ((rows, "rows"), (positions, "positions"), (seq_of_token, "seq_of_token"), (block_table, "block_table")):
        _i32(t, name)
    _angles_ok(angles, qkv.shape[-2], head_dim, "attention_decode_fused")
    _need(qkv.dtype == torch.float32 and qkv.dim() in (2, 3) and qkv.is_contiguous(), "attention_decode_fused: float32 qkv")
    parts = qkv.shape[0] if qkv.dim() == 3 else 1
    n_tokens = qkv.shape[-2]
    _need(qkv.shape[-1] == (n_q + 2 * n_kv) * head_dim, "attention_decode_fused: qkv width is not (n_q + 2 n_kv) head_dim")
    _need(attention_decode_fused_ok(head_dim, rotary_dim, inv_freq is not None, parts),
          "attention_decode_fused: head size a multiple of 128, rotated over its whole width, at most 4 slabs")
    _need(out.shape == (n_tokens, n_q * head_dim) and out.dtype == torch.bfloat16 and out.is_contiguous(),
          "attention_decode_fused: out is bfloat16 [tokens, n_q head_dim]")
    _need(k_cache.dtype == torch.bfloat16 and k_cache.shape == v_cache.shape and k_cache.shape[1] == n_kv
          and k_cache.shape[3] == head_dim and n_q % n_kv == 0, "attention_decode_fused: cache shape")
    for w, name in ((q_norm_w, "q_norm_w"), (k_norm_w, "k_norm_w")):
        _need(w is None or (w.dtype == torch.float32 and w.numel() == head_dim), f"attention_decode_fused: {name} float32 [head_dim]")
    _need(inv_freq is None or (inv_freq.dtype == torch.float32 and inv_freq.numel() == head_dim // 2),
          "attention_decode_fused: inv_freq float32 [head_dim / 2]")
    group = n_q // n_kv
    _need(group <= 16, "attention_decode_fused: more than 16 query heads per key/value head are refused")
    n_items = rows.numel()
    part_acc, part_ml, arrivals = _decode_workspace(workspace, n_items, n_kv, "attention_decode_fused")
    max_splits = part_ml.numel() // max(1, n_items * n_q * 2)
    span = min(max_context, window) if window else max_context
    need = (span + DECODE_SPLIT - 1) // DECODE_SPLIT + (1 if window else 0)
    grid = grid_splits if grid_splits is not None else max(1, min(need, max_splits))
    _need(part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32
          and part_acc.numel() >= n_items * n_q * max_splits * head_dim and need <= max_splits,
          "attention_decode_fused: workspace too small for this context")
    defines = {"HEAD_DIM": head_dim, "GROUP": group}
    fn = _fn("attention_decode", "kipp_attention_decode_fused",
             [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_int] + [_c_ptr] * 9 + [_c_int] * 6
             + [_c_float, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr], defines)
    null = lambda t: _ptr(t) if t is not None else None
    _check(fn(_ptr(qkv), parts, n_tokens, null(q_norm_w), null(k_norm_w), float(eps), null(inv_freq), null(angles),
              1 if write_kv else 0,
              _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(part_acc), _ptr(part_ml), _ptr(rows), _ptr(positions),
              _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], n_items, n_q, n_kv, head_dim,
              k_cache.shape[2], float(scale), int(window), grid, max_splits, _ptr(arrivals), int(bool(out_steps_major)), _stream()),
           "attention_decode_fused")
    return out


def attention_decode_workspace(n_items: int, n_q: int, head_dim: int, max_context: int, device) -> tuple:
    """(part_acc, part_ml, arrivals): room for every split's partial result, and a count per (token, key/value
    head) of the splits that have finished, which is zero between launches (the last to finish merges and sets
    it back).  One launch at a time may use a workspace."""
    max_splits = (max_context + DECODE_SPLIT_MIN - 1) // DECODE_SPLIT_MIN + 1       # the shortest splits a launch may take
    return (torch.empty(n_items * n_q * max_splits * head_dim, dtype=torch.float32, device=device),
            torch.empty(n_items * n_q * max_splits * 2, dtype=torch.float32, device=device),
            torch.zeros(n_items * n_q, dtype=torch.int32, device=device))


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                      item_seq: torch.Tensor, item_tile: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                      positions: torch.Tensor, block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int,
                      scale: float, window: int = 0, tile_rows: int = 128, cuts=None, capped: bool = False, chunked: bool = False,
                      sink: bool = False) -> torch.Tensor:
    """Attention of prompt portions: work item i is the `item_tile[i]`-th tile
    of `tile_rows` (128, 64 or 32) query rows of sequence `item_seq[i]`.
    `chunked`: the build in which `window` is the length of a chunk: position p sees the keys from p - p % window on.
    `sink`: the build that adds one to the softmax's denominator (a key of score 0 that has no value); not with `cuts`.
    `capped`: the build whose scores pass tanh: `scale` is then the cap c, and q comes multiplied by (the score's
    scale / c), so that a weight is exp(c tanh(q . k scale / c) - maximum).

    `cuts` = (split_keys, item_split, merge_rows, merge_cuts, workspace): the keys are cut at multiples of
    `split_keys` (a multiple of 64), work item i takes cut `item_split[i]` of its tile's keys, and the rows
    `merge_rows[j]` (each with `merge_cuts[j]` cuts) are merged afterwards, in the order of the cuts.
    `workspace` = (part_acc, part_ml) float32 from `attention_prefill_workspace`.  For few, long work items,
    which alone would leave most compute units idle; not with a window."""
    _dev(q, k_cache, v_cache, out, item_seq, item_tile, q_start, q_len, positions, block_table)
    _need(tile_rows in (32, 64, 128), "attention_prefill: tiles of 32, 64 or 128 query rows")
    for t, name in ((item_seq, "item_seq"), (item_tile, "item_tile"), (q_start, "q_start"), (q_len, "q_len"),
                    (positions, "positions"), (block_table, "block_table")):
        _i32(t, name)
    _attn_common(q, k_cache, v_cache, out, n_q, n_kv, head_dim, "attention_prefill")
    _need(item_seq.numel() == item_tile.numel(), "attention_prefill: one tile index per work item")
    _need(block_table.shape[1] <= PREFILL_MAX_BLOCKS, "attention_prefill: more pages per sequence than the kernel stages")
    _need(not chunked or window > 0, "attention_prefill: a chunk's length must be positive")
    _need(not (sink and cuts is not None), "attention_prefill: the added one in the denominator does not go with cuts of the keys")
    split_keys, item_split, merge_rows, merge_cuts, part_acc, part_ml, max_splits = 0, None, None, None, None, None, 0
    if cuts is not None:
        split_keys, item_split, merge_rows, merge_cuts, (part_acc, part_ml) = cuts
        _dev(item_split, merge_rows, merge_cuts, part_acc, part_ml)
        for t, name in ((item_split, "item_split"), (merge_rows, "merge_rows"), (merge_cuts, "merge_cuts")):
            _i32(t, name)
        rows = q.shape[0]
        max_splits = part_ml.numel() // max(1, rows * n_q * 2)
        _need(window == 0 and split_keys > 0 and split_keys % 64 == 0 and item_split.numel() == item_seq.numel()
              and merge_rows.numel() == merge_cuts.numel() and part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32
              and max_splits >= 1 and part_acc.numel() >= rows * n_q * max_splits * head_dim,
              "attention_prefill: cuts need no window, a multiple of 64 keys, one cut per work item and a workspace for every row")
    fn = _fn("attention_prefill", "kipp_attention_prefill",
             [_c_ptr] * 10 + [_c_int] * 6 + [_c_float, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int,
                                             _c_ptr], attention_build_defines(head_dim, None, capped, chunked, sink))
    _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(item_seq), _ptr(item_tile), _ptr(q_start),
              _ptr(q_len), _ptr(positions), _ptr(block_table), block_table.shape[1], item_seq.numel(), n_q, n_kv,
              head_dim, k_cache.shape[2], float(scale), int(window), int(tile_rows), _ptr(item_split), int(split_keys),
              _ptr(part_acc), _ptr(part_ml), int(max_splits), _ptr(merge_rows), _ptr(merge_cuts),
              merge_rows.numel() if merge_rows is not None else 0, _stream()), "attention_prefill")
    return out


def attention_prefill_workspace(rows: int, n_q: int, head_dim: int, max_splits: int, device) -> tuple:
    """(part_acc, part_ml) for `attention_prefill(..., cuts=...)`: sums and (maximum, denominator) of every cut."""
    return (torch.empty(rows * n_q * max_splits * head_dim, dtype=torch.float32, device=device),
            torch.empty(rows * n_q * max_splits * 2, dtype=torch.float32, device=device))


# --------------------------------------------------------------------------- matrix products

SKINNY_MAX_ROWS = 64     # rows the few-rows kernel takes
SKINNY_BEST_ROWS = 12    # ... and rows up to which it is the faster one (each wave reads its rows of x itself; beyond, x staged in LDS wins:
                         # with rows in steps-major order a step at 12 rows takes 3.02 ms this way against 3.22, at 16 rows 3.58 against 3.56)
ROWS_MAX_ROWS = 256      # rows of the kernel that stages x through LDS
ROWS_BEST_ROWS = 192     # beyond these the product built for hundreds of rows is faster where it takes the shape (measured)


def gemm_rows_ok(m: int, k: int) -> bool:
    """Shapes our own streaming products take: at most 256 rows, K a multiple of 8 and at least 32."""
    return 0 < m <= ROWS_MAX_ROWS and k % 8 == 0 and k >= 32


def gemm_skinny_ok(m: int, k: int) -> bool:
    """Shapes the few-rows kernel takes: at most 64 rows, K a multiple of 8 and at least 32."""
    return 0 < m <= SKINNY_MAX_ROWS and k % 8 == 0 and k >= 32


def _tile(block: torch.Tensor) -> torch.Tensor:
    """[16 t, K] rows -> [tile][step of 32 columns][lane][8 values], lane l = row l % 16, columns 8 (l / 16) .. + 7."""
    rows, k = block.shape
    return block.view(rows // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1)


def _pad_rows(block: torch.Tensor, multiple: int) -> torch.Tensor:
    rest = -block.shape[0] % multiple
    return block if not rest else torch.cat([block, torch.zeros((rest, block.shape[1]), dtype=block.dtype, device=block.device)])


def tile_weight(w: torch.Tensor) -> torch.Tensor:
    """The streaming layout of a bfloat16 matrix [N, K], K a multiple of 32: the
    1 KB a wave reads in one step (16 rows x 32 columns) is contiguous,
    [tile of 16 rows][step of 32 columns][lane][8 values] with lane l holding row
    l % 16 and columns 8 (l / 16) .. + 7 of the step.  The rows are padded to
    whole tiles with zeros."""
    _need(w.dim() == 2 and w.dtype == torch.bfloat16, "tile_weight: a bfloat16 matrix")
    _need(w.shape[1] % 32 == 0, "tile_weight: K a multiple of 32")
    return _tile(_pad_rows(w, 16))


def tile_weight_pairs(w_gate_up: torch.Tensor) -> torch.Tensor:
    """The streaming layout of [gate; up] ([2 I, K]) for the product that ends in
    SwiGLU: tile t holds gate rows 8 t .. 8 t + 7 over up rows 8 t .. 8 t + 7, so
    that one tile gives 8 finished outputs (I padded to a multiple of 8 with zeros).
    As a plain tiled matrix it is the weight with its rows in that order."""
    _need(w_gate_up.dim() == 2 and w_gate_up.dtype == torch.bfloat16, "tile_weight_pairs: a bfloat16 matrix")
    two_inner, k = w_gate_up.shape
    _need(k % 32 == 0 and two_inner % 2 == 0, "tile_weight_pairs: K a multiple of 32, gate and up of equal height")
    inner = two_inner // 2
    gate, up = _pad_rows(w_gate_up[:inner], 8), _pad_rows(w_gate_up[inner:], 8)
    return _tile(torch.cat([gate.view(-1, 8, k), up.view(-1, 8, k)], dim=1).view(-1, k))


def tile_weight_device(w: torch.Tensor, gate_up: bool = False) -> torch.Tensor:
    """`tile_weight(w)` (or `tile_weight_pairs(w)` with `gate_up`) by the kernel that hosts without torch use."""
    _dev(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and w.is_contiguous() and w.shape[1] % 32 == 0,
          "tile_weight_device: a contiguous bfloat16 matrix, K a multiple of 32")
    n, k = w.shape
    _need(not gate_up or n % 2 == 0, "tile_weight_device: gate and up of equal height")
    inner = n // 2 if gate_up else 0
    tile_count = (inner + 7) // 8 if gate_up else (n + 15) // 16
    out = torch.empty(tile_count * 16 * k, dtype=torch.bfloat16, device=w.device)
    fn = _fn("elementwise", "kipp_tile_weight", [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(w), _ptr(out), n, k, inner, _stream()), "tile_weight_device")
    return out


def pairs_width(inner: int) -> int:
    """Columns of a product from paired tiles: 16 for every 8 outputs."""
    return 16 * ((inner + 7) // 8)


def _tiles_ok(tiles, n: int, k: int, what: str) -> int:
    if tiles is None:
        return 0
    _need(tiles.dtype == torch.bfloat16 and tiles.is_contiguous() and k % 32 == 0
          and tiles.numel() == ((n + 15) // 16) * 16 * k, f"{what}: the tiled weight does not match [N, K]")
    return 1


def _row_scale_args(row_scale, m: int, what: str):
    """(sumsq pointer, parts, eps) of `row_scale` = (sumsq, parts, eps), sumsq float32 [M, parts rounded up to 4]."""
    if row_scale is None:
        return None, 0, 0.0
    sumsq, parts, eps = row_scale
    _dev(sumsq)
    _need(m <= 16 and sumsq.dtype == torch.float32 and sumsq.dim() == 2 and parts > 0
          and tuple(sumsq.shape) == (m, (parts + 3) // 4 * 4) and sumsq.is_contiguous(),
          f"{what}: row_scale is (float32 [M, parts rounded up to 4], parts, eps), for at most 16 rows")
    return _ptr(sumsq), int(parts), float(eps)


def gemm_skinny_parts(n: int, k: int, max_parts: int) -> int:
    """Slabs `gemm_skinny` cuts a product against a weight [n, k] into when it may use up to `max_parts`."""
    return build.library("gemm_skinny").kipp_gemm_skinny_parts(int(n), int(k), int(max_parts))


def steps_major(rows: torch.Tensor) -> torch.Tensor:
    """bfloat16 rows [M, K] (K a multiple of 32) as [K / 32][M][32], the order the few-rows products may read and write
    their rows in (`x_steps_major`, `out_steps_major`): what a wave reads of x in one step is then one run of memory."""
    m, k = rows.shape
    _need(k % 32 == 0, "steps_major: whole runs of 32 columns")
    return rows.view(m, k // 32, 32).transpose(0, 1).contiguous().view(m, k)


def from_steps_major(rows: torch.Tensor) -> torch.Tensor:
    """The inverse of `steps_major`: [K / 32][M][32] (held as a tensor of shape [M, K]) back to [M, K]."""
    m, k = rows.shape
    return rows.view(k // 32, m, 32).transpose(0, 1).contiguous().view(m, k)


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, max_parts: int = 1, tiles: torch.Tensor = None,
                row_scale=None, add_norm=None, x_steps_major: bool = False, out_steps_major: bool = False):
    """float32 [parts, M, N] whose sum over parts is x . w^T, for M <= 64 rows of
    bfloat16 x against bfloat16 w [N, K].  parts <= max_parts is chosen from the
    shape (1 when the weight has many rows).  With `tiles` (tile_weight(w)) the
    weight is streamed from that layout.

    `row_scale` = (sumsq [M, P rounded up to 4], P, eps), M <= 16: row t of the
    product is multiplied by rsqrt(sum(sumsq[t, :P]) / K + eps), i.e. x holds rows
    of an RMS norm that still lack their scale.
    `add_norm` = (residual float32 [M, N], norm_weight float32 [N]), M <= 16: the product
    (in one part) is added to `residual` in place by the kernel itself and the
    call returns (rows, sumsq) instead: rows = bfloat16(residual * norm_weight)
    and sumsq [M, P rounded up to 4] with P = ceil(N / 16) sums a row: (sumsq, P, eps)
    is the `row_scale` of the next product.
    `x_steps_major`: x holds its values as `steps_major` orders them; `out_steps_major`: so do the rows that
    `add_norm` returns (both need the width in question to be a multiple of 32)."""
    _dev(x, w)
    m, k = x.shape
    n = w.shape[0]
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 operands")
    _need(w.shape == (n, k), "gemm_skinny: shapes do not match")
    _need(gemm_skinny_ok(m, k), "gemm_skinny: at most 64 rows, K a multiple of 8 and at least 32")
    _need(not x_steps_major or k % 32 == 0, "gemm_skinny: rows in steps-major order need K a multiple of 32")
    _need(not out_steps_major or (add_norm is not None and n % 32 == 0), "gemm_skinny: steps-major rows come from add_norm, N a multiple of 32")
    lib = build.library("gemm_skinny")
    tiled = _tiles_ok(tiles, n, k, "gemm_skinny")
    sumsq, sumsq_parts, eps = _row_scale_args(row_scale, m, "gemm_skinny")
    residual = norm_w = rows = sumsq_out = out = None
    if add_norm is None:
        parts = lib.kipp_gemm_skinny_parts(n, k, int(max_parts))
        out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
    else:
        residual, norm_w = add_norm
        _dev(residual, norm_w)
        _need(m <= 16 and residual.dtype == torch.float32 and residual.shape == (m, n) and residual.is_contiguous(),
              "gemm_skinny: the residual is float32 [M, N], at most 16 rows")
        _need(norm_w.dtype == torch.float32 and norm_w.numel() == n, "gemm_skinny: the norm weight is float32 [N]")
        rows = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        sumsq_out = torch.empty((m, ((n + 15) // 16 + 3) // 4 * 4), dtype=torch.float32, device=x.device)
    fn = _fn("gemm_skinny", "kipp_gemm_skinny",
             [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float,
              _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(tiles if tiled else w), _ptr(out), m, n, k, int(max_parts), tiled, sumsq, sumsq_parts, eps,
              _ptr(residual), _ptr(norm_w), _ptr(rows), _ptr(sumsq_out), int(bool(x_steps_major)), int(bool(out_steps_major)),
              _stream()), "gemm_skinny")
    return out if add_norm is None else (rows, sumsq_out)


def scale_rows(rows: torch.Tensor, sumsq: torch.Tensor, parts: int, eps: float, out: torch.Tensor,
               steps_major: bool = False) -> torch.Tensor:
    """out[t] = rows[t] * rsqrt(sum(sumsq[t, :parts]) / width + eps), bfloat16: the rows of an RMS norm
    from what `gemm_skinny(..., add_norm=...)` returns, for a consumer that does not take `row_scale`
    (`steps_major`: `rows` were written in that order; `out` is [M, width] rows all the same)."""
    _dev(rows, sumsq, out)
    m, width = rows.shape
    _need(rows.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.shape == rows.shape
          and sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[0] == m and 0 < parts <= sumsq.shape[1]
          and sumsq.is_contiguous(), "scale_rows: shapes or types differ")
    fn = _fn("elementwise", "kipp_scale_rows", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr])
    _check(fn(_ptr(rows), _ptr(sumsq), _ptr(out), m, width, int(parts), sumsq.shape[1], float(eps), int(bool(steps_major)), _stream()),
           "scale_rows")
    return out


def gemm_rows(x: torch.Tensor, w: torch.Tensor, max_parts: int = 1, tiles: torch.Tensor = None,
              pairs: bool = False, cut: int = 0) -> torch.Tensor:
    """float32 [parts, M, N] whose sum over parts is x . w^T, for 8 < M <= 256 rows
    (any M <= 256 is taken): the rows of x are staged through LDS and shared by
    the waves of a workgroup.  `pairs`: `tiles` is tile_weight_pairs(w), w = [gate; up];
    the product then has `pairs_width(inner)` columns in the order of those tiles
    (what `swiglu(..., pairs=True)` takes).
    `cut` (measurements and tests): 10 x waves of a workgroup (4 to 8) + tiles of 16 rows a wave (1 or 2),
    with exactly `max_parts` parts of K."""
    _dev(x, w)
    m, k = x.shape
    n = w.shape[0]
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows: bfloat16 operands")
    _need(w.shape == (n, k), "gemm_rows: shapes do not match")
    _need(0 < m <= ROWS_MAX_ROWS and k % 8 == 0, "gemm_rows: at most 256 rows and K a multiple of 8")
    if pairs:
        _need(tiles is not None and n % 2 == 0, "gemm_rows: pairs need the paired tiles of [gate; up]")
        n = pairs_width(n // 2)
    lib = build.library("gemm_rows")
    parts = lib.kipp_gemm_rows_parts(m, n, k, int(max_parts)) if not cut else min(int(max_parts), max(1, k // rows_chunk(m)))
    out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
    tiled = _tiles_ok(tiles, n, k, "gemm_rows")
    fn = _fn("gemm_rows", "kipp_gemm_rows", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(tiles if tiled else w), _ptr(out), m, n, k, int(max_parts), tiled, int(cut), _stream()), "gemm_rows")
    return out


def rows_chunk(m: int) -> int:
    """Columns of x that `gemm_rows` stages at a time (every part of K is at least one such chunk)."""
    return 64 if m > 128 else (128 if m > 64 else 256)


def gemm_rows_swiglu_pays(m: int, two_inner: int, k: int) -> bool:
    """Whether `gemm_rows_swiglu` is the faster way for this shape (it does not split K: where the weight has too few
    rows for that, the split product and `swiglu` are faster)."""
    return bool(build.library("gemm_rows").kipp_gemm_rows_swiglu_pays(int(m), int(two_inner), int(k)))


def gemm_rows_swiglu(x: torch.Tensor, tiles: torch.Tensor, out: torch.Tensor, cut: int = 0) -> torch.Tensor:
    """out[M, I] (bfloat16) = silu(x . w_gate^T) * (x . w_up^T) for up to 256 rows; `tiles` = tile_weight_pairs([gate; up]).
    `cut`: as in `gemm_rows`."""
    _dev(x, tiles, out)
    m, k = x.shape
    inner = out.shape[1]
    _need(x.dtype == torch.bfloat16 and tiles.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.is_contiguous()
          and x.is_contiguous(), "gemm_rows_swiglu: bfloat16 operands and output")
    _need(0 < m <= ROWS_MAX_ROWS and k % 32 == 0 and out.shape[0] == m, "gemm_rows_swiglu: at most 256 rows and K a multiple of 32")
    _tiles_ok(tiles, pairs_width(inner), k, "gemm_rows_swiglu")
    fn = _fn("gemm_rows", "kipp_gemm_rows_swiglu", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(tiles), _ptr(out), m, 2 * inner, k, int(cut), _stream()), "gemm_rows_swiglu")
    return out


def gemm_skinny_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, tiles: torch.Tensor = None,
                       row_scale=None, x_steps_major: bool = False, out_steps_major: bool = False) -> torch.Tensor:
    """out[M, I] (bfloat16) = silu(x . w_gate^T) * (x . w_up^T), w_gate_up = [gate; up] of [2 I, K];
    `tiles` = tile_weight_pairs(w_gate_up).  The same bits from both layouts.
    `row_scale`, `x_steps_major`: as in `gemm_skinny` (both products are scaled before the activation);
    `out_steps_major`: `out` is written in the order of `steps_major` (I a multiple of 32)."""
    _dev(x, w_gate_up, out)
    m, k = x.shape
    two_inner = w_gate_up.shape[0]
    _need(x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          "gemm_skinny_swiglu: bfloat16 operands and output")
    _need(w_gate_up.shape == (two_inner, k) and two_inner % 2 == 0 and out.shape == (m, two_inner // 2),
          "gemm_skinny_swiglu: shapes do not match")
    _need(gemm_skinny_ok(m, k), "gemm_skinny_swiglu: at most 64 rows, K a multiple of 8 and at least 32")
    _need((not x_steps_major or k % 32 == 0) and (not out_steps_major or (two_inner // 2) % 32 == 0),
          "gemm_skinny_swiglu: rows in steps-major order need their width to be a multiple of 32")
    tiled = _tiles_ok(tiles, pairs_width(two_inner // 2), k, "gemm_skinny_swiglu")
    sumsq, sumsq_parts, eps = _row_scale_args(row_scale, m, "gemm_skinny_swiglu")
    fn = _fn("gemm_skinny", "kipp_gemm_skinny_swiglu",
             [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(tiles if tiled else w_gate_up), _ptr(out), m, two_inner, k, tiled, sumsq, sumsq_parts, eps,
              int(bool(x_steps_major)), int(bool(out_steps_major)), _stream()), "gemm_skinny_swiglu")
    return out


TILES_END = {"slabs": 0, "swiglu": 1, "bf16": 2}


def gemm_tiles_ok(m: int, k: int, n: int = 1) -> bool:
    """Shapes the product for prompt portions takes: K a multiple of 32 (any number of rows; it is built for
    hundreds), each operand under 4 GiB (a lane's offset into it is 32 bits wide)."""
    return m > 0 and k > 0 and k % 32 == 0 and max(m, n) * k * 2 < 2**32


def gemm_tiles_parts(m: int, n: int, k: int, end: str = "slabs", max_parts: int = 1) -> int:
    """Parts of K the launcher plans for a product of these sizes when it may use up to `max_parts`."""
    return int(build.library("gemm_tiles").kipp_gemm_tiles_parts(int(m), int(n), int(k), TILES_END[end], int(max_parts)))


def gemm_tiles(x: torch.Tensor, w: torch.Tensor, end: str = "slabs", max_parts: int = 1, force: int = 0) -> torch.Tensor:
    """x [M, K] . w [N, K]^T on the matrix cores for many rows, bfloat16 operands, float32 accumulation.
    end "slabs": float32 [parts, M, N] whose sum over parts is the product (parts <= max_parts, chosen from the shape);
    "swiglu": w = [gate; up] of [2 I, K], the result is bfloat16 [M, I] = silu(x . gate^T) * (x . up^T);
    "bf16": bfloat16 [M, N].  `force` = 100 wm + 10 wn + parts (+ 1000: workgroups of 8 waves, four across, wave tiles
    4 x 2 or 2 x 2; + 2000, bfloat16 ends: those for the whole rounds of 256 tiles and smaller tiles for the columns
    that are left, 8 waves on half the rows or, + 10000 r, 4 waves on 256 x 64, 128 x 128 or 128 x 64 outputs) takes
    that cut instead of the planned one (the runtime's timed choice, tests)."""
    _dev(x, w)
    m, k = x.shape
    n = w.shape[0]
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_tiles: bfloat16 operands")
    _need(w.shape == (n, k) and gemm_tiles_ok(m, k), "gemm_tiles: shapes do not match, or K is no multiple of 32")
    _need(end in TILES_END, f"gemm_tiles: end {end!r} is not one of {sorted(TILES_END)}")
    code = TILES_END[end]
    lib = build.library("gemm_tiles")
    if end == "slabs":
        parts = force % 10 if force else lib.kipp_gemm_tiles_parts(m, n, k, code, int(max_parts))
        _need(parts >= 1, "gemm_tiles: no cut for these sizes")
        out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
    elif end == "swiglu":
        _need(n % 2 == 0, "gemm_tiles: [gate; up] has an even number of rows")
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    fn = _fn("gemm_tiles", "kipp_gemm_tiles", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(w), _ptr(out), m, n, k, code, int(max_parts), int(force), _stream()), "gemm_tiles")
    return out


def gemm_f32(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M,N] = x[M,K] . w[N,K]^T in true float32 (w float32 or bfloat16)."""
    _dev(x, w, out)
    _need(x.dtype == torch.float32 and out.dtype == torch.float32, "gemm_f32: x and out are float32")
    m, k = x.shape
    n = w.shape[0]
    _need(w.shape == (n, k) and out.shape == (m, n), "gemm_f32: shapes do not match [M,K] x [N,K] -> [M,N]")
    fn = _fn("gemm_f32", "kipp_gemm_f32", [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(w), _code(w), _ptr(out), m, n, k, _stream()), "gemm_f32")
    return out


# --------------------------------------------------------------------------- probe

def stream_read(buffer: torch.Tensor, workgroups: int, depth: int = 8) -> int:
    """Reads `buffer` once with `workgroups` x 4 waves, `depth` 16-byte loads a lane in
    flight; returns the bytes read (what the grid covers in whole rings)."""
    _dev(buffer)
    _need(buffer.is_contiguous() and depth in (4, 8, 16), "stream_read: a contiguous buffer, depth 4, 8 or 16")
    lib = build.library("probe")
    fn = lib.kipp_probe_stream_read
    fn.restype = ctypes.c_longlong
    fn.argtypes = [_c_ptr, ctypes.c_longlong, _c_int, _c_int, _c_ptr, _c_ptr]
    sink = torch.zeros(1, dtype=torch.int32, device=buffer.device)
    got = fn(_ptr(buffer), buffer.numel() * buffer.element_size(), int(workgroups), int(depth), _ptr(sink), _stream())
    _need(got > 0, "stream_read: buffer too small for this grid")
    return int(got)


def mfma_rate(data: torch.Tensor, workgroups: int, accumulators: int, iters: int) -> int:
    """Launches the probe that only multiplies (32x32x16 bfloat16 products from registers, `accumulators` = 8 or 16
    independent sums a wave, `workgroups` of 4 waves); `data`: 16 KiB whose bits are the operands.  Returns the
    floating-point operations launched."""
    _dev(data)
    _need(data.is_contiguous() and data.numel() * data.element_size() == 16384 and accumulators in (8, 16),
          "mfma_rate: 16 KiB of operand bits, 8 or 16 accumulators")
    fn = build.library("probe").kipp_probe_mfma_rate
    fn.restype = ctypes.c_longlong
    fn.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]
    sink = torch.zeros(1, dtype=torch.int32, device=data.device)
    got = fn(_ptr(data), int(workgroups), int(accumulators), int(iters), _ptr(sink), _stream())
    _need(got > 0, "mfma_rate: refused")
    return int(got)


# --------------------------------------------------------------------------- sampling

def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, out)
    _i32(out, "argmax output")
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and out.numel() == logits.shape[0],
          "argmax: float32 [rows, vocab] and one int32 per row")
    rows = logits.shape[0]
    scratch = torch.empty(build.library("sampling").kipp_argmax_scratch_floats(rows), dtype=torch.float32, device=logits.device)
    fn = _fn("sampling", "kipp_argmax", [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr])
    _check(fn(_ptr(logits), _ptr(out), rows, logits.shape[1], _ptr(scratch), _stream()), "argmax")
    return out


def row_nll(logits: torch.Tensor, targets: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[r] = -log softmax(logits[r])[targets[r]] in float64 (the maximum in float32, exponentials and their sum in
    float64): what a perplexity run adds up."""
    _dev(logits, targets, out)
    _i32(targets, "targets")
    rows = logits.shape[0]
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "row_nll: float32 [rows, vocab]")
    _need(targets.numel() == rows and out.numel() == rows and out.dtype == torch.float64, "row_nll: one target and one float64 a row")
    fn = _fn("sampling", "kipp_row_nll", [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr])
    _check(fn(_ptr(logits), rows, logits.shape[1], _ptr(targets), _ptr(out), _stream()), "row_nll")
    return out


def adjust_logits(logits: torch.Tensor, begin: torch.Tensor, biases: torch.Tensor, token: torch.Tensor, value: torch.Tensor,
                  repetition: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor) -> torch.Tensor:
    """Logit bias and the penalties over recent tokens, applied to rows of float32 logits in place, in the host
    sampler's order and with its float operations: row r's entries are begin[r] .. begin[r + 1], the first biases[r]
    of them biases (value: the bias), the others distinct recent tokens (value: how often each occurs); tokens lie
    inside the vocabulary."""
    _dev(logits, begin, biases, token, value, repetition, presence, frequency)
    _i32(begin, "begin")
    _i32(biases, "biases")
    _i32(token, "token")
    rows = logits.shape[0]
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "adjust_logits: float32 [rows, vocab]")
    _need(begin.numel() == rows + 1 and all(t.numel() == rows for t in (biases, repetition, presence, frequency)),
          "adjust_logits: one value per row, rows + 1 begins")
    _need(token.numel() == value.numel() and all(t.dtype == torch.float32 for t in (value, repetition, presence, frequency)),
          "adjust_logits: one float32 value per entry, float32 penalties")
    fn = _fn("sampling", "kipp_adjust_logits", [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr])
    _check(fn(_ptr(logits), rows, logits.shape[1], _ptr(begin), _ptr(biases), _ptr(token), _ptr(value), _ptr(repetition),
              _ptr(presence), _ptr(frequency), _stream()), "adjust_logits")
    return logits


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """One token for each row of float32 logits: greedy where temperature <= 0,
    else temperature sampling with top-k (0: off), min-p (0: off) and top-p, using
    the row's uniform draw in [0, 1) (float64) made on the host."""
    _dev(logits, temperature, top_k, top_p, min_p, uniform, out)
    _i32(top_k, "top_k")
    _i32(out, "sample output")
    rows = logits.shape[0]
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample: float32 [rows, vocab]")
    _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32 and min_p.dtype == torch.float32
          and uniform.dtype == torch.float64, "sample: float32 parameters and float64 draws")
    _need(all(t.numel() == rows for t in (temperature, top_k, top_p, min_p, uniform, out)), "sample: one value per row")
    _need(logits.shape[1] < (1 << 24), "sample: the vocabulary must be below 2^24")
    fn = _fn("sampling", "kipp_sample", [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr])
    _check(fn(_ptr(logits), rows, logits.shape[1], _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(min_p),
              _ptr(uniform), _ptr(out), _stream()), "sample")
    return out
