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


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     rows: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                     n_q: int, n_kv: int, head_dim: int, scale: float, window: int, max_context: int,
                     workspace: tuple, grid_splits: Optional[int] = None) -> torch.Tensor:
    """Attention of single query tokens (batch rows `rows`) over their pages.
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
    defines = {"HEAD_DIM": head_dim, "GROUP": group}
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
                      scale: float, window: int = 0, tile_rows: int = 128, cuts=None) -> torch.Tensor:
    """Attention of prompt portions: work item i is the `item_tile[i]`-th tile
    of `tile_rows` (128, 64 or 32) query rows of sequence `item_seq[i]`.

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
                                             _c_ptr], {"HEAD_DIM": head_dim})
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
