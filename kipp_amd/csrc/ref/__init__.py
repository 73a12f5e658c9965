"""The scalar C references of the kernels (`ref_ops.c`), callable from Python on NumPy arrays.

They are compiled into the C host's library (its scalar path is made of them); this module binds the same functions
so that a kernel test can set each kernel beside its reference.  Arrays are float32 (bfloat16 storage: uint16 bits).
"""
from __future__ import annotations

import ctypes

import numpy as np

_lib = None
F32, BF16 = 0, 1


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        from ...host import build
        _lib = ctypes.CDLL(build.library_path("host-only"))
        vp, sz, i32, f32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float
        _lib.ref_embed.argtypes = [vp, i32, vp, vp, sz, sz]
        _lib.ref_rms_norm.argtypes = [vp, vp, vp, sz, f32]
        _lib.ref_matvec.argtypes = [vp, i32, vp, vp, sz, sz]
        _lib.ref_head_norm.argtypes = [vp, sz, sz, vp, f32]
        _lib.ref_rope.argtypes = [vp, sz, ctypes.c_int32, vp, i32]
        _lib.ref_softmax.argtypes = [vp, sz]
        _lib.ref_silu.argtypes, _lib.ref_silu.restype = [f32], f32
        _lib.ref_swiglu.argtypes = [vp, vp, sz]
        _lib.ref_kv_write.argtypes = [vp, vp, i32, vp, sz, sz, sz, sz, vp, vp]
        _lib.ref_paged_gqa.argtypes = [vp, vp, vp, i32, vp, sz, sz, sz, sz, sz, sz, f32, vp, vp]
        _lib.ref_causal_gqa.argtypes = [vp, vp, vp, sz, sz, sz, sz, sz, f32, vp, vp]
        _lib.ref_argmax.argtypes, _lib.ref_argmax.restype = [vp, sz], ctypes.c_uint32
        _lib.ref_float_to_bf16.argtypes, _lib.ref_float_to_bf16.restype = [f32], ctypes.c_uint16
        _lib.ref_bf16_to_float.argtypes, _lib.ref_bf16_to_float.restype = [ctypes.c_uint16], f32
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _stored(a: np.ndarray):
    """(array, dtype code) of a weight or cache: float32 as it is, uint16 as bfloat16 bits."""
    if a.dtype == np.uint16:
        return np.ascontiguousarray(a), BF16
    return _f32(a), F32


def embed(table: np.ndarray, tokens) -> np.ndarray:
    table, code = _stored(table)
    tokens = np.ascontiguousarray(tokens, dtype=np.int32)
    out = np.empty((len(tokens), table.shape[1]), dtype=np.float32)
    lib().ref_embed(_p(table), code, _p(tokens), _p(out), len(tokens), table.shape[1])
    return out


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    x, weight = _f32(x), _f32(weight)
    out = np.empty_like(x)
    for r in range(x.shape[0]):
        lib().ref_rms_norm(_p(x[r]), _p(weight), _p(out[r]), x.shape[1], eps)
    return out


def linear(x: np.ndarray, weight: np.ndarray) -> np.ndarray:
    """x [M, K] . weight [N, K]^T, row by row through the matvec."""
    x = _f32(x)
    weight, code = _stored(weight)
    out = np.empty((x.shape[0], weight.shape[0]), dtype=np.float32)
    for r in range(x.shape[0]):
        lib().ref_matvec(_p(weight), code, _p(x[r]), _p(out[r]), weight.shape[0], weight.shape[1])
    return out


def swiglu(gate_up: np.ndarray) -> np.ndarray:
    gate_up = _f32(gate_up)
    inner = gate_up.shape[1] // 2
    out = np.empty((gate_up.shape[0], inner), dtype=np.float32)
    for r in range(gate_up.shape[0]):
        lib().ref_swiglu(_p(gate_up[r]), _p(out[r]), inner)
    return out


def head_norm_rope(values: np.ndarray, heads: int, d: int, weight, eps: float, positions, inv_freq, rotary_dim: int,
                   interleaved: bool = False) -> np.ndarray:
    """Per-head norm (weight None: none) and rotation (inv_freq None: none) of [tokens, heads * d]."""
    out = _f32(values).copy()
    w = _f32(weight) if weight is not None else None
    f = _f32(inv_freq) if inv_freq is not None else None
    for t in range(out.shape[0]):
        lib().ref_head_norm(_p(out[t]), heads, d, _p(w) if w is not None else None, eps)
        if f is not None:
            for h in range(heads):
                lib().ref_rope(ctypes.c_void_p(out[t].ctypes.data + 4 * h * d), rotary_dim, int(positions[t]), _p(f), int(interleaved))
    return out


def kv_write(k_cache: np.ndarray, v_cache: np.ndarray, table_row, pos: int, k: np.ndarray, v: np.ndarray) -> None:
    """k, v [n_kv, d] of the token at `pos` into caches [pages, n_kv, page, d] (float32 or bfloat16 bits), in place."""
    code = BF16 if k_cache.dtype == np.uint16 else F32
    table_row = np.ascontiguousarray(table_row, dtype=np.int32)
    k, v = _f32(k), _f32(v)
    lib().ref_kv_write(_p(k_cache), _p(v_cache), code, _p(table_row), k_cache.shape[2], k_cache.shape[1], k_cache.shape[3], pos, _p(k), _p(v))


def paged_gqa(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, table_row, pos: int, n_q: int, scale: float,
              window: int = 0) -> np.ndarray:
    """One query token [n_q * d] at `pos` over its sequence's pages: [n_q * d]."""
    code = BF16 if k_cache.dtype == np.uint16 else F32
    q = _f32(q)
    table_row = np.ascontiguousarray(table_row, dtype=np.int32)
    n_kv, page, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    scores = np.empty(pos + 1, dtype=np.float32)
    out = np.empty(n_q * d, dtype=np.float32)
    lib().ref_paged_gqa(_p(q), _p(k_cache), _p(v_cache), code, _p(table_row), page, n_q, n_kv, d, pos, window, scale, _p(scores), _p(out))
    return out


def argmax(values: np.ndarray) -> int:
    values = _f32(values)
    return int(lib().ref_argmax(_p(values), values.size))


def bf16_bits(a) -> np.ndarray:
    """float32 values rounded to bfloat16 (nearest, ties to even), as uint16 bits."""
    a = _f32(a)
    fn = lib().ref_float_to_bf16
    return np.array([fn(float(v)) for v in a.ravel()], dtype=np.uint16).reshape(a.shape)
