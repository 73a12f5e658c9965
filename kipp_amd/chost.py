"""A thin wrapper of the C host (`kipp_amd/host`, built into `libkipp_amd.so`).

Everything here is a call into the C library: a model opened from a folder,
sessions, the step function, the sampler.  Nothing is computed in Python and
no tensor library is involved; logits come back as NumPy arrays.

    model = CModel("folder", path="gpu-bf16", page_tokens=16, kv_pool_pages=64)
    a = model.session()
    logits = model.step([(a, [5, 17, 3], [0, 2])])        # float32 [2, vocab]
    token = sample(logits[1], temperature=0.8, top_p=0.9, rng=Rng(7))

Errors of the library are raised as `KippError` with the library's code name
(kipp.h's: argument, io, format, unsupported, memory, range, internal).
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import numpy as np

from .host import build as _build

PATHS = {"gpu-bf16": 0, "gpu-fp32": 1, "cpu-fp32": 2}
DTYPE_PATHS = {"bfloat16": "gpu-bf16", "float32": "gpu-fp32"}
_MAX_STOP = 8

_u32p = ctypes.POINTER(ctypes.c_uint32)
_f32p = ctypes.POINTER(ctypes.c_float)


class _Error(ctypes.Structure):
    _fields_ = [("code", ctypes.c_int), ("message", ctypes.c_char * 2048)]


class _OpenConfig(ctypes.Structure):
    _fields_ = [("path", ctypes.c_int), ("page_tokens", ctypes.c_uint32), ("kv_pool_pages", ctypes.c_uint32),
                ("max_sessions", ctypes.c_uint32), ("max_step_tokens", ctypes.c_uint32), ("share_prefixes", ctypes.c_int),
                ("device", ctypes.c_int), ("kernel_dir", ctypes.c_char_p), ("page_order", _u32p), ("eager_steps", ctypes.c_int)]


class _ModelInfo(ctypes.Structure):
    _fields_ = [("architecture", ctypes.c_char_p), ("path", ctypes.c_int), ("block_count", ctypes.c_uint32),
                ("embedding_length", ctypes.c_uint32), ("feed_forward_length", ctypes.c_uint32),
                ("attention_head_count", ctypes.c_uint32), ("attention_head_count_kv", ctypes.c_uint32),
                ("attention_head_dim", ctypes.c_uint32), ("vocab_size", ctypes.c_uint32), ("context_length", ctypes.c_uint32),
                ("rope_theta", ctypes.c_float), ("rms_norm_eps", ctypes.c_float), ("tied_embeddings", ctypes.c_int),
                ("stop_tokens", ctypes.c_uint32 * _MAX_STOP), ("stop_token_count", ctypes.c_uint32),
                ("page_tokens", ctypes.c_uint32), ("cache_groups", ctypes.c_uint32), ("mapped_bytes", ctypes.c_uint64),
                ("weight_bytes", ctypes.c_uint64), ("cache_bytes", ctypes.c_uint64)]


class _SessionInfo(ctypes.Structure):
    _fields_ = [("capacity", ctypes.c_uint32), ("length", ctypes.c_uint32), ("adopted_tokens", ctypes.c_uint32),
                ("cache_bytes", ctypes.c_uint64)]


class _PoolStats(ctypes.Structure):
    _fields_ = [("total_blocks", ctypes.c_uint32), ("free_blocks", ctypes.c_uint32), ("reused_blocks_total", ctypes.c_uint64),
                ("evicted_blocks_total", ctypes.c_uint64)]


class _StepItem(ctypes.Structure):
    _fields_ = [("session", ctypes.c_void_p), ("tokens", _u32p), ("token_count", ctypes.c_size_t), ("want", _u32p),
                ("want_count", ctypes.c_size_t)]


class _BatchItem(ctypes.Structure):
    _fields_ = [("session", ctypes.c_void_p), ("tokens", _u32p), ("token_count", ctypes.c_size_t), ("logits", _f32p)]


class _SampleParams(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_p", ctypes.c_float), ("top_k", ctypes.c_uint32), ("min_p", ctypes.c_float),
                ("frequency_penalty", ctypes.c_float), ("presence_penalty", ctypes.c_float), ("repetition_penalty", ctypes.c_float),
                ("recent_tokens", _u32p), ("recent_count", ctypes.c_size_t), ("logit_bias_tokens", _u32p),
                ("logit_bias_values", _f32p), ("logit_bias_count", ctypes.c_size_t)]


class _SchedulerConfig(ctypes.Structure):
    _fields_ = [("max_step_tokens", ctypes.c_uint32), ("prefill_chunk", ctypes.c_uint32), ("max_running", ctypes.c_uint32),
                ("keep_last_logits", ctypes.c_int)]


class _Request(ctypes.Structure):
    _fields_ = [("id", ctypes.c_uint64), ("prompt", _u32p), ("prompt_count", ctypes.c_size_t), ("max_new_tokens", ctypes.c_uint32),
                ("params", _SampleParams), ("seed", ctypes.c_uint64), ("stop_tokens", ctypes.c_uint32 * _MAX_STOP),
                ("stop_token_count", ctypes.c_uint32)]


class _Produced(ctypes.Structure):
    _fields_ = [("id", ctypes.c_uint64), ("token", ctypes.c_uint32)]


class _Result(ctypes.Structure):
    _fields_ = [("id", ctypes.c_uint64), ("reason", ctypes.c_int), ("output", _u32p), ("output_count", ctypes.c_size_t),
                ("error", ctypes.c_char_p)]


class _SchedulerStats(ctypes.Structure):
    _fields_ = [(name, ctypes.c_uint64) for name in ("requests", "refused", "finished", "failed", "failed_steps", "prompt_tokens",
                                                     "generated_tokens", "prefix_tokens_reused", "steps", "waits_for_pages",
                                                     "waits_for_prefix")] + \
               [("queue_wait_seconds_sum", ctypes.c_double), ("queue_wait_count", ctypes.c_uint64), ("ttft_seconds_sum", ctypes.c_double),
                ("ttft_count", ctypes.c_uint64), ("decode_seconds_sum", ctypes.c_double)]


FINISH_REASONS = {0: None, 1: "length", 2: "stop", 3: "cancelled", 4: "failed"}


class KippError(RuntimeError):
    def __init__(self, code: str, message: str):
        super().__init__(f"{code}: {message}")
        self.code, self.message = code, message


_libs = {}


def library(variant: str = "gpu") -> ctypes.CDLL:
    """The loaded C library: "gpu" (every path) or "host-only" (cpu-fp32 alone; needs no HIP to load)."""
    lib = _libs.get(variant)
    if lib is None:
        if variant == "gpu":
            # A process has ONE HIP runtime: the first one loaded serves every library that names it.  Where PyTorch
            # is installed it ships its own, which it must get whether it is imported before or after this library, so
            # it is loaded first here.  Nothing else of it is used.
            try:
                import torch  # noqa: F401
            except ImportError:
                pass
        lib = ctypes.CDLL(_build.library_path(variant))
        vp, sz, u32, err = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.POINTER(_Error)
        sigs = {
            "kipp_model_open_ex": [ctypes.c_char_p, ctypes.POINTER(_OpenConfig), ctypes.POINTER(vp), err],
            "kipp_model_close": [vp, err],
            "kipp_model_get_info": [vp, ctypes.POINTER(_ModelInfo)],
            "kipp_model_is_stop_token": [vp, u32],
            "kipp_model_kv_pool_stats": [vp, u32, ctypes.POINTER(_PoolStats)],
            "kipp_session_create": [vp, u32, ctypes.POINTER(vp), err],
            "kipp_session_reset": [vp, err],
            "kipp_session_truncate": [vp, u32, err],
            "kipp_session_get_info": [vp, ctypes.POINTER(_SessionInfo)],
            "kipp_session_eval": [vp, _u32p, sz, _f32p, sz, err],
            "kipp_session_eval_n": [vp, _u32p, sz, _f32p, u32, err],
            "kipp_session_eval_scored": [vp, _u32p, sz, _f32p, u32, err],
            "kipp_session_match_prefix": [vp, _u32p, sz, _u32p, err],
            "kipp_eval_batch": [vp, ctypes.POINTER(_BatchItem), sz, err],
            "kipp_model_eval": [vp, _u32p, sz, _f32p, sz, err],
            "kipp_step": [vp, ctypes.POINTER(_StepItem), sz, _f32p, sz, err],
            "kipp_step_argmax": [vp, ctypes.POINTER(_StepItem), sz, _u32p, sz, err],
            "kipp_step_nll": [vp, ctypes.POINTER(_StepItem), sz, _u32p, ctypes.POINTER(ctypes.c_double), sz, err],
            "kipp_step_sample": [vp, ctypes.POINTER(_StepItem), sz, ctypes.POINTER(_SampleParams), ctypes.POINTER(ctypes.c_double), _u32p, sz, err],
            "kipp_step_sample_logits": [vp, ctypes.POINTER(_StepItem), sz, ctypes.POINTER(_SampleParams), ctypes.POINTER(ctypes.c_double), _u32p, sz,
                                        _f32p, sz, err],
            "kipp_sample_ex": [_f32p, sz, ctypes.POINTER(_SampleParams), ctypes.POINTER(ctypes.c_uint64), _u32p, err],
            "kipp_test_scramble_session_kv": [vp, err],
            "kipp_scheduler_create": [vp, ctypes.POINTER(_SchedulerConfig), ctypes.POINTER(vp), err],
            "kipp_scheduler_add": [vp, ctypes.POINTER(_Request), err],
            "kipp_scheduler_cancel": [vp, ctypes.c_uint64, err],
            "kipp_scheduler_step": [vp, ctypes.POINTER(_Produced), sz, ctypes.POINTER(sz), err],
            "kipp_scheduler_idle": [vp],
            "kipp_scheduler_result": [vp, ctypes.c_uint64, ctypes.POINTER(_Result)],
            "kipp_scheduler_collect": [vp, ctypes.c_uint64],
            "kipp_scheduler_get_stats": [vp, ctypes.POINTER(_SchedulerStats)],
        }
        for name, argtypes in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, ctypes.c_int
        lib.kipp_session_destroy.argtypes, lib.kipp_session_destroy.restype = [vp], None
        lib.kipp_rng_uniform.argtypes, lib.kipp_rng_uniform.restype = [ctypes.POINTER(ctypes.c_uint64)], ctypes.c_double
        lib.kipp_scheduler_destroy.argtypes, lib.kipp_scheduler_destroy.restype = [vp], None
        lib.kipp_scheduler_last_logits.argtypes, lib.kipp_scheduler_last_logits.restype = [vp, ctypes.c_uint64], _f32p
        lib.kipp_test_fail_forward_after.argtypes, lib.kipp_test_fail_forward_after.restype = [vp, ctypes.c_int], None
        lib.kipp_error_code_name.argtypes, lib.kipp_error_code_name.restype = [ctypes.c_int], ctypes.c_char_p
        lib.kipp_test_graph_replays.argtypes, lib.kipp_test_graph_replays.restype = [vp], ctypes.c_uint64
        lib.kipp_test_cut_attention_steps.argtypes, lib.kipp_test_cut_attention_steps.restype = [vp], ctypes.c_uint64
        lib.kipp_test_session_pages.argtypes = [vp, u32, ctypes.POINTER(ctypes.c_int32), sz]
        lib.kipp_test_session_pages.restype = sz
        _libs[variant] = lib
    return lib


def _raise(lib, error: _Error):
    raise KippError(lib.kipp_error_code_name(error.code).decode(), error.message.decode("utf-8", "replace"))


def _u32(values: Sequence[int]):
    array = np.ascontiguousarray(np.asarray(values, dtype=np.uint32))
    return array, array.ctypes.data_as(_u32p)


class CSession:
    def __init__(self, model: "CModel", handle: int):
        self.model, self.handle = model, handle

    def _info(self) -> _SessionInfo:
        info = _SessionInfo()
        self.model.lib.kipp_session_get_info(self.handle, ctypes.byref(info))
        return info

    @property
    def length(self) -> int:
        return self._info().length

    @property
    def adopted_tokens(self) -> int:
        return self._info().adopted_tokens

    def pages(self, group: int = 0):
        out = (ctypes.c_int32 * 65536)()
        n = self.model.lib.kipp_test_session_pages(self.handle, group, out, 65536)
        return list(out[:n])

    def eval(self, tokens: Sequence[int]) -> np.ndarray:
        return self.model._rows(self.model.lib.kipp_session_eval, self, tokens, 1, sized=True)[0]

    def eval_n(self, tokens: Sequence[int], rows: int) -> np.ndarray:
        return self.model._rows(self.model.lib.kipp_session_eval_n, self, tokens, rows)

    def eval_scored(self, tokens: Sequence[int], rows: int) -> np.ndarray:
        return self.model._rows(self.model.lib.kipp_session_eval_scored, self, tokens, rows)

    def match_prefix(self, tokens: Sequence[int]) -> int:
        keep, ptr = _u32(tokens)
        matched, error = ctypes.c_uint32(0), _Error()
        if self.model.lib.kipp_session_match_prefix(self.handle, ptr, len(keep), ctypes.byref(matched), ctypes.byref(error)) != 0:
            _raise(self.model.lib, error)
        return matched.value

    def truncate(self, length: int) -> None:
        error = _Error()
        if self.model.lib.kipp_session_truncate(self.handle, length, ctypes.byref(error)) != 0:
            _raise(self.model.lib, error)

    def reset(self) -> None:
        error = _Error()
        if self.model.lib.kipp_session_reset(self.handle, ctypes.byref(error)) != 0:
            _raise(self.model.lib, error)

    def scramble(self) -> None:
        """Reverse its block tables, the pages' contents moving along (a test's way to show that results do not depend on
        where pages lie)."""
        error = _Error()
        if self.model.lib.kipp_test_scramble_session_kv(self.handle, ctypes.byref(error)) != 0:
            _raise(self.model.lib, error)

    def destroy(self) -> None:
        if self.handle is not None:
            self.model.lib.kipp_session_destroy(self.handle)
            self.model.sessions.discard(self)
            self.handle = None


class CModel:
    def __init__(self, folder: str, path: str = "gpu-bf16", page_tokens: int = 16, kv_pool_pages: int = 0, max_sessions: int = 64,
                 max_step_tokens: int = 4096, share_prefixes: bool = True, device: int = 0, kernel_dir: Optional[str] = None,
                 page_order: Optional[Sequence[int]] = None, variant: Optional[str] = None, eager_steps: bool = False):
        if path not in PATHS:
            raise ValueError(f"path is one of {sorted(PATHS)}")
        self.lib = library(variant or ("host-only" if path == "cpu-fp32" and variant is None else "gpu"))
        if path != "cpu-fp32" and kernel_dir is None:
            # what this model launches is compiled now if it is not built yet, and the manifest names it
            from .config import load_config
            from .csrc import build
            from .csrc.variants import model_variants
            _, cfg = load_config(folder)
            build.build_all(model_variants(cfg.model_spec(), "bfloat16" if path == "gpu-bf16" else "float32"))
            build.write_manifest()
            kernel_dir = build._lib_dir()
        order = _u32(page_order) if page_order is not None else (None, None)
        config = _OpenConfig(PATHS[path], page_tokens, kv_pool_pages, max_sessions, max_step_tokens, int(share_prefixes), device,
                             kernel_dir.encode() if kernel_dir else None, order[1], int(eager_steps))
        handle, error = ctypes.c_void_p(), _Error()
        if self.lib.kipp_model_open_ex(folder.encode(), ctypes.byref(config), ctypes.byref(handle), ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        self.handle = handle
        self.sessions = set()
        info = _ModelInfo()
        self.lib.kipp_model_get_info(self.handle, ctypes.byref(info))
        self.info = info
        self.vocab_size = info.vocab_size
        self.context_length = info.context_length

    @property
    def graph_replays(self) -> int:
        """Steps that ran from a recording since the model was opened."""
        return int(self.lib.kipp_test_graph_replays(self.handle))

    @property
    def cut_attention_steps(self) -> int:
        """Work lists of prompt portions whose keys were cut over more workgroups since the model was opened."""
        return int(self.lib.kipp_test_cut_attention_steps(self.handle))

    def session(self, capacity: int = 0) -> CSession:
        handle, error = ctypes.c_void_p(), _Error()
        if self.lib.kipp_session_create(self.handle, capacity, ctypes.byref(handle), ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        s = CSession(self, handle)
        self.sessions.add(s)
        return s

    def step(self, entries: Sequence[Tuple[CSession, Sequence[int], Sequence[int]]]) -> Optional[np.ndarray]:
        """One batch of (session, its next tokens, wanted places): float32 [wanted, vocab], or None if nothing is wanted."""
        items = (_StepItem * len(entries))()
        keep = []
        wanted = 0
        for i, (session, tokens, want) in enumerate(entries):
            t, tp = _u32(tokens)
            w, wp = _u32(want)
            keep.append((t, w))
            items[i] = _StepItem(session.handle, tp, len(t), wp if len(w) else None, len(w))
            wanted += len(w)
        out = np.empty((wanted, self.vocab_size), dtype=np.float32)
        error = _Error()
        if self.lib.kipp_step(self.handle, items, len(entries), out.ctypes.data_as(_f32p), out.size, ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return out if wanted else None

    def step_argmax(self, entries: Sequence[Tuple[CSession, Sequence[int], Sequence[int]]]) -> List[int]:
        """The same batch, answered with the index of the largest logit at every wanted place (found where the path computes)."""
        items = (_StepItem * len(entries))()
        keep = []
        wanted = 0
        for i, (session, tokens, want) in enumerate(entries):
            t, tp = _u32(tokens)
            w, wp = _u32(want)
            keep.append((t, w))
            items[i] = _StepItem(session.handle, tp, len(t), wp if len(w) else None, len(w))
            wanted += len(w)
        out = np.zeros(max(wanted, 1), dtype=np.uint32)
        error = _Error()
        if self.lib.kipp_step_argmax(self.handle, items, len(entries), out.ctypes.data_as(_u32p), wanted, ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return [int(t) for t in out[:wanted]]

    def step_nll(self, entries: Sequence[Tuple[CSession, Sequence[int], Sequence[int]]], targets: Sequence[int]) -> np.ndarray:
        """The same batch, answered with -log softmax(row)[target] (float64) for every wanted place, computed where the
        path computes: `targets` has one token a wanted place, in order."""
        items = (_StepItem * len(entries))()
        keep = []
        wanted = 0
        for i, (session, tokens, want) in enumerate(entries):
            t, tp = _u32(tokens)
            w, wp = _u32(want)
            keep.append((t, w))
            items[i] = _StepItem(session.handle, tp, len(t), wp if len(w) else None, len(w))
            wanted += len(w)
        if len(targets) != wanted:
            raise ValueError("one target for every wanted place")
        tg, tgp = _u32(targets if wanted else [0])
        out = np.zeros(max(wanted, 1), dtype=np.float64)
        error = _Error()
        if self.lib.kipp_step_nll(self.handle, items, len(entries), tgp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), wanted,
                                  ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return out[:wanted]

    def step_sample(self, entries: Sequence[Tuple[CSession, Sequence[int], Sequence[int]]], choices: Sequence[dict], logits: bool = False):
        """The same batch, answered with one token for every wanted place, chosen where the path computes as kipp_sample_ex
        would: `choices` has, for each wanted place in order, the sampler's parameters by name (temperature, top_p, top_k,
        min_p, frequency_penalty, presence_penalty, repetition_penalty, recent, logit_bias) and `uniform`, the draw.
        With `logits` the result is (tokens, the wanted rows of logits as the model left them)."""
        items = (_StepItem * len(entries))()
        keep = []
        wanted = 0
        for i, (session, tokens, want) in enumerate(entries):
            t, tp = _u32(tokens)
            w, wp = _u32(want)
            keep.append((t, w))
            items[i] = _StepItem(session.handle, tp, len(t), wp if len(w) else None, len(w))
            wanted += len(w)
        if len(choices) != wanted:
            raise ValueError("one choice for every wanted place")
        params = (_SampleParams * max(wanted, 1))()
        draws = (ctypes.c_double * max(wanted, 1))()
        for r, c in enumerate(choices):
            recent, rp = _u32(c.get("recent", ()))
            bias = c.get("logit_bias") or {}
            bt, btp = _u32(list(bias.keys()))
            bv = np.ascontiguousarray(np.asarray(list(bias.values()), dtype=np.float32))
            keep.append((recent, bt, bv))
            params[r] = _SampleParams(c.get("temperature", 0.0), c.get("top_p", 1.0), c.get("top_k", 0), c.get("min_p", 0.0),
                                      c.get("frequency_penalty", 0.0), c.get("presence_penalty", 0.0), c.get("repetition_penalty", 1.0),
                                      rp if len(recent) else None, len(recent), btp if len(bt) else None,
                                      bv.ctypes.data_as(_f32p) if len(bv) else None, len(bt))
            draws[r] = c.get("uniform", 0.0)
        out = np.zeros(max(wanted, 1), dtype=np.uint32)
        error = _Error()
        if logits:
            rows = np.empty((wanted, self.vocab_size), dtype=np.float32)
            if self.lib.kipp_step_sample_logits(self.handle, items, len(entries), params, draws, out.ctypes.data_as(_u32p), wanted,
                                                rows.ctypes.data_as(_f32p), rows.size, ctypes.byref(error)) != 0:
                _raise(self.lib, error)
            return [int(t) for t in out[:wanted]], rows
        if self.lib.kipp_step_sample(self.handle, items, len(entries), params, draws, out.ctypes.data_as(_u32p), wanted, ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return [int(t) for t in out[:wanted]]

    def singles(self, sessions: Sequence[CSession]) -> "CSingles":
        """A step of one token a session, made ready once: `CSingles.step` then costs one call into the library."""
        return CSingles(self, sessions)

    def eval(self, tokens: Sequence[int]) -> np.ndarray:
        """kipp.h's evaluation without a session: the logits of the last of up to 256 tokens."""
        t, tp = _u32(tokens)
        out = np.empty(self.vocab_size, dtype=np.float32)
        error = _Error()
        if self.lib.kipp_model_eval(self.handle, tp, len(t), out.ctypes.data_as(_f32p), out.size, ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return out

    def eval_batch(self, entries: Sequence[Tuple[CSession, Sequence[int]]]) -> np.ndarray:
        """kipp.h's batched call: every session's tokens appended, the logits of each one's last token."""
        out = np.empty((len(entries), self.vocab_size), dtype=np.float32)
        items = (_BatchItem * len(entries))()
        keep = []
        for i, (session, tokens) in enumerate(entries):
            t, tp = _u32(tokens)
            keep.append(t)
            items[i] = _BatchItem(session.handle, tp, len(t), out[i].ctypes.data_as(_f32p))
        error = _Error()
        if self.lib.kipp_eval_batch(self.handle, items, len(entries), ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return out

    def _rows(self, fn, session: CSession, tokens: Sequence[int], rows: int, sized: bool = False) -> np.ndarray:
        t, tp = _u32(tokens)
        out = np.empty((rows, self.vocab_size), dtype=np.float32)
        error = _Error()
        last = out.size if sized else rows
        if fn(session.handle, tp, len(t), out.ctypes.data_as(_f32p), last, ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return out

    def pool_stats(self, group: int = 0) -> dict:
        stats = _PoolStats()
        if self.lib.kipp_model_kv_pool_stats(self.handle, group, ctypes.byref(stats)) != 0:
            raise KippError("argument", f"no cache group {group}")
        return {"total_blocks": stats.total_blocks, "free_blocks": stats.free_blocks,
                "reused_blocks_total": stats.reused_blocks_total, "evicted_blocks_total": stats.evicted_blocks_total}

    def is_stop_token(self, token: int) -> bool:
        return bool(self.lib.kipp_model_is_stop_token(self.handle, token))

    def close(self) -> None:
        if self.handle is not None:
            for s in list(self.sessions):
                s.destroy()
            error = _Error()
            if self.lib.kipp_model_close(self.handle, ctypes.byref(error)) != 0:
                _raise(self.lib, error)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


class CSingles:
    """Sessions that each bring one token a step and want its largest logit's index (greedy decoding): the items of
    kipp_step_argmax are built once, so a step is `tokens` in, one call, `out` back, with no Python for every session."""

    def __init__(self, model: CModel, sessions: Sequence[CSession]):
        self.model, self.n = model, len(sessions)
        self.tokens = np.zeros(self.n, dtype=np.uint32)       # what the next step feeds
        self.out = np.zeros(max(self.n, 1), dtype=np.uint32)  # what the last step chose
        self._want = np.zeros(1, dtype=np.uint32)
        self._items = (_StepItem * self.n)()
        base = self.tokens.ctypes.data
        for i, session in enumerate(sessions):
            self._items[i] = _StepItem(session.handle, ctypes.cast(base + 4 * i, _u32p), 1, self._want.ctypes.data_as(_u32p), 1)

    def step(self, feed_back: bool = False) -> np.ndarray:
        """One step from `self.tokens`; returns `self.out`.  `feed_back`: the chosen tokens are the next step's."""
        error = _Error()
        if self.model.lib.kipp_step_argmax(self.model.handle, self._items, self.n, self.out.ctypes.data_as(_u32p), self.n,
                                           ctypes.byref(error)) != 0:
            _raise(self.model.lib, error)
        if feed_back:
            self.tokens[:] = self.out[:self.n]
        return self.out


class CScheduler:
    """The C scheduler (`host/scheduler.c`) over a `CModel`: requests in, (request, token) pairs out."""

    def __init__(self, model: CModel, max_step_tokens: int = 2048, prefill_chunk: int = 512, max_running: int = 0,
                 keep_last_logits: bool = False):
        self.model, self.lib = model, model.lib
        config = _SchedulerConfig(max_step_tokens, prefill_chunk, max_running, int(keep_last_logits))
        handle, error = ctypes.c_void_p(), _Error()
        if self.lib.kipp_scheduler_create(model.handle, ctypes.byref(config), ctypes.byref(handle), ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        self.handle = handle
        self._produced = (_Produced * 1024)()

    def add(self, request_id: int, prompt: Sequence[int], max_new_tokens: int, temperature: float = 0.0, top_p: float = 1.0,
            top_k: int = 0, min_p: float = 0.0, frequency_penalty: float = 0.0, presence_penalty: float = 0.0,
            repetition_penalty: float = 1.0, logit_bias: Optional[dict] = None, seed: int = 1, stop_tokens: Sequence[int] = ()) -> None:
        p, pp = _u32(prompt)
        bias = logit_bias or {}
        bt, btp = _u32(list(bias.keys()))
        bv = np.ascontiguousarray(np.asarray(list(bias.values()), dtype=np.float32))
        params = _SampleParams(temperature, top_p, top_k, min_p, frequency_penalty, presence_penalty, repetition_penalty, None, 0,
                               btp if len(bt) else None, bv.ctypes.data_as(_f32p) if len(bv) else None, len(bt))
        stops = (ctypes.c_uint32 * _MAX_STOP)(*list(stop_tokens)[:_MAX_STOP])
        request = _Request(request_id, pp, len(p), max_new_tokens, params, seed, stops, len(stop_tokens))
        error = _Error()
        if self.lib.kipp_scheduler_add(self.handle, ctypes.byref(request), ctypes.byref(error)) != 0:
            _raise(self.lib, error)

    def step(self):
        """One step; the (request id, token) pairs that became known."""
        count, error = ctypes.c_size_t(0), _Error()
        if self.lib.kipp_scheduler_step(self.handle, self._produced, 1024, ctypes.byref(count), ctypes.byref(error)) != 0:
            _raise(self.lib, error)
        return [(int(self._produced[i].id), int(self._produced[i].token)) for i in range(min(count.value, 1024))]

    @property
    def idle(self) -> bool:
        return bool(self.lib.kipp_scheduler_idle(self.handle))

    def run(self, max_steps: int = 100000) -> None:
        steps = 0
        while not self.idle and steps < max_steps:
            self.step()
            steps += 1

    def cancel(self, request_id: int) -> None:
        error = _Error()
        if self.lib.kipp_scheduler_cancel(self.handle, request_id, ctypes.byref(error)) != 0:
            _raise(self.lib, error)

    def result(self, request_id: int) -> dict:
        out = _Result()
        if self.lib.kipp_scheduler_result(self.handle, request_id, ctypes.byref(out)) != 0:
            raise KeyError(request_id)
        return {"id": int(out.id), "finish_reason": FINISH_REASONS[out.reason], "output": [int(out.output[i]) for i in range(out.output_count)],
                "error": (out.error or b"").decode("utf-8", "replace")}

    def last_logits(self, request_id: int) -> Optional[np.ndarray]:
        ptr = self.lib.kipp_scheduler_last_logits(self.handle, request_id)
        return np.ctypeslib.as_array(ptr, shape=(self.model.vocab_size,)).copy() if ptr else None

    def collect(self, request_id: int) -> None:
        if self.lib.kipp_scheduler_collect(self.handle, request_id) != 0:
            raise KeyError(request_id)

    @property
    def stats(self) -> dict:
        st = _SchedulerStats()
        self.lib.kipp_scheduler_get_stats(self.handle, ctypes.byref(st))
        return {name: getattr(st, name) for name, _ in _SchedulerStats._fields_}

    def destroy(self) -> None:
        if self.handle is not None:
            self.lib.kipp_scheduler_destroy(self.handle)
            self.handle = None


class Rng:
    """The caller-owned state of the sampler's generator (xorshift64*, nonzero)."""

    def __init__(self, seed: int):
        self.state = ctypes.c_uint64(seed)

    def uniform(self, variant: str = "host-only") -> float:
        """The next draw in [0, 1), as kipp_sample_ex takes it."""
        return float(library(variant).kipp_rng_uniform(ctypes.byref(self.state)))


def sample(logits: np.ndarray, temperature: float = 0.0, top_p: float = 1.0, top_k: int = 0, min_p: float = 0.0,
           frequency_penalty: float = 0.0, presence_penalty: float = 0.0, repetition_penalty: float = 1.0,
           recent: Sequence[int] = (), logit_bias: Optional[dict] = None, rng: Optional[Rng] = None, variant: str = "host-only") -> int:
    """kipp_sample_ex of the C library."""
    lib = library(variant)
    values = np.ascontiguousarray(logits, dtype=np.float32)
    r, rp = _u32(list(recent))
    bias = logit_bias or {}
    bt, btp = _u32(list(bias.keys()))
    bv = np.ascontiguousarray(np.asarray(list(bias.values()), dtype=np.float32))
    params = _SampleParams(temperature, top_p, top_k, min_p, frequency_penalty, presence_penalty, repetition_penalty,
                           rp if len(r) else None, len(r), btp if len(bt) else None,
                           bv.ctypes.data_as(_f32p) if len(bv) else None, len(bt))
    token, error = ctypes.c_uint32(0), _Error()
    state = ctypes.byref(rng.state) if rng is not None else None
    if lib.kipp_sample_ex(values.ctypes.data_as(_f32p), values.size, ctypes.byref(params), state, ctypes.byref(token), ctypes.byref(error)) != 0:
        _raise(lib, error)
    return int(token.value)
