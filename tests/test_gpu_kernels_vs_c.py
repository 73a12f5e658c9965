"""Every kernel beside its scalar C reference (kipp_amd/csrc/ref/ref_ops.c, pinned against the plain NumPy
implementation in tests/test_ref_ops.py): the reference keeps a scalar host function beside each of its kernels and
gates the kernel against it (/root/reference/README.md:110-112).  float32 kernels agree with the scalar float32 sums to
rounding; bfloat16 kernels are compared on the same (rounded) operands."""
import math

import numpy as np
import pytest
import torch

from kipp_amd.csrc import ref
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32_TOL, BF16_TOL = 1e-11, 2e-5


def _ops():
    from kipp_amd.csrc import ops
    return ops


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def _bits(t: torch.Tensor) -> np.ndarray:
    """A bfloat16 tensor's values as the uint16 bits the C references take for bfloat16 storage."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _rounded(a: np.ndarray) -> np.ndarray:
    return torch.tensor(a).bfloat16().float().numpy()


def test_embed_rmsnorm_swiglu_argmax():
    ops = _ops()
    rng = np.random.default_rng(0)
    table = torch.tensor(rng.normal(size=(301, 72))).bfloat16()
    tokens = rng.integers(0, 301, size=19)
    got = ops.embed(table.to(DEV), _t(tokens, torch.int32), torch.empty(19, 72, device=DEV))
    assert np.array_equal(got.cpu().numpy(), ref.embed(_bits(table), tokens))
    for width, rows in ((72, 5), (2560, 3), (5000, 2)):
        x = rng.normal(size=(rows, width)).astype(np.float32)
        w = (1 + 0.1 * rng.normal(size=width)).astype(np.float32)
        got = ops.rmsnorm(_t(x), _t(w), 1e-6, torch.empty(rows, width, device=DEV))
        assert plain.nmse(got.cpu().numpy(), ref.rms_norm(x, w, 1e-6)) < F32_TOL
        delta = rng.normal(size=(2, rows, width)).astype(np.float32)        # two slabs of a split product, added in order
        xd = _t(x)
        got = ops.rmsnorm(xd, _t(w), 1e-6, torch.empty(rows, width, dtype=torch.bfloat16, device=DEV), delta=_t(delta))
        summed = (x + delta[0]) + delta[1]
        assert np.array_equal(xd.cpu().numpy(), summed)
        assert plain.nmse(got.float().cpu().numpy(), ref.rms_norm(summed, w, 1e-6)) < BF16_TOL
    for inner, rows in ((200, 7), (9728, 2), (204, 3)):
        gu = (3 * rng.normal(size=(rows, 2 * inner))).astype(np.float32)
        got = ops.swiglu(_t(gu), torch.empty(rows, inner, device=DEV))
        assert plain.nmse(got.cpu().numpy(), ref.swiglu(gu)) < F32_TOL
    for vocab in (5, 509, 151936):
        logits = rng.normal(size=(3, vocab)).astype(np.float32)
        logits[1, [vocab // 3, vocab - 1]] = logits[1].max() + 1.0             # a tie: the lowest index
        out = ops.argmax(_t(logits), torch.empty(3, dtype=torch.int32, device=DEV)).cpu().numpy()
        assert [int(t) for t in out] == [ref.argmax(row) for row in logits]


@pytest.mark.parametrize("m,n,k", [(1, 77, 64), (5, 300, 2560), (8, 2560, 9728), (17, 200, 96), (64, 640, 352), (130, 509, 160),
                                   (300, 257, 96), (700, 1300, 2560)])
def test_products(m, n, k):
    """The float32 product, and each bfloat16 product that takes the shape (few rows, staged rows, tiles, with the
    weight as rows and in the streaming layout), against the scalar matvec over the same operands."""
    ops = _ops()
    rng = np.random.default_rng(m + n + k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    w = (rng.normal(size=(n, k)) * 0.1).astype(np.float32)
    want = ref.linear(x, w)
    got = ops.gemm_f32(_t(x), _t(w), torch.empty(m, n, device=DEV))
    assert plain.nmse(got.cpu().numpy(), want) < F32_TOL
    xb, wb = torch.tensor(x).bfloat16(), torch.tensor(w).bfloat16()
    want = ref.linear(xb.float().numpy(), _bits(wb))                             # bfloat16 operands, widened element by element
    got = ops.gemm_f32(_t(xb.float().numpy()), wb.to(DEV), torch.empty(m, n, device=DEV))
    assert plain.nmse(got.cpu().numpy(), want) < F32_TOL
    tiles = ops.tile_weight(wb.to(DEV)) if k % 32 == 0 else None
    ran = 0
    if ops.gemm_skinny_ok(m, k):
        for t in (None, tiles):
            got = ops.gemm_skinny(xb.to(DEV), wb.to(DEV), max_parts=8, tiles=t).sum(dim=0)
            assert plain.nmse(got.cpu().numpy(), want) < 1e-10
            ran += 1
    if ops.gemm_rows_ok(m, k):
        for t in (None, tiles):
            got = ops.gemm_rows(xb.to(DEV), wb.to(DEV), max_parts=12, tiles=t).sum(dim=0)
            assert plain.nmse(got.cpu().numpy(), want) < 1e-10
            ran += 1
    if ops.gemm_tiles_ok(m, k, n):
        got = ops.gemm_tiles(xb.to(DEV), wb.to(DEV), "slabs", max_parts=4).sum(dim=0)
        assert plain.nmse(got.cpu().numpy(), want) < 1e-10
        ran += 1
    assert ran > 0


def _paged(rng, seq_lens, n_kv, d, page, dtype, extra=3):
    blocks = [-(-n // page) for n in seq_lens]
    total = sum(blocks) + extra
    order = rng.permutation(total)
    table = np.zeros((len(seq_lens), max(blocks)), dtype=np.int32)
    at = 0
    for s, b in enumerate(blocks):
        table[s, :b] = order[at:at + b]
        at += b
    k = torch.tensor(rng.normal(size=(total, n_kv, page, d)) + 0.5, dtype=dtype)
    v = torch.tensor(rng.normal(size=(total, n_kv, page, d)) + 1.0, dtype=dtype)      # a DC offset in V
    return table, k, v


def _stored(t: torch.Tensor) -> np.ndarray:
    return _bits(t) if t.dtype == torch.bfloat16 else t.numpy()


@pytest.mark.parametrize("n_q,n_kv,d,page,rotary", [(4, 2, 16, 16, 16), (3, 1, 48, 8, 32), (8, 2, 128, 16, 128), (5, 1, 256, 16, 256)])
@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_norm_rotation_and_cache_write(n_q, n_kv, d, page, rotary, mode):
    ops = _ops()
    rng = np.random.default_rng(d + n_q)
    seq_lens, q_lens = [40, 9, 1], [7, 9, 1]
    cdt = torch.float32 if mode == "f32" else torch.bfloat16
    table, k, v = _paged(rng, seq_lens, n_kv, d, page, cdt)
    positions, seq_of = [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        positions += list(range(n - ql, n))
        seq_of += [s] * ql
    t = len(positions)
    qkv = rng.normal(size=(t, (n_q + 2 * n_kv) * d)).astype(np.float32)
    qw, kw = (1 + 0.1 * rng.normal(size=(2, d))).astype(np.float32)
    inv_freq = np.power(np.float64(10000.0), -(2.0 * np.arange(rotary // 2)) / rotary).astype(np.float32)
    kd, vd = k.to(DEV), v.to(DEV)
    q_out = ops.qk_norm_rope_kv_write(_t(qkv), torch.empty(t, n_q * d, dtype=cdt, device=DEV), kd, vd, _t(positions, torch.int32),
                                      _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d, _t(qw), _t(kw), 1e-6,
                                      _t(inv_freq), rotary)
    q_ref = ref.head_norm_rope(qkv[:, :n_q * d], n_q, d, qw, 1e-6, positions, inv_freq, rotary)
    k_ref = ref.head_norm_rope(qkv[:, n_q * d:(n_q + n_kv) * d], n_kv, d, kw, 1e-6, positions, inv_freq, rotary)
    tol = 1e-10 if mode == "f32" else 1e-5                 # sines and cosines of the device against the host's
    assert plain.nmse(q_out.float().cpu().numpy(), q_ref) < tol
    k_c, v_c = _stored(k).copy(), _stored(v).copy()
    for i, (pos, s) in enumerate(zip(positions, seq_of)):
        ref.kv_write(k_c, v_c, table[s], pos, k_ref[i].reshape(n_kv, d), qkv[i, (n_q + n_kv) * d:].reshape(n_kv, d))
    if mode == "f32":
        assert plain.nmse(kd.cpu().numpy(), k_c) < tol and np.array_equal(vd.cpu().numpy(), v_c)
    else:
        widen = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)      # noqa: E731
        assert plain.nmse(kd.float().cpu().numpy(), widen(k_c)) < tol and np.array_equal(_bits(vd), v_c)


@pytest.mark.parametrize("n_q,n_kv,d,page", [(4, 2, 16, 16), (6, 3, 48, 8), (8, 2, 128, 16), (4, 1, 128, 32), (2, 1, 256, 16)])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_kernels(n_q, n_kv, d, page, window):
    """The generic kernel in both precisions, the kernel for portions and the one for single tokens, each against the
    scalar paged attention over the same pages through the same scrambled table."""
    ops = _ops()
    rng = np.random.default_rng(n_q * 100 + d + window)
    seq_lens, q_lens = [1, 70, 300, 33, 150], [1, 1, 130, 33, 1]
    scale = 1.0 / math.sqrt(d)
    for dtype in (torch.float32, torch.bfloat16):
        table, k, v = _paged(rng, seq_lens, n_kv, d, page, dtype)
        positions, seq_of, q_start = [], [], []
        for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
            q_start.append(len(positions))
            positions += list(range(n - ql, n))
            seq_of += [s] * ql
        t = len(positions)
        q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=dtype)
        k_c, v_c = _stored(k), _stored(v)
        want = np.stack([ref.paged_gqa(q[i].float().numpy(), k_c, v_c, table[seq_of[i]], positions[i], n_q, scale, window) for i in range(t)])
        args = (_t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32))
        out = ops.paged_attention_generic(q.to(DEV), k.to(DEV), v.to(DEV), torch.empty(t, n_q * d, dtype=dtype, device=DEV), *args,
                                          n_q, n_kv, d, scale, window)
        assert plain.nmse(out.float().cpu().numpy(), want) < (F32_TOL if dtype == torch.float32 else BF16_TOL)
        if dtype != torch.bfloat16:
            continue
        out = torch.zeros(t, n_q * d, dtype=dtype, device=DEV)
        portions = [s for s in range(len(seq_lens)) if q_lens[s] > 1]
        tiles = [(s, tile) for s in portions for tile in range(-(-q_lens[s] // 128))]
        ops.attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), out, _t([s for s, _ in tiles], torch.int32), _t([tile for _, tile in tiles], torch.int32),
                              _t(q_start, torch.int32), _t(q_lens, torch.int32), args[0], args[2], n_q, n_kv, d, scale, window)
        singles = [q_start[s] for s in range(len(seq_lens)) if q_lens[s] == 1]
        longest = max(seq_lens[s] for s in range(len(seq_lens)) if q_lens[s] == 1)
        space = ops.attention_decode_workspace(len(singles), n_q, d, longest, DEV)
        ops.attention_decode(q.to(DEV), k.to(DEV), v.to(DEV), out, _t(singles, torch.int32), args[0], args[1], args[2], n_q, n_kv, d, scale,
                             window, longest, space)
        assert plain.nmse(out.float().cpu().numpy(), want) < BF16_TOL
