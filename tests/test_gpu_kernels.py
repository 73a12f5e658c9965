"""Each HIP kernel alone against a plain float64 reference, at sizes other
than the engine tests use (ragged widths, odd head counts, several head sizes)."""
import math

import numpy as np
import pytest
import torch

from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from kipp_amd.csrc import ops
    return ops


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def _rel(got, ref):
    return plain.nmse(got, ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    ops = _ops()
    rng = np.random.default_rng(0)
    table = torch.tensor(rng.normal(size=(301, 72)), dtype=dtype)
    tokens = rng.integers(0, 301, size=19)
    out = ops.embed(table.to(DEV), _t(tokens, torch.int32), torch.empty(19, 72, device=DEV))
    assert torch.equal(out.cpu(), table.float()[tokens])


@pytest.mark.parametrize("width,rows", [(2, 1), (72, 5), (2560, 3), (5000, 2), (1536, 4), (8192, 2), (8196, 2), (2560, 300), (1028, 256)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(width, rows, out_dtype):
    """Rows of every width class: up to 256 rows of more than 1,024 columns take a workgroup of 512 or 1,024 threads under
    bfloat16 (1,536; 2,560 and 1,028; 5,000 and 8,192 in two passes), more rows or wider ones the workgroups of 256."""
    ops = _ops()
    rng = np.random.default_rng(width)
    x = rng.normal(size=(rows, width)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=width)).astype(np.float32)
    eps = 1e-5
    ref = plain.rms_norm(x, w, eps)
    got = ops.rmsnorm(_t(x), _t(w), eps, torch.empty(rows, width, dtype=out_dtype, device=DEV))
    tol = 1e-12 if out_dtype == torch.float32 else 1e-5
    assert _rel(got.float().cpu().numpy(), ref) < tol
    # with the residual add fused in: x is updated in place
    delta = rng.normal(size=(rows, width)).astype(np.float32)
    xd = _t(x)
    got = ops.rmsnorm(xd, _t(w), eps, torch.empty(rows, width, dtype=out_dtype, device=DEV), delta=_t(delta))
    assert np.array_equal(xd.cpu().numpy(), x + delta)
    assert _rel(got.float().cpu().numpy(), plain.rms_norm(x + delta, w, eps)) < tol


def test_rmsnorm_reference_vector():
    # /root/reference/tests/kipp_test.c:88-96: x=[3,4], w=1, eps=0 -> x / sqrt(12.5)
    ops = _ops()
    got = ops.rmsnorm(_t([[3.0, 4.0]]), _t([1.0, 1.0]), 0.0, torch.empty(1, 2, device=DEV)).cpu().numpy()[0]
    assert np.allclose(got, np.array([3.0, 4.0]) / math.sqrt(12.5), rtol=1e-6)


@pytest.mark.parametrize("inner,rows", [(1, 1), (200, 7), (9728, 2), (204, 3)])
def test_swiglu(inner, rows):
    ops = _ops()
    rng = np.random.default_rng(inner)
    gu = (3 * rng.normal(size=(rows, 2 * inner))).astype(np.float32)
    ref = plain.silu(gu[:, :inner].astype(np.float64)) * gu[:, inner:]
    got = ops.swiglu(_t(gu), torch.empty(rows, inner, device=DEV))
    assert _rel(got.cpu().numpy(), ref) < 1e-12
    gub = torch.tensor(gu).bfloat16()
    refb = plain.silu(gub[:, :inner].double().numpy()) * gub[:, inner:].double().numpy()
    got = ops.swiglu(gub.to(DEV), torch.empty(rows, inner, dtype=torch.bfloat16, device=DEV))
    assert _rel(got.float().cpu().numpy(), refb) < 1e-5
    # /root/reference/tests/kipp_test.c:130-132
    got = ops.swiglu(_t([[0.0, 1.0, 5.0, 2.0]]), torch.empty(1, 2, device=DEV)).cpu().numpy()[0]
    assert abs(got[0]) < 1e-7 and abs(got[1] - 1.4621172) < 1e-6


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 2, 3), (5, 77, 130), (64, 64, 16), (130, 509, 80), (17, 200, 2560)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_gemm_f32(m, n, k, wdtype):
    ops = _ops()
    rng = np.random.default_rng(m * 1000 + n)
    x = rng.normal(size=(m, k)).astype(np.float32)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=wdtype)
    ref = x.astype(np.float64) @ w.double().numpy().T
    got = ops.gemm_f32(_t(x), w.to(DEV), torch.empty(m, n, device=DEV))
    assert _rel(got.cpu().numpy(), ref) < 1e-12
    # integer-valued inputs: float32 sums are exact, so any tiling fault shows at tolerance 0
    xi = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
    wi = rng.integers(-3, 4, size=(n, k)).astype(np.float32)
    got = ops.gemm_f32(_t(xi), _t(wi).to(wdtype), torch.empty(m, n, device=DEV))
    assert np.array_equal(got.cpu().numpy(), xi @ wi.T)


def test_gemm_f32_reference_vector():
    # /root/reference/tests/kipp_test.c:98-108
    ops = _ops()
    got = ops.gemm_f32(_t([[2.0, -1.0, 0.5]]), _t([[1, 2, 3], [-1, 0.5, 0]]), torch.empty(1, 2, device=DEV))
    assert np.allclose(got.cpu().numpy(), [[1.5, -2.5]])


def test_gemm_f32_rows_do_not_depend_on_the_batch():
    ops = _ops()
    rng = np.random.default_rng(5)
    x = rng.normal(size=(150, 333)).astype(np.float32)
    w = rng.normal(size=(90, 333)).astype(np.float32)
    full = ops.gemm_f32(_t(x), _t(w), torch.empty(150, 90, device=DEV)).cpu().numpy()
    for lo, hi in [(0, 1), (63, 66), (149, 150), (70, 133)]:
        part = ops.gemm_f32(_t(x[lo:hi]), _t(w), torch.empty(hi - lo, 90, device=DEV)).cpu().numpy()
        assert np.array_equal(part, full[lo:hi])


def _paged_setup(rng, seq_lens, n_kv, d, page, dtype, extra_pages=3):
    """Random caches and a scrambled page table for sequences of the given lengths."""
    blocks = [-(-n // page) for n in seq_lens]
    total = sum(blocks) + extra_pages
    perm = rng.permutation(total)
    max_blocks = max(blocks)
    table = np.zeros((len(seq_lens), max_blocks), dtype=np.int32)
    at = 0
    for s, b in enumerate(blocks):
        table[s, :b] = perm[at:at + b]
        at += b
    k = torch.tensor(rng.normal(size=(total, n_kv, page, d)) + 0.5, dtype=dtype)
    v = torch.tensor(rng.normal(size=(total, n_kv, page, d)) + 1.0, dtype=dtype)  # a DC offset in V
    return table, k, v


def _gather(cache, table_row, n, page):
    out = []
    for s in range(n):
        out.append(cache[table_row[s // page], :, s % page, :].double().numpy())
    return np.stack(out)  # [n, n_kv, d]


@pytest.mark.parametrize("n_q,n_kv,d,page", [(4, 2, 16, 16), (6, 3, 48, 8), (5, 1, 80, 4), (8, 8, 128, 16), (2, 1, 256, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 37])
def test_paged_attention_generic(n_q, n_kv, d, page, dtype, window):
    ops = _ops()
    rng = np.random.default_rng(n_q * 100 + d + window)
    seq_lens = [1, 70, 130, 33]              # tokens in the cache after this step
    q_lens = [1, 1, 21, 33]                  # of which the last q_len are this step's queries
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, dtype)
    positions, seq_of = [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        positions += list(range(n - ql, n))
        seq_of += [s] * ql
    t = len(positions)
    q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=dtype)
    scale = 1.0 / math.sqrt(d)
    out = ops.paged_attention_generic(q.to(DEV), k.to(DEV), v.to(DEV), torch.empty(t, n_q * d, dtype=dtype, device=DEV),
                                      _t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32),
                                      n_q, n_kv, d, scale, window)
    ref = np.zeros((t, n_q, d))
    qd = q.double().numpy().reshape(t, n_q, d)
    for i, (pos, s) in enumerate(zip(positions, seq_of)):
        ks, vs = _gather(k, table[s], pos + 1, page), _gather(v, table[s], pos + 1, page)
        lo = max(0, pos - window + 1) if window else 0
        for h in range(n_q):
            g = h // (n_q // n_kv)
            p = plain.softmax((ks[lo:, g] @ qd[i, h]) * scale)
            ref[i, h] = p @ vs[lo:, g]
    tol = 1e-11 if dtype == torch.float32 else 2e-5
    assert _rel(out.float().cpu().numpy().reshape(t, n_q, d), ref) < tol


def test_attention_reference_vector():
    # /root/reference/tests/kipp_test.c:135-175: 2 tokens, 32 query heads over 8 key/value heads,
    # q = k = 0, v0 = 1, v1 = 3 -> token 0 gives 1.0, token 1 gives 2.0
    ops = _ops()
    n_q, n_kv, d, page = 32, 8, 128, 16
    k = torch.zeros(1, n_kv, page, d, device=DEV)
    v = torch.zeros(1, n_kv, page, d, device=DEV)
    v[0, :, 0, :] = 1.0
    v[0, :, 1, :] = 3.0
    q = torch.zeros(2, n_q * d, device=DEV)
    out = ops.paged_attention_generic(q, k, v, torch.empty_like(q), _t([0, 1], torch.int32), _t([0, 0], torch.int32),
                                      _t([[0]], torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), 0).cpu().numpy()
    assert np.allclose(out[0], 1.0) and np.allclose(out[1], 2.0)


@pytest.mark.parametrize("n_q,n_kv,d,page,rotary", [(4, 2, 16, 16, 16), (3, 1, 48, 8, 48), (8, 2, 128, 16, 128), (2, 2, 64, 4, 32),
                                                  (5, 1, 256, 16, 256), (9, 3, 128, 8, 128), (4, 2, 128, 16, 64)])
@pytest.mark.parametrize("mode", ["f32", "bf16"])
@pytest.mark.parametrize("norm", [True, False])
def test_qk_norm_rope_kv_write(n_q, n_kv, d, page, rotary, mode, norm):
    ops = _ops()
    rng = np.random.default_rng(d + n_q)
    seq_lens, q_lens = [40, 9, 1], [7, 9, 1]
    cdt = torch.float32 if mode == "f32" else torch.bfloat16
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, cdt)
    k0, v0 = k.clone(), v.clone()
    positions, seq_of = [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        positions += list(range(n - ql, n))
        seq_of += [s] * ql
    t = len(positions)
    qkv = rng.normal(size=(t, (n_q + 2 * n_kv) * d)).astype(np.float32)
    qw = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    kw = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    eps, theta = 1e-5, 10000.0
    half = rotary // 2
    inv_freq = np.power(np.float64(theta), -(2.0 * np.arange(half)) / rotary).astype(np.float32)
    kd, vd = k.to(DEV), v.to(DEV)
    q_out = ops.qk_norm_rope_kv_write(
        _t(qkv), torch.empty(t, n_q * d, dtype=cdt, device=DEV), kd, vd,
        _t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d,
        _t(qw) if norm else None, _t(kw) if norm else None, eps, _t(inv_freq), rotary)

    # the same with the angles of the step made beforehand: the same bits
    k2, v2 = k.to(DEV), v.to(DEV)
    table_of_angles = ops.rotary_angles(_t(positions, torch.int32), _t(inv_freq), torch.empty(t, rotary, device=DEV))
    q2 = ops.qk_norm_rope_kv_write(
        _t(qkv), torch.empty(t, n_q * d, dtype=cdt, device=DEV), k2, v2,
        _t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d,
        _t(qw) if norm else None, _t(kw) if norm else None, eps, None, rotary, angles=table_of_angles)
    assert torch.equal(q2, q_out) and torch.equal(k2, kd) and torch.equal(v2, vd)
    want = np.float32(np.array(positions, dtype=np.float32)[:, None] * inv_freq[None, :]).astype(np.float64)
    got_angles = table_of_angles.cpu().numpy()
    assert np.abs(got_angles[:, :half] - np.cos(want)).max() < 1e-6 and np.abs(got_angles[:, half:] - np.sin(want)).max() < 1e-6

    def ref_heads(x, n_heads, w):
        x = x.astype(np.float64)
        if norm:
            x = plain.head_norm(x, n_heads, d, w, eps)
        xh = x.reshape(t, n_heads, d)
        rot = plain.rope(xh[..., :rotary].reshape(t, n_heads * rotary), n_heads, rotary, positions, theta)
        xh = np.concatenate([rot.reshape(t, n_heads, rotary), xh[..., rotary:]], axis=-1)
        return xh
    q_ref = ref_heads(qkv[:, :n_q * d], n_q, qw)
    k_ref = ref_heads(qkv[:, n_q * d:(n_q + n_kv) * d], n_kv, kw)
    v_ref = qkv[:, (n_q + n_kv) * d:].reshape(t, n_kv, d)
    tol = 1e-11 if mode == "f32" else 1e-5
    assert _rel(q_out.float().cpu().numpy().reshape(t, n_q, d), q_ref) < tol
    kc, vc = kd.cpu(), vd.cpu()
    touched = torch.zeros(k.shape[0], page, dtype=torch.bool)
    for i, (pos, s) in enumerate(zip(positions, seq_of)):
        pg, slot = table[s, pos // page], pos % page
        touched[pg, slot] = True
        assert _rel(kc[pg, :, slot, :].float().numpy(), k_ref[i]) < tol
        assert _rel(vc[pg, :, slot, :].float().numpy(), v_ref[i]) < (1e-14 if mode == "f32" else 1e-5)
    # every slot that no token of the step maps to is untouched
    keep = ~touched[:, None, :, None].expand_as(k)
    assert torch.equal(kc[keep], k0[keep]) and torch.equal(vc[keep], v0[keep])


@pytest.mark.parametrize("n_q,n_kv,d,rotary", [(4, 2, 16, 16), (3, 1, 48, 32), (2, 1, 128, 128), (2, 2, 256, 64)])
def test_rotary_pairing_of_neighbours(n_q, n_kv, d, rotary):
    """pairing "interleaved": pair i is (2i, 2i + 1).  It is the half pairing of a head whose rotated dims are
    reordered, evens first, then odds: checked against the plain rotation of the reordered head, and head
    sizes that the half pairing rotates in registers take the general kernel here."""
    ops = _ops()
    rng = np.random.default_rng(d)
    t, page = 11, 8
    positions = list(range(20, 20 + t))
    table = np.arange(4, dtype=np.int32)[None, :]
    k = torch.zeros(4, n_kv, page, d, device=DEV)
    v = torch.zeros_like(k)
    qkv = rng.normal(size=(t, (n_q + 2 * n_kv) * d)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    inv_freq = np.power(np.float64(300.0), -(2.0 * np.arange(rotary // 2)) / rotary).astype(np.float32)
    q = ops.qk_norm_rope_kv_write(_t(qkv), torch.empty(t, n_q * d, device=DEV), k, v, _t(positions, torch.int32),
                                  _t([0] * t, torch.int32), _t(table, torch.int32), n_q, n_kv, d, _t(w), _t(w), 1e-6,
                                  _t(inv_freq), rotary, pairing="interleaved").cpu().numpy().reshape(t, n_q, d)
    order = np.concatenate([np.arange(0, rotary, 2), np.arange(1, rotary, 2)])

    def ref(x, heads):
        xh = plain.head_norm(x.astype(np.float64), heads, d, w, 1e-6).reshape(t, heads, d)
        rot = plain.rope(xh[..., order].reshape(t, heads * rotary), heads, rotary, positions, 300.0).reshape(t, heads, rotary)
        out = xh.copy()
        out[..., order] = rot
        return out
    assert _rel(q, ref(qkv[:, :n_q * d], n_q)) < 1e-11
    k_ref = ref(qkv[:, n_q * d:(n_q + n_kv) * d], n_kv)
    kc = k.cpu().numpy()
    for i, pos in enumerate(positions):
        assert _rel(kc[pos // page, :, pos % page, :], k_ref[i]) < 1e-11
    with pytest.raises(Exception):
        ops.qk_norm_rope_kv_write(_t(qkv), torch.empty(t, n_q * d, device=DEV), k, v, _t(positions, torch.int32),
                                  _t([0] * t, torch.int32), _t(table, torch.int32), n_q, n_kv, d, None, None, 1e-6,
                                  _t(inv_freq), rotary, pairing="pairs of three")


def test_rope_reference_vector():
    # /root/reference/tests/kipp_test.c:110-123: d=4, pos 1, theta 1e4, x=[1,2,3,4]:
    # pair (0,2) turns by 1.0, pair (1,3) by 0.01
    ops = _ops()
    k = torch.zeros(1, 1, 4, 16, device=DEV)
    v = torch.zeros_like(k)
    x = np.zeros((1, 3 * 16), dtype=np.float32)
    x[0, :4] = [1, 2, 3, 4]
    inv_freq = np.array([1.0, 0.01], dtype=np.float32)
    q = ops.qk_norm_rope_kv_write(_t(x), torch.empty(1, 16, device=DEV), k, v, _t([1], torch.int32), _t([0], torch.int32),
                                  _t([[0]], torch.int32), 1, 1, 16, None, None, 0.0, _t(inv_freq), 4).cpu().numpy()[0]
    c, s, c2, s2 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    assert np.allclose(q[:4], [c - 3 * s, 2 * c2 - 4 * s2, 3 * c + s, 4 * c2 + 2 * s2], rtol=1e-6)


@pytest.mark.parametrize("vocab,rows", [(1, 1), (509, 3), (151936, 2)])
def test_argmax(vocab, rows):
    ops = _ops()
    rng = np.random.default_rng(vocab)
    logits = rng.normal(size=(rows, vocab)).astype(np.float32)
    if vocab > 10:
        logits[0, 7] = logits[0, vocab - 3] = 50.0   # a tie: the lowest index wins
    got = ops.argmax(_t(logits), torch.empty(rows, dtype=torch.int32, device=DEV)).cpu().numpy()
    assert np.array_equal(got, np.argmax(logits, axis=1))


# ----------------------------------------------------------------------------- bfloat16 kernels

def _attention_reference(q, k, v, table, positions, seq_of, n_q, n_kv, d, page, window):
    t = len(positions)
    scale = 1.0 / math.sqrt(d)
    ref = np.zeros((t, n_q, d))
    qd = q.double().numpy().reshape(t, n_q, d)
    cache = {}
    for i, (pos, s) in enumerate(zip(positions, seq_of)):
        if s not in cache or cache[s][0].shape[0] < pos + 1:
            n = max(p for p, ss in zip(positions, seq_of) if ss == s) + 1
            cache[s] = (_gather(k, table[s], n, page), _gather(v, table[s], n, page))
        ks, vs = cache[s]
        lo = max(0, pos - window + 1) if window else 0
        for h in range(n_q):
            g = h // (n_q // n_kv)
            p = plain.softmax((ks[lo:pos + 1, g] @ qd[i, h]) * scale)
            ref[i, h] = p @ vs[lo:pos + 1, g]
    return ref


@pytest.mark.parametrize("n_q,n_kv,d,page", [(32, 8, 128, 16), (6, 2, 48, 8), (4, 4, 64, 4), (16, 1, 32, 16), (8, 2, 256, 32), (2, 1, 16, 16)])
@pytest.mark.parametrize("window", [0, 300])
def test_attention_decode(n_q, n_kv, d, page, window):
    ops = _ops()
    rng = np.random.default_rng(n_q * 7 + d + window)
    seq_lens = [1, 70, 300, 700, 256, 257, 513]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    # a batch in which the decode tokens are not the first rows: rows 1, 3, 4, ... of a larger batch
    t = len(seq_lens) + 3
    rows = [1, 3, 4, 5, 7, 8, 9]
    positions = [0] * t
    seq_of = [0] * t
    for r, (s, n) in zip(rows, enumerate(seq_lens)):
        positions[r], seq_of[r] = n - 1, s
    q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=torch.bfloat16)
    out = torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV)
    ws = ops.attention_decode_workspace(len(rows), n_q, d, max(seq_lens), DEV)
    ops.attention_decode(q.to(DEV), k.to(DEV), v.to(DEV), out, _t(rows, torch.int32), _t(positions, torch.int32),
                         _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), window,
                         max(seq_lens), ws)
    ref = _attention_reference(q[rows], k, v, table, [positions[r] for r in rows], [seq_of[r] for r in rows],
                               n_q, n_kv, d, page, window)
    got = out.float().cpu().numpy().reshape(t, n_q, d)
    assert _rel(got[rows], ref) < 1e-5
    untouched = [r for r in range(t) if r not in rows]
    assert not got[untouched].any()


@pytest.mark.parametrize("n_seqs,n_q,n_kv,d,page,window,longest", [
    (6, 32, 8, 128, 16, 0, 4500), (6, 32, 8, 128, 16, 600, 4500), (6, 6, 2, 48, 8, 0, 4500), (6, 16, 1, 32, 16, 0, 4500),
    (12, 32, 8, 128, 16, 0, 4500),          # a dozen sequences: the kernel that streams through LDS, in ranges
    (8, 16, 8, 64, 16, 0, 9500)])           # long contexts at a head size the LDS kernel does not take: long ranges
def test_attention_decode_merged_by_the_last_workgroup_gives_the_bits_of_the_merge_launch(n_seqs, n_q, n_kv, d, page, window, longest):
    """The splits of a head are merged by whichever of their workgroups finishes last, from partial results
    written through to memory, or (without the arrival counts in the workspace) by a launch of its own: the same
    sums in the same order, so the same bits, in each of the three kernels.  Several launches on one workspace,
    with other contexts each time (a count that was not set back, or a partial result read before it arrived,
    would show), one to two dozen splits a head, a sequence of one split among them."""
    ops = _ops()
    rng = np.random.default_rng(n_q + d + window + n_seqs)
    ws = ops.attention_decode_workspace(n_seqs, n_q, d, longest, DEV)
    assert len(ws) == 3 and ws[2].dtype == torch.int32 and not ws[2].any()
    for launch in range(4 if longest < 5000 else 2):
        seq_lens = [int(n) for n in rng.integers(longest // 2, longest, size=n_seqs - 1)] + [int(rng.integers(1, 190))]
        if launch % 2:
            seq_lens[0] = int(rng.integers(260, 600))
        table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
        rows = list(range(n_seqs))
        positions = [n - 1 for n in seq_lens]
        q = torch.tensor(rng.normal(size=(n_seqs, n_q * d)), dtype=torch.bfloat16).to(DEV)
        args = (k.to(DEV), v.to(DEV))
        idx = (_t(rows, torch.int32), _t(positions, torch.int32), _t(rows, torch.int32), _t(table, torch.int32))
        here, apart = (torch.zeros(n_seqs, n_q * d, dtype=torch.bfloat16, device=DEV) for _ in range(2))
        ws[0].fill_(float("nan"))
        ops.attention_decode(q, *args, here, *idx, n_q, n_kv, d, 1 / math.sqrt(d), window, max(seq_lens), ws)
        torch.cuda.synchronize()
        assert not ws[2].any(), f"launch {launch}: a count was not set back"
        ops.attention_decode(q, *args, apart, *idx, n_q, n_kv, d, 1 / math.sqrt(d), window, max(seq_lens), ws[:2])
        assert torch.equal(here, apart), f"launch {launch}"
        if launch == 0:
            some = [0, n_seqs - 1]
            ref = _attention_reference(q.cpu()[some], k, v, table, [positions[i] for i in some], some, n_q, n_kv, d, page, window)
            assert _rel(here.float().cpu().numpy().reshape(n_seqs, n_q, d)[some], ref) < 1e-5


@pytest.mark.parametrize("n_q,n_kv,d,page,window", [(32, 8, 128, 16, 0), (32, 8, 128, 16, 1500), (6, 2, 48, 8, 0), (2, 1, 16, 16, 700)])
def test_attention_decode_of_many_rows(n_q, n_kv, d, page, window):
    """The kernel that walks long ranges of keys with a running maximum (built here so that it
    takes over at 1,024 keys instead of 8,192): contexts on both sides of its range and block
    edges (128, 129, 1024, 1025, 2049), the first token, rows that are not the first of the batch."""
    ops = _ops()
    inner = ops._fn

    def early(lib, name, argtypes, defines=None):
        return inner(lib, name, argtypes, dict(defines, STREAM_FROM=1024) if lib == "attention_decode" else defines)
    ops._fn = early
    try:
        _many_rows(ops, n_q, n_kv, d, page, window)
    finally:
        ops._fn = inner


def _many_rows(ops, n_q, n_kv, d, page, window):
    rng = np.random.default_rng(n_q + d + window)
    n_rows = 512 // n_kv + 8
    edge = [1, 2, 127, 128, 129, 255, 256, 257, 1023, 1024, 1025, 2047, 2048, 2049, 2300]
    seq_lens = (edge + [int(x) for x in rng.integers(1, 2300, size=n_rows)])[:n_rows]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    t = n_rows + 2
    rows = list(range(2, t))
    positions, seq_of = [0] * t, [0] * t
    for r, (sq, n) in zip(rows, enumerate(seq_lens)):
        positions[r], seq_of[r] = n - 1, sq
    q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=torch.bfloat16)
    out = torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV)
    ws = ops.attention_decode_workspace(n_rows, n_q, d, max(seq_lens), DEV)
    ops.attention_decode(q.to(DEV), k.to(DEV), v.to(DEV), out, _t(rows, torch.int32), _t(positions, torch.int32),
                         _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), window,
                         max(seq_lens), ws)
    got = out.float().cpu().numpy().reshape(t, n_q, d)
    check = list(range(len(edge))) + list(range(len(edge), n_rows, 7))        # the plain form is slow: the edges and a sample
    ref = _attention_reference(q[[rows[i] for i in check]], k, v, table, [positions[rows[i]] for i in check],
                               [seq_of[rows[i]] for i in check], n_q, n_kv, d, page, window)
    assert _rel(got[[rows[i] for i in check]], ref) < 1e-5
    assert not got[:2].any()


def _whole_contexts(ops):
    """The kernels built so that the one in which a workgroup walks a whole context takes every launch
    it can (head size 128, pages of 16 keys and more), not only those of many sequences."""
    inner = ops._fn

    def forced(lib, name, argtypes, defines=None):
        return inner(lib, name, argtypes, dict(defines, RING_FROM_PAIRS=1) if lib == "attention_decode" else defines)
    return inner, forced


@pytest.mark.parametrize("n_q,n_kv,d,page,window", [(32, 8, 128, 16, 0), (32, 8, 128, 16, 300), (16, 1, 128, 32, 0), (16, 1, 128, 16, 5000)])
def test_attention_decode_over_whole_contexts(n_q, n_kv, d, page, window):
    """A workgroup a (sequence, key/value head), keys and values streamed through LDS: contexts of one
    key, at block edges (15, 16, 17, 63, 64, 65), around a stage's and a range's end (4095, 4096, 4097, 8200),
    rows that are not the first of the batch."""
    ops = _ops()
    inner, forced = _whole_contexts(ops)
    ops._fn = forced
    try:
        rng = np.random.default_rng(n_q + page + window)
        seq_lens = [1, 2, 15, 16, 17, 63, 64, 65, 128, 300, 777, 1024, 2049] + ([4095, 4096, 4097, 8200] if n_kv == 1 else [])
        table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
        t = len(seq_lens) + 2
        rows = list(range(2, t))
        positions, seq_of = [0] * t, [0] * t
        for r, (sq, n) in zip(rows, enumerate(seq_lens)):
            positions[r], seq_of[r] = n - 1, sq
        q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=torch.bfloat16)
        out = torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV)
        ws = ops.attention_decode_workspace(len(rows), n_q, d, max(seq_lens), DEV)
        ops.attention_decode(q.to(DEV), k.to(DEV), v.to(DEV), out, _t(rows, torch.int32), _t(positions, torch.int32),
                             _t(seq_of, torch.int32), _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), window,
                             max(seq_lens), ws)
        ref = _attention_reference(q[rows], k, v, table, [positions[r] for r in rows], [seq_of[r] for r in rows],
                                   n_q, n_kv, d, page, window)
        got = out.float().cpu().numpy().reshape(t, n_q, d)
        for i, r in enumerate(rows):
            assert _rel(got[r], ref[i]) < 1e-5, f"context of {seq_lens[i]} keys"
        assert not got[:2].any()
    finally:
        ops._fn = inner


@pytest.mark.parametrize("window", [0, 2500])
def test_attention_decode_of_a_dozen_sequences_in_ranges(window):
    """12 sequences of 8 key/value heads are 96 workgroups when each walks a whole context: behind 2,000 to
    3,000 keys the streaming kernel takes them in ranges that give 256 (here 1,152 keys), merged in order;
    contexts at the ranges' edges, both forms of the kernel, the same bits from both."""
    ops = _ops()
    n_q, n_kv, d, page = 32, 8, 128, 16
    longest = 3072
    assert ops.attention_decode_streams(12, n_kv, d, n_q // n_kv, page, longest, window)
    rng = np.random.default_rng(33 + window)
    seq_lens = [2100, 3000, 1151, 1152, 1153, 1, 2304, 2305, 500, 3072, 17, 2700]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    t = len(seq_lens)
    rows, positions, seq_of = list(range(t)), [n - 1 for n in seq_lens], list(range(t))
    qkv = _t(rng.normal(size=(t, (n_q + 2 * n_kv) * d)).astype(np.float32))
    inv_freq = _t(np.power(1e6, -(2.0 * np.arange(d // 2)) / d).astype(np.float32))
    args = (_t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32))
    ws = ops.attention_decode_workspace(t, n_q, d, longest, DEV)
    k1, v1 = k.to(DEV), v.to(DEV)
    q = ops.qk_norm_rope_kv_write(qkv, torch.empty(t, n_q * d, dtype=torch.bfloat16, device=DEV), k1, v1, *args, n_q, n_kv, d,
                                  None, None, 0.0, inv_freq, d, write_kv=True)
    want = ops.attention_decode(q, k1, v1, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV), _t(rows, torch.int32),
                                *args, n_q, n_kv, d, 1 / math.sqrt(d), window, longest, ws)
    k2, v2 = k.to(DEV), v.to(DEV)
    got = ops.attention_decode_fused(qkv, k2, v2, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                     _t(rows, torch.int32), *args, n_q, n_kv, d, None, None, 0.0, inv_freq, d, True,
                                     1 / math.sqrt(d), window, longest, ws)
    assert torch.equal(got, want) and torch.equal(k1, k2) and torch.equal(v1, v2)
    major = ops.attention_decode_fused(qkv, k.to(DEV), v.to(DEV), torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                       _t(rows, torch.int32), *args, n_q, n_kv, d, None, None, 0.0, inv_freq, d, True,
                                       1 / math.sqrt(d), window, longest, ws, out_steps_major=True)
    assert torch.equal(ops.from_steps_major(major), want)
    ref = _attention_reference(q.cpu(), k1.cpu(), v1.cpu(), table, positions, seq_of, n_q, n_kv, d, page, window)
    out = want.float().cpu().numpy().reshape(t, n_q, d)
    for i in range(t):
        assert _rel(out[i], ref[i]) < 1e-5, f"context of {seq_lens[i]} keys"


@pytest.mark.parametrize("window", [0, 6000, 8000])
def test_attention_decode_of_few_long_sequences(window):
    """Four sequences of several thousand keys: the streaming kernel takes them in ranges of 1,024 keys
    (what gives 256 workgroups), with the merge kernel behind it; contexts at the ranges' edges.  With a
    window of 6,000 the ranges would be shorter than that and the split kernel stays."""
    ops = _ops()
    n_q, n_kv, d, page = 8, 8, 128, 16
    assert ops.attention_decode_streams(4, n_kv, d, 1, page, 9000) and not ops.attention_decode_streams(4, n_kv, d, 1, page, 2000)
    assert ops.attention_decode_streams(4, n_kv, d, 1, page, 9000, 8000) and not ops.attention_decode_streams(4, n_kv, d, 1, page, 9000, 6000)
    rng = np.random.default_rng(17 + window)
    seq_lens = [9000, 1024, 1025, 7168]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    rows = list(range(4))
    positions = [n - 1 for n in seq_lens]
    q = torch.tensor(rng.normal(size=(4, n_q * d)), dtype=torch.bfloat16)
    out = torch.zeros(4, n_q * d, dtype=torch.bfloat16, device=DEV)
    ws = ops.attention_decode_workspace(4, n_q, d, max(seq_lens), DEV)
    ops.attention_decode(q.to(DEV), k.to(DEV), v.to(DEV), out, _t(rows, torch.int32), _t(positions, torch.int32),
                         _t(rows, torch.int32), _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), window, max(seq_lens), ws)
    ref = _attention_reference(q, k, v, table, positions, rows, n_q, n_kv, d, page, window)
    got = out.float().cpu().numpy().reshape(4, n_q, d)
    for i in range(4):
        assert _rel(got[i], ref[i]) < 1e-5, f"context of {seq_lens[i]} keys"


def test_attention_decode_in_longer_splits():
    """8 sequences of 8 key/value heads behind 2,100 to 2,700 keys: splits of 256 keys would be more workgroups
    than fit at once, so both forms of the kernel cut the keys every 320 (a recorded graph asks for the longest
    context of its bucket: the splits beyond a sequence's position leave at once).  Against the plain attention,
    and the same bits from both forms."""
    ops = _ops()
    n_q, n_kv, d, page = 32, 8, 128, 16
    rng = np.random.default_rng(21)
    seq_lens = [2100, 2700, 2561, 320, 321, 1, 2239, 2240]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    t = len(seq_lens)
    rows, positions, seq_of = list(range(t)), [n - 1 for n in seq_lens], list(range(t))
    width = (n_q + 2 * n_kv) * d
    qkv = _t(rng.normal(size=(t, width)).astype(np.float32))
    inv_freq = _t(np.power(1e6, -(2.0 * np.arange(d // 2)) / d).astype(np.float32))
    args = (_t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32))
    longest = 3072                                     # what a graph recorded for this bucket of contexts asks for
    ws = ops.attention_decode_workspace(t, n_q, d, longest, DEV)
    k1, v1 = k.to(DEV), v.to(DEV)
    q = ops.qk_norm_rope_kv_write(qkv, torch.empty(t, n_q * d, dtype=torch.bfloat16, device=DEV), k1, v1, *args, n_q, n_kv, d,
                                  None, None, 0.0, inv_freq, d, write_kv=True)
    want = ops.attention_decode(q, k1, v1, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV), _t(rows, torch.int32),
                                *args, n_q, n_kv, d, 1 / math.sqrt(d), 0, longest, ws)
    k2, v2 = k.to(DEV), v.to(DEV)
    got = ops.attention_decode_fused(qkv, k2, v2, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                     _t(rows, torch.int32), *args, n_q, n_kv, d, None, None, 0.0, inv_freq, d, True,
                                     1 / math.sqrt(d), 0, longest, ws)
    assert torch.equal(got, want) and torch.equal(k1, k2) and torch.equal(v1, v2)
    major = ops.attention_decode_fused(qkv, k.to(DEV), v.to(DEV), torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                       _t(rows, torch.int32), *args, n_q, n_kv, d, None, None, 0.0, inv_freq, d, True,
                                       1 / math.sqrt(d), 0, longest, ws, out_steps_major=True)
    assert torch.equal(ops.from_steps_major(major), want)
    ref = _attention_reference(q.cpu(), k1.cpu(), v1.cpu(), table, positions, seq_of, n_q, n_kv, d, page, 0)
    assert _rel(want.float().cpu().numpy().reshape(t, n_q, d), ref) < 1e-5


_PROJECTION_GEOMETRIES = [(32, 8, 128, 16), (8, 1, 128, 8), (16, 1, 128, 16), (3, 3, 128, 4), (8, 2, 256, 32), (4, 2, 256, 16)]


@pytest.mark.parametrize("n_q,n_kv,d,page,whole", [g + (False,) for g in _PROJECTION_GEOMETRIES]
                         + [g + (True,) for g in _PROJECTION_GEOMETRIES if g[2] == 128 and g[3] % 16 == 0])
@pytest.mark.parametrize("window,norm,slabs,write_kv", [(0, True, 1, True), (300, True, 3, True), (0, False, 2, True), (0, True, 1, False)])
def test_attention_decode_from_the_projection(n_q, n_kv, d, page, window, norm, slabs, write_kv, whole):
    """Decode attention that starts from the QKV projection's output: the same bits
    in the attention output and in the cache as the rotary kernel followed by the
    attention kernel, at split edges (256, 257, 513) and for the first token.  `whole`: the
    kernels in which a workgroup walks a whole context (head size 128, pages of 16 and more)."""
    ops = _ops()
    inner, forced = _whole_contexts(ops)
    ops._fn = forced if whole else inner
    try:
        _from_the_projection(ops, n_q, n_kv, d, page, window, norm, slabs, write_kv)
    finally:
        ops._fn = inner


def _from_the_projection(ops, n_q, n_kv, d, page, window, norm, slabs, write_kv):
    rng = np.random.default_rng(n_q * 5 + d + window + slabs)
    seq_lens = [1, 70, 300, 700, 256, 257, 513]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    t = len(seq_lens)
    rows = list(range(t))
    positions = [n - 1 for n in seq_lens]
    seq_of = list(range(t))
    width = (n_q + 2 * n_kv) * d
    qkv = _t(rng.normal(size=(slabs, t, width)).astype(np.float32))
    if slabs == 1:
        qkv = qkv[0]
    qw = _t((1 + 0.1 * rng.normal(size=d)).astype(np.float32)) if norm else None
    kw = _t((1 + 0.1 * rng.normal(size=d)).astype(np.float32)) if norm else None
    inv_freq = _t(np.power(1e6, -(2.0 * np.arange(d // 2)) / d).astype(np.float32))
    args = (_t(positions, torch.int32), _t(seq_of, torch.int32), _t(table, torch.int32))
    ws = ops.attention_decode_workspace(t, n_q, d, max(seq_lens), DEV)
    # two kernels
    k1, v1 = k.to(DEV), v.to(DEV)
    q = ops.qk_norm_rope_kv_write(qkv, torch.empty(t, n_q * d, dtype=torch.bfloat16, device=DEV), k1, v1, *args, n_q, n_kv, d,
                                  qw, kw, 1e-6, inv_freq, d, write_kv=write_kv)
    want = ops.attention_decode(q, k1, v1, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV), _t(rows, torch.int32),
                                *args, n_q, n_kv, d, 1 / math.sqrt(d), window, max(seq_lens), ws)
    # one kernel
    k2, v2 = k.to(DEV), v.to(DEV)
    got = ops.attention_decode_fused(qkv, k2, v2, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                     _t(rows, torch.int32), *args, n_q, n_kv, d, qw, kw, 1e-6, inv_freq, d, write_kv,
                                     1 / math.sqrt(d), window, max(seq_lens), ws)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    k3, v3 = k.to(DEV), v.to(DEV)
    angles = ops.rotary_angles(args[0], inv_freq, torch.empty(t, d, device=DEV))
    again = ops.attention_decode_fused(qkv, k3, v3, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                       _t(rows, torch.int32), *args, n_q, n_kv, d, qw, kw, 1e-6, None, d, write_kv,
                                       1 / math.sqrt(d), window, max(seq_lens), ws, angles=angles)
    assert torch.equal(again, got) and torch.equal(k3, k2) and torch.equal(v3, v2)
    assert write_kv != torch.equal(k2.cpu(), k)            # the cache changed exactly when it was to be written
    assert torch.equal(got, want)
    # the rows in the order a few-rows product reads them in: the same values, merged by the last split's workgroup
    # or by a launch of its own
    for workspace in (ws, ws[:2]):
        k4, v4 = k.to(DEV), v.to(DEV)
        major = ops.attention_decode_fused(qkv, k4, v4, torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                           _t(rows, torch.int32), *args, n_q, n_kv, d, qw, kw, 1e-6, inv_freq, d, write_kv,
                                           1 / math.sqrt(d), window, max(seq_lens), workspace, out_steps_major=True)
        assert torch.equal(ops.from_steps_major(major), want) and torch.equal(k4, k2) and torch.equal(v4, v2)
    assert not ops.attention_decode_fused_ok(64, 64, True) and not ops.attention_decode_fused_ok(128, 64, True)
    assert ops.attention_decode_fused_ok(128, 64, False)


@pytest.mark.parametrize("n_q,n_kv,d,page", [(32, 8, 128, 16), (6, 2, 48, 8), (4, 4, 64, 4), (3, 1, 80, 16), (2, 1, 256, 32), (2, 2, 16, 8),
                                             (4, 2, 128, 4), (5, 1, 128, 64)])
@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("tile_rows", [128, 64, 32])
def test_attention_prefill(n_q, n_kv, d, page, window, tile_rows):
    """Tiles of 128 query rows, and of 64 and 32 (what the mixer asks for where tiles of 128 would leave
    compute units idle): the same result whichever way a portion is cut into work items."""
    ops = _ops()
    rng = np.random.default_rng(n_q * 11 + d + window)
    seq_lens = [130, 64, 300, 5, 257]      # tokens in the cache after this step
    q_lens = [130, 2, 100, 5, 129]         # this step's portion of each
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    positions, seq_of, q_start = [], [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        q_start.append(len(positions))
        positions += list(range(n - ql, n))
        seq_of += [s] * ql
    t = len(positions)
    items = [(s, tile) for s, ql in enumerate(q_lens) for tile in range(-(-ql // tile_rows))]
    q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=torch.bfloat16)
    out = ops.attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                _t([i[0] for i in items], torch.int32), _t([i[1] for i in items], torch.int32),
                                _t(q_start, torch.int32), _t(q_lens, torch.int32), _t(positions, torch.int32),
                                _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), window, tile_rows=tile_rows)
    ref = _attention_reference(q, k, v, table, positions, seq_of, n_q, n_kv, d, page, window)
    got = out.float().cpu().numpy().reshape(t, n_q, d)
    for i in range(t):
        assert _rel(got[i], ref[i]) < 2e-5, f"row {i}: position {positions[i]} of sequence {seq_of[i]}"


@pytest.mark.parametrize("n_q,n_kv,d,page", [(8, 2, 128, 16), (6, 2, 48, 8), (3, 1, 80, 16), (2, 2, 16, 8)])
@pytest.mark.parametrize("split_keys", [64, 192, 512])
def test_attention_prefill_with_the_keys_cut(n_q, n_kv, d, page, split_keys):
    """The keys of a work item cut at multiples of `split_keys`, the cuts merged afterwards: portions that begin
    at position 0 and deep in a sequence, a tile whose rows lie on both sides of a cut's edge (rows before the
    edge have nothing in the cut behind it), a row count that is no multiple of the tile."""
    ops = _ops()
    rng = np.random.default_rng(n_q * 7 + d + split_keys)
    seq_lens = [700, 130, 330, 64]
    q_lens = [150, 130, 2, 5]
    table, k, v = _paged_setup(rng, seq_lens, n_kv, d, page, torch.bfloat16)
    positions, seq_of, q_start = [], [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        q_start.append(len(positions))
        positions += list(range(n - ql, n))
        seq_of += [s] * ql
    t = len(positions)
    items, merge_rows, merge_cuts = [], [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        for tile in range(-(-ql // 128)):
            rows = min(128, ql - tile * 128)
            last = n - ql + tile * 128 + rows - 1
            cuts = last // split_keys + 1
            items += [(s, tile, c) for c in range(cuts)]
            merge_rows += list(range(q_start[s] + tile * 128, q_start[s] + tile * 128 + rows))
            merge_cuts += [cuts] * rows
    rng.shuffle(items)                                           # any order of the work items
    space = ops.attention_prefill_workspace(t, n_q, d, max(merge_cuts), DEV)
    space[0].fill_(float("nan"))                                 # whatever the workspace held before is never read
    space[1].fill_(float("nan"))
    q = torch.tensor(rng.normal(size=(t, n_q * d)), dtype=torch.bfloat16)
    cuts = (split_keys, _t([i[2] for i in items], torch.int32), _t(merge_rows, torch.int32), _t(merge_cuts, torch.int32), space)
    out = ops.attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                                _t([i[0] for i in items], torch.int32), _t([i[1] for i in items], torch.int32),
                                _t(q_start, torch.int32), _t(q_lens, torch.int32), _t(positions, torch.int32),
                                _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), 0, cuts=cuts)
    ref = _attention_reference(q, k, v, table, positions, seq_of, n_q, n_kv, d, page, 0)
    got = out.float().cpu().numpy().reshape(t, n_q, d)
    for i in range(t):
        assert _rel(got[i], ref[i]) < 2e-5, f"row {i}: position {positions[i]} of sequence {seq_of[i]}"
    with pytest.raises(Exception):                               # a window is not cut
        ops.attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros(t, n_q * d, dtype=torch.bfloat16, device=DEV),
                              _t([i[0] for i in items], torch.int32), _t([i[1] for i in items], torch.int32),
                              _t(q_start, torch.int32), _t(q_lens, torch.int32), _t(positions, torch.int32),
                              _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), 100, cuts=cuts)


@pytest.mark.parametrize("rise", [3.0, 40.0, 400.0, -40.0])
def test_attention_prefill_with_a_moving_maximum(rise):
    """The head-size-128 kernel takes its exponents against a maximum that follows the true one
    only after it has moved by 2^8: here every query's scores rise (or fall) along the keys by
    `rise` in all, in small steps, so the reference is stale on most tiles and renewed on some."""
    ops = _ops()
    n_q, n_kv, d, page = 4, 2, 128, 16
    rng = np.random.default_rng(int(abs(rise)))
    n, ql = 900, 200
    table, k, v = _paged_setup(rng, [n], n_kv, d, page, torch.bfloat16)
    positions = list(range(n - ql, n))
    q = torch.tensor(rng.normal(size=(ql, n_q * d)), dtype=torch.bfloat16)
    # a direction every query has the component 1 along: key s gets `rise * s / n * sqrt(d)` of it on top of noise
    kk = 0.05 * k.clone().float()
    qq = q.float().reshape(ql, n_q, d).clone()
    qq[:, :, 0] = 1.0
    for s_ in range(n):
        kk[table[0, s_ // page], :, s_ % page, 0] = rise * s_ / n * math.sqrt(d)
    q, kk = qq.reshape(ql, n_q * d).to(torch.bfloat16), kk.to(torch.bfloat16)
    items = list(range(-(-ql // ops.PREFILL_ROWS)))
    out = ops.attention_prefill(q.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(ql, n_q * d, dtype=torch.bfloat16, device=DEV),
                                _t([0] * len(items), torch.int32), _t(items, torch.int32), _t([0], torch.int32),
                                _t([ql], torch.int32), _t(positions, torch.int32), _t(table, torch.int32), n_q, n_kv, d,
                                1 / math.sqrt(d), 0)
    ref = _attention_reference(q, kk, v, table, positions, [0] * ql, n_q, n_kv, d, page, 0)
    got = out.float().cpu().numpy().reshape(ql, n_q, d)
    assert np.isfinite(got).all()
    for i in range(ql):
        assert _rel(got[i], ref[i]) < 2e-5, f"row {i}"


@pytest.mark.parametrize("kernel", ["decode", "prefill"])
def test_one_far_key_among_hundreds_decides(kernel):
    """Random values would hide a key that is skipped or read from the wrong
    page: here one far key has by far the largest score, so the output must be
    its value row."""
    ops = _ops()
    n_q, n_kv, d, page = 8, 2, 128, 16
    rng = np.random.default_rng(3)
    n = 777
    for far in (0, 15, 16, 255, 256, 511, 640, 776):
        table, k, v = _paged_setup(rng, [n], n_kv, d, page, torch.bfloat16)
        qv = rng.normal(size=(1, n_q * d))
        q = torch.tensor(qv, dtype=torch.bfloat16)
        kk = k.clone()
        for g in range(n_kv):   # the far key of head g points along query head 4 g
            kk[table[0, far // page], g, far % page, :] = 6.0 * q[0].reshape(n_q, d)[4 * g]
        if kernel == "decode":
            ws = ops.attention_decode_workspace(1, n_q, d, n, DEV)
            out = ops.attention_decode(q.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(1, n_q * d, dtype=torch.bfloat16, device=DEV),
                                       _t([0], torch.int32), _t([n - 1], torch.int32), _t([0], torch.int32),
                                       _t(table, torch.int32), n_q, n_kv, d, 1 / math.sqrt(d), 0, n, ws)
        else:
            q2 = torch.cat([torch.zeros(1, n_q * d, dtype=torch.bfloat16), q])
            out = ops.attention_prefill(q2.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(2, n_q * d, dtype=torch.bfloat16, device=DEV),
                                        _t([0], torch.int32), _t([0], torch.int32), _t([0], torch.int32), _t([2], torch.int32),
                                        _t([n - 2, n - 1], torch.int32), _t(table, torch.int32), n_q, n_kv, d,
                                        1 / math.sqrt(d), 0)[1:]
        got = out.float().cpu().numpy().reshape(n_q, d)
        for g in range(n_kv):
            want = v[table[0, far // page], g, far % page, :].float().numpy()
            assert np.abs(got[4 * g] - want).max() < 0.02, f"far key {far}, head {4 * g}"


@pytest.mark.parametrize("m", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("n,k,max_parts", [(16, 32, 1), (77, 80, 1), (2560, 200, 8), (2560, 9728, 8), (509, 2560, 2), (6144, 2560, 1),
                                           (40, 4096, 8)])
def test_gemm_skinny(m, n, k, max_parts):
    ops = _ops()
    rng = np.random.default_rng(m + n)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_skinny(x.to(DEV), w.to(DEV), max_parts)
    assert 1 <= out.shape[0] <= max_parts and tuple(out.shape[1:]) == (m, n)
    ref = x.double().numpy() @ w.double().numpy().T
    assert _rel(out.sum(dim=0).cpu().numpy(), ref) < 1e-11
    xi = torch.tensor(rng.integers(-3, 4, size=(m, k)), dtype=torch.bfloat16)
    wi = torch.tensor(rng.integers(-3, 4, size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_skinny(xi.to(DEV), wi.to(DEV), max_parts).sum(dim=0)
    assert np.array_equal(out.cpu().numpy(), xi.float().numpy() @ wi.float().numpy().T)
    if k % 32 == 0:      # the same product from the streaming layout: the same sums in the same order
        wd = w.to(DEV)
        assert torch.equal(ops.gemm_skinny(x.to(DEV), wd, max_parts, tiles=ops.tile_weight(wd)),
                           ops.gemm_skinny(x.to(DEV), wd, max_parts))


@pytest.mark.parametrize("m", [1, 3, 4, 5, 8, 11, 16])
@pytest.mark.parametrize("n,k,tiled", [(16, 32, True), (77, 80, False), (2560, 4096, True), (2560, 9728, True),
                                       (100, 2560, False), (200, 4096, True), (36, 512, True), (5120, 1024, True), (12288, 256, True)])
def test_gemm_skinny_adds_the_residual_and_prepares_the_norm(m, n, k, tiled):
    """The product's own kernel adds it to the residual and writes the rows and partial sums that the
    next product scales its rows by: the chain residual add -> RMS norm -> product without a norm
    kernel (12,288 columns: more partial sums than a lane asks for at once)."""
    ops = _ops()
    rng = np.random.default_rng(m + n + k)
    x = torch.tensor(rng.normal(size=(m, k)) / math.sqrt(k), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=torch.bfloat16)
    norm_w = torch.tensor(1.0 + 0.1 * rng.normal(size=n), dtype=torch.float32)
    residual0 = torch.tensor(rng.normal(size=(m, n)) * 3.0, dtype=torch.float32)
    wd = w.to(DEV)
    tiles = ops.tile_weight(wd) if tiled else None
    eps = 1e-3
    ref_x = residual0.double().numpy() + x.double().numpy() @ w.double().numpy().T
    residual = residual0.to(DEV)
    rows, sumsq = ops.gemm_skinny(x.to(DEV), wd, tiles=tiles, add_norm=(residual, norm_w.to(DEV)))
    assert _rel(residual.cpu().numpy(), ref_x) < 1e-11
    # the rows are exactly bfloat16(new residual * norm weight), the partial sums add up to the rows' sums of squares
    assert torch.equal(rows, (residual * norm_w.to(DEV)).bfloat16())
    parts = (n + 15) // 16
    assert sumsq.shape == (m, (parts + 3) // 4 * 4)
    assert np.allclose(sumsq[:, :parts].sum(dim=1).cpu().numpy(), (residual.double() ** 2).sum(dim=1).cpu().numpy(), rtol=1e-5)
    # the same sums as the product launched alone, in one part, and added afterwards
    assert torch.equal(residual, residual0.to(DEV) + ops.gemm_skinny(x.to(DEV), wd, 1, tiles=tiles)[0])
    # the next product, scaled by the rows' norms, against the product of the normalized rows (up to 16 rows)
    if n % 8 == 0 and n >= 32:
        n2 = 48
        w2 = torch.tensor(rng.normal(size=(n2, n)) / math.sqrt(n), dtype=torch.bfloat16)
        got = ops.gemm_skinny(rows, w2.to(DEV), 4, row_scale=(sumsq, parts, eps)).sum(dim=0)
        normed = ref_x / np.sqrt((ref_x ** 2).mean(axis=1, keepdims=True) + eps) * norm_w.double().numpy()
        ref = normed @ w2.double().numpy().T
        assert _rel(got.cpu().numpy(), ref) < 2e-5
        # the rows alone, for a consumer that does not scale
        finished = ops.scale_rows(rows, sumsq, parts, eps, torch.empty_like(rows))
        assert _rel(finished.float().cpu().numpy(), normed) < 2e-5
        act = ops.gemm_skinny_swiglu(rows, torch.cat([w2, w2]).to(DEV), torch.empty(m, n2, dtype=torch.bfloat16, device=DEV),
                                     row_scale=(sumsq, parts, eps))
        assert _rel(act.float().cpu().numpy(), plain.silu(ref) * ref) < 3e-5


@pytest.mark.parametrize("n,k", [(20, 64), (16, 32), (151, 96), (2560, 4096), (38, 2560)])
def test_tile_weight_by_the_kernel(n, k):
    """The kernel that lays a matrix out for streaming (what the C host calls at load) against the torch form."""
    ops = _ops()
    w = torch.randn(n, k).bfloat16().to(DEV)
    assert torch.equal(ops.tile_weight_device(w), ops.tile_weight(w))
    if n % 2 == 0:
        assert torch.equal(ops.tile_weight_device(w, gate_up=True), ops.tile_weight_pairs(w))


@pytest.mark.parametrize("m", [1, 2, 5, 8])
@pytest.mark.parametrize("n,k", [(96, 64), (2560, 4096), (160, 320)])
def test_few_rows_products_with_rows_in_steps_major_order(m, n, k):
    """The few-rows products read x, and write the rows they make for the next product, as [width / 32][rows][32] when told
    so: the same bits as from and to [rows][width], for the plain product, the residual's end, the activation's end and the
    kernel that finishes a norm's rows."""
    ops = _ops()
    torch.manual_seed(m * 1000 + n)
    x = torch.randn(m, k).bfloat16().to(DEV)
    w = (torch.randn(n, k) * 0.1).bfloat16().to(DEV)
    tiles = ops.tile_weight(w)
    xm = ops.steps_major(x)
    assert torch.equal(ops.from_steps_major(xm), x)
    for t in (None, tiles):
        assert torch.equal(ops.gemm_skinny(xm, w, 4, tiles=t, x_steps_major=True), ops.gemm_skinny(x, w, 4, tiles=t))
    # the residual's end: rows and sums from either order of x, into either order of the rows
    norm_w = (1 + 0.1 * torch.randn(n)).to(DEV)
    res = torch.randn(m, n).to(DEV)
    want_res = res.clone()
    want_rows, want_ss = ops.gemm_skinny(x, w, tiles=tiles, add_norm=(want_res, norm_w))
    for x_major, out_major in ((True, False), (False, True), (True, True)):
        got_res = res.clone()
        rows, ss = ops.gemm_skinny(xm if x_major else x, w, tiles=tiles, add_norm=(got_res, norm_w), x_steps_major=x_major, out_steps_major=out_major)
        parts = (n + 15) // 16                                     # the sums a row has (its stride is rounded up to 4)
        assert torch.equal(got_res, want_res) and torch.equal(ss[:, :parts], want_ss[:, :parts])
        assert torch.equal(ops.from_steps_major(rows) if out_major else rows, want_rows)
        fin = ops.scale_rows(rows, ss, parts, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV), steps_major=out_major)
        assert torch.equal(fin, ops.scale_rows(want_rows, want_ss, parts, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV)))
    # the activation's end ([gate; up] of n / 2 rows each, when n / 2 is a multiple of 32)
    if (n // 2) % 32 == 0:
        for t in (None, ops.tile_weight_pairs(w)):
            want = ops.gemm_skinny_swiglu(x, w, torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV), tiles=t)
            got = ops.gemm_skinny_swiglu(xm, w, torch.empty(m, n // 2, dtype=torch.bfloat16, device=DEV), tiles=t, x_steps_major=True,
                                         out_steps_major=True)
            assert torch.equal(ops.from_steps_major(got), want)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(torch.zeros(2, 40, dtype=torch.bfloat16, device=DEV), torch.zeros(16, 40, dtype=torch.bfloat16, device=DEV), x_steps_major=True)


def test_tile_weight_layout():
    ops = _ops()
    w = torch.arange(20 * 64, dtype=torch.float32).reshape(20, 64).bfloat16()          # 20 rows: the second tile is padded
    t = ops.tile_weight(w.to(DEV)).cpu().view(2, 2, 64, 8)                               # [tile][step][lane][8]
    for tile, step, lane in [(0, 0, 0), (0, 1, 17), (1, 0, 3), (1, 1, 63), (1, 0, 4)]:
        row, col = 16 * tile + lane % 16, 32 * step + 8 * (lane // 16)
        want = w[row, col:col + 8] if row < 20 else torch.zeros(8, dtype=torch.bfloat16)
        assert torch.equal(t[tile, step, lane], want)
    # [gate; up] of 10 + 10 rows in pairs: tile 0 = gate rows 0..7 over up rows 0..7, tile 1 = gate 8, 9 (then zeros) over up 8, 9
    two = ops.tile_weight_pairs(w.to(DEV)).cpu().view(2, 2, 64, 8)
    assert torch.equal(two[0, 1, 16 + 3], w[3, 32 + 8:32 + 16]) and torch.equal(two[0, 0, 32 + 8 + 5], w[10 + 5, 16:24])
    assert torch.equal(two[1, 1, 1], w[9, 32:40]) and torch.equal(two[1, 0, 48 + 9], w[10 + 9, 24:32])
    assert not two[1, 0, 2].any() and not two[1, 1, 8 + 2].any()
    assert ops.pairs_width(10) == 32 and ops.pairs_width(9728) == 2 * 9728
    with pytest.raises(ops.KernelError):
        ops.tile_weight(torch.zeros(16, 40, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(torch.zeros(2, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(20, 64, dtype=torch.bfloat16, device=DEV),
                        tiles=torch.zeros(16 * 64, dtype=torch.bfloat16, device=DEV))   # tiles of another matrix


@pytest.mark.parametrize("m", [1, 17, 32, 33, 64, 65, 81, 113, 128, 129, 177, 200, 256])
@pytest.mark.parametrize("n,k,max_parts", [(16, 32, 1), (77, 80, 4), (2560, 264, 8), (2560, 9728, 16), (509, 2560, 2), (6144, 2560, 16),
                                           (70000, 512, 1)])
def test_gemm_rows(m, n, k, max_parts):
    """Up to 64 rows x is staged in chunks of 256 columns, from 65 rows on in chunks of 128, from 129 of 64."""
    ops = _ops()
    rng = np.random.default_rng(m + n)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_rows(x.to(DEV), w.to(DEV), max_parts)
    assert 1 <= out.shape[0] <= max_parts and tuple(out.shape[1:]) == (m, n)
    ref = x.double().numpy() @ w.double().numpy().T
    assert _rel(out.sum(dim=0).cpu().numpy(), ref) < 1e-11
    xi = torch.tensor(rng.integers(-3, 4, size=(m, k)), dtype=torch.bfloat16)
    wi = torch.tensor(rng.integers(-3, 4, size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_rows(xi.to(DEV), wi.to(DEV), max_parts).sum(dim=0)
    assert np.array_equal(out.cpu().numpy(), xi.float().numpy() @ wi.float().numpy().T)
    if k % 32 == 0:
        wd = w.to(DEV)
        assert torch.equal(ops.gemm_rows(x.to(DEV), wd, max_parts, tiles=ops.tile_weight(wd)),
                           ops.gemm_rows(x.to(DEV), wd, max_parts))


ROWS_CUTS = [41, 51, 61, 71, 81, 52, 62, 72, 82]        # 10 x waves of a workgroup + tiles of 16 rows a wave


@pytest.mark.parametrize("m", [13, 16, 40, 64, 100, 200])
@pytest.mark.parametrize("n,k,parts", [(77, 544, 1), (2560, 1024, 3), (509, 2560, 2), (1200, 320, 1)])
def test_gemm_rows_workgroups_of_any_size(m, n, k, parts):
    """A workgroup of 4 to 8 waves, one or two tiles of 16 rows of W a wave: an output element is summed over K in the
    same order whatever the workgroup, so every cut with the same parts of K gives the same bits."""
    ops = _ops()
    rng = np.random.default_rng(m + n + parts)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16).to(DEV)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=torch.bfloat16).to(DEV)
    tiles = ops.tile_weight(w)
    ref = x.double().cpu().numpy() @ w.double().cpu().numpy().T
    first = None
    for cut in ROWS_CUTS:
        out = ops.gemm_rows(x, w, parts, tiles=tiles, cut=cut)
        assert out.shape == (parts, m, n)
        if first is None:
            first = out
            assert _rel(out.sum(dim=0).cpu().numpy(), ref) < 1e-11
        assert torch.equal(out, first), f"cut {cut}"
        assert torch.equal(ops.gemm_rows(x, w, parts, cut=cut), first), f"cut {cut}, from rows"
    with pytest.raises(ops.KernelError):
        ops.gemm_rows(x, w, parts, tiles=tiles, cut=31)
    with pytest.raises(ops.KernelError):
        ops.gemm_rows(x, w, parts, tiles=tiles, cut=83)


@pytest.mark.parametrize("m", [13, 16, 33, 64, 90, 256])
@pytest.mark.parametrize("inner,k", [(16, 32), (77, 96), (9728, 2560), (1001, 512), (300, 1056)])
def test_gemm_rows_swiglu(m, inner, k):
    """The gate and up products of a few dozen rows with the activation at their end, from the paired tiles, K not split:
    against the plain activation of the exact products, the same bits as the product in one slab followed by the activation
    kernel, and the same from every workgroup size."""
    ops = _ops()
    rng = np.random.default_rng(m + inner)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16).to(DEV)
    w = torch.tensor(rng.normal(size=(2 * inner, k)) / math.sqrt(k), dtype=torch.bfloat16).to(DEV)
    tiles = ops.tile_weight_pairs(w)
    gu = x.double().cpu().numpy() @ w.double().cpu().numpy().T
    ref = plain.silu(gu[:, :inner]) * gu[:, inner:]
    new = lambda: torch.full((m, inner), 7.0, dtype=torch.bfloat16, device=DEV)
    got = ops.gemm_rows_swiglu(x, tiles, new())
    assert _rel(got.float().cpu().numpy(), ref) < 1e-5
    two = ops.swiglu(ops.gemm_rows(x, w, 1, tiles=tiles, pairs=True), new(), pairs=True)
    assert torch.equal(got, two)
    for cut in ROWS_CUTS:
        assert torch.equal(ops.gemm_rows_swiglu(x, tiles, new(), cut=cut), got), f"cut {cut}"
    assert ops.gemm_rows_swiglu_pays(64, 2 * 9728, 2560) and not ops.gemm_rows_swiglu_pays(128, 2 * 9728, 2560)
    assert not ops.gemm_rows_swiglu_pays(64, 2 * 512, 2560)          # too few rows of W to go round without splitting K


TILE_CUTS = [0, 441, 442, 444, 421, 422, 243, 221, 224, 431, 432, 232, 1421, 1422, 1424, 1221]      # 100 wm + 10 wn + parts (+ 1000: 8 waves; + 2000: whole rounds of those, the rest smaller; + 10000 r: the rest's tile); 0: what the launcher plans


@pytest.mark.parametrize("force", TILE_CUTS)
@pytest.mark.parametrize("m,n,k", [(257, 300, 64), (300, 2560, 96), (513, 77, 2560), (1000, 640, 352), (64, 16, 32)])
def test_gemm_tiles_float32_end(m, n, k, force):
    """The product for prompt portions, every wave tile and split of K, at sizes that end inside tiles on both
    sides (and one smaller than any tile): against float64, and exactly on small integers."""
    ops = _ops()
    if force % 10 > k // 32:
        pytest.skip("more parts than steps of K")
    rng = np.random.default_rng(m + n + force)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_tiles(x.to(DEV), w.to(DEV), "slabs", max_parts=4, force=force)
    assert tuple(out.shape[1:]) == (m, n) and (out.shape[0] == force % 10 if force else 1 <= out.shape[0] <= 4)
    ref = x.double().numpy() @ w.double().numpy().T
    assert _rel(out.sum(dim=0).cpu().numpy(), ref) < 1e-11
    xi = torch.tensor(rng.integers(-3, 4, size=(m, k)), dtype=torch.bfloat16)
    wi = torch.tensor(rng.integers(-3, 4, size=(n, k)), dtype=torch.bfloat16)
    out = ops.gemm_tiles(xi.to(DEV), wi.to(DEV), "slabs", max_parts=4, force=force).sum(dim=0)
    assert np.array_equal(out.cpu().numpy(), xi.float().numpy() @ wi.float().numpy().T)


@pytest.mark.parametrize("force", [0, 441, 421, 241, 221, 1421, 1221, 2421, 32421])
@pytest.mark.parametrize("m,inner,k", [(257, 150, 64), (600, 9728 // 8, 160), (300, 24, 2560), (2050, 1300, 96), (2050, 4804, 64)])
def test_gemm_tiles_swiglu_and_bfloat16_ends(m, inner, k, force):
    """W = [gate; up]: silu(x . gate^T) * (x . up^T) rounded once, at the end (gate first: the other way round
    gives another result), also where the launcher cuts the columns into two kinds of tiles (as planned, or
    forced with + 2000: whole rounds of 8-wave tiles and the rest of the columns in smaller ones, which the
    last size has); and the plain bfloat16 end.  Widths that are no multiple of 8 take the store of single values."""
    ops = _ops()
    rng = np.random.default_rng(m + inner + force)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(2 * inner, k)) * 0.3, dtype=torch.bfloat16)
    act = ops.gemm_tiles(x.to(DEV), w.to(DEV), "swiglu", force=force)
    assert act.dtype == torch.bfloat16 and tuple(act.shape) == (m, inner)
    both = x.double().numpy() @ w.double().numpy().T
    ref = plain.silu(both[:, :inner]) * both[:, inner:]
    assert _rel(act.float().cpu().numpy(), ref) < 2e-5
    assert _rel(act.float().cpu().numpy(), plain.silu(both[:, inner:]) * both[:, :inner]) > 1e-2
    rounded = ops.gemm_tiles(x.to(DEV), w.to(DEV), "bf16", force=force)
    assert rounded.dtype == torch.bfloat16 and _rel(rounded.float().cpu().numpy(), both) < 2e-5
    # bit for bit what rounding the float32 end gives
    exact = ops.gemm_tiles(x.to(DEV), w.to(DEV), "slabs", force=force)[0]
    assert torch.equal(rounded, exact.to(torch.bfloat16))


def test_gemm_tiles_cuts_with_the_same_parts_give_the_same_bits():
    """An output element is summed over K in the same order whatever the wave tile and the number of waves: every
    cut with the same parts of K gives the same bits (the runtime relies on it when it takes the fastest of them)."""
    ops = _ops()
    rng = np.random.default_rng(3)
    x = torch.tensor(rng.normal(size=(700, 2560)), dtype=torch.bfloat16).to(DEV)
    w = torch.tensor(rng.normal(size=(1300, 2560)) * 0.05, dtype=torch.bfloat16).to(DEV)
    for parts, cuts in ((1, (441, 431, 421, 241, 221, 1421, 1221)), (2, (442, 432, 422, 222, 1422)), (4, (444, 424, 1424))):
        base = ops.gemm_tiles(x, w, "slabs", max_parts=4, force=cuts[0])
        assert base.shape[0] == parts
        for cut in cuts[1:]:
            assert torch.equal(ops.gemm_tiles(x, w, "slabs", max_parts=4, force=cut), base), cut
    gated = ops.gemm_tiles(x, w, "swiglu", force=441)
    for cut in (0, 421, 241, 221, 1421):
        assert torch.equal(ops.gemm_tiles(x, w, "swiglu", force=cut), gated), cut
    # wide enough for whole rounds of tiles and a rest
    x = torch.tensor(rng.normal(size=(2050, 96)), dtype=torch.bfloat16).to(DEV)
    w = torch.tensor(rng.normal(size=(2 * 4800, 96)) * 0.3, dtype=torch.bfloat16).to(DEV)
    gated = ops.gemm_tiles(x, w, "swiglu", force=441)
    for cut in (0, 1421, 2421, 12421, 22421, 32421):
        assert torch.equal(ops.gemm_tiles(x, w, "swiglu", force=cut), gated), cut


def test_gemm_tiles_refuses_what_it_cannot_do():
    ops = _ops()
    x = torch.zeros(300, 40, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception):
        ops.gemm_tiles(x, torch.zeros(64, 40, dtype=torch.bfloat16, device=DEV))            # K no multiple of 32
    with pytest.raises(Exception):
        ops.gemm_tiles(x.float(), torch.zeros(64, 40, device=DEV))                             # float32 operands
    with pytest.raises(Exception):
        ops.gemm_tiles(torch.zeros(300, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(63, 64, dtype=torch.bfloat16, device=DEV),
                       "swiglu")                                                               # an odd number of rows is no [gate; up]


def test_consumers_add_slabs_in_order():
    """The rotary kernels and SwiGLU take a product that comes in slabs."""
    ops = _ops()
    rng = np.random.default_rng(12)
    for d in (32, 128):                                    # through LDS, and in registers
        n_q, n_kv, page, t = 4, 2, 8, 5
        slabs = rng.normal(size=(3, t, (n_q + 2 * n_kv) * d)).astype(np.float32)
        whole = slabs[0] + slabs[1] + slabs[2]
        table = np.arange(4, dtype=np.int32).reshape(1, 4)
        inv_freq = np.power(1e4, -(2.0 * np.arange(d // 2)) / d).astype(np.float32)
        outs = []
        for qkv in (slabs, whole):
            k, v = torch.zeros(4, n_kv, page, d, device=DEV), torch.zeros(4, n_kv, page, d, device=DEV)
            q = ops.qk_norm_rope_kv_write(_t(qkv), torch.empty(t, n_q * d, device=DEV), k, v, _t(np.arange(t), torch.int32),
                                          _t(np.zeros(t), torch.int32), _t(table, torch.int32), n_q, n_kv, d,
                                          _t(np.ones(d)), _t(np.ones(d)), 1e-6, _t(inv_freq), d)
            outs.append((q.cpu(), k.cpu(), v.cpu()))
        assert all(torch.equal(a, b) for a, b in zip(*outs))
    gu = rng.normal(size=(4, 6, 2 * 40)).astype(np.float32)
    a = ops.swiglu(_t(gu), torch.empty(6, 40, device=DEV)).cpu()
    b = ops.swiglu(_t(gu[0] + gu[1] + gu[2] + gu[3]), torch.empty(6, 40, device=DEV)).cpu()
    assert torch.equal(a, b)


def test_stream_read_probe_covers_the_buffer():
    """The bandwidth yardstick reads whole rings only and says how many bytes that was."""
    ops = _ops()
    buf = torch.zeros(3 * 2**20 + 5, dtype=torch.int32, device=DEV)
    for groups, depth in ((8, 4), (32, 8), (5, 16)):
        got = ops.stream_read(buf, groups, depth)
        ring = groups * 4 * depth * 1024
        assert got % ring == 0 and buf.numel() * 4 - ring < got <= buf.numel() * 4
    with pytest.raises(ops.KernelError):
        ops.stream_read(torch.zeros(1024, dtype=torch.int32, device=DEV), 64, 8)    # less than two rings a wave
    torch.cuda.synchronize()


def test_gemm_skinny_refuses_what_it_cannot_do():
    ops = _ops()
    x = torch.zeros(2, 8, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x, torch.zeros(16, 8, dtype=torch.bfloat16, device=DEV))        # K below 32
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(torch.zeros(2, 36, dtype=torch.bfloat16, device=DEV), torch.zeros(16, 36, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("m,inner,k", [(1, 16, 32), (8, 200, 80), (64, 9728, 2560), (5, 77, 40), (33, 100, 2560), (7, 77, 96)])
def test_gemm_skinny_swiglu(m, inner, k):
    ops = _ops()
    rng = np.random.default_rng(m + inner)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(2 * inner, k)) / math.sqrt(k), dtype=torch.bfloat16)
    out = ops.gemm_skinny_swiglu(x.to(DEV), w.to(DEV), torch.empty(m, inner, dtype=torch.bfloat16, device=DEV))
    gu = x.double().numpy() @ w.double().numpy().T
    ref = plain.silu(gu[:, :inner]) * gu[:, inner:]
    assert _rel(out.float().cpu().numpy(), ref) < 1e-5
    if k % 32 == 0:
        wd = w.to(DEV)
        tiled = ops.gemm_skinny_swiglu(x.to(DEV), wd, torch.empty(m, inner, dtype=torch.bfloat16, device=DEV),
                                       tiles=ops.tile_weight_pairs(wd))
        assert torch.equal(tiled, out)


@pytest.mark.parametrize("m,inner,k,max_parts", [(17, 16, 32, 1), (40, 77, 96, 4), (64, 9728, 2560, 12), (100, 200, 256, 2), (128, 1001, 512, 3)])
def test_gate_up_product_from_paired_tiles(m, inner, k, max_parts):
    """Many rows: the product streamed from the paired tiles has its columns tile by tile (8 gates, 8 ups);
    the activation kernel reads them so, one slab or several."""
    ops = _ops()
    rng = np.random.default_rng(m + inner)
    x = torch.tensor(rng.normal(size=(m, k)), dtype=torch.bfloat16)
    w = torch.tensor(rng.normal(size=(2 * inner, k)) / math.sqrt(k), dtype=torch.bfloat16)
    wd = w.to(DEV)
    y = ops.gemm_rows(x.to(DEV), wd, max_parts, tiles=ops.tile_weight_pairs(wd), pairs=True)
    assert y.shape[1:] == (m, ops.pairs_width(inner)) and 1 <= y.shape[0] <= max_parts
    got = ops.swiglu(y, torch.empty(m, inner, dtype=torch.bfloat16, device=DEV), pairs=True)
    gu = x.double().numpy() @ w.double().numpy().T
    ref = plain.silu(gu[:, :inner]) * gu[:, inner:]
    assert _rel(got.float().cpu().numpy(), ref) < 1e-5
    # the same columns as the plain product, only in another order
    plain_y = ops.gemm_rows(x.to(DEV), wd, max_parts).sum(dim=0).cpu()
    # column c of the paired product: tile c // 16, gate (c % 16 < 8) or up of feature 8 (c // 16) + c % 8
    cols = [(c, 8 * (c // 16) + c % 8, c % 16 >= 8) for c in range(ops.pairs_width(inner))]
    keep = [c for c, f, _ in cols if f < inner]
    order = {c: (inner + f if is_up else f) for c, f, is_up in cols}
    assert _rel(y.sum(dim=0).cpu().numpy()[:, keep], plain_y.numpy()[:, [order[c] for c in keep]]) < 1e-10


@pytest.mark.parametrize("rows,width,n_parts,out_dtype", [(3, 80, 4, torch.float32), (20, 2560, 7, torch.bfloat16), (5, 1536, 2, torch.bfloat16),
                                                       (4, 5120, 9, torch.bfloat16), (300, 2560, 3, torch.bfloat16)])
def test_rmsnorm_adds_slabs_in_order(rows, width, n_parts, out_dtype):
    """The slabs of a split product are added to the residual one after the other, whatever the workgroup's size."""
    ops = _ops()
    rng = np.random.default_rng(8 + rows)
    x = rng.normal(size=(rows, width)).astype(np.float32)
    parts = rng.normal(size=(n_parts, rows, width)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=width)).astype(np.float32)
    xd = _t(x)
    got = ops.rmsnorm(xd, _t(w), 1e-6, torch.empty(rows, width, dtype=out_dtype, device=DEV), delta=_t(parts))
    total = x.copy()
    for p in parts:
        total = total + p
    assert np.array_equal(xd.cpu().numpy(), total)
    assert _rel(got.float().cpu().numpy(), plain.rms_norm(total, w, 1e-6)) < (1e-12 if out_dtype == torch.float32 else 1e-5)


@pytest.mark.parametrize("vocab", [509, 151936])
def test_device_sampler_agrees_with_the_host_sampler(vocab):
    """Same logits, same parameters, same uniform draw: the same token."""
    from kipp_amd.sampling import SampleParams, XorShift64Star, sample
    ops = _ops()
    rng = np.random.default_rng(vocab)
    cases = []
    for temperature in (0.0, 0.3, 0.8, 1.5):
        for top_k in (0, 1, 5, 40):
            for top_p in (1.0, 0.9, 0.3, 1e-6):
                for min_p in (0.0, 0.05, 0.5):
                    cases.append((temperature, top_k, top_p, min_p))
    cases = cases[:: 3 if vocab > 1000 else 1]
    rows = len(cases)
    logits = (rng.normal(size=(rows, vocab)) * rng.choice([0.3, 2.0, 6.0], size=(rows, 1))).astype(np.float32)
    logits[::2, 17] = logits[::2, 400] = logits[::2].max(axis=1) + 0.25    # two equal maxima: the lower id comes first
    logits[1::4, 100:140] = -30.0                                           # many equal values far below
    seeds = rng.integers(1, 2 ** 62, size=rows)
    uniforms = [XorShift64Star(int(s)).uniform() for s in seeds]
    got = ops.sample(_t(logits), _t([c[0] for c in cases]), _t([c[1] for c in cases], torch.int32),
                     _t([c[2] for c in cases]), _t([c[3] for c in cases]), _t(uniforms, torch.float64),
                     torch.empty(rows, dtype=torch.int32, device=DEV)).cpu().tolist()
    for i, (temperature, top_k, top_p, min_p) in enumerate(cases):
        want = sample(logits[i], SampleParams(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p),
                      XorShift64Star(int(seeds[i])))
        assert got[i] == want, f"row {i}: T={temperature} top_k={top_k} top_p={top_p} min_p={min_p}: {got[i]} != {want}"


@pytest.mark.parametrize("vocab", [509, 151936])
def test_bias_and_penalties_on_the_device_are_the_host_sampler_s(vocab):
    """Rows with a bias, with every penalty alone and together, with recent tokens that repeat and that lie outside the
    vocabulary, beside rows with nothing: the changed logits are the host sampler's bit for bit (each step one IEEE
    operation, in its order), and so is the token then chosen for the same draw."""
    from kipp_amd.sampling import SampleParams, XorShift64Star, apply_bias_and_penalties, logit_change_entries, sample
    ops = _ops()
    rng = np.random.default_rng(vocab + 1)
    recents = [[], [3, 7, 3, 3, 100, 7], list(rng.integers(0, vocab, 64)), [5, vocab + 3, 5, 9], [vocab - 1] * 64]
    settings = [dict(), dict(logit_bias={4: 2.5, 100: -7.0, vocab + 9: 1.0}), dict(repetition_penalty=1.3), dict(presence_penalty=0.7),
                dict(frequency_penalty=0.31), dict(repetition_penalty=0.8, presence_penalty=-0.2, frequency_penalty=0.05, logit_bias={3: 1.1, 7: -0.3}),
                dict(repetition_penalty=0.0, frequency_penalty=1e-3)]
    cases = [(SampleParams(temperature=t, top_p=0.9, **kw), recent) for kw in settings for recent in recents for t in (0.0, 0.9)]
    rows = len(cases)
    logits = (rng.normal(size=(rows, vocab)) * 3.0).astype(np.float32)
    begin, biases, tokens, values = [0], [], [], []
    for params, recent in cases:
        t, v, n_bias = logit_change_entries(params, recent, vocab) if params.changes_logits else ([], [], 0)
        tokens += t
        values += v
        biases.append(n_bias)
        begin.append(len(tokens))
    device = _t(logits)
    ops.adjust_logits(device, _t(begin, torch.int32), _t(biases, torch.int32), _t(tokens or [0], torch.int32)[:len(tokens)],
                      _t(values or [0.0])[:len(tokens)], _t([p.repetition_penalty for p, _ in cases]),
                      _t([p.presence_penalty for p, _ in cases]), _t([p.frequency_penalty for p, _ in cases]))
    got = device.cpu().numpy()
    changed = 0
    for i, (params, recent) in enumerate(cases):
        want = apply_bias_and_penalties(logits[i], params, recent)
        assert np.array_equal(got[i], want), f"row {i}: {params} recent {recent[:8]}: {np.flatnonzero(got[i] != want)[:5]}"
        changed += int(not np.array_equal(want, logits[i]))
    assert changed >= rows // 2
    seeds = rng.integers(1, 2 ** 62, size=rows)
    picked = ops.sample(device, _t([p.temperature for p, _ in cases]), _t([0] * rows, torch.int32), _t([0.9] * rows), _t([0.0] * rows),
                        _t([XorShift64Star(int(s)).uniform() for s in seeds], torch.float64), torch.empty(rows, dtype=torch.int32, device=DEV)).cpu().tolist()
    for i, (params, recent) in enumerate(cases):
        assert picked[i] == sample(logits[i], params, XorShift64Star(int(seeds[i])), recent), i


@pytest.mark.parametrize("vocab", [509, 151936])
def test_row_nll_against_float64(vocab):
    """-log softmax at a target: the maximum in float32, exponentials and sum in float64, as the perplexity run of the
    reference adds it up; rows with a far outlier and with equal values."""
    ops = _ops()
    rng = np.random.default_rng(vocab + 5)
    rows = 9
    logits = (rng.normal(size=(rows, vocab)) * rng.choice([0.5, 4.0, 12.0], size=(rows, 1))).astype(np.float32)
    logits[1, 7] = 80.0
    logits[2] = 0.25
    targets = rng.integers(0, vocab, rows)
    targets[1] = 7
    got = ops.row_nll(_t(logits), _t(targets, torch.int32), torch.empty(rows, dtype=torch.float64, device=DEV)).cpu().numpy()
    wide = logits.astype(np.float64)
    top = wide.max(axis=1)
    want = top + np.log(np.exp(wide - top[:, None]).sum(axis=1)) - wide[np.arange(rows), targets]
    assert np.allclose(got, want, rtol=1e-13, atol=1e-13), np.abs(got - want).max()
    assert abs(got[2] - np.log(vocab)) < 1e-12 and got[1] < 1e-6


def test_device_sampler_orders_equal_logits_by_their_ids():
    """Rows of many equal logits, zeros of both signs among them (-0.0 equals 0.0: such candidates are ordered by their ids
    alone, as the host sampler's comparison orders them), quantized values, and every sampling option: the host's token."""
    from kipp_amd.sampling import SampleParams, XorShift64Star, sample
    ops = _ops()
    rng = np.random.default_rng(77)
    vocab, rows = 4096, 192
    logits = (np.round(rng.normal(size=(rows, vocab)) * rng.choice([0.05, 0.5, 2.0], size=(rows, 1)) * 4) / 4).astype(np.float32)
    assert (np.signbit(logits) & (logits == 0)).any() and ((~np.signbit(logits)) & (logits == 0)).any()
    t = rng.choice([0.2, 0.7, 1.0, 1.6], size=rows).astype(np.float32)
    k = rng.choice([0, 0, 1, 3, 50, 900, 2000], size=rows).astype(np.int32)
    p = rng.choice([1.0, 1.0, 0.95, 0.5, 0.1], size=rows).astype(np.float32)
    m = rng.choice([0.0, 0.0, 0.02, 0.3], size=rows).astype(np.float32)
    seeds = rng.integers(1, 2 ** 62, size=rows)
    got = ops.sample(_t(logits), _t(t), _t(k, torch.int32), _t(p), _t(m), _t([XorShift64Star(int(s)).uniform() for s in seeds], torch.float64),
                     torch.empty(rows, dtype=torch.int32, device=DEV)).cpu().tolist()
    for i in range(rows):
        want = sample(logits[i], SampleParams(temperature=float(t[i]), top_k=int(k[i]), top_p=float(p[i]), min_p=float(m[i])), XorShift64Star(int(seeds[i])))
        assert got[i] == want, f"row {i}: T={t[i]} top_k={k[i]} top_p={p[i]} min_p={m[i]}: {got[i]} != {want}"


@pytest.mark.parametrize("vocab", [509, 151936])
def test_device_sampler_at_the_ends_of_the_draw(vocab):
    """A draw of 0 takes the first candidate (the largest logit, the lowest id among equals); a draw just under 1 the last
    one that is kept: the smallest logit within 20 of the largest after the temperature (the highest id among equals), or the
    k-th largest under top-k.  Rows of many candidates (walked level by level) and of few (finished in LDS)."""
    ops = _ops()
    rng = np.random.default_rng(vocab + 9)
    rows = 8
    logits = (rng.normal(size=(rows, vocab)) * np.array([0.05, 0.05, 3.0, 3.0, 9.0, 9.0, 0.05, 9.0])[:, None]).astype(np.float32)
    logits[1, 5] = logits[1, 77] = logits[1].max() + 1.0          # equal maxima
    logits[3, 100:110] = logits[3].min()                           # equal minima
    temperature = np.array([0.8, 1.0, 0.8, 1.3, 0.5, 0.9, 0.8, 0.9], dtype=np.float32)
    top_k = np.array([0, 0, 0, 0, 0, 0, 7, 7], dtype=np.int32)
    for draw in (0.0, 1.0 - 2.0 ** -53):
        got = ops.sample(_t(logits), _t(temperature), _t(top_k, torch.int32), _t([1.0] * rows), _t([0.0] * rows),
                         _t([draw] * rows, torch.float64), torch.empty(rows, dtype=torch.int32, device=DEV)).cpu().tolist()
        for r in range(rows):
            scaled = logits[r] * (np.float32(1.0) / temperature[r])
            order = sorted(range(vocab), key=lambda i: (-float(scaled[i]), i))
            kept = [i for i in order if scaled[i] >= scaled.max() - np.float32(20.0)]
            if top_k[r]:
                kept = kept[:top_k[r]]
            assert got[r] == (kept[0] if draw == 0.0 else kept[-1]), (r, draw, got[r], kept[0], kept[-1], len(kept))


def test_device_sampler_follows_the_distribution():
    ops = _ops()
    from kipp_amd.sampling import XorShift64Star
    logits = np.array([0.0, 3.0, -1.0, 2.5, 1.0, -40.0], dtype=np.float32)
    n = 4000
    r = XorShift64Star(5)
    u = [r.uniform() for _ in range(n)]
    got = ops.sample(_t(np.tile(logits, (n, 1))), _t([0.7] * n), _t([0] * n, torch.int32), _t([1.0] * n), _t([0.0] * n),
                     _t(u, torch.float64), torch.empty(n, dtype=torch.int32, device=DEV)).cpu().numpy()
    p = np.exp((logits[:5] - logits.max()) / 0.7)
    p /= p.sum()
    counts = np.bincount(got, minlength=6)
    assert np.abs(counts[:5] / n - p).max() < 0.03 and counts[5] == 0


@pytest.mark.parametrize("kernel", ["generic", "decode", "prefill"])
def test_window_edge(kernel):
    """With a window of W the key at pos - W + 1 is the oldest one seen and the key at pos - W is
    not: each of the two is given by far the largest score in turn."""
    ops = _ops()
    n_q, n_kv, d, page, window = 8, 2, 128, 16, 300
    rng = np.random.default_rng(9)
    n = 700
    for offset, seen in ((window - 1, True), (window, False)):
        table, k, v = _paged_setup(rng, [n], n_kv, d, page, torch.bfloat16)
        q = torch.tensor(rng.normal(size=(1, n_q * d)), dtype=torch.bfloat16)
        far = n - 1 - offset
        kk = k.clone()
        for g in range(n_kv):
            kk[table[0, far // page], g, far % page, :] = 6.0 * q[0].reshape(n_q, d)[4 * g]
        args = dict(n_q=n_q, n_kv=n_kv, head_dim=d, scale=1 / math.sqrt(d), window=window)
        i32 = lambda x: _t(x, torch.int32)
        if kernel == "generic":
            out = ops.paged_attention_generic(q.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(1, n_q * d, dtype=torch.bfloat16, device=DEV),
                                              i32([n - 1]), i32([0]), i32(table), **args)
        elif kernel == "decode":
            ws = ops.attention_decode_workspace(1, n_q, d, n, DEV)
            out = ops.attention_decode(q.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(1, n_q * d, dtype=torch.bfloat16, device=DEV),
                                       i32([0]), i32([n - 1]), i32([0]), i32(table), max_context=n, workspace=ws, **args)
        else:
            q2 = torch.cat([torch.zeros(1, n_q * d, dtype=torch.bfloat16), q])
            out = ops.attention_prefill(q2.to(DEV), kk.to(DEV), v.to(DEV), torch.zeros(2, n_q * d, dtype=torch.bfloat16, device=DEV),
                                        i32([0]), i32([0]), i32([0]), i32([2]), i32([n - 2, n - 1]), i32(table), **args)[1:]
        got = out.float().cpu().numpy().reshape(n_q, d)
        for g in range(n_kv):
            want = v[table[0, far // page], g, far % page, :].float().numpy()
            close = np.abs(got[4 * g] - want).max() < 0.02
            assert close == seen, f"{kernel}: key at distance {offset} (window {window}) seen={close}, expected {seen}"
