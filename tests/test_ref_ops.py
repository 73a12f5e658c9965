"""The scalar C references of the kernels (kipp_amd/csrc/ref/ref_ops.c) against the plain NumPy implementation and
the vectors of the reference's own tests: the C functions are what the kernel tests and the C host's scalar path
compare with, so they are pinned here first, without a GPU."""
import math

import numpy as np
import pytest

from kipp_amd.csrc import ref
from tests.plain import qwen3_plain as plain


def test_bfloat16_rounding_vectors():
    # /root/reference/tests/kipp_test.c:56-62
    lib = ref.lib()
    assert lib.ref_float_to_bf16(1.0) == 0x3f80 and lib.ref_float_to_bf16(-2.0) == 0xc000
    assert math.isinf(lib.ref_bf16_to_float(0x7f80)) and lib.ref_bf16_to_float(lib.ref_float_to_bf16(1.00390625)) == 1.0
    import torch
    values = np.random.default_rng(0).normal(size=4000).astype(np.float32) * 100
    assert np.array_equal(ref.bf16_bits(values), torch.tensor(values).bfloat16().view(torch.int16).numpy().view(np.uint16))


def test_the_c_references_are_the_plain_formulas():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(5, 72)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=72)).astype(np.float32)
    assert plain.nmse(ref.rms_norm(x, w, 1e-5), plain.rms_norm(x, w, 1e-5)) < 1e-12
    # /root/reference/tests/kipp_test.c:88-96
    assert np.allclose(ref.rms_norm(np.array([[3.0, 4.0]]), np.ones(2), 0.0)[0], np.array([3.0, 4.0]) / math.sqrt(12.5), rtol=1e-6)
    m = rng.normal(size=(31, 72)).astype(np.float32)
    assert plain.nmse(ref.linear(x, m), plain.linear(x, m)) < 1e-12
    assert np.allclose(ref.linear(np.array([[2.0, -1.0, 0.5]]), np.array([[1, 2, 3], [-1, 0.5, 0]])), [[1.5, -2.5]])   # kipp_test.c:98-108
    bits = ref.bf16_bits(m)
    widened = (bits.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(ref.linear(x, bits), ref.linear(x, widened))
    gu = (3 * rng.normal(size=(4, 2 * 50))).astype(np.float32)
    assert plain.nmse(ref.swiglu(gu), plain.silu(gu[:, :50].astype(np.float64)) * gu[:, 50:]) < 1e-12
    assert abs(ref.lib().ref_silu(1.0) - 0.7310586) < 1e-6 and ref.lib().ref_silu(0.0) == 0.0                          # kipp_test.c:130-132
    table = rng.normal(size=(40, 24)).astype(np.float32)
    assert np.array_equal(ref.embed(table, [3, 39, 0]), table[[3, 39, 0]])
    assert ref.argmax(np.array([1.0, 3.0, 3.0, 2.0])) == 1


@pytest.mark.parametrize("interleaved", [False, True])
def test_head_norm_and_rotation(interleaved):
    rng = np.random.default_rng(2)
    heads, d, rotary = 3, 16, 8
    values = rng.normal(size=(6, heads * d)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    positions = np.array([0, 1, 5, 40, 41, 1000])
    inv_freq = np.power(10000.0, -(2.0 * np.arange(rotary // 2)) / rotary).astype(np.float32)
    got = ref.head_norm_rope(values, heads, d, w, 1e-6, positions, inv_freq, rotary, interleaved)
    normed = plain.head_norm(values, heads, d, w, 1e-6)
    if not interleaved:
        want = normed.reshape(6, heads, d).copy()
        want[..., :rotary] = plain.rope(normed.reshape(6, heads, d)[..., :rotary].reshape(6, heads * rotary), heads, rotary, positions,
                                        10000.0).reshape(6, heads, rotary)
        assert plain.nmse(got, want.reshape(6, heads * d)) < 1e-11
    else:
        # interleaved pairing is the half pairing of the head with its rotated dims reordered (evens first, then odds)
        order = np.concatenate([np.arange(0, rotary, 2), np.arange(1, rotary, 2)])
        heads_in = normed.reshape(6, heads, d)
        turned = plain.rope(heads_in[..., order].reshape(6, heads * rotary), heads, rotary, positions, 10000.0).reshape(6, heads, rotary)
        assert plain.nmse(got.reshape(6, heads, d)[..., order], turned) < 1e-11
        assert plain.nmse(got.reshape(6, heads, d)[..., rotary:], heads_in[..., rotary:]) < 1e-13    # dims beyond the rotated ones: normed only
    assert plain.nmse(got[0], normed[0]) < 1e-13       # position 0 turns nothing


@pytest.mark.parametrize("window", [0, 7])
def test_paged_attention_over_a_scrambled_table(window):
    """Keys and values written through a block table into pages in a scrambled order, then read back by the paged
    attention: equal to the plain causal attention over the same keys, for every position."""
    rng = np.random.default_rng(3)
    n_q, n_kv, d, page, n = 6, 2, 16, 4, 23
    pages = 9
    table = rng.permutation(pages)[: -(-n // page)].astype(np.int32)
    q = rng.normal(size=(n, n_q * d)).astype(np.float32)
    k = rng.normal(size=(n, n_kv * d)).astype(np.float32)
    v = (rng.normal(size=(n, n_kv * d)) + 1.0).astype(np.float32)
    for stored in (np.float32, np.uint16):
        k_cache = np.zeros((pages, n_kv, page, d), dtype=stored)
        v_cache = np.zeros((pages, n_kv, page, d), dtype=stored)
        for pos in range(n):
            ref.kv_write(k_cache, v_cache, table, pos, k[pos].reshape(n_kv, d), v[pos].reshape(n_kv, d))
        if stored == np.uint16:
            kk = (ref.bf16_bits(k).astype(np.uint32) << 16).view(np.float32)
            vv = (ref.bf16_bits(v).astype(np.uint32) << 16).view(np.float32)
        else:
            kk, vv = k, v
        want = plain.causal_gqa(q, kk, vv, n_q, n_kv, d, window=window or None)
        got = np.stack([ref.paged_gqa(q[pos], k_cache, v_cache, table, pos, n_q, 1 / math.sqrt(d), window) for pos in range(n)])
        assert plain.nmse(got, want) < 1e-11
    # what lies in the pages is where the table says: position 5 is slot 1 of the table's second page
    assert np.array_equal(k_cache.view(np.uint16)[table[1], :, 1, :], ref.bf16_bits(k[5]).reshape(n_kv, d))
