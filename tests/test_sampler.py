"""The host sampler: vectors of its own that show each rule, and then the reference's own sampler
tests, vector for vector (/root/reference/tests/kipp_test.c:502-540, 586-694)."""
import numpy as np
import pytest

from kipp_amd.sampling import SampleParams, XorShift64Star, sample

LOGITS = np.array([0.0, 3.0, -1.0, 2.5, 1.0, -40.0], dtype=np.float32)


def test_xorshift64star_by_hand():
    # /root/reference/src/kipp.c:3322-3329 with state 1
    x = 1
    x ^= x >> 12
    x ^= (x << 25) & (2 ** 64 - 1)
    x ^= x >> 27
    r = XorShift64Star(1)
    assert r.next_u64() == (x * 2685821657736338717) % 2 ** 64 and r.state == x
    assert 0.0 <= r.uniform() < 1.0
    with pytest.raises(ValueError):
        XorShift64Star(0)


def test_greedy_and_degenerate_cases_return_the_argmax():
    assert sample(LOGITS, SampleParams(), None) == 1
    tie = np.array([1.0, 5.0, 5.0], dtype=np.float32)
    assert sample(tie, SampleParams(), None) == 1                        # lowest index wins ties
    rng = XorShift64Star(7)
    assert sample(LOGITS, SampleParams(temperature=1.0, top_p=1e-6), rng) == 1
    assert sample(LOGITS, SampleParams(temperature=1.0, top_k=1), rng) == 1
    r2 = XorShift64Star(7)
    sample(LOGITS, SampleParams(temperature=0.0), r2)
    assert r2.state == 7                                                  # greedy never touches the generator


def test_same_seed_same_tokens_and_the_tail_is_never_drawn():
    a = [sample(LOGITS, SampleParams(temperature=1.5), r) for r in [XorShift64Star(42)] for _ in range(200)]
    b = [sample(LOGITS, SampleParams(temperature=1.5), r) for r in [XorShift64Star(42)] for _ in range(200)]
    assert a == b and 1 in a and 3 in a and 5 not in a                    # token 5 is more than 20 below the maximum


def test_bad_parameters():
    rng = XorShift64Star(1)
    for bad in (SampleParams(temperature=1.0, top_p=0.0), SampleParams(temperature=1.0, top_p=1.5),
                SampleParams(temperature=1.0, min_p=-0.1), SampleParams(temperature=1.0, min_p=1.1)):
        with pytest.raises(ValueError):
            sample(LOGITS, bad, rng)
    with pytest.raises(ValueError):
        sample(LOGITS, SampleParams(temperature=1.0), None)


def test_bias_and_penalties():
    assert sample(LOGITS, SampleParams(logit_bias={2: 10.0}), None) == 2
    # repetition penalty 5.0 on token 1 (3.0 -> 0.6) lets token 3 win
    assert sample(LOGITS, SampleParams(repetition_penalty=5.0), None, recent=[1]) == 3
    # a negative logit is multiplied, not divided
    neg = np.array([-1.0, -2.0], dtype=np.float32)
    assert sample(neg, SampleParams(repetition_penalty=3.0), None, recent=[0]) == 1
    assert sample(LOGITS, SampleParams(presence_penalty=1.0), None, recent=[1, 1]) == 3
    assert sample(LOGITS, SampleParams(frequency_penalty=0.3), None, recent=[1, 1]) == 3
    assert sample(LOGITS, SampleParams(frequency_penalty=0.3), None, recent=[1]) == 1


def test_min_p_and_top_k_cut_the_tail():
    rng = XorShift64Star(3)
    drawn = {sample(LOGITS, SampleParams(temperature=1.0, min_p=0.5), rng) for _ in range(300)}
    assert drawn == {1, 3}                                                # exp(-0.5) = 0.61 stays, exp(-2) goes
    drawn = {sample(LOGITS, SampleParams(temperature=1.0, top_k=3), rng) for _ in range(600)}
    assert drawn == {1, 3, 4}
    drawn = {sample(LOGITS, SampleParams(temperature=1.0, top_p=0.6), rng) for _ in range(300)}
    assert drawn == {1, 3}                                                # 0.55 alone is short of 0.6 of the mass


def test_distribution_matches_softmax():
    rng = XorShift64Star(99)
    n = 20000
    counts = np.bincount([sample(LOGITS, SampleParams(temperature=0.7), rng) for _ in range(n)], minlength=6)
    p = np.exp((LOGITS[:5] - LOGITS.max()) / 0.7)
    p /= p.sum()
    assert np.abs(counts[:5] / n - p).max() < 0.012 and counts[5] == 0


# ------------------------------------------------------------------------------------------------
# The reference's own sampler tests, vector for vector, through the interface that carries its
# names (`kipp_amd.api.sample` / `sample_ex` / `KippError`).

def test_reference_test_sampler():
    # /root/reference/tests/kipp_test.c:502-540 (test_sampler)
    from kipp_amd.api import ERROR_ARGUMENT, KippError, sample as kipp_sample
    logits = np.array([0.1, 4.0, -1.0, 3.5, 0.0, -7.0, 2.0, 1.0], dtype=np.float32)
    assert kipp_sample(logits, 0.0, 1.0, None) == 1
    rng = XorShift64Star(42)
    assert kipp_sample(logits, 1.0, 1.0e-6, rng) == 1
    first = kipp_sample(logits, 1.0, 0.9, XorShift64Star(42))
    token = kipp_sample(logits, 1.0, 0.9, XorShift64Star(42))
    assert token == first and token < 8
    seen = [0] * 8
    rng = XorShift64Star(7)
    for _ in range(200):
        token = kipp_sample(logits, 1.5, 1.0, rng)
        assert token < 8
        seen[token] = 1
    assert seen[1] and seen[3]
    assert not seen[5]
    zero_rng = XorShift64Star(1)
    zero_rng.state = 0
    for call in (lambda: kipp_sample(None, 0.0, 1.0, None),
                 lambda: kipp_sample(logits, 1.0, 0.0, rng),
                 lambda: kipp_sample(logits, 1.0, 1.5, rng),
                 lambda: kipp_sample(logits, 1.0, 1.0, zero_rng)):
        with pytest.raises(KippError) as e:
            call()
        assert e.value.code == ERROR_ARGUMENT


def test_reference_test_sample_ex():
    # /root/reference/tests/kipp_test.c:586-647 (test_sample_ex)
    from kipp_amd.api import ERROR_ARGUMENT, KippError, sample_ex
    logits = np.array([1.0, 5.0, 2.0, 4.0, 0.0, 3.0], dtype=np.float32)
    rng = XorShift64Star(99)
    # greedy over bias-adjusted logits: token 4 is lifted above the rest
    assert sample_ex(logits, SampleParams(temperature=0.0, top_p=1.0, repetition_penalty=1.0, logit_bias={4: 10.0}), None) == 4
    # top_k = 1 with temperature always returns the argmax
    topk = SampleParams(temperature=1.0, top_p=1.0, top_k=1, repetition_penalty=1.0)
    for _ in range(20):
        assert sample_ex(logits, topk, rng) == 1
    # repetition penalty: logit[1] 5.0 / 2 = 2.5, now below logit[3] = 4.0
    penalized = SampleParams(temperature=0.0, top_p=1.0, repetition_penalty=2.0)
    assert sample_ex(logits, penalized, None, recent=[1, 1, 1, 1]) == 3
    # min_p keeps only the dominant token
    peaked = np.array([10.0, 0.0, 0.0, 0.0], dtype=np.float32)
    minp = SampleParams(temperature=1.0, top_p=1.0, min_p=0.5, repetition_penalty=1.0)
    rng = XorShift64Star(7)
    for _ in range(20):
        assert sample_ex(peaked, minp, rng) == 0
    with pytest.raises(KippError) as e:
        sample_ex(logits, SampleParams(temperature=1.0, top_p=1.0, min_p=1.5, repetition_penalty=1.0), rng)
    assert e.value.code == ERROR_ARGUMENT


def test_reference_test_sample_fast_paths():
    # /root/reference/tests/kipp_test.c:655-694: a zero-valued bias forces the path that copies the logits; both
    # paths give the same token from the same generator state and leave the generator in the same state
    from kipp_amd.api import sample_ex
    logits = np.array([np.float32((i * 37 + 11) % 29) * np.float32(0.35) - np.float32((i * 13) % 7) for i in range(64)],
                      dtype=np.float32)
    for temperature in (0.0, 0.8):
        for seed in (1, 7, 99, 12345):
            fast = SampleParams(temperature=temperature, top_p=0.9, top_k=40, repetition_penalty=1.0)
            slow = SampleParams(temperature=temperature, top_p=0.9, top_k=40, repetition_penalty=1.0, logit_bias={3: 0.0})
            assert not fast.changes_logits and slow.changes_logits
            fast_rng, slow_rng = XorShift64Star(seed), XorShift64Star(seed)
            assert sample_ex(logits, fast, fast_rng) == sample_ex(logits, slow, slow_rng)
            assert fast_rng.state == slow_rng.state and (fast_rng.state == seed) == (temperature == 0.0)
