"""The session interface, after the reference's gates for its cached path
(/root/reference/tests/kipp_test.c:2488-2730, 1684-2026): every check there that
does not need the pinned checkpoint, against the plain implementation."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model(model_folders):
    from kipp_amd.api import Model
    m = Model.open(model_folders[("b", "float32")], dtype="float32", kv_pool_blocks=64, page_tokens=8)
    yield m
    assert not m.sessions
    m.close()


@pytest.fixture(scope="module")
def reference(model_folders):
    toks = H.random_tokens(50, 96, 509)            # three pages and more
    return toks, H.plain_logits(model_folders[("b", "float32")], toks)


def test_cached_decode_equals_recompute_at_every_position(model, reference):
    toks, ref = reference
    s = model.session_create(len(toks))
    for i, t in enumerate(toks[:40]):
        H.assert_close(s.eval([t])[None], ref[i:i + 1], H.NMSE_F32, f"position {i}")
    assert s.get_info().length == 40
    s.destroy()


def test_multi_token_prefill_equals_token_by_token_and_rows_are_bitwise(model, reference):
    toks, ref = reference
    a, b = model.session_create(96), model.session_create(96)
    whole = a.eval_n(toks, 96)
    H.assert_close(whole, ref, H.NMSE_F32, "eval_n")
    singles = np.stack([b.eval([t]) for t in toks])
    assert np.array_equal(whole, singles)          # rows reproduce single-token evaluation bit for bit
    a.destroy()
    b.destroy()


def test_capacity_and_argument_checks(model, reference):
    from kipp_amd.api import ERROR_ARGUMENT, ERROR_RANGE, KippError
    toks, _ = reference
    for bad in (0, 257):
        with pytest.raises(KippError) as e:
            model.session_create(bad)
        assert e.value.code == ERROR_RANGE
    s = model.session_create(10)
    with pytest.raises(KippError) as e:
        s.eval([])
    assert e.value.code == ERROR_ARGUMENT
    s.eval(toks[:10])                              # exactly the capacity
    with pytest.raises(KippError) as e:
        s.eval([1])
    assert e.value.code == ERROR_RANGE and s.length == 10
    with pytest.raises(KippError) as e:
        s.eval_n(toks[:0] + [1], 2)
    t = model.session_create(4)
    with pytest.raises(KippError):
        t.eval([509])                              # outside the vocabulary
    assert t.length == 0
    with pytest.raises(KippError):
        model.close()                              # sessions are alive
    s.destroy()
    t.destroy()
    s.destroy()                                    # twice is harmless


def test_reset_truncate_resume_and_independence(model, reference):
    toks, ref = reference
    s, other = model.session_create(96), model.session_create(96)
    other.eval(H.random_tokens(7, 30, 509))        # a neighbour must not disturb s
    s.eval(toks[:70])
    s.truncate(37)                                 # in the middle of a page
    assert s.length == 37
    other.eval([3])
    H.assert_close(s.eval_n(toks[37:60], 23), ref[37:60], H.NMSE_F32, "truncate and resume")
    s.reset()
    assert s.length == 0
    H.assert_close(s.eval_n(toks[:20], 20), ref[:20], H.NMSE_F32, "after reset")
    from kipp_amd.api import KippError
    with pytest.raises(KippError):
        s.truncate(21)
    s.destroy()
    other.destroy()


def test_batch_of_sessions_equals_isolated_and_rejects_duplicates(model, reference):
    from kipp_amd.api import KippError
    toks, ref = reference
    a, b, c = (model.session_create(96) for _ in range(3))
    a.eval(toks[:33])
    b.eval(toks[:7])
    got = model.eval_batch([(a, toks[33:34]), (b, toks[7:40]), (c, toks[:61])])
    for row, upto in zip(got, (34, 40, 61)):
        H.assert_close(row[None], ref[upto - 1:upto], H.NMSE_F32, f"batch item ending at {upto}")
    with pytest.raises(KippError):
        model.eval_batch([(a, [1]), (a, [2])])
    assert a.length == 34
    for s in (a, b, c):
        s.destroy()


def test_published_prefix_is_adopted_and_a_small_pool_fails_cleanly(model_folders, reference):
    from kipp_amd.api import ERROR_RANGE, KippError, Model
    toks, ref = reference
    m = Model.open(model_folders[("b", "float32")], dtype="float32", kv_pool_blocks=13, page_tokens=8)
    a = m.session_create(96)
    a.eval(toks[:70])
    a.destroy()                                    # publishes 8 full pages
    b = m.session_create(96)
    assert b.match_prefix(toks) == 64
    H.assert_close(b.eval_n(toks[64:90], 26), ref[64:90], H.NMSE_F32, "adopted prefix")
    assert m.kv_pool_stats().reused_pages_total >= 8
    c = m.session_create(96)                       # 12 of 13 pages are held: a long prompt cannot fit
    with pytest.raises(KippError) as e:
        c.eval(toks[:30])
    assert e.value.code == ERROR_RANGE and c.length == 0
    H.assert_close(b.eval_n(toks[90:96], 6), ref[90:96], H.NMSE_F32, "neighbour unharmed")
    c.eval(toks[:8])                               # one page still fits
    for s in (b, c):
        s.destroy()
    stateless = m.eval(toks[:20])
    H.assert_close(stateless[None], ref[19:20], H.NMSE_F32, "stateless evaluation")
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_session_that_is_reset_decodes_over_its_new_pages(model_folders, dtype):
    """A request id that is closed and opened again names a new request with other pages.  Single-token
    steps keep their block tables on the device from step to step and copy a row only when it changed:
    the row of the old request must not serve the new one."""
    from kipp_amd.api import Model
    folder = model_folders[("b", dtype)]
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
    m = Model.open(folder, dtype=dtype, kv_pool_blocks=64, page_tokens=8)
    first, second = H.random_tokens(70, 30, 509), H.random_tokens(71, 30, 509)
    ref_first, ref_second = H.plain_logits(folder, first), H.plain_logits(folder, second)
    s = m.session_create(64)
    s.eval(first[:20])
    for i in range(20, 26):
        H.assert_close(s.eval([first[i]])[None], ref_first[i:i + 1], tol, f"first timeline, position {i}")
    pages_before = list(s._req.tables[0])
    s.reset()
    s.eval(second[:20])
    assert list(s._req.tables[0]) != pages_before       # the case the test is for: same id, other pages
    for i in range(20, 30):
        H.assert_close(s.eval([second[i]])[None], ref_second[i:i + 1], tol, f"after reset, position {i}")
    s.destroy()
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_generations_on_one_engine(model_folders, dtype):
    """The second run's requests take rows of recorded steps that the first run's requests held."""
    from kipp_amd import generate
    from kipp_amd.engine import Engine
    from tests.test_gpu_entry import _follows_plain_argmax
    folder = model_folders[("a", dtype)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=1024, share_prefixes=False)
    margin = 1e-5 if dtype == "float32" else 0.03
    for run in range(3):
        prompts = [H.random_tokens(300 + 10 * run + i, n, 256) for i, n in enumerate([7 + run, 21, 3])]
        outputs = generate(engine, prompts, max_new_tokens=12)
        for prompt, out in zip(prompts, outputs):
            assert len(out) == 12
            _follows_plain_argmax(folder, prompt, out, margin)
    engine.cache.check()


def test_eval_n_reproduces_single_tokens_bitwise_and_eval_scored_within_tolerance(model_folders):
    """/root/reference/src/kipp.h:190-213: `eval_n` rows are the bits of single-token evaluation (so a greedy
    choice cannot flip between verification and decoding); `eval_scored` may run all rows through kernels
    that reduce in another order and agrees within tolerance.  Under bfloat16 the two differ."""
    from kipp_amd.api import Model
    folder = model_folders[("b", "bfloat16")]
    toks = H.random_tokens(81, 60, 509)
    ref = H.plain_logits(folder, toks)
    m = Model.open(folder, dtype="bfloat16", kv_pool_blocks=64, page_tokens=8)
    a, b, c = (m.session_create(64) for _ in range(3))
    exact = a.eval_n(toks, 25)
    scored = b.eval_scored(toks, 25)
    c.eval(toks[:35])
    singles = np.stack([c.eval([t]) for t in toks[35:]])
    assert np.array_equal(exact, singles)
    assert not np.array_equal(scored, singles)
    H.assert_close(scored, ref[35:], H.NMSE_BF16["tiny"], "eval_scored")
    H.assert_close(exact, ref[35:], H.NMSE_BF16["tiny"], "eval_n")
    assert a.length == b.length == c.length == 60
    # all or nothing: 5 tokens that do not fit leave the session as it was, also when some of them ran
    d = m.session_create(10)
    d.eval(toks[:8])
    from kipp_amd.api import KippError
    with pytest.raises(KippError):
        d.eval_n(toks[8:13], 3)
    assert d.length == 8
    for s in (a, b, c, d):
        s.destroy()
    m.close()
