"""The layer sizes of the benchmark shape (Qwen3-4B: hidden 2560, 32 query and 8
key/value heads of 128, SwiGLU 9728, vocabulary 151936, tied), with two layers
so that the plain implementation stays affordable: the kernels run at the
sizes they are measured at, against the same plain reference."""
import numpy as np
import pytest

from tests import helpers as H
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def real_folder(tmp_path_factory):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    cfg = shape_config("qwen3-4b")
    cfg["num_hidden_layers"] = 2
    folder = str(tmp_path_factory.mktemp("real") / "qwen3-4b-2layers")
    write_random_model(folder, cfg, seed=21, dtype="bfloat16")
    return folder


@pytest.fixture(scope="module")
def real_reference(real_folder):
    cfg, weights = plain.load_folder(real_folder)
    requests = {"p": H.random_tokens(1, 150, 151936), "q": H.random_tokens(2, 37, 151936), "r": H.random_tokens(3, 70, 151936)}
    refs = {}
    for rid, toks in requests.items():
        refs[rid] = plain.forward_whole(cfg, weights, toks)
    return requests, refs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_layer_sizes_match_plain(real_folder, real_reference, dtype):
    from kipp_amd.engine import Engine
    requests, refs = real_reference
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16
    for cut, maker in (("whole", H.whole), ("tail", lambda r: H.tail_one_by_one(r, 20)), ("mixed", lambda r: H.mixed(r, seed=4))):
        steps = maker(requests)
        engine = Engine.from_folder(real_folder, dtype=dtype, page_size=16, num_pages=H.peak_pages(requests, steps, 16),
                                    max_requests=4, share_prefixes=False)
        got = H.replay(engine, requests, steps)
        for rid in requests:
            H.assert_close(got[rid], refs[rid], tol, f"4B sizes/{dtype}/{cut}/{rid}")
            if dtype == "float32":
                assert np.array_equal(got[rid].argmax(axis=1), refs[rid].argmax(axis=1))
        del engine
