"""The build helper on the CPU, with a stand-in for the compiler: what it prints must not be able to
hold the build up, and a failure must carry the compiler's words."""
import os
import stat
import sys

import pytest

from kipp_amd.csrc import build

FAKE = """#!{python}
import sys
out = sys.argv[sys.argv.index("-o") + 1]
for i in range(4000):                       # far more than a pipe holds
    print("warning: line %d of a long list of warnings that nobody reads before the compiler ends" % i)
if {fail}:
    print("error: this source does not compile")
    sys.exit(1)
open(out, "wb").write(b"not a library")
"""


def _fake_compiler(tmp_path, fail):
    path = tmp_path / ("hipcc_fails" if fail else "hipcc_talks")
    path.write_text(FAKE.format(python=sys.executable, fail=fail))
    path.chmod(path.stat().st_mode | stat.S_IXUSR)
    return str(path)


@pytest.mark.timeout(60)
def test_a_talkative_compiler_does_not_hold_the_build_up(tmp_path, monkeypatch):
    monkeypatch.setenv("HIPCC", _fake_compiler(tmp_path, fail=False))
    monkeypatch.setenv("KIPP_AMD_BUILD_DIR", str(tmp_path / "lib"))
    build.build_all([("elementwise", {"TALKS": 1})])
    out, _, _ = build.library_path("elementwise", {"TALKS": 1})
    assert os.path.exists(out) and open(out, "rb").read() == b"not a library"
    assert not [f for f in os.listdir(os.path.dirname(out)) if f.endswith(".log") or f.endswith(".tmp")]


@pytest.mark.timeout(60)
def test_a_failed_compile_says_what_the_compiler_said(tmp_path, monkeypatch):
    monkeypatch.setenv("HIPCC", _fake_compiler(tmp_path, fail=True))
    monkeypatch.setenv("KIPP_AMD_BUILD_DIR", str(tmp_path / "lib"))
    with pytest.raises(build.BuildError, match="this source does not compile"):
        build.build_all([("elementwise", {"FAILS": 1})])
    out, _, _ = build.library_path("elementwise", {"FAILS": 1})
    assert not os.path.exists(out)
    assert not [f for f in os.listdir(os.path.dirname(out)) if f.endswith(".log") or f.endswith(".tmp")]
