"""Compile the C host into one shared library, `_lib/libkipp_amd.<hash>.so`.

The hash covers every source of the host, the scalar references it is made of
and the flags, so a changed source is never served by a stale library.  Built
at first use if it is not there (gcc, a few seconds).  `variant="host-only"`
leaves the GPU's table out (no HIP needed to compile or load: what the
sanitizer build of the host logic uses); `sanitize=True` adds AddressSanitizer
and UndefinedBehaviorSanitizer for executables that link the sources
directly (`test_program`).
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import tempfile
from typing import List, Tuple

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.path.join(os.path.dirname(HERE), "csrc", "ref")
SOURCES = ["error.c", "json.c", "config.c", "safetensors.c", "pool.c", "cache.c", "runtime.c", "backend_cpu.c", "parts.c",
           "model.c", "step.c", "scheduler.c", "sampler.c", "hooks.c"]
GPU_SOURCES = ["backend_hip.c"]
# -ffp-contract=off: a sum's bits must not depend on how the compiler happened to fuse a loop
FLAGS = ["-std=c11", "-O2", "-fPIC", "-D_GNU_SOURCE", "-ffp-contract=off", "-Wall", "-Wextra", "-Werror=implicit-function-declaration"]
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


class HostBuildError(RuntimeError):
    pass


def _compiler() -> str:
    for cand in (os.environ.get("CC"), shutil.which("gcc"), shutil.which("cc"), shutil.which("clang")):
        if cand and (os.path.exists(cand) or shutil.which(cand)):
            return cand
    raise HostBuildError("no C compiler found (set CC)")


def _sources(gpu: bool) -> List[str]:
    files = [os.path.join(HERE, f) for f in SOURCES + (GPU_SOURCES if gpu else [])]
    files.append(os.path.join(REF, "ref_ops.c"))
    return files


def _digest(files: List[str], flags: List[str]) -> str:
    h = hashlib.sha1()
    headers = [os.path.join(HERE, f) for f in sorted(os.listdir(HERE)) if f.endswith(".h")] + [os.path.join(REF, "ref_ops.h")]
    for path in files + headers:
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(flags).encode())
    return h.hexdigest()[:10]


def _out_dir() -> str:
    path = os.path.join(HERE, "_lib")
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return path
    except OSError:
        path = os.path.join(tempfile.gettempdir(), f"kipp_amd-{os.getuid()}", "host_lib")
        os.makedirs(path, exist_ok=True)
        return path


def _flags(gpu: bool, sanitize: bool) -> Tuple[List[str], List[str]]:
    compile_flags = list(FLAGS)
    link = ["-lm", "-ldl"]
    if gpu:
        compile_flags += ["-I", os.path.join(ROCM, "include")]
        link += ["-L", os.path.join(ROCM, "lib"), "-lamdhip64", f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}"]
    else:
        compile_flags += ["-DKIPP_NO_HIP"]
    if sanitize:
        compile_flags += ["-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"]
    return compile_flags, link


def _run(cmd: List[str], what: str) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise HostBuildError(f"{what} failed (exit {proc.returncode}):\n{' '.join(cmd)}\n{proc.stdout}{proc.stderr}")


def library_path(variant: str = "gpu", force: bool = False) -> str:
    """The built shared library: "gpu" (all three paths) or "host-only" (cpu-fp32 alone)."""
    gpu = variant == "gpu"
    if variant not in ("gpu", "host-only"):
        raise ValueError("variant is 'gpu' or 'host-only'")
    files = _sources(gpu)
    compile_flags, link = _flags(gpu, False)
    name = f"libkipp_amd{'' if gpu else '_host'}.{_digest(files, compile_flags + link)}.so"
    in_tree = os.path.join(HERE, "_lib", name)
    if os.path.exists(in_tree) and not force:
        return in_tree
    out = os.path.join(_out_dir(), name)
    if os.path.exists(out) and not force:
        return out
    tmp = f"{out}.{os.getpid()}.tmp"
    _run([_compiler()] + compile_flags + ["-shared"] + files + ["-o", tmp] + link, "compiling the C host")
    os.replace(tmp, out)
    for stale in os.listdir(os.path.dirname(out)):
        prefix = "libkipp_amd." if gpu else "libkipp_amd_host."
        if stale.startswith(prefix) and stale.endswith(".so") and stale != name:
            try:
                os.remove(os.path.join(os.path.dirname(out), stale))
            except OSError:
                pass
    return out


def cli_path(force: bool = False) -> str:
    """The built command line of the C host (`kipp_cli.c` linked against the library's sources): `_lib/kipp.<hash>`."""
    files = [os.path.join(HERE, "kipp_cli.c")] + _sources(True)
    compile_flags, link = _flags(True, False)
    name = f"kipp.{_digest(files, compile_flags + link)}"
    in_tree = os.path.join(HERE, "_lib", name)
    if os.path.exists(in_tree) and not force:
        return in_tree
    out = os.path.join(_out_dir(), name)
    if os.path.exists(out) and not force:
        return out
    tmp = f"{out}.{os.getpid()}.tmp"
    _run([_compiler()] + compile_flags + files + ["-o", tmp] + link, "compiling the command line of the C host")
    os.replace(tmp, out)
    for stale in os.listdir(os.path.dirname(out)):
        if stale.startswith("kipp.") and not stale.endswith(".so") and stale != name and ".tmp" not in stale:
            try:
                os.remove(os.path.join(os.path.dirname(out), stale))
            except OSError:
                pass
    return out


def test_program(source: str, out: str, sanitize: bool = True) -> str:
    """An executable of `source` (a C file with main) linked with the host's sources without the GPU's table,
    by default under AddressSanitizer and UndefinedBehaviorSanitizer."""
    compile_flags, link = _flags(False, sanitize)
    _run([_compiler()] + compile_flags + ["-I", HERE, source] + _sources(False) + ["-o", out] + link, "compiling a test program of the C host")
    return out


test_program.__test__ = False


if __name__ == "__main__":
    import sys
    if "--cli" in sys.argv:
        print(cli_path())           # what bin/kipp-c runs: built if it is not there
    else:
        print(library_path("gpu", force=True))
        print(library_path("host-only", force=True))
        print(cli_path(force=True))
