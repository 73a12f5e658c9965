"""Compile the HIP sources for gfx950 and load them with ctypes.

Each `.hip` file becomes one shared library under `_lib/`; the file name holds
a hash of the source, the shared headers, the flags and the specialisation
constants, so a changed source is never served by a stale library.  A library
is compiled at its first use if it is not there (a line is printed when that
starts and every few seconds until it ends); `build_all` compiles a list in
parallel.  If the package folder cannot be written, libraries go to
`$KIPP_AMD_BUILD_DIR` or a per-user folder under the system's temp folder.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import Dict, Iterable, Optional, Tuple

ARCH = "gfx950"
HERE = os.path.dirname(os.path.abspath(__file__))
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unused-result"]

_loaded: Dict[str, ctypes.CDLL] = {}


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels cannot be compiled (set HIPCC or install ROCm)")


def _lib_dir() -> str:
    override = os.environ.get("KIPP_AMD_BUILD_DIR")
    if override:
        os.makedirs(override, exist_ok=True)
        return override
    path = os.path.join(HERE, "_lib")
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return path
    except OSError:
        path = os.path.join(tempfile.gettempdir(), f"kipp_amd-{os.getuid()}", "_lib")
        os.makedirs(path, exist_ok=True)
        return path


def _defines_tag(defines: Optional[dict]) -> Tuple[str, list]:
    if not defines:
        return "", []
    items = sorted(defines.items())
    return "." + ".".join(f"{k}{v}" for k, v in items), [f"-D{k}={v}" for k, v in items]


def library_path(name: str, defines: Optional[dict] = None) -> Tuple[str, list, str]:
    src = os.path.join(HERE, name + ".hip")
    if not os.path.exists(src):
        raise BuildError(f"no kernel source {src}")
    tag, dflags = _defines_tag(defines)
    h = hashlib.sha1()
    headers = sorted(f for f in os.listdir(HERE) if f.endswith(".h"))
    for path in [src] + [os.path.join(HERE, f) for f in headers]:
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + dflags).encode())
    fname = f"libkipp_{name}{tag}.{h.hexdigest()[:10]}.so"
    # a library built in-tree is used even when the build folder is elsewhere
    in_tree = os.path.join(HERE, "_lib", fname)
    if os.path.exists(in_tree):
        return in_tree, dflags, src
    return os.path.join(_lib_dir(), fname), dflags, src


def _start(name: str, defines: Optional[dict]):
    out, dflags, src = library_path(name, defines)
    if os.path.exists(out):
        return out, None, None
    tmp = f"{out}.{os.getpid()}.tmp"
    cmd = [_hipcc()] + FLAGS + dflags + ["-I", HERE, src, "-o", tmp]
    # what the compiler prints goes to a file: through a pipe that nobody reads before the compiler
    # ends, a long list of warnings would fill the pipe and the compiler would wait for ever
    with open(tmp + ".log", "w") as log:
        proc = subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT)     # the child keeps its own handle
    return out, tmp, proc


def _say(msg: str) -> None:
    print(f"kipp_amd: {msg}", file=sys.stderr, flush=True)


def _finish(name, out, tmp, proc, started) -> None:
    proc.wait()
    log = ""
    try:
        with open(tmp + ".log", "r", errors="replace") as f:
            log = f.read()
        os.remove(tmp + ".log")
    except OSError:
        pass
    if proc.returncode != 0 or not os.path.exists(tmp):
        try:
            os.remove(tmp)
        except OSError:
            pass
        raise BuildError(f"hipcc failed for {name}.hip (exit {proc.returncode}):\n{log}")
    os.replace(tmp, out)
    _say(f"compiled {os.path.basename(out)} in {time.time() - started:.0f} s")


def build_all(specs: Iterable[Tuple[str, Optional[dict]]], jobs: int = 8, force: bool = False) -> None:
    """Compile every (name, defines) that is not built yet, `jobs` at a time."""
    pending = []
    for name, defines in specs:
        out, _, _ = library_path(name, defines)
        if force and os.path.exists(out):
            os.remove(out)
            out, _, _ = library_path(name, defines)
        if not os.path.exists(out) and (name, tuple(sorted((defines or {}).items()))) not in [(p[0], tuple(sorted((p[1] or {}).items()))) for p in pending]:
            pending.append((name, defines))
    running = []
    started = time.time()
    last = started
    while pending or running:
        while pending and len(running) < jobs:
            name, defines = pending.pop(0)
            out, tmp, proc = _start(name, defines)
            if proc is not None:
                _say(f"compiling {name}.hip{_defines_tag(defines)[0]} for {ARCH} ...")
                running.append((name, out, tmp, proc, time.time()))
        for item in list(running):
            if item[3].poll() is not None:
                running.remove(item)
                _finish(*item)
        if running:
            time.sleep(0.2)
            if time.time() - last > 10:
                last = time.time()
                _say(f"still compiling {', '.join(r[0] for r in running)} ({last - started:.0f} s)")
    if started != last or force or not os.path.exists(os.path.join(HERE, "_lib", "MANIFEST")):
        write_manifest()


def write_manifest() -> Optional[str]:
    """`MANIFEST` in the in-tree folder: a line "<name>[.<CONSTANT><value>...] <file>" for every library there that is the
    current build of its source (a host that is no Python, the C one, finds the kernels by it).  Returns its
    path, or None where the folder cannot be written."""
    import re
    folder = os.path.join(HERE, "_lib")
    if not os.path.isdir(folder):
        return None
    lines = []
    for f in sorted(os.listdir(folder)):
        m = re.fullmatch(r"libkipp_([a-z0-9_]+?)((?:\.[A-Z_]+[0-9]+)*)\.([0-9a-f]{10})\.so", f)
        if not m:
            continue
        name, tag = m.group(1), m.group(2)
        defines = {k: int(v) for k, v in re.findall(r"\.([A-Z_]+?)([0-9]+)(?=\.|$)", tag)} or None
        try:
            current = os.path.basename(library_path(name, defines)[0])
        except BuildError:
            continue
        if current == f:
            lines.append(f"{name}{tag} {f}")
    try:
        tmp = os.path.join(folder, f".MANIFEST.{os.getpid()}")
        with open(tmp, "w") as out:
            out.write("\n".join(lines) + "\n")
        os.replace(tmp, os.path.join(folder, "MANIFEST"))
    except OSError:
        return None
    return os.path.join(folder, "MANIFEST")


def library(name: str, defines: Optional[dict] = None) -> ctypes.CDLL:
    """The loaded library of `name`.hip with these constants, compiled if absent."""
    key = name + _defines_tag(defines)[0]
    lib = _loaded.get(key)
    if lib is None:
        out, _, _ = library_path(name, defines)
        if not os.path.exists(out):
            build_all([(name, defines)])
            out, _, _ = library_path(name, defines)
        try:
            lib = ctypes.CDLL(out)
        except OSError as e:
            raise BuildError(f"cannot load {out}: {e}") from e
        _loaded[key] = lib
    return lib


def loaded_libraries() -> Dict[str, str]:
    return {k: v._name for k, v in _loaded.items()}


def clean_stale(keep: Iterable[Tuple[str, Optional[dict]]] = ()) -> None:
    """Remove left-over temporary files from the in-tree folder and, when `keep`
    is given, every library that is not the current build of one of its entries."""
    folder = os.path.join(HERE, "_lib")
    if not os.path.isdir(folder):
        return
    wanted = {os.path.basename(library_path(name, defines)[0]) for name, defines in keep}
    for f in os.listdir(folder):
        if f.endswith(".tmp") or (wanted and f.endswith(".so") and f not in wanted):
            os.remove(os.path.join(folder, f))
