"""Compiles the HIP sources of this folder for gfx950, one shared library per family.

The reference compiles every kernel source at build time with ``hipcc --genco
--offload-arch=... -O3`` and fails with the compiler's output
(rocml-kernels/build.rs:10-59).  Here each family (``elementwise``, ``gemm``,
``attention``, ``sampling``) becomes ``_build/lib<family>.so`` next to the sources;
a family is compiled when it is first needed and no library built from the present
sources is there (a hash of the sources and flags is kept beside each library), so a
fresh checkout works without a build step and an edited kernel is never run from an
old library.  ``python -m rocml_amd.csrc.build``
compiles all of them again.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, List

from ..errors import ExtensionMissingError

SRC_DIR = os.path.dirname(os.path.abspath(__file__))
FAMILIES = ("elementwise", "gemm", "attention", "sampling")
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

_lock = threading.Lock()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise ExtensionMissingError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dir() -> str:
    """``_build`` beside the sources, or a per-user folder under the temporary
    directory when the checkout cannot be written."""
    local = os.path.join(SRC_DIR, "_build")
    if os.path.isdir(local) and all(is_current(os.path.join(local, f"lib{f}.so"), f) for f in FAMILIES):
        return local
    if _writable_dir(local):
        return local
    alt = os.path.join(tempfile.gettempdir(), f"rocml_amd_build_{os.getuid()}")
    if _writable_dir(alt):
        return alt
    raise ExtensionMissingError(f"neither {local} nor {alt} can be written")


def source_hash(family: str) -> str:
    """Hash of what a family's library is made from: its source, the headers of this folder that
    it includes (directly or through another of them) and the compiler flags."""
    h = hashlib.sha256(" ".join([ARCH, *FLAGS]).encode())
    names, todo = [], [f"{family}.hip"]
    while todo:
        name = todo.pop()
        if name in names:
            continue
        names.append(name)
        with open(os.path.join(SRC_DIR, name), "r", encoding="utf-8") as f:
            for line in f:
                line = line.strip()
                if line.startswith("#include \""):
                    inc = line.split('"')[1]
                    if os.path.exists(os.path.join(SRC_DIR, inc)):
                        todo.append(inc)
    for name in sorted(names):
        with open(os.path.join(SRC_DIR, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    return h.hexdigest()


def is_current(path: str, family: str) -> bool:
    """Whether ``path`` exists and was built from the present sources."""
    try:
        with open(path + ".srchash", "r", encoding="utf-8") as f:
            return os.path.exists(path) and f.read().strip() == source_hash(family)
    except OSError:
        return False


def library_path(family: str) -> str:
    local = os.path.join(SRC_DIR, "_build", f"lib{family}.so")
    if is_current(local, family):
        return local
    return os.path.join(build_dir(), f"lib{family}.so")


def _compile(family: str, out_path: str, log: List[str]) -> None:
    src = os.path.join(SRC_DIR, f"{family}.hip")
    tmp = f"{out_path}.{os.getpid()}.tmp"
    env = dict(os.environ)
    # hipcc keeps a cache under HOME; an empty or unwritable HOME must not stop it.
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    cmd = [_hipcc(), f"--offload-arch={ARCH}", *FLAGS, src, "-o", tmp]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                          cwd=SRC_DIR)
    output = "\n".join(line for line in proc.stdout.splitlines()
                       if "is not a recognized feature for this target" not in line)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        log.append(f"hipcc failed for {family}.hip:\n{output}")
        return
    os.replace(tmp, out_path)
    with open(out_path + ".srchash", "w", encoding="utf-8") as f:
        f.write(source_hash(family))


def build(families: Iterable[str] = FAMILIES, force: bool = True, quiet: bool = False) -> Dict[str, str]:
    """Compiles the named families (in parallel) and returns their library paths.
    With ``force=False`` a family whose library was built from the present sources is left alone.  Prints a line
    when it starts, every few seconds while the compiler runs, and when it ends."""
    with _lock:
        out_dir = build_dir() if not force else (
            os.path.join(SRC_DIR, "_build") if _writable_dir(os.path.join(SRC_DIR, "_build")) else build_dir())
        todo = []
        paths = {}
        for fam in families:
            if fam not in FAMILIES:
                raise ExtensionMissingError(f"unknown kernel family {fam!r}")
            path = os.path.join(out_dir, f"lib{fam}.so")
            paths[fam] = path
            if force or not is_current(path, fam):
                todo.append(fam)
        if not todo:
            return paths

        def say(msg: str) -> None:
            if not quiet:
                print(f"[rocml_amd] {msg}", file=sys.stderr, flush=True)

        say(f"compiling HIP kernels for {ARCH}: {', '.join(todo)} -> {out_dir}")
        log: List[str] = []
        threads = [threading.Thread(target=_compile, args=(fam, paths[fam], log)) for fam in todo]
        start = time.time()
        for t in threads:
            t.start()
        while any(t.is_alive() for t in threads):
            for t in threads:
                t.join(timeout=5.0)
                if t.is_alive():
                    break
            if any(t.is_alive() for t in threads):
                say(f"  still compiling ({time.time() - start:.0f} s)")
        if log:
            raise ExtensionMissingError("\n".join(log))
        say(f"compiled in {time.time() - start:.1f} s")
        return paths


def ensure(family: str) -> str:
    """Path of a family's library, compiling it first if it does not exist or is older than
    its sources."""
    path = library_path(family)
    if is_current(path, family):
        return path
    return build([family], force=False)[family]


if __name__ == "__main__":
    build(force=True)
