"""Compiles the HIP sources under csrc/ into one shared library for gfx950.

`hipcc` is called directly, one process per source file, and the objects are linked into
`libbeholdd_hip.so` next to this file.  A stamp beside the library records a hash of the
sources and flags, so a library built from other sources is built again.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIB_NAME = "libbeholdd_hip.so"

# No fast-math: the kernels start running maxima at -inf and test logits for finiteness.
# The packed-fp32 feature is switched off for device code (the host pass warns that it does
# not know the feature; that is harmless).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


class BuildError(RuntimeError):
    pass


def source_page_size() -> int:
    """Tokens in one page of the key/value cache: `BH_PAGE` of csrc/layout.h, the one place that says so.
    (The built library reports the same number as `bh_page_size()`; this reads it where no library is loaded.)"""
    with open(os.path.join(CSRC, "layout.h"), "r", encoding="utf-8") as handle:
        for line in handle:
            words = line.split()
            if len(words) >= 3 and words[0] == "#define" and words[1] == "BH_PAGE":
                return int(words[2])
    raise BuildError("csrc/layout.h does not define BH_PAGE")


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                     "the HIP kernel library cannot be built")


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    digest.update(" ".join(HIPCC_FLAGS).encode())
    for path in sources() + sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")):
        digest.update(os.path.basename(path).encode())
        with open(path, "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=folder, delete=True)
        probe.close()
        return True
    except OSError:
        return False


def library_dir() -> str:
    """The package's own folder, or a per-user temporary folder when the package is read-only."""
    if _writable(HERE):
        return HERE
    fallback = os.path.join(tempfile.gettempdir(), f"beholdd_hip_{os.getuid()}")
    os.makedirs(fallback, exist_ok=True)
    return fallback


def library_path() -> str:
    in_tree = os.path.join(HERE, LIB_NAME)
    if os.path.exists(in_tree):
        return in_tree
    return os.path.join(library_dir(), LIB_NAME)


def is_current(path: str | None = None) -> bool:
    path = path or library_path()
    stamp = path + ".stamp"
    if not (os.path.exists(path) and os.path.exists(stamp)):
        return False
    with open(stamp, "r", encoding="utf-8") as handle:
        return handle.read().strip() == source_hash()


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = library_dir()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    jobs = jobs or max(1, min(16, os.cpu_count() or 1))
    say = (lambda text: print(f"[beholdd build] {text}", file=sys.stderr, flush=True)) if verbose else (lambda text: None)
    pending = list(sources())
    say(f"compiling {len(pending)} HIP sources for gfx950 with {hipcc}")
    running: list = []
    objects = []
    started = time.time()
    last_note = started
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    while pending or running:
        while pending and len(running) < jobs:
            src = pending.pop(0)
            obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
            objects.append(obj)
            command = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
            running.append((src, subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                                  text=True, env=env)))
        for item in list(running):
            src, process = item
            if process.poll() is None:
                continue
            output = process.stdout.read()
            running.remove(item)
            if process.returncode != 0:
                for _, other in running:
                    other.kill()
                raise BuildError(f"hipcc failed on {src}:\n{output}")
            say(f"compiled {os.path.basename(src)} ({time.time() - started:.0f} s)")
        if running:
            time.sleep(0.2)
            if time.time() - last_note > 15:
                last_note = time.time()
                say(f"still compiling {', '.join(os.path.basename(s) for s, _ in running)} "
                    f"({time.time() - started:.0f} s)")
    target = os.path.join(out_dir, LIB_NAME)
    tmp_target = target + f".tmp{os.getpid()}"
    link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp_target, *objects],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if link.returncode != 0:
        raise BuildError(f"linking {LIB_NAME} failed:\n{link.stdout}")
    os.replace(tmp_target, target)
    with open(target + ".stamp", "w", encoding="utf-8") as handle:
        handle.write(source_hash() + "\n")
    say(f"linked {target} ({time.time() - started:.0f} s)")
    return target


def build_plain_twins(out_dir: str, selftest: bool = False) -> str:
    """Compile csrc/plain_twins.cpp with the host compiler: a shared library of the kernels' plain twins, or with
    `selftest` a program of its own, built with the address and undefined-behaviour sanitizers, that checks the
    twins against the reference's test vectors.  Returns the path of what was built."""
    compiler = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++")
    if not compiler:
        raise BuildError("no host C++ compiler (g++) was found")
    source = os.path.join(CSRC, "plain_twins.cpp")
    os.makedirs(out_dir, exist_ok=True)
    if selftest:
        target = os.path.join(out_dir, "plain_twins_selftest")
        command = [compiler, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                   "-DBH_TWINS_SELFTEST", "-I", CSRC, source, "-o", target]
    else:
        target = os.path.join(out_dir, "libbeholdd_plain.so")
        command = [compiler, "-std=c++17", "-O2", "-shared", "-fPIC", "-I", CSRC, source, "-o", target]
    done = subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if done.returncode != 0:
        raise BuildError(f"{' '.join(command)} failed:\n{done.stdout}")
    return target


def ensure_built(verbose: bool = True) -> str:
    """The path of a library that matches the sources, building it when none does."""
    path = library_path()
    if is_current(path):
        return path
    return build(verbose=verbose)
