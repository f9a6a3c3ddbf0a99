"""Compiles the HIP sources for gfx950 into shared libraries, one per source file.

A library's file name carries a hash of its source, the shared header and the
compiler flags, so a library that exists is always the one its source asks for;
a changed source compiles again at its next use.  Libraries are written next to
the sources (the folder travels with the checkout); if that folder cannot be
written, a per-user folder under the temporary directory is used.

`ensure([...])` compiles only what is asked for, several files at a time, and
prints a line when each file starts and ends and every few seconds meanwhile.
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

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# packed 32-bit float instructions are switched off for every kernel
# and the first kernel arguments arrive in scalar registers with the wavefront (the command
# processor preloads them) instead of being fetched by the kernel's first instructions
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-mllvm", "-amdgpu-kernarg-preload-count=16",
         "-Wno-unused-command-line-argument"]
HEADERS = ["common.h", "qk_prep.h", "tinyinfer_kernels.h", "tinyinfer_kernels_tuning.h"]
# flags of single libraries.  The attention kernels rescale their MFMA accumulators with
# vector instructions; kept in the accumulation registers they would be copied out and back
# on every turn of the loop, so their MFMAs are told to work on ordinary vector registers.
EXTRA_FLAGS: Dict[str, List[str]] = {
    "attention_bf16": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}

def _discover() -> Dict[str, str]:
    """library name -> source file: every `*.hip` in this folder is a kernel library of its own, named for
    the file.  A new kernel file needs no entry anywhere."""
    return {f[:-4]: f for f in sorted(os.listdir(HERE)) if f.endswith(".hip")}


SOURCES: Dict[str, str] = _discover()
# libraries no model needs (measurement helpers): built with everything else, never on a model's behalf
ON_DEMAND = ("measure",)


def libraries_for(dtype: str) -> List[str]:
    """The kernel libraries a model of this dtype needs: every one except those whose name ends in `_bf16`
    when the engine runs in float32 (what a first call compiles)."""
    return [n for n in SOURCES if n not in ON_DEMAND and (dtype == "bfloat16" or not n.endswith("_bf16"))]


# the host library (configuration, weights, parts, cache manager, step function, scheduler, sampler
# and the C interface the Python package binds): C++17, no device code
PKG = os.path.dirname(HERE)
HOST_SOURCES = ["config/json.cpp", "config/config.cpp", "ops/ops.cpp", "parts/parts.cpp", "weights/weights.cpp",
                "models/model.cpp", "cache/cache_manager.cpp", "engine/engine.cpp", "engine/scheduler.cpp",
                "sampling/sampler.cpp", "engine/c_api.cpp"]
HOST_HEADERS = ["include/inference.h", "weights/weights.h", "csrc/tinyinfer_kernels.h"]
HOST_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-Wall", "-Wno-unused-function"]
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                     "the HIP kernels cannot be compiled")


def _digest(name: str) -> str:
    h = hashlib.sha256()
    for f in [SOURCES[name]] + HEADERS:
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(FLAGS + EXTRA_FLAGS.get(name, [])).encode())
    return h.hexdigest()[:12]


def _lib_dirs() -> List[str]:
    """Where a library may lie: beside the sources first, then the per-user folder."""
    tmp = os.path.join(tempfile.gettempdir(), f"tinyinfer_amd_{os.getuid()}")
    return [HERE, tmp]


def lib_name(name: str) -> str:
    return f"libti_{name}.{_digest(name)}.so"


def find(name: str):
    fn = lib_name(name)
    for d in _lib_dirs():
        p = os.path.join(d, fn)
        if os.path.isfile(p):
            return p
    return None


def _writable_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError(f"no folder to write the kernel libraries to (tried {_lib_dirs()})")


def _say(msg: str) -> None:
    print(f"[tinyinfer build] {msg}", file=sys.stderr, flush=True)


def _compile(name: str, out_dir: str) -> str:
    src = os.path.join(HERE, SOURCES[name])
    final = os.path.join(out_dir, lib_name(name))
    part = final + f".{os.getpid()}.part"
    env = dict(os.environ)
    # the compiler keeps caches under HOME; give it one if the user has none
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    t0 = time.time()
    _say(f"compiling {SOURCES[name]} for {ARCH} ...")
    proc = subprocess.run([_hipcc()] + FLAGS + EXTRA_FLAGS.get(name, []) + [src, "-o", part], cwd=HERE, env=env,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(part):
            os.remove(part)
        raise BuildError(f"hipcc failed on {SOURCES[name]}:\n{proc.stdout}")
    os.replace(part, final)
    # libraries of older versions of this source are of no use any more
    for f in os.listdir(out_dir):
        if f.startswith(f"libti_{name}.") and f.endswith(".so") and f != os.path.basename(final):
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    _say(f"compiled {SOURCES[name]} in {time.time() - t0:.1f} s")
    return final


def ensure(names: Iterable[str], force: bool = False) -> Dict[str, str]:
    """Paths of the libraries `names`, compiling those that are not there
    (all of them with `force`)."""
    names = list(names)
    for n in names:
        if n not in SOURCES:
            raise BuildError(f"unknown kernel library {n!r}; known: {sorted(SOURCES)}")
    paths: Dict[str, str] = {}
    todo = []
    for n in names:
        p = None if force else find(n)
        if p:
            paths[n] = p
        else:
            todo.append(n)
    if not todo:
        return paths
    out_dir = _writable_dir()
    errors: List[BaseException] = []
    done = threading.Event()

    def work(n):
        try:
            paths[n] = _compile(n, out_dir)
        except BaseException as e:  # noqa: BLE001
            errors.append(e)

    def heartbeat():
        t0 = time.time()
        while not done.wait(10.0):
            _say(f"still compiling ({time.time() - t0:.0f} s) ...")

    threads = [threading.Thread(target=work, args=(n,)) for n in todo]
    hb = threading.Thread(target=heartbeat, daemon=True)
    hb.start()
    limit = max(1, min(8, os.cpu_count() or 1))
    for i in range(0, len(threads), limit):
        for t in threads[i:i + limit]:
            t.start()
        for t in threads[i:i + limit]:
            t.join()
    done.set()
    if errors:
        raise errors[0]
    return paths


def _host_digest() -> str:
    h = hashlib.sha256()
    for f in HOST_SOURCES + HOST_HEADERS:
        with open(os.path.join(PKG, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()[:12]


def host_lib_name() -> str:
    return f"libtinyinfer.{_host_digest()}.so"


def find_host():
    for d in _lib_dirs():
        p = os.path.join(d, host_lib_name())
        if os.path.isfile(p):
            return p
    return None


def ensure_host(force: bool = False) -> str:
    """Path of the host library, compiled (its files several at a time) if it is not there."""
    p = None if force else find_host()
    if p:
        return p
    cxx = shutil.which("g++") or shutil.which("c++") or os.path.join(ROCM, "llvm", "bin", "clang++")
    if not cxx or not os.path.isfile(cxx):
        raise BuildError("no C++ compiler found (g++, c++, or ROCm's clang++): the host library cannot be compiled")
    out_dir = _writable_dir()
    final = os.path.join(out_dir, host_lib_name())
    work = tempfile.mkdtemp(prefix="tinyinfer_host_")
    t0 = time.time()
    _say(f"compiling the host library ({len(HOST_SOURCES)} files) ...")
    errors: List[str] = []
    objects = []

    def one(src):
        obj = os.path.join(work, src.replace("/", "_") + ".o")
        objects.append(obj)
        proc = subprocess.run([cxx] + HOST_FLAGS + ["-I" + os.path.join(ROCM, "include"), "-c", os.path.join(PKG, src), "-o", obj],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            errors.append(f"{src}:\n{proc.stdout}")

    done = threading.Event()

    def heartbeat():
        while not done.wait(10.0):
            _say(f"still compiling the host library ({time.time() - t0:.0f} s) ...")

    threading.Thread(target=heartbeat, daemon=True).start()
    threads = [threading.Thread(target=one, args=(s,)) for s in HOST_SOURCES]
    limit = max(1, min(8, os.cpu_count() or 1))
    for i in range(0, len(threads), limit):
        for t in threads[i:i + limit]:
            t.start()
        for t in threads[i:i + limit]:
            t.join()
    try:
        if errors:
            raise BuildError("the host library does not compile:\n" + "\n".join(errors))
        part = final + f".{os.getpid()}.part"
        proc = subprocess.run([cxx, "-shared", "-o", part] + objects + ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-ldl",
                                                                          "-lpthread", "-Wl,-rpath," + os.path.join(ROCM, "lib")],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise BuildError(f"the host library does not link:\n{proc.stdout}")
        os.replace(part, final)
    finally:
        done.set()
        shutil.rmtree(work, ignore_errors=True)
    for f in os.listdir(out_dir):
        if f.startswith("libtinyinfer.") and f.endswith(".so") and f != os.path.basename(final):
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    _say(f"compiled the host library in {time.time() - t0:.1f} s")
    return final


# programs beside the libraries: name -> source (C++17, linked with the host library)
TOOLS: Dict[str, str] = {"trace_run": "engine/trace_run.cpp"}


def tool_name(name: str) -> str:
    h = hashlib.sha256()
    with open(os.path.join(PKG, TOOLS[name]), "rb") as fh:
        h.update(fh.read())
    h.update(_host_digest().encode())
    return f"tinyinfer_{name}.{h.hexdigest()[:12]}"


def ensure_tool(name: str, force: bool = False) -> str:
    """Path of the program `name`, compiled and linked with the host library if it is not there."""
    fn = tool_name(name)
    if not force:
        for d in _lib_dirs():
            if os.path.isfile(os.path.join(d, fn)):
                return os.path.join(d, fn)
    host = ensure_host()
    cxx = shutil.which("g++") or shutil.which("c++") or os.path.join(ROCM, "llvm", "bin", "clang++")
    out_dir = os.path.dirname(host)
    final = os.path.join(out_dir, fn)
    part = final + f".{os.getpid()}.part"
    t0 = time.time()
    _say(f"compiling {TOOLS[name]} ...")
    proc = subprocess.run([cxx, "-std=c++17", "-O2", "-D__HIP_PLATFORM_AMD__", os.path.join(PKG, TOOLS[name]), "-o", part, host,
                           "-Wl,-rpath," + out_dir, "-Wl,-rpath," + os.path.join(ROCM, "lib")],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(part):
            os.remove(part)
        raise BuildError(f"{TOOLS[name]} does not compile:\n{proc.stdout}")
    os.replace(part, final)
    for f in os.listdir(out_dir):
        if f.startswith(f"tinyinfer_{name}.") and f != fn and not f.endswith(".part"):
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    _say(f"compiled {TOOLS[name]} in {time.time() - t0:.1f} s")
    return final


def write_manifest() -> None:
    """kernels.manifest beside the libraries: `name file` a line, for programs that use the host library
    without this package (it looks the kernel libraries up there)."""
    for d in _lib_dirs():
        lines = []
        for n in SOURCES:
            p = os.path.join(d, lib_name(n))
            if os.path.isfile(p):
                lines.append(f"{n} {os.path.basename(p)}")
        if lines:
            try:
                with open(os.path.join(d, "kernels.manifest"), "w") as f:
                    f.write("\n".join(lines) + "\n")
            except OSError:
                pass


def build_all(force: bool = True) -> Dict[str, str]:
    paths = ensure([n for n, s in SOURCES.items() if os.path.isfile(os.path.join(HERE, s))], force=force)
    paths["host"] = ensure_host(force=force)
    for tool in TOOLS:
        paths[tool] = ensure_tool(tool, force=force)
    write_manifest()
    return paths


if __name__ == "__main__":
    for k, v in build_all().items():
        print(k, v)
