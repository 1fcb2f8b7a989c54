"""Building and finding the native libraries.

Four kinds of shared library, all built from the sources beside this file:

* `core`  - the id pool of the cache manager (C++, host only, g++);
* `ops`   - the HIP kernels that do not depend on the head size (hipcc, gfx950);
* `library` - the calls of the vendor's matrix-product library for large products (hipcc, linked with hipBLASLt);
* `attn_d<D>` - the attention kernels for head size D (hipcc, `-DDISTIE_HEAD_DIM=D`; the matrix-core
  kernels for multiples of 16, the wave-per-token kernel for every even size).

A library's file name carries a hash of its sources and flags, so a stale build is never
loaded. Libraries live in `distie_amd/_lib/` (in-tree); if that folder cannot be written,
in a per-user folder under the temporary directory. `ensure(name)` returns the path and
compiles first if the file is not there, printing a line when it starts and every few
seconds while it waits, so a first call in a fresh checkout shows progress.
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
from pathlib import Path
from typing import List

SRC = Path(__file__).resolve().parent
ARCH = "gfx950"
# packed-fp32 instructions are switched off: some of their forms gave wrong results on this hardware
HIP_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]
CXX_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-pthread"]

OPS_SOURCES = ["elementwise.hip", "gemm.hip", "gemv.hip", "decode_products.hip", "sampling.hip"]
ATTN_SOURCES = ["attention.hip"]
LIBRARY_SOURCES = ["library_products.hip"]
LINK_LIBS = {"library": ["-lhipblaslt"]}
HEADERS = ["common.h"]
OPS_HEADERS = ["no_alloc.h", "packed.h"]


class BuildError(RuntimeError):
    pass


def _say(text: str) -> None:
    print(f"[distie_amd] {text}", file=sys.stderr, flush=True)


def _hash(files: List[str], flags: List[str]) -> str:
    h = hashlib.sha256()
    headers = HEADERS + (OPS_HEADERS if files == OPS_SOURCES else [])
    for name in files + headers:
        path = SRC / name
        if path.is_file():
            h.update(name.encode())
            h.update(path.read_bytes())
    h.update(" ".join(flags).encode())
    return h.hexdigest()[:10]


def _spec(name: str):
    """-> (sources, compiler, flags)"""
    if name == "core":
        return ["block_pool.cpp"], os.environ.get("CXX", "g++"), list(CXX_FLAGS)
    if name == "ops":
        return list(OPS_SOURCES), _hipcc(), list(HIP_FLAGS)
    if name == "library":
        return list(LIBRARY_SOURCES), _hipcc(), list(HIP_FLAGS)
    if name.startswith("attn_d"):
        dim = int(name[len("attn_d"):])
        if dim < 2 or dim > 256 or dim % 2:
            raise BuildError(f"attention kernels are built for even head sizes up to 256, not {dim}")
        return list(ATTN_SOURCES), _hipcc(), list(HIP_FLAGS) + [f"-DDISTIE_HEAD_DIM={dim}"]
    raise BuildError(f"no native library named {name}")


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    raise BuildError("hipcc not found: the HIP kernels cannot be built (looked at $HIPCC, PATH, /opt/rocm/bin)")


def _folders() -> List[Path]:
    own = SRC.parent / "_lib"
    shared = Path(tempfile.gettempdir()) / f"distie_amd_lib_{os.getuid()}"
    return [own, shared]


def file_name(name: str) -> str:
    sources, _, flags = _spec(name)
    return f"libdistie_{name}.{_hash(sources, flags)}.so"


def find(name: str):
    target = file_name(name)
    for folder in _folders():
        path = folder / target
        if path.is_file():
            return path
    return None


def _writable_folder() -> Path:
    for folder in _folders():
        try:
            folder.mkdir(parents=True, exist_ok=True)
            probe = folder / f".probe_{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return folder
        except OSError:
            continue
    raise BuildError("no writable folder for the native libraries")


def _run(cmd: List[str], what: str) -> None:
    started = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())   # hipcc wants a HOME for its caches
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, cwd=str(SRC), env=env)
    lines: List[bytes] = []
    reader = threading.Thread(target=lambda: lines.extend(proc.stdout.readlines()), daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=10)
            break
        except subprocess.TimeoutExpired:
            _say(f"still compiling {what} ({int(time.time() - started)} s)")
    reader.join()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{b''.join(lines).decode(errors='replace')}")


def build(name: str, force: bool = False) -> Path:
    """Compile library `name` (always, if `force`), and return its path."""
    existing = None if force else find(name)
    if existing is not None:
        return existing
    sources, compiler, flags = _spec(name)
    folder = _writable_folder()
    target = folder / file_name(name)
    _say(f"compiling {name} ({', '.join(sources)}) for {ARCH if compiler != os.environ.get('CXX', 'g++') else 'the host'} ...")
    started = time.time()
    scratch = Path(tempfile.mkdtemp(prefix="distie_build_", dir=str(folder)))
    try:
        objects = []
        errors: List[BaseException] = []

        def compile_one(src: str) -> None:
            obj = scratch / (Path(src).stem + ".o")
            lang = ["-x", "hip"] if src.endswith(".hip") else []
            try:
                _run([compiler] + flags + lang + ["-c", str(SRC / src), "-o", str(obj)], f"{name}/{src}")
            except BaseException as exc:  # noqa: BLE001 - reported below
                errors.append(exc)

        threads = [threading.Thread(target=compile_one, args=(s,)) for s in sources]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        if errors:
            raise errors[0]
        objects = [str(scratch / (Path(s).stem + ".o")) for s in sources]
        link_flags = [f for f in flags if not f.startswith("-D")]
        staging = scratch / target.name
        libs = LINK_LIBS.get(name, [])
        if libs:
            libs = [f"-L{Path(compiler).resolve().parent.parent / 'lib'}"] + libs
        _run([compiler] + link_flags + ["-shared"] + objects + libs + ["-o", str(staging)], f"{name} (link)")
        os.replace(staging, target)
    finally:
        shutil.rmtree(scratch, ignore_errors=True)
    # older builds of the same library are of no use any more
    for old in folder.glob(f"libdistie_{name}.*.so"):
        if old != target:
            try:
                old.unlink()
            except OSError:
                pass
    _say(f"built {target.name} in {time.time() - started:.0f} s")
    return target


def ensure(name: str) -> Path:
    """Path of library `name`, built now if it is not there yet."""
    return build(name, force=False)


DEFAULT_HEAD_DIMS = (16, 32, 40, 48, 64, 80, 96, 112, 128, 256)


def build_all(head_dims=DEFAULT_HEAD_DIMS, force: bool = True) -> List[Path]:
    out = [build("core", force), build("ops", force), build("library", force)]
    for d in head_dims:
        out.append(build(f"attn_d{d}", force))
    return out


if __name__ == "__main__":
    for path in build_all():
        print(path)
