"""Compile the HIP sources under ``lockstep_amd/csrc`` into shared libraries.

Two kinds of library exist:

``core``            every kernel whose code does not depend on a model size
                    (matrix products, norms, rotation and cache write, SwiGLU,
                    embedding, arg-max);
``attention<D>``    the attention kernels for one head size ``D``; a model
                    needs only its own.

A library's file name carries a hash of its sources and flags, so a stale
build is never loaded.  Libraries are written next to the package
(``lockstep_amd/_lib``) when that folder can be written, otherwise to a
per-user folder under the system's temporary directory.  ``load`` compiles at
the first call what is not there yet and says so on stderr while it works.
There is no fallback: without the library (and without ``hipcc`` to make it)
the import of the kernels fails.
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

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-ffp-contract=off", "-Wno-pass-failed",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-shared", "-fPIC",
]
CORE_SOURCES = ("core.hip", "gemm.hip", "sample.hip")
ATTENTION_SOURCES = ("attention.hip",)


class BuildError(RuntimeError):
    pass


def _headers(sources) -> tuple:
    """The headers of this folder that ``sources`` include, directly or through one another."""
    found: list[str] = []
    queue = list(sources)
    while queue:
        text = (CSRC / queue.pop(0)).read_text()
        for line in text.splitlines():
            line = line.strip()
            if line.startswith('#include "'):
                name = line.split('"')[1]
                if name not in found and (CSRC / name).is_file():
                    found.append(name)
                    queue.append(name)
    return tuple(sorted(found))


def _hash(sources, defines) -> str:
    digest = hashlib.sha256()
    for name in tuple(sources) + _headers(sources):
        digest.update(name.encode())
        digest.update((CSRC / name).read_bytes())
    digest.update(" ".join(FLAGS + list(defines)).encode())
    return digest.hexdigest()[:12]


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        handle, probe = tempfile.mkstemp(prefix=".probe-", dir=folder)
        os.close(handle)
        os.unlink(probe)
        return True
    except OSError:
        return False


def lib_dirs() -> list[Path]:
    """Folders searched for built libraries, the first writable one is built into."""
    in_tree = Path(__file__).resolve().parent.parent / "_lib"
    user = Path(tempfile.gettempdir()) / f"lockstep_amd-{os.getuid()}" / "_lib"
    return [in_tree, user]


def _target(kind: str, sources, defines) -> str:
    return f"liblockstep_{kind}-{_hash(sources, defines)}.so"


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).is_file():
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); the kernels cannot be built")


def _run(cmd, what: str) -> None:
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    proc = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed for {what}:\n{' '.join(cmd)}\n{proc.stderr[-4000:]}")


def _compile(kind: str, sources, defines, out: Path) -> None:
    """Compile ``sources`` into the shared library ``out``: every source to an object file of its own,
    side by side, then one link (a library of several sources takes as long as its slowest one)."""
    hipcc = find_hipcc()
    compile_flags = [f for f in FLAGS if f != "-shared"]
    started = time.time()
    print(f"[lockstep_amd] compiling {kind} kernels for {ARCH} -> {out.name}", file=sys.stderr, flush=True)
    done = threading.Event()

    def ticker():
        while not done.wait(15.0):
            print(f"[lockstep_amd] ... still compiling {kind} ({time.time() - started:.0f} s)",
                  file=sys.stderr, flush=True)

    thread = threading.Thread(target=ticker, daemon=True)
    thread.start()
    objects = [out.with_name(f"{out.name}.{Path(s).stem}.o") for s in sources]
    try:
        if len(sources) == 1:
            _run([hipcc, *FLAGS, *defines, "-o", str(out), str(CSRC / sources[0])], kind)
        else:
            errors: list = []

            def one(source, obj):
                try:
                    _run([hipcc, *compile_flags, *defines, "-c", "-o", str(obj), str(CSRC / source)], f"{kind} ({source})")
                except Exception as exc:  # noqa: BLE001 - reported below
                    errors.append(exc)

            workers = [threading.Thread(target=one, args=pair) for pair in zip(sources, objects)]
            for w in workers:
                w.start()
            for w in workers:
                w.join()
            if errors:
                raise errors[0]
            _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(out), *[str(o) for o in objects]], kind)
    finally:
        done.set()
        for obj in objects:
            if obj.exists():
                obj.unlink()
    print(f"[lockstep_amd] compiled {kind} in {time.time() - started:.1f} s", file=sys.stderr, flush=True)


def build(kind: str, sources, defines=(), force: bool = False) -> Path:
    """Return the path of the library, compiling it if it is missing (or ``force``)."""
    name = _target(kind, sources, defines)
    if not force:
        for folder in lib_dirs():
            if (folder / name).is_file():
                return folder / name
    for folder in lib_dirs():
        if not _writable(folder):
            continue
        for stale in folder.glob(f"liblockstep_{kind}-*.so"):
            if stale.name != name:
                try:
                    stale.unlink()
                except OSError:
                    pass
        tmp = folder / f".{name}.{os.getpid()}.{threading.get_ident()}.tmp"
        try:
            _compile(kind, sources, list(defines), tmp)
            os.replace(tmp, folder / name)
        finally:
            if tmp.exists():
                tmp.unlink()
        return folder / name
    raise BuildError(f"no writable folder for built kernels among {[str(d) for d in lib_dirs()]}")


def build_core(force: bool = False) -> Path:
    # LOCKSTEP_CORE_DEFINES: further -D switches for the core library (the tuning macros at the top of the
    # sources), for measurements; the file name carries them in its hash like every other flag
    extra = tuple(os.environ.get("LOCKSTEP_CORE_DEFINES", "").split())
    return build("core", CORE_SOURCES, extra, force)


def build_attention(head_dim: int, force: bool = False) -> Path:
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise BuildError(
            f"head size {head_dim} is not supported: the attention kernels take multiples of 16 from 16 to 256")
    return build(f"attention{head_dim}", ATTENTION_SOURCES, (f"-DLS_HEAD_DIM={head_dim}",), force)


MUTANT_DEFINE = "-DLS_MUTANTS"


def build_core_mutants(force: bool = False) -> Path:
    """The core library with its switchable wrong variants compiled in (positive controls of the
    tests); a file of its own, never loaded by the engine."""
    return build("core.mutants", CORE_SOURCES, (MUTANT_DEFINE,), force)


def build_attention_mutants(head_dim: int, force: bool = False) -> Path:
    return build(f"attention{head_dim}.mutants", ATTENTION_SOURCES, (f"-DLS_HEAD_DIM={head_dim}", MUTANT_DEFINE), force)


DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 128, 256)
MUTANT_HEAD_DIMS = (16, 32, 128)     # the head sizes of the tests that use the controls


def build_all(head_dims=DEFAULT_HEAD_DIMS, force: bool = True, mutants: bool = True) -> list[Path]:
    """Compile the core library and the attention library of each head size,
    a few at a time; with ``mutants`` also the control libraries of the tests."""
    jobs = [lambda: build_core(force)] + [lambda d=d: build_attention(d, force) for d in head_dims]
    if mutants:
        jobs += [lambda: build_core_mutants(force)] + [lambda d=d: build_attention_mutants(d, force)
                                                       for d in MUTANT_HEAD_DIMS]
    results: list = [None] * len(jobs)
    errors: list = []

    def run(i):
        try:
            results[i] = jobs[i]()
        except Exception as exc:  # noqa: BLE001 - reported below
            errors.append(exc)

    width = max(1, min(4, (os.cpu_count() or 2) // 2))
    for lo in range(0, len(jobs), width):
        threads = [threading.Thread(target=run, args=(i,)) for i in range(lo, min(lo + width, len(jobs)))]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    if errors:
        raise errors[0]
    return results
