"""Compiling and loading the two native libraries.

``libpagedllm_host.so``  the host runtime (cache manager, scheduler, sampler), g++.
``libpagedllm_hip.so``   the gfx950 kernels, hipcc.

Both are built in-tree under ``_build/`` (or, when the package folder cannot be
written, under the temporary folder).  A library is rebuilt when its sources
have changed since it was built.  Nothing here falls back to anything: when a
library cannot be built or loaded the error says so.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path

from .errors import TensorError

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC = PACKAGE_DIR / "csrc"
GPU_ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={GPU_ARCH}", "-O3", "-fPIC", "-std=c++17",
    # packed 32-bit float operations are not to be generated on this hardware
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HOST_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra"]

_lock = threading.Lock()
_loaded: dict = {}


def _say(message: str) -> None:
    print(f"[paged-llm-rs_amd] {message}", file=sys.stderr, flush=True)


def build_dir() -> Path:
    """Where built libraries live: in-tree when writable, else a per-user temporary folder."""
    override = os.environ.get("PAGEDLLM_BUILD_DIR")
    if override:
        path = Path(override)
        path.mkdir(parents=True, exist_ok=True)
        return path
    path = PACKAGE_DIR / "_build"
    try:
        path.mkdir(exist_ok=True)
        probe = path / f".write_probe_{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return path
    except OSError:
        tag = hashlib.sha256(str(PACKAGE_DIR).encode()).hexdigest()[:12]
        path = Path(tempfile.gettempdir()) / f"paged_llm_rs_amd_{os.getuid()}_{tag}"
        path.mkdir(parents=True, exist_ok=True)
        return path


def _sources(kind: str) -> list:
    folder = CSRC / kind
    suffixes = (".hip",) if kind == "hip" else (".cpp",)
    return sorted(p for p in folder.iterdir() if p.suffix in suffixes)


def _fingerprint(kind: str) -> str:
    h = hashlib.sha256()
    folder = CSRC / kind
    for p in sorted(folder.iterdir()):
        if p.suffix in (".hip", ".cpp", ".hpp", ".h"):
            h.update(p.name.encode())
            h.update(p.read_bytes())
    h.update(" ".join(HIP_FLAGS if kind == "hip" else HOST_FLAGS).encode())
    return h.hexdigest()


def library_path(kind: str) -> Path:
    return build_dir() / f"libpagedllm_{kind}.so"


def is_current(kind: str) -> bool:
    lib = library_path(kind)
    stamp = lib.with_suffix(".stamp")
    return lib.exists() and stamp.exists() and stamp.read_text().strip() == _fingerprint(kind)


def _run_all(commands: list, what: str) -> None:
    """Run compile commands side by side, saying now and then that they still run."""
    # What a compiler prints goes to a file: a pipe that nobody reads while the compiler runs holds 64 KB,
    # and a compiler with more warnings than that would wait for ever.
    logs = {name: tempfile.TemporaryFile(mode="w+") for name, _ in commands}
    pending = {name: subprocess.Popen(cmd, stdout=logs[name], stderr=subprocess.STDOUT) for name, cmd in commands}
    started = time.time()
    last = started
    outputs = {}
    while pending:
        for name, proc in list(pending.items()):
            if proc.poll() is not None:
                logs[name].seek(0)
                outputs[name] = (proc.returncode, logs[name].read())
                logs[name].close()
                del pending[name]
        if pending:
            time.sleep(0.2)
            if time.time() - last > 10:
                last = time.time()
                _say(f"still compiling {what}: {', '.join(pending)} ({int(last - started)} s)")
    failed = {n: out for n, (code, out) in outputs.items() if code != 0}
    if failed:
        text = "\n".join(f"--- {n} ---\n{out}" for n, out in failed.items())
        raise TensorError(f"compiling {what} failed:\n{text}")


def build(kind: str, force: bool = False) -> Path:
    """Compile one library (``host`` or ``hip``) unless it is current."""
    with _lock:
        lib = library_path(kind)
        if not force and is_current(kind):
            return lib
        compiler = shutil.which("hipcc") or "/opt/rocm/bin/hipcc" if kind == "hip" else shutil.which("g++")
        if not compiler or not Path(compiler).exists():
            raise TensorError(f"no compiler for the {kind} library ({'hipcc' if kind == 'hip' else 'g++'} not found)")
        sources = _sources(kind)
        obj_dir = build_dir() / f"obj_{kind}"
        obj_dir.mkdir(exist_ok=True)
        flags = HIP_FLAGS if kind == "hip" else HOST_FLAGS
        _say(f"compiling the {kind} library ({len(sources)} files) with {Path(compiler).name} into {build_dir()}")
        objects = []
        commands = []
        for src in sources:
            obj = obj_dir / (src.stem + ".o")
            objects.append(str(obj))
            commands.append((src.name, [compiler, *flags, "-c", str(src), "-o", str(obj)]))
        started = time.time()
        _run_all(commands, f"the {kind} library")
        tmp = lib.with_suffix(f".tmp{os.getpid()}.so")
        link = [compiler, "-shared", "-fPIC", "-o", str(tmp), *objects]
        if kind == "hip":
            link.insert(1, f"--offload-arch={GPU_ARCH}")
        _run_all([("link", link)], f"the {kind} library")
        os.replace(tmp, lib)
        lib.with_suffix(".stamp").write_text(_fingerprint(kind) + "\n")
        _say(f"built {lib.name} in {time.time() - started:.0f} s")
        _loaded.pop(kind, None)
        return lib


def load(kind: str) -> ctypes.CDLL:
    """The loaded library, built first when it is missing or stale."""
    if kind in _loaded:
        return _loaded[kind]
    lib = build(kind)
    try:
        handle = ctypes.CDLL(str(lib))
    except OSError as e:
        raise TensorError(f"loading {lib} failed: {e}") from e
    _loaded[kind] = handle
    return handle


def build_all(force: bool = True) -> None:
    build("host", force=force)
    build("hip", force=force)
