"""Compiling and loading the HIP modules.

Each ``csrc/<module>.hip`` becomes one shared library built with plain ``hipcc`` for
gfx950 and loaded through ``ctypes``; entry points are ``extern "C"`` functions that
take raw device pointers and a HIP stream.  ``csrc/<module>.cpp`` (the host-side core of the
cache manager) is plain C++ built with the host compiler the same way.  A module is compiled the first time it
is asked for (and again when its source or the flags change); the engine asks only
for the modules its model's parts name.  Built libraries live in ``csrc/_build`` of
the checkout, or in a per-user temporary folder if that is not writable.
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
from typing import Dict, Iterable, List

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc")
CSRC = os.path.normpath(CSRC)
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-shared", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-pass-failed"]
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC", "-Wall"]
HOST_MODULES = ("hostcore",)                      # plain C++, no GPU code
MODULES = ("common", "attention", "mamba2", "ssd", "gemm", "decode", "sampling", "microbench") + HOST_MODULES

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                           "the HIP kernels cannot be built and there is no other code path")


def _host_compiler() -> str:
    for candidate in (os.environ.get("CXX"), "g++", "c++", "clang++", "/opt/rocm/llvm/bin/clang++"):
        found = candidate and (candidate if os.path.isfile(candidate) else shutil.which(candidate))
        if found:
            return found
    raise KernelBuildError("no C++ compiler was found (looked at $CXX, g++, c++, clang++); "
                           "the host-side core cannot be built and there is no other code path")


def _main_source(module: str) -> str:
    return os.path.join(CSRC, f"{module}.cpp" if module in HOST_MODULES else f"{module}.hip")


def _sources(module: str) -> List[str]:
    main = _main_source(module)
    if not os.path.isfile(main):
        raise KernelBuildError(f"no such kernel module: {main}")
    if module in HOST_MODULES:
        return [main]
    headers = sorted(os.path.join(CSRC, name) for name in os.listdir(CSRC) if name.endswith(".h"))
    return [main] + headers


def _stamp(module: str) -> str:
    digest = hashlib.sha256()
    digest.update(" ".join(HOST_FLAGS if module in HOST_MODULES else FLAGS).encode())
    for path in _sources(module):
        with open(path, "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()


def _build_dirs() -> List[str]:
    in_tree = os.path.join(CSRC, "_build")
    user = os.path.join(tempfile.gettempdir(), f"macllm_infer_amd_build_{os.getuid()}")
    return [in_tree, user]


def _find_built(module: str, stamp: str):
    for folder in _build_dirs():
        library = os.path.join(folder, f"{module}.so")
        marker = library + ".stamp"
        if os.path.isfile(library) and os.path.isfile(marker):
            with open(marker) as handle:
                if handle.read().strip() == stamp:
                    return library
    return None


def _writable_build_dir() -> str:
    for folder in _build_dirs():
        try:
            os.makedirs(folder, exist_ok=True)
            probe = os.path.join(folder, f".probe_{os.getpid()}_{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return folder
        except OSError:
            continue
    raise KernelBuildError(f"no writable folder for built kernels among {_build_dirs()}")


def compile_module(module: str, force: bool = False, quiet: bool = False) -> str:
    """Compile one module if it is not built for the current source; return the library path."""
    stamp = _stamp(module)
    if not force:
        built = _find_built(module, stamp)
        if built:
            return built
    folder = _writable_build_dir()
    library = os.path.join(folder, f"{module}.so")
    scratch = os.path.join(folder, f"{module}.{os.getpid()}.tmp.so")
    if module in HOST_MODULES:
        command = [_host_compiler()] + HOST_FLAGS + [_main_source(module), "-o", scratch]
        what = f"host module '{module}'"
    else:
        command = [_hipcc()] + FLAGS + [_main_source(module), "-o", scratch]
        what = f"HIP module '{module}' for {ARCH}"
    if not quiet:
        print(f"[macllm_infer_amd] compiling {what} ...", file=sys.stderr, flush=True)
    started = time.time()
    environment = dict(os.environ)
    environment.setdefault("HOME", tempfile.gettempdir())
    process = subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                               env=environment, cwd=folder)
    output: List[str] = []
    reader = threading.Thread(target=lambda: output.append(process.stdout.read()), daemon=True)
    reader.start()
    while True:
        try:
            process.wait(timeout=15)
            break
        except subprocess.TimeoutExpired:
            if not quiet:
                print(f"[macllm_infer_amd]   still compiling '{module}' ({time.time() - started:.0f} s)",
                      file=sys.stderr, flush=True)
    reader.join()
    if process.returncode != 0:
        if os.path.exists(scratch):
            os.remove(scratch)
        raise KernelBuildError(f"{command[0]} failed for module '{module}':\n{''.join(output)}")
    os.replace(scratch, library)
    with open(library + ".stamp", "w") as handle:
        handle.write(stamp)
    if not quiet:
        print(f"[macllm_infer_amd] built '{module}' in {time.time() - started:.0f} s -> {library}",
              file=sys.stderr, flush=True)
    return library


def compile_modules(modules: Iterable[str], force: bool = False, quiet: bool = False) -> Dict[str, str]:
    """Compile several modules side by side."""
    modules = list(dict.fromkeys(modules))
    results: Dict[str, str] = {}
    errors: List[BaseException] = []

    def work(name: str) -> None:
        try:
            results[name] = compile_module(name, force=force, quiet=quiet)
        except BaseException as error:      # re-raised below, in the caller's thread
            errors.append(error)

    threads = [threading.Thread(target=work, args=(name,)) for name in modules]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    if errors:
        raise errors[0]
    return results


def load_module(module: str) -> ctypes.CDLL:
    """The loaded library of ``module``; compiles it first if need be.  There is no fallback:
    a module that cannot be built or loaded is an error."""
    with _lock:
        if module not in _loaded:
            path = compile_module(module)
            try:
                _loaded[module] = ctypes.CDLL(path)
            except OSError as error:
                raise KernelBuildError(f"cannot load {path}: {error}") from error
        return _loaded[module]


def ensure_modules(modules: Iterable[str]) -> None:
    needed = [name for name in dict.fromkeys(modules) if name not in _loaded]
    if needed:
        compile_modules(needed)
        for name in needed:
            load_module(name)
