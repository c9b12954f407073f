"""Builds and loads the gfx950 kernel modules.

A module is one shared library made from sources under ``nnis_amd/csrc`` with
``hipcc --offload-arch=gfx950`` and loaded through ``ctypes``.  ``core`` holds
the kernels whose sizes are run-time arguments; attention is compiled per head
size (``attn_hd<N>``), so a first call compiles what the model at hand needs
and nothing else.  A built library is named after a hash of its sources and
flags: a stale one is never loaded.

There is no fallback: if a module is neither built nor buildable the call
fails with ``KernelError``.
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
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

from ..errors import KernelError

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib")
ARCH = "gfx950"
# packed 32-bit float instructions are switched off for all device code
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# Per source: the matrix instructions keep their sums in the ordinary vector registers.  Left to itself the
# compiler puts them into the accumulation registers and moves them to and fro: in the tiled product's loop 48
# moves a step for 16 matrix instructions, in the decode attention with keys on lanes 336 for 144.  (With the
# sums in vector registers the prefill attention's four-column kernels at 64 channels keep 17 to 26 registers
# in scratch memory, all outside their loops over the keys; no other kernel of either file spills.)
_VECTOR_SUMS = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
PREBUILT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 192, 256)

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


@dataclass(frozen=True)
class ModuleRecipe:
    """What a module is made from: source files and the headers they include (names inside ``directory``),
    preprocessor definitions, and extra compiler flags per source."""

    sources: Tuple[str, ...]
    headers: Tuple[str, ...] = ()
    defines: Tuple[Tuple[str, str], ...] = ()
    source_flags: Tuple[Tuple[str, Tuple[str, ...]], ...] = ()
    directory: str = CSRC
    host_only: bool = False  # plain C++ for the host compiler: no device code, no GPU needed to run it

    def flags_of(self, source: str) -> List[str]:
        return [flag for name, flags in self.source_flags if name == source for flag in flags]


_modules: Dict[str, ModuleRecipe] = {}
_families: Dict[str, Callable[[str], ModuleRecipe]] = {}  # by prefix: the rest of a module's name -> its recipe


def register_module(name: str, sources: Sequence[str], headers: Sequence[str] = (), defines: Optional[Dict[str, str]] = None,
                    source_flags: Optional[Dict[str, Sequence[str]]] = None, directory: str = CSRC, replace: bool = False,
                    host_only: bool = False) -> None:
    """Makes ``load_module(name)`` build and load a library from ``sources``
    under ``directory`` (every flag of the library's own kernels applies; the
    library's headers are on the include path).  A part that brings kernels
    of its own registers them here and declares their entry points with
    ``ops.bind``; nothing else in the library has to know the module.  The
    module exports ``const char* nnis_last_error()`` (``common.h`` has the
    helpers that fill it), and its entry points return 0 or an error."""
    if name in _modules and not replace:
        raise KernelError(f"kernel module {name!r} is registered already")
    _modules[name] = ModuleRecipe(tuple(sources), tuple(headers), tuple(sorted((defines or {}).items())),
                                  tuple(sorted((k, tuple(v)) for k, v in (source_flags or {}).items())), directory, host_only)


def register_module_family(prefix: str, recipe: Callable[[str], ModuleRecipe], replace: bool = False) -> None:
    """Modules compiled per size: ``load_module(prefix + rest)`` builds what ``recipe(rest)`` describes."""
    if prefix in _families and not replace:
        raise KernelError(f"kernel module family {prefix!r} is registered already")
    _families[prefix] = recipe


def _attention_recipe(rest: str) -> ModuleRecipe:
    try:
        head_dim = int(rest)
    except ValueError:
        raise KernelError(f"unknown kernel module 'attn_hd{rest}'") from None
    return ModuleRecipe(("attention.hip",), ("common.h",), (("NNIS_HEAD_DIM", str(head_dim)),), (("attention.hip", tuple(_VECTOR_SUMS)),))


# the library's own modules: ``core`` holds the kernels whose sizes are run-time arguments; attention is compiled per head size
register_module("core", ["elementwise.hip", "gemm.hip", "gemm_mfma.hip", "gemm_fused.hip", "sampling.hip"],
                headers=["common.h", "epilogue.h", "nnis_noalloc.h"], source_flags={"gemm_mfma.hip": _VECTOR_SUMS})
register_module_family("attn_hd", _attention_recipe)
# plain host references of the kernels' operations, for the tests (no device code: the host compiler builds them)
register_module("reference", ["reference.cpp"], host_only=True)
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-ffp-contract=off"]  # a multiply-add is fused only where the source says fmaf


def _say(message: str) -> None:
    print(f"[nnis_amd] {message}", file=sys.stderr, flush=True)


def module_recipe(module: str) -> ModuleRecipe:
    """What a module name is made from."""
    if module in _modules:
        return _modules[module]
    for prefix, recipe in _families.items():
        if module.startswith(prefix):
            return recipe(module[len(prefix):])
    raise KernelError(f"unknown kernel module {module!r}")


def _module_hash(recipe: ModuleRecipe) -> str:
    digest = hashlib.sha256()
    for name in recipe.headers + recipe.sources:
        path = os.path.join(recipe.directory, name)
        if not os.path.exists(path):
            path = os.path.join(CSRC, name)  # (a module from elsewhere may include the library's headers)
        with open(path, "rb") as handle:
            digest.update(name.encode())
            digest.update(handle.read())
    digest.update(" ".join(HOST_FLAGS if recipe.host_only else FLAGS).encode())
    digest.update(repr(sorted((name, list(flags)) for name, flags in recipe.source_flags if name in recipe.sources)).encode())
    digest.update(repr(sorted(recipe.defines)).encode())
    return digest.hexdigest()[:12]


def module_filename(module: str) -> str:
    return f"libnnis_{module}-{_module_hash(module_recipe(module))}.so"


def _fallback_dir() -> str:
    base = os.environ.get("TMPDIR") or tempfile.gettempdir()
    path = os.path.join(base, f"nnis_amd-lib-{os.getuid()}")
    os.makedirs(path, exist_ok=True)
    return path


def find_built(module: str) -> Optional[str]:
    name = module_filename(module)
    for directory in (LIB_DIR, _fallback_dir()):
        path = os.path.join(directory, name)
        if os.path.exists(path):
            return path
    return None


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise KernelError("hipcc was not found (PATH, $HIPCC, /opt/rocm/bin): the HIP kernels cannot be built")


def _host_compiler() -> str:
    for candidate in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if candidate and (os.path.isabs(candidate) and os.path.exists(candidate) or shutil.which(candidate)):
            return shutil.which(candidate) or candidate
    raise KernelError("no host C++ compiler was found (CXX, g++, c++, clang++): the plain references cannot be built")


def _run_with_heartbeat(commands: List[Tuple[str, List[str]]], env: Dict[str, str]) -> None:
    """Runs the commands in parallel, printing a line when each starts and
    ends and one every 20 s in between."""
    running = []
    for label, command in commands:
        _say(f"compiling {label} ...")
        running.append((label, subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env)))
    started = time.time()
    last = started
    failures = []
    pending = list(running)
    while pending:
        still = []
        for label, process in pending:
            try:
                output, _ = process.communicate(timeout=0.5)
            except subprocess.TimeoutExpired:
                still.append((label, process))
                continue
            if process.returncode != 0:
                failures.append((label, output.decode(errors="replace")))
            else:
                _say(f"compiled {label} ({time.time() - started:.0f} s)")
        pending = still
        if pending and time.time() - last > 20:
            last = time.time()
            _say(f"still compiling {', '.join(label for label, _ in pending)} ({last - started:.0f} s)")
    if failures:
        text = "\n".join(f"--- {label} ---\n{output}" for label, output in failures)
        raise KernelError(f"hipcc failed:\n{text}")


def build_module(module: str, force: bool = False) -> str:
    """Compiles one module and returns the library's path."""
    recipe = module_recipe(module)
    sources, defines = list(recipe.sources), dict(recipe.defines)
    name = module_filename(module)
    if not force:
        found = find_built(module)
        if found:
            return found
    hipcc = _host_compiler() if recipe.host_only else _hipcc()
    base_flags = HOST_FLAGS if recipe.host_only else FLAGS
    try:
        os.makedirs(LIB_DIR, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=LIB_DIR, delete=True)
        probe.close()
        out_dir = LIB_DIR
    except OSError:
        out_dir = _fallback_dir()
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env.get("HOME", "/nonexistent"), os.W_OK):
        env["HOME"] = _fallback_dir()  # the compiler may keep a cache under HOME
    work = tempfile.mkdtemp(prefix=f"nnis_{module}_", dir=_fallback_dir())
    try:
        define_flags = [f"-D{k}={v}" for k, v in sorted(defines.items())]
        objects = []
        commands = []
        for source in sources:
            obj = os.path.join(work, source + ".o")
            objects.append(obj)
            commands.append(
                (f"{source} [{module}] for {'the host' if recipe.host_only else ARCH}", [hipcc] + base_flags + recipe.flags_of(source) + define_flags
                 + ["-I", recipe.directory, "-I", CSRC, "-c", os.path.join(recipe.directory, source), "-o", obj])
            )
        _run_with_heartbeat(commands, env)
        tmp_out = os.path.join(work, name)
        link = [hipcc, "-shared", "-fPIC", "-o", tmp_out] if recipe.host_only else [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp_out]
        _run_with_heartbeat([(f"link {module}", link + objects)], env)
        final = os.path.join(out_dir, name)
        shutil.move(tmp_out, final)
        # older builds of the same module are of no use any more
        prefix = f"libnnis_{module}-"
        for other in os.listdir(out_dir):
            if other.startswith(prefix) and other != name and other.endswith(".so"):
                try:
                    os.remove(os.path.join(out_dir, other))
                except OSError:
                    pass
        return final
    finally:
        shutil.rmtree(work, ignore_errors=True)


def load_module(module: str, build_if_missing: bool = True) -> ctypes.CDLL:
    with _lock:
        if module in _loaded:
            return _loaded[module]
        path = find_built(module)
        if path is None:
            if not build_if_missing:
                raise KernelError(f"kernel module {module} is not built ({module_filename(module)} not found under {LIB_DIR})")
            _say(f"kernel module {module} is not built yet; building it now")
            path = build_module(module)
        try:
            lib = ctypes.CDLL(path)
        except OSError as error:
            raise KernelError(f"cannot load {path}: {error}") from None
        lib.nnis_last_error.restype = ctypes.c_char_p
        lib.nnis_last_error.argtypes = []
        _loaded[module] = lib
        return lib


def all_prebuilt_modules() -> List[str]:
    return ["core", "reference"] + [f"attn_hd{d}" for d in PREBUILT_HEAD_DIMS]


def build_all(force: bool = True, jobs: int = 4) -> List[str]:
    """Compiles every module (used by the repository's build check)."""
    from concurrent.futures import ThreadPoolExecutor

    modules = all_prebuilt_modules()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        return list(pool.map(lambda m: build_module(m, force=force), modules))
