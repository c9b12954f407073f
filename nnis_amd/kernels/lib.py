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
from typing import Dict, List, Optional, Tuple

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
SOURCE_FLAGS = {"gemm_mfma.hip": _VECTOR_SUMS, "attention.hip": _VECTOR_SUMS}
HEADERS = {"core": ["common.h", "epilogue.h", "nnis_noalloc.h"], "attention": ["common.h"]}  # what a module's sources include
CORE_SOURCES = ["elementwise.hip", "gemm.hip", "gemm_mfma.hip", "gemm_fused.hip", "sampling.hip"]
ATTENTION_SOURCES = ["attention.hip"]
PREBUILT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 192, 256)

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def _say(message: str) -> None:
    print(f"[nnis_amd] {message}", file=sys.stderr, flush=True)


def module_recipe(module: str) -> Tuple[List[str], Dict[str, str]]:
    """Sources and preprocessor definitions of a module name."""
    if module == "core":
        return [s for s in CORE_SOURCES if os.path.exists(os.path.join(CSRC, s))], {}
    if module.startswith("attn_hd"):
        head_dim = int(module[len("attn_hd"):])
        return list(ATTENTION_SOURCES), {"NNIS_HEAD_DIM": str(head_dim)}
    raise KernelError(f"unknown kernel module {module!r}")


def _module_hash(sources: List[str], defines: Dict[str, str]) -> str:
    digest = hashlib.sha256()
    headers = HEADERS["attention" if sources == ATTENTION_SOURCES else "core"]
    for name in headers + sources:
        with open(os.path.join(CSRC, name), "rb") as handle:
            digest.update(name.encode())
            digest.update(handle.read())
    digest.update(" ".join(FLAGS).encode())
    digest.update(repr(sorted((name, flags) for name, flags in SOURCE_FLAGS.items() if name in sources)).encode())
    digest.update(repr(sorted(defines.items())).encode())
    return digest.hexdigest()[:12]


def module_filename(module: str) -> str:
    sources, defines = module_recipe(module)
    return f"libnnis_{module}-{_module_hash(sources, defines)}.so"


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


def _run_with_heartbeat(commands: List[Tuple[str, List[str]]], env: Dict[str, str]) -> None:
    """Runs the commands in parallel, printing a line when each starts and
    ends and one every 20 s in between."""
    running = []
    for label, command in commands:
        _say(f"compiling {label} for {ARCH} ...")
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
    sources, defines = module_recipe(module)
    name = module_filename(module)
    if not force:
        found = find_built(module)
        if found:
            return found
    hipcc = _hipcc()
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
                (f"{source} [{module}]", [hipcc] + FLAGS + SOURCE_FLAGS.get(source, []) + define_flags + ["-I", CSRC, "-c", os.path.join(CSRC, source), "-o", obj])
            )
        _run_with_heartbeat(commands, env)
        tmp_out = os.path.join(work, name)
        _run_with_heartbeat([(f"link {module}", [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp_out] + objects)], env)
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
    return ["core"] + [f"attn_hd{d}" for d in PREBUILT_HEAD_DIMS]


def build_all(force: bool = True, jobs: int = 4) -> List[str]:
    """Compiles every module (used by the repository's build check)."""
    from concurrent.futures import ThreadPoolExecutor

    modules = all_prebuilt_modules()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        return list(pool.map(lambda m: build_module(m, force=force), modules))
