"""Kernel modules as a registry: the library's own are entries of it, and a
part from elsewhere adds its sources without a change to the library (here the
toy kernel that tests/test_gpu_parts.py runs on the GPU: compiled for gfx950,
which needs no GPU)."""

import ctypes
import os
import shutil

import pytest

from nnis_amd.errors import KernelError
from nnis_amd.kernels import lib

HERE = os.path.dirname(os.path.abspath(__file__))


def test_the_librarys_modules_are_registered_like_any_other():
    core = lib.module_recipe("core")
    assert "gemm_mfma.hip" in core.sources and "common.h" in core.headers and core.directory == lib.CSRC
    attention = lib.module_recipe("attn_hd96")
    assert attention.sources == ("attention.hip",) and dict(attention.defines) == {"NNIS_HEAD_DIM": "96"}
    assert lib.module_filename("attn_hd96") != lib.module_filename("attn_hd64")  # a size of its own, a library of its own
    for unknown in ("nothing", "attn_hdx"):
        with pytest.raises(KernelError, match="unknown kernel module"):
            lib.module_recipe(unknown)
    with pytest.raises(KernelError, match="registered already"):
        lib.register_module("core", ["gemm.hip"])


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_a_module_from_elsewhere_is_built_and_named_by_its_sources(tmp_path):
    lib.register_module("toy_mean", ["toy_running_mean.hip"], headers=["common.h"], directory=HERE, replace=True)
    name = lib.module_filename("toy_mean")
    path = lib.build_module("toy_mean")  # (compiles only if this very source is not built yet)
    assert os.path.basename(path) == name and os.path.exists(path)
    handle = ctypes.CDLL(path)
    assert hasattr(handle, "toy_running_mean") and hasattr(handle, "nnis_last_error")
    # another source under the same module name is another library: a stale build is never loaded
    other = tmp_path / "toy_running_mean.hip"
    other.write_text(open(os.path.join(HERE, "toy_running_mean.hip")).read() + "\n// changed\n")
    lib.register_module("toy_mean", ["toy_running_mean.hip"], headers=["common.h"], directory=str(tmp_path), replace=True)
    assert lib.module_filename("toy_mean") != name
    lib.register_module("toy_mean", ["toy_running_mean.hip"], headers=["common.h"], directory=HERE, replace=True)
