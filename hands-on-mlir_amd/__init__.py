"""MI355X-native runtime kernel library for Hands-on-MLIR's lowered BERT graphs.

The product is the C-ABI shared library ``lib/libhom_amdgpu_runner_utils.so``
(sources in ``csrc/``, interface in ``/include``) plus the C++ host driver
``lib/libhom_bert_driver.so``.  This Python package only builds them and binds
them with ctypes for tests and benchmarks.
"""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
RUNTIME_LIB = os.path.join(LIB_DIR, "libhom_amdgpu_runner_utils.so")
DRIVER_LIB = os.path.join(LIB_DIR, "libhom_bert_driver.so")
ENGINE_LIB = os.path.join(LIB_DIR, "libhom_execution_engine.so")


def build(jobs: int = 8, force: bool = True) -> None:
    """Compile every HIP source for gfx950 (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", CSRC_DIR, f"-j{jobs}"]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)


def libraries_built() -> bool:
    return os.path.exists(RUNTIME_LIB) and os.path.exists(DRIVER_LIB)
