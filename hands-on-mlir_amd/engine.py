"""ctypes binding of the execution engine (include/hom_execution_engine.h): loads a
module compiled by hands-on-opt and calls it through the reference's packed
calling convention.  For tests and examples; nothing here computes."""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_void_p

from . import ENGINE_LIB
from .hom_runtime import CUnrankedMemRef, load_runtime

_lib = None


def load_engine():
    global _lib
    if _lib is None:
        if not os.path.exists(ENGINE_LIB):
            raise RuntimeError(f"{ENGINE_LIB} is missing: build it with __graft_entry__.build()")
        lib = ctypes.CDLL(ENGINE_LIB)
        lib.homEngineOpen.restype, lib.homEngineOpen.argtypes = c_void_p, [c_char_p]
        lib.homEngineArgNum.restype, lib.homEngineArgNum.argtypes = c_int32, [c_void_p, c_char_p]
        lib.homEngineInvoke.restype = c_int
        lib.homEngineInvoke.argtypes = [c_void_p, c_char_p, POINTER(c_void_p), c_int32]
        lib.homEngineDealloc.restype, lib.homEngineDealloc.argtypes = c_int, [c_void_p, c_char_p]
        lib.homEngineClose.restype, lib.homEngineClose.argtypes = None, [c_void_p]
        lib.homEngineLastError.restype, lib.homEngineLastError.argtypes = c_char_p, [c_void_p]
        _lib = lib
    return _lib


class Engine:
    """mlir::hands_on_mlir::ExecutionEngine's role: ``Engine(path).invoke("forward", ...)``."""

    def __init__(self, path):
        load_runtime()  # the module resolves the operator entry points against it
        self._lib = load_engine()
        self._h = self._lib.homEngineOpen(os.fsencode(path))
        if not self._h:
            raise OSError(self._lib.homEngineLastError(None).decode())

    def arg_num(self, func="forward"):
        return self._lib.homEngineArgNum(self._h, func.encode())

    def invoke(self, func, memrefs, returns_memref=True):
        """memrefs: MemRef arguments in order.  Returns the CUnrankedMemRef result (its
        descriptor is malloc'd by the module and owned by the caller) or None."""
        keep, slots = [], []
        for m in memrefs:
            rank, desc = c_int64(m.rank), c_void_p(ctypes.cast(m.descriptor, c_void_p).value)
            keep += [rank, desc]
            slots += [ctypes.addressof(rank), ctypes.addressof(desc)]
        result = CUnrankedMemRef(0, None)
        if returns_memref:
            slots.append(ctypes.addressof(result))
        arr = (c_void_p * len(slots))(*slots)
        if self._lib.homEngineInvoke(self._h, func.encode(), arr, len(slots)) != 0:
            raise RuntimeError(self._lib.homEngineLastError(self._h).decode())
        return result if returns_memref else None

    def dealloc(self, func="forward"):
        if self._lib.homEngineDealloc(self._h, func.encode()) != 0:
            raise RuntimeError(self._lib.homEngineLastError(self._h).decode())

    def close(self):
        if self._h:
            self._lib.homEngineClose(self._h)
            self._h = None
