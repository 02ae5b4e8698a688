"""The execution engine (include/hom_execution_engine.h) against a stand-in for a
module compiled by hands-on-opt (tests/modules/bert_encoder_module.cpp): the
reference's packed calling convention, init/argNum/dealloc protocol and
ownership rules (ExecutionEngine.h:27-171, ExtractInitFunc.cpp:60-276,
UnifyLLVMFuncInterface.cpp:60-131)."""
import ctypes
import importlib
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DIMS = dict(layers=2, hidden=128, heads=2, ffn=512, bs=3, seq=64, vocab=1000)


def build_module(tmp_path, extra=()):
    pkg = importlib.import_module("hands-on-mlir_amd")
    out = str(tmp_path / "libbert_module.so")
    d = DIMS
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           f"-I{ROOT}/include",
           f"-DHOM_LAYERS={d['layers']}", f"-DHOM_HIDDEN={d['hidden']}", f"-DHOM_HEADS={d['heads']}",
           f"-DHOM_FFN={d['ffn']}", f"-DHOM_BATCH={d['bs']}", f"-DHOM_SEQ={d['seq']}",
           f"-DHOM_VOCAB={d['vocab']}", *extra,
           os.path.join(ROOT, "tests", "modules", "bert_encoder_module.cpp"),
           f"-L{pkg.LIB_DIR}", "-lhom_amdgpu_runner_utils", f"-Wl,-rpath,{pkg.LIB_DIR}", "-o", out]
    subprocess.run(cmd, check=True)
    return out


def test_engine_header_symbols_exported():
    import re
    pkg = importlib.import_module("hands-on-mlir_amd")
    text = open(os.path.join(ROOT, "include", "hom_execution_engine.h")).read()
    names = set(re.findall(r"\b(homEngine\w+)\s*\(", text))
    assert names == {"homEngineOpen", "homEngineArgNum", "homEngineInvoke", "homEngineDealloc",
                     "homEngineClose", "homEngineLastError"}
    lib = ctypes.CDLL(pkg.ENGINE_LIB)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"


def test_engine_loads_module_and_reports_errors(tmp_path):
    engine = importlib.import_module("hands-on-mlir_amd.engine")
    with pytest.raises(OSError):
        engine.Engine(str(tmp_path / "missing.so"))
    e = engine.Engine(build_module(tmp_path))
    try:
        assert e.arg_num("forward") == 2 + 4 * DIMS["layers"] + 6
        assert e.arg_num("backward") == -1
        with pytest.raises(RuntimeError, match="_hom_ciface_backward"):
            e.invoke("backward", [])
    finally:
        e.close()


@pytest.mark.gpu
def test_compiled_masked_lm_module_through_engine(gpu, rt, oracle, synth, tmp_path, monkeypatch):
    """The stand-in module with the LM head (-DHOM_LM_HEAD): forward returns logits [b, s, vocab], as the
    module the reference's examples/torch/bert/bert.cu loads does."""
    import torch
    engine = importlib.import_module("hands-on-mlir_amd.engine")
    weights = importlib.import_module("hands-on-mlir_amd.weights")
    enc_test = importlib.import_module("test_gpu_encoder")
    d = dict(DIMS, vocab=1002)
    model = synth.bert_encoder(config=43, **d)
    model["lens"][:] = [64, 9, 40]
    model["mask"] = synth.mask_from_lengths(model["lens"], d["seq"])
    consts = [model["word"], model["pos_type"]]
    for w in model["weights"]:
        consts += [w[k] for k in ("wqkv", "wo", "w1", "w2")]
    consts += [model["w_transform"], np.ascontiguousarray(model["word"].T)]
    for i, c in enumerate(consts):
        weights.write_binary(str(tmp_path), i, c)
    monkeypatch.setenv("HOM_CONSTANT_DIR", str(tmp_path))
    monkeypatch.setitem(DIMS, "vocab", 1002)
    e = engine.Engine(build_module(tmp_path, ("-DHOM_LM_HEAD",)))
    try:
        assert e.arg_num("forward") == 2 + 4 * d["layers"] + 2 + 8
        ids = torch.from_numpy(model["ids"]).cuda()
        mask = torch.from_numpy(model["mask"].astype(np.int64)).cuda()
        M = rt.MemRef.from_tensor
        res = e.invoke("forward", [M(ids), M(mask)])
        ptr, sizes, strides = rt.read_descriptor(res)
        assert res.rank == 3 and sizes == [d["bs"], d["seq"], d["vocab"]]
        out = torch.empty(sizes, dtype=torch.float16, device="cuda")
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        torch.cuda.synchronize()
        assert hip.hipMemcpy(out.data_ptr(), ptr, out.numel() * 2, 3) == 0
        logits = out.cpu().numpy()
        libc = ctypes.CDLL("libc.so.6")
        libc.free.argtypes = [ctypes.c_void_p]
        libc.free(res.descriptor)
        h_or = enc_test.oracle_forward(oracle, model, "erf").astype(np.float16)
        want = enc_test.lm_head_oracle(oracle, h_or, model, "erf").reshape(d["bs"], d["seq"], d["vocab"])
        for b, n in enumerate(model["lens"]):
            err = np.abs(logits[b, :n].astype(np.float64) - want[b, :n])
            assert (err <= 1e-2 + 1e-3 * np.abs(want[b, :n])).all(), (b, err.max())
        e.dealloc("forward")
    finally:
        e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["manifest", "nvte"])
def test_compiled_module_through_engine(gpu, rt, oracle, synth, tmp_path, monkeypatch, variant):
    import torch
    engine = importlib.import_module("hands-on-mlir_amd.engine")
    weights = importlib.import_module("hands-on-mlir_amd.weights")
    enc_test = importlib.import_module("test_gpu_encoder")
    d = DIMS
    model = synth.bert_encoder(config=43, **d)
    model["lens"][:] = [64, 9, 40]
    model["mask"] = synth.mask_from_lengths(model["lens"], d["seq"])
    nk = variant == "nvte"
    consts = [model["word"], model["pos_type"]]
    for w in model["weights"]:
        consts += [w[k].T.copy() if nk else w[k] for k in ("wqkv", "wo", "w1", "w2")]
    for i, c in enumerate(consts):
        # half of them as text, half as binary files: both formats reach the same bits
        (weights.write_text if i % 2 else weights.write_binary)(str(tmp_path), i, c)
    monkeypatch.setenv("HOM_CONSTANT_DIR", str(tmp_path))
    e = engine.Engine(build_module(tmp_path, ("-DHOM_USE_NVTE",) if nk else ()))
    try:
        ids = torch.from_numpy(model["ids"]).cuda()
        mask = torch.from_numpy(model["mask"].astype(np.int64)).cuda()
        M = rt.MemRef.from_tensor
        outs = []
        for _ in range(2):  # the second call reuses the tensors the first one initialised
            res = e.invoke("forward", [M(ids), M(mask)])
            ptr, sizes, strides = rt.read_descriptor(res)
            assert res.rank == 3 and sizes == [d["bs"], d["seq"], d["hidden"]]
            out = torch.empty(sizes, dtype=torch.float16, device="cuda")
            hip = ctypes.CDLL("libamdhip64.so")
            hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
            torch.cuda.synchronize()
            assert hip.hipMemcpy(out.data_ptr(), ptr, out.numel() * 2, 3) == 0
            outs.append(out.cpu().numpy())
            # the result's descriptor belongs to the caller (bert.cu:169 frees it)
            libc = ctypes.CDLL("libc.so.6")
            libc.free.argtypes = [ctypes.c_void_p]
            libc.free(res.descriptor)
        assert np.array_equal(outs[0], outs[1])
        want = enc_test.oracle_forward(oracle, model, "tanh" if nk else "erf")
        enc_test.check(outs[0], want, model["lens"], f"compiled module ({variant})")
        e.dealloc("forward")
    finally:
        e.close()
