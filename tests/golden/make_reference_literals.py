"""Extract the numeric literals that the reference's example drivers use as test
inputs (they are data, not code) into reference_literals.json.

Run in the authoring container only (needs /root/reference); the JSON it writes
is what the tests read.  Sources:
  examples/torch/layernorm/cuda/verify.py:3-55   matrices a (4x32), b (32x8), c (8x16)
  examples/torch/layernorm/cuda/layernorm.cu:24-26   2x10 layer-norm input
  examples/torch/elementwise/add.cu:21-26   a (3x3x3), b (3x1x3)
  examples/torch/bert_attention/cuSeqLen.cu:18-19,26   bs, seq_len, row lengths
  examples/torch/linear/cuda/b.cu:17,28-38,47,61   GEMM constant case
"""
import json
import os
import re

REF = "/root/reference/examples/torch"


def floats(text):
    return [float(x) for x in re.findall(r"-?\d+\.?\d*(?:e-?\d+)?", text)]


def triple_quoted(src, name):
    m = re.search(name + r' = """(.*?)"""', src, re.S)
    rows = [floats(line) for line in m.group(1).strip().split("\n") if line.strip()]
    return rows


def braces_after(src, marker):
    i = src.index(marker)
    j = src.index("{", i)
    k = src.index("}", j)
    return floats(src[j + 1:k])


out = {}
v = open(os.path.join(REF, "layernorm/cuda/verify.py")).read()
out["verify_a"] = triple_quoted(v, "a")
out["verify_b"] = triple_quoted(v, "b")
out["verify_c"] = triple_quoted(v, "c")
out["verify_eps_stats"] = 1e-5   # verify.py:78
out["verify_eps_ln"] = 1e-6      # verify.py:89
ln = open(os.path.join(REF, "layernorm/cuda/layernorm.cu")).read()
out["layernorm_2x10"] = braces_after(ln, "float host_ptr[]")
add = open(os.path.join(REF, "elementwise/add.cu")).read()
out["add_a_3x3x3"] = braces_after(add, "float host_ptr_a[]")
out["add_b_3x1x3"] = braces_after(add, "float host_ptr_b[]")
cs = open(os.path.join(REF, "bert_attention/cuSeqLen.cu")).read()
out["cuseqlen_bs"] = int(re.search(r"bs = (\d+)", cs).group(1))
out["cuseqlen_seq"] = int(re.search(r"seq_len = (\d+)", cs).group(1))
out["cuseqlen_lengths"] = [int(x) for x in braces_after(cs, "int32_t data[]")]
out["gemm_const"] = {"m": 512, "n": 768, "k": 768, "a": 0.1, "b": 0.2,
                     "expect": 768 * 0.02, "tol": 1e-1}  # b.cu:17,28-38,61
assert len(out["verify_a"]) == 4 and len(out["verify_a"][0]) == 32
assert len(out["verify_b"]) == 32 and len(out["verify_b"][0]) == 8
assert len(out["verify_c"]) == 8 and len(out["verify_c"][0]) == 16
assert len(out["layernorm_2x10"]) == 20
assert len(out["add_a_3x3x3"]) == 27 and len(out["add_b_3x1x3"]) == 9
here = os.path.dirname(os.path.abspath(__file__))
json.dump(out, open(os.path.join(here, "reference_literals.json"), "w"), indent=1)
print("wrote reference_literals.json")
