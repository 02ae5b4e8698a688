"""Thin Python handle on the C++ BERT driver (csrc/bert_driver.cpp) for tests
and benchmarks: uploads seeded weights, runs the lowered encoder's call list
eagerly or as a replayed HIP graph, fetches the output."""
import ctypes

import numpy as np

from . import hom_runtime as rt


class BertEncoder:
    ROLES = ("qkv", "out", "ffn1", "ffn2", "transform", "decoder")

    def __init__(self, layers, hidden, heads, ffn, bs, seq, vocab, gemm_mode=1, gelu_form="erf",
                 lm_head=False, role_layout=None, fold_layernorm=False):
        """role_layout: optional {role: "kn" | "nk"} pinning the weight layout (and with it the entry
        point: cutlassGemmF16 / nvteGemmF16) of individual GEMM roles; others are decided by the driver.
        fold_layernorm: run the call list whose per-layer layer norms are folded into the GEMMs around them
        (homGemmFoldedLayernormF16; row-major weights for every role, erf GELU); takes effect in load()."""
        self.fold_layernorm = fold_layernorm
        if fold_layernorm:
            role_layout = dict(role_layout or {}, qkv="kn", out="kn", ffn1="kn", ffn2="kn")
        self.drv = rt.load_driver()
        self.dims = dict(layers=layers, hidden=hidden, heads=heads, ffn=ffn, bs=bs, seq=seq, vocab=vocab)
        self.gemm_mode = gemm_mode
        layout = (ctypes.c_int32 * 6)(*[-1] * 6)
        for role, lay in (role_layout or {}).items():
            layout[self.ROLES.index(role)] = {"kn": 0, "nk": 1}[lay]
        self.h = self.drv.homBertCreateWithLayout(layers, hidden, heads, ffn, bs, seq, vocab, gemm_mode,
                                                  1 if gelu_form == "tanh" else 0, layout)
        if not self.h:
            raise ValueError("homBertCreateWithLayout refused the configuration (a GELU role of an erf-GELU "
                             "graph pinned to [N, K] weights: nvteGemmF16 computes the tanh form only)")
        self.lm_head = lm_head
        if lm_head:
            assert self.drv.homBertEnableLmHead(self.h) == 0, "homBertEnableLmHead failed"

    def close(self):
        if self.h:
            self.drv.homBertDestroy(self.h)
            self.h = None

    def _upload(self, layer, which, arr):
        arr = np.ascontiguousarray(arr, np.float16)
        rc = self.drv.homBertUpload(self.h, layer, which, arr.ctypes.data_as(ctypes.c_void_p), arr.size)
        assert rc == 0, f"upload failed ({rc})"

    def load(self, model):
        """model: dict from synth.bert_encoder().  Weights are [K, N]; the nvte
        path wants them as [N, K], which the compiler would transpose at compile
        time (HOMNVGPULegalizeGemmPass)."""
        nk = [bool(self.drv.homBertRoleIsNK(self.h, r)) for r in range(6)]
        for l, w in enumerate(model["weights"]):
            for which, key in enumerate(("wqkv", "wo", "w1", "w2")):
                self._upload(l, which, w[key].T if nk[which] else w[key])
        self._upload(0, 4, model["word"])
        self._upload(0, 5, model["pos_type"])
        if self.lm_head:
            # the decoder is tied to the word embeddings (BertForMaskedLM): logits = t . word^T, so the
            # [K, N] operand of the manifest path is word^T and the [N, K] operand of the nvte path is word
            self._upload(0, 6, model["w_transform"].T if nk[4] else model["w_transform"])
            self._upload(0, 7, model["word"] if nk[5] else model["word"].T)
        if self.fold_layernorm:
            # (after the uploads: the column sums of Wqkv and W1 are computed from the device copies)
            if self.drv.homBertFoldLayernorm(self.h) != 0:
                raise ValueError("the driver refused to fold the layer norms for this configuration")

    def set_inputs(self, ids=None, mask=None, hidden=None):
        p = lambda a, dt: (np.ascontiguousarray(a, dt).ctypes.data_as(ctypes.c_void_p)
                           if a is not None else None)
        keep = [np.ascontiguousarray(a, dt) if a is not None else None
                for a, dt in ((ids, np.int64), (mask, np.int64), (hidden, np.float16))]
        ptrs = [a.ctypes.data_as(ctypes.c_void_p) if a is not None else None for a in keep]
        assert self.drv.homBertSetInputs(self.h, *ptrs) == 0

    def forward(self, from_ids=True):
        self.drv.homBertForward(self.h, int(from_ids))

    def capture(self, from_ids=True):
        assert self.drv.homBertCapture(self.h, int(from_ids)) == 0

    @property
    def stream(self):
        """The hipStream_t (as an integer) this encoder's calls are enqueued on."""
        return self.drv.homBertGetStream(self.h)

    def replay(self):
        assert self.drv.homBertReplay(self.h) == 0

    def output(self):
        d = self.dims
        out = np.empty((d["bs"], d["seq"], d["hidden"]), np.float16)
        assert self.drv.homBertGetOutput(self.h, out.ctypes.data_as(ctypes.c_void_p)) == 0
        return out

    def logits(self):
        d = self.dims
        out = np.empty((d["bs"], d["seq"], d["vocab"]), np.float16)
        assert self.drv.homBertGetLogits(self.h, out.ctypes.data_as(ctypes.c_void_p)) == 0
        return out

    def time(self, steps, warmup, graph=True, from_ids=True):
        ms = self.drv.homBertTime(self.h, steps, warmup, int(graph), int(from_ids))
        assert ms > 0, "timing failed"
        return ms

    def set_gemm_choice(self, role, gemm_num, split_k=1):
        """Pin the manifest kernel (1-based) of one GEMM role ("qkv", "out", "ffn1", "ffn2")."""
        idx = ("qkv", "out", "ffn1", "ffn2").index(role)
        if self.drv.homBertSetGemmChoice(self.h, idx, gemm_num, split_k) != 0:
            raise ValueError(f"bad kernel choice {gemm_num}/{split_k} for {role}")

    def role_is_nk(self, role):
        return bool(self.drv.homBertRoleIsNK(self.h, self.ROLES.index(role)))

    def gemm_choices(self):
        buf = (ctypes.c_int32 * 8)()
        self.drv.homBertGetGemmChoices(self.h, buf)
        names = ("qkv", "out", "ffn1", "ffn2")
        return {n: (buf[2 * i], buf[2 * i + 1]) for i, n in enumerate(names)}
