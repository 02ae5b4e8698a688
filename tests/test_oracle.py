"""Pins the CPU oracle: against the literals the reference's example drivers
hold, against numpy / scipy / torch library routines, and against closed-form
identities chosen so that a dropped term, a wrong sign or index or a transposed
operand fails at least one of them."""
import numpy as np
import pytest
import scipy.special
import torch


# ------------------------------------------------------------------ fp16 ----
def test_half_conversions_match_numpy(oracle):
    L = oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    got = np.array([L.hom_oracle_half_to_float(int(h)) for h in allh], np.float32)
    ok = (got == ref) | (np.isnan(got) & np.isnan(ref))
    assert ok.all()
    g = np.random.default_rng(0)
    bits = g.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    edge = np.array([0x33000000, 0x33000001, 0x32ffffff, 0x387fc000, 0x387fe000, 0x38800000,
                     0x477fe000, 0x477fefff, 0x477ff000, 0x47800000, 0x3f801000, 0x3f803000,
                     0x00000001, 0x7f800000, 0x80000000, 0x38000000, 0x387fffff], np.uint32)
    bits = np.concatenate([bits, edge, edge | np.uint32(0x80000000)])
    f = bits.view(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([L.hom_oracle_float_to_half(float(x)) if not np.isnan(x) else 0x7e00 for x in f],
                   np.uint16)
    nan = np.isnan(f)
    assert (got[~nan] == want[~nan]).all()


# ------------------------------------------------------------------ GELU ----
def test_gelu_forms(oracle):
    x = np.linspace(-8, 8, 4001)
    erf = oracle.gelu(x, "erf")
    assert np.allclose(erf, 0.5 * x * (1 + scipy.special.erf(x / np.sqrt(2))), rtol=0, atol=1e-15)
    t = torch.tensor(x, dtype=torch.float64)
    assert np.allclose(erf, torch.nn.functional.gelu(t).numpy(), atol=1e-12)
    tanh = oracle.gelu(x, "tanh")
    assert np.allclose(tanh, torch.nn.functional.gelu(t, approximate="tanh").numpy(), atol=1e-12)
    poly = oracle.gelu(x, "poly")
    # identities: GELU(0) = 0, GELU(x) - GELU(-x) = x, -> x for large x
    for f in (erf, tanh, poly):
        assert f[2000] == 0.0
        assert np.allclose(f - f[::-1], x, atol=1e-12)
        assert abs(f[-1] - 8.0) < 1e-6
    # the three forms differ by less than 1e-3 absolute (A&S 7.1.27 erf error 5e-4)
    assert np.abs(erf - tanh).max() < 1e-3
    assert np.abs(erf - poly).max() < 1.5e-3
    assert np.abs(erf - poly).max() > 1e-5  # and they are not the same function


# ------------------------------------------------------------------ GEMM ----
def _rand16(g, shape, std=1.0):
    return (g.standard_normal(shape) * std).astype(np.float16)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (5, 7, 3), (33, 17, 65), (64, 128, 96)])
def test_gemm_matches_numpy(oracle, M, N, K):
    g = np.random.default_rng(M * 1000 + N * 10 + K)
    A, B, C = _rand16(g, (M, K)), _rand16(g, (K, N)), _rand16(g, (M, N))
    want = 0.5 * (A.astype(np.float64) @ B.astype(np.float64)) + 2.0 * C.astype(np.float64)
    got = oracle.gemm(A, B, C, alpha=0.5, beta=2.0)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    # B given as [N, K] must give the same result (catches a transposed operand)
    got_nk = oracle.gemm(A, np.ascontiguousarray(B.T), C, alpha=0.5, beta=2.0, b_is_nk=True)
    assert np.array_equal(got, got_nk)
    # bias row and per-batch broadcast
    bias = _rand16(g, (1, N))
    assert np.allclose(oracle.gemm(A, B, bias, beta=1.0),
                       A.astype(np.float64) @ B.astype(np.float64) + bias.astype(np.float64),
                       rtol=1e-6, atol=1e-6)
    # beta == 0 ignores C entirely
    assert np.array_equal(oracle.gemm(A, B, None), oracle.gemm(A, B, C, beta=0.0))


def test_gemm_identity_and_onehot_are_exact(oracle):
    g = np.random.default_rng(1)
    A = _rand16(g, (16, 16))
    eye = np.eye(16, dtype=np.float16)
    assert np.array_equal(oracle.gemm(A, eye), A.astype(np.float32))
    assert np.array_equal(oracle.gemm(eye, A), A.astype(np.float32))
    onehot = np.zeros((16, 4), np.float16)
    onehot[3, 0] = onehot[5, 1] = onehot[0, 2] = onehot[15, 3] = 1
    assert np.array_equal(oracle.gemm(A, onehot), A[:, [3, 5, 0, 15]].astype(np.float32))


def test_gemm_reference_constant_case(oracle, literals):
    c = literals["gemm_const"]  # b.cu: A = 0.1, B = 0.2, expect K * 0.02 within 1e-1
    A = np.full((c["m"], c["k"]), c["a"], np.float16)
    B = np.full((c["k"], c["n"]), c["b"], np.float16)
    out = oracle.gemm(A, B)
    assert np.abs(out - c["expect"]).max() < c["tol"]
    exact = c["k"] * float(np.float16(c["a"])) * float(np.float16(c["b"]))
    assert np.allclose(out, exact, rtol=1e-6)


def test_gemm_verify_py_matrices(oracle, literals):
    a = np.array(literals["verify_a"], np.float16)
    b = np.array(literals["verify_b"], np.float16)
    ab = oracle.gemm(a, b)
    want = (torch.tensor(a.astype(np.float32)) @ torch.tensor(b.astype(np.float32))).numpy()
    assert np.allclose(ab, want, rtol=1e-5, atol=1e-5)
    # rstd / -mean*rstd, formulas of verify.py:72-80
    var, mean = oracle.row_stats(ab, literals["verify_eps_stats"])
    t = torch.tensor(want, dtype=torch.float64)
    m, sqm = t.mean(-1), (t * t).mean(-1)
    v = 1 / torch.sqrt(sqm - m * m + literals["verify_eps_stats"])
    assert np.allclose(var, v.numpy(), rtol=1e-4)
    assert np.allclose(mean, (-m * v).numpy(), rtol=1e-4)


def test_row_stats_constant_row_is_finite(oracle):
    """E[x^2] - E[x]^2 of a constant row is zero up to rounding, possibly negative: the clamp keeps
    var = 1/sqrt(eps) finite for the tiny eps BERT uses, and mean = -x * var."""
    x = np.full((3, 768), 0.1, np.float32)
    x[1] = -7.3
    x[2] = 1000.25
    var, mean = oracle.row_stats(x, 1e-12)
    assert np.isfinite(var).all() and np.isfinite(mean).all()
    # The true variance of a constant row is exactly 0, so var = 1/sqrt(eps) = 1e6 wherever the fp64
    # rounding of E[x^2] - E[x]^2 (at most 2 n 2^-53 x^2, a sequential sum of n products) is far below
    # eps, and never above it (the clamp); where the rounding is comparable to eps it can only lower var,
    # to no less than 1/sqrt(that bound + eps).  mean is -x * var in every case.
    xs = x[:, 0].astype(np.float64)
    slack = 2 * 768 * 2.0 ** -53 * xs ** 2
    assert (var <= 1e6 * (1 + 1e-6)).all()
    assert (var >= (1 - 1e-6) / np.sqrt(slack + 1e-12)).all()
    assert slack[0] < 1e-14 and abs(var[0] - 1e6) <= 1e-3 * 1e6
    assert np.allclose(mean, -xs * var.astype(np.float64), rtol=1e-6, atol=0)
    # a row with spread is untouched by the clamp
    g = np.random.default_rng(5)
    y = g.standard_normal((4, 64)).astype(np.float32)
    v, m = oracle.row_stats(y, 1e-5)
    assert np.allclose(v, 1 / np.sqrt(y.astype(np.float64).var(-1) + 1e-5), rtol=1e-5)
    assert np.allclose(m, -y.astype(np.float64).mean(-1) * v, rtol=1e-4, atol=1e-6)


def test_gemm_activation_epilogue(oracle):
    g = np.random.default_rng(2)
    A, B = _rand16(g, (8, 32)), _rand16(g, (32, 8), 0.3)
    lin = oracle.gemm(A, B).astype(np.float64)
    assert np.allclose(oracle.gemm(A, B, act="gelu_erf"), oracle.gelu(lin, "erf"), atol=1e-6)
    assert np.allclose(oracle.gemm(A, B, act="gelu_tanh"), oracle.gelu(lin, "tanh"), atol=1e-6)


# ------------------------------------------------------------- LayerNorm ----
def test_layernorm_reference_literal(oracle, literals):
    x = np.array(literals["layernorm_2x10"], np.float32).reshape(2, 10)
    # layernorm.cu feeds torch.manual_seed(42); torch.rand(1, 2, 10) printed to 4 digits
    torch.manual_seed(42)
    assert np.allclose(torch.rand(1, 2, 10).numpy()[0], x, atol=5e-5)
    got = oracle.layernorm_f32(x, 1e-5)
    want = torch.nn.functional.layer_norm(torch.tensor(x), (10,), eps=1e-5).numpy()
    assert np.allclose(got, want, atol=1e-6)


def test_layernorm_f16_matches_torch_and_invariants(oracle):
    g = np.random.default_rng(3)
    x = _rand16(g, (37, 96), 2.0) + np.float16(1.5)
    got = oracle.layernorm_f16(x, 1e-12)
    want = torch.nn.functional.layer_norm(torch.tensor(x.astype(np.float64)), (96,), eps=1e-12).numpy()
    assert np.allclose(got, want, atol=1e-5)
    assert np.abs(got.mean(-1)).max() < 1e-6
    assert np.allclose(got.var(-1), 1.0, atol=1e-5)
    const = np.full((3, 64), 0.75, np.float16)
    assert np.array_equal(oracle.layernorm_f16(const, 1e-5), np.zeros((3, 64), np.float32))
    # residual + affine superset; with gamma = 1, beta = 0, res = 0 it is the plain form bit for bit
    res, gam, bet = _rand16(g, (37, 96)), _rand16(g, (96,), 0.02) + np.float16(1), _rand16(g, (96,), 0.02)
    full = oracle.layernorm_f16(x, 1e-12, res=res, gamma=gam, beta=bet)
    s = x.astype(np.float64) + res.astype(np.float64)
    want = torch.nn.functional.layer_norm(torch.tensor(s), (96,), torch.tensor(gam.astype(np.float64)),
                                          torch.tensor(bet.astype(np.float64)), eps=1e-12).numpy()
    assert np.allclose(full, want, atol=1e-5)
    plain = oracle.layernorm_f16(x, 1e-12, res=np.zeros_like(x), gamma=np.ones(96, np.float16),
                                 beta=np.zeros(96, np.float16))
    assert np.array_equal(plain, got)


# ------------------------------------------------------------ cu_seqlens ----
def test_cu_seqlens_reference_case(oracle, literals):
    bs, seq, lens = literals["cuseqlen_bs"], literals["cuseqlen_seq"], literals["cuseqlen_lengths"]
    mask = np.array([[1 if j < lens[i % 8] else 0 for j in range(seq)] for i in range(bs)], np.int64)
    want = [0, 64, 76, 107, 139, 172, 206, 241, 277, 341, 353, 384, 416, 449, 483, 518, 554]
    assert oracle.cu_seqlens(mask).tolist() == want
    assert oracle.cu_seqlens(mask.astype(np.int32)).tolist() == want
    assert oracle.cu_seqlens(np.zeros((3, 5), np.int64)).tolist() == [0, 0, 0, 0]
    assert oracle.cu_seqlens(np.ones((3, 5), np.int64)).tolist() == [0, 5, 10, 15]


# ----------------------------------------------------------- elementwise ----
def test_elementwise_reference_literal(oracle, literals):
    a = np.array(literals["add_a_3x3x3"], np.float32).reshape(3, 3, 3)
    b = np.array(literals["add_b_3x1x3"], np.float32).reshape(3, 1, 3)
    assert np.array_equal(oracle.elementwise("add", a, b), a + b)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_elementwise_all_broadcast_patterns(oracle, dtype):
    g = np.random.default_rng(4)
    a = (g.standard_normal((3, 4, 5)) + 3).astype(dtype)
    for mask in range(8):
        shape = tuple(1 if mask >> i & 1 else a.shape[i] for i in range(3))
        b = (g.standard_normal(shape) + 3).astype(dtype)
        for op, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
            want = fn(a.astype(np.float32), b.astype(np.float32)).astype(dtype)
            assert np.array_equal(oracle.elementwise(op, a, b), want), (mask, op)


def test_gather_is_a_row_copy(oracle):
    g = np.random.default_rng(5)
    table = _rand16(g, (50, 24))
    idx = g.integers(0, 50, size=(3, 7))
    assert np.array_equal(oracle.gather(idx, table), table[idx])


# ------------------------------------------------------------- attention ----
def _sdpa(qkv, lens, heads, scale):
    bs, seq, w = qkv.shape
    d = w // (3 * heads)
    t = torch.tensor(qkv.astype(np.float64)).reshape(bs, seq, 3, heads, d)
    q, k, v = (t[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    keymask = torch.arange(seq)[None, :] < torch.tensor(lens)[:, None]
    out = torch.nn.functional.scaled_dot_product_attention(
        q, k, v, attn_mask=keymask[:, None, None, :], scale=scale)
    return out.permute(0, 2, 1, 3).reshape(bs, seq, heads * d).numpy()


def test_attention_matches_sdpa_on_valid_rows(oracle):
    g = np.random.default_rng(6)
    bs, seq, heads, d = 3, 24, 2, 8
    qkv = _rand16(g, (bs, seq, 3 * heads * d))
    lens = np.array([24, 7, 1], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    got = oracle.attention(qkv, cu, heads, 0.3)
    want = _sdpa(qkv, lens, heads, 0.3)
    for b in range(bs):
        assert np.allclose(got[b, :lens[b]], want[b, :lens[b]], atol=1e-6)
        assert not got[b, lens[b]:].any()  # padded query rows are defined as zeros


def test_attention_invariants_and_layout(oracle):
    g = np.random.default_rng(7)
    bs, seq, heads, d = 2, 16, 3, 4
    qkv = _rand16(g, (bs, seq, 3, heads, d))
    lens = np.array([16, 9], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    base = oracle.attention(qkv.reshape(bs, seq, -1), cu, heads, 0.5)
    # V constant per head -> O equals that constant (rows of P sum to 1)
    c = qkv.copy()
    c[:, :, 2, :, :] = np.float16(0.625)
    out = oracle.attention(c.reshape(bs, seq, -1), cu, heads, 0.5)
    assert np.allclose(out[0], 0.625, atol=1e-6) and np.allclose(out[1, :9], 0.625, atol=1e-6)
    # permuting the valid keys (K and V rows together) leaves O unchanged
    p = qkv.copy()
    perm = g.permutation(9)
    p[1, :9, 1:] = qkv[1, perm, 1:]
    out = oracle.attention(p.reshape(bs, seq, -1), cu, heads, 0.5)
    assert np.allclose(out[1, :9], base[1, :9], atol=1e-6)
    # masked keys do not matter
    m = qkv.copy()
    m[1, 9:, 1:] = np.float16(100.0)
    out = oracle.attention(m.reshape(bs, seq, -1), cu, heads, 0.5)
    assert np.allclose(out[1, :9], base[1, :9], atol=1e-6)
    # layout [3][heads][d]: a head whose V is one-hot in d returns that pattern
    # only in that head's slice of the output
    z = np.zeros((1, 4, 3, heads, d), np.float16)
    z[:, :, 2, 1, 2] = 1.0
    out = oracle.attention(z.reshape(1, 4, -1), np.array([0, 4], np.int32), heads, 1.0)
    want = np.zeros((1, 4, heads, d), np.float32)
    want[:, :, 1, 2] = 1.0
    assert np.array_equal(out.reshape(1, 4, heads, d), want)


# --------------------------------------------------------------- encoder ----
def _torch_encoder(h, weights, lens, layers, bs, seq, hidden, heads, ffn, gelu):
    """Independent fp64 encoder built from torch ops (post-LN, no biases)."""
    x = torch.tensor(h.astype(np.float64)).reshape(bs, seq, hidden)
    keymask = torch.arange(seq)[None, :] < torch.tensor(lens)[:, None]
    d = hidden // heads
    off = 0
    w = torch.tensor(weights.astype(np.float64))

    def take(k, n):
        nonlocal off
        m = w[off:off + k * n].reshape(k, n)
        off += k * n
        return m
    for _ in range(layers):
        wqkv, wo, w1, w2 = take(hidden, 3 * hidden), take(hidden, hidden), take(hidden, ffn), take(ffn, hidden)
        qkv = (x @ wqkv).reshape(bs, seq, 3, heads, d)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        a = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=keymask[:, None, None, :])
        a = a.permute(0, 2, 1, 3).reshape(bs, seq, hidden)
        a = a * keymask[:, :, None]  # padded query rows are zeros by definition
        x = torch.nn.functional.layer_norm(a @ wo + x, (hidden,), eps=1e-12)
        f = torch.nn.functional.gelu(x @ w1, approximate="tanh" if gelu == "tanh" else "none")
        x = torch.nn.functional.layer_norm(f @ w2 + x, (hidden,), eps=1e-12)
    return x.numpy()


@pytest.mark.parametrize("gelu", ["erf", "tanh"])
def test_encoder_composition_matches_torch(oracle, gelu):
    g = np.random.default_rng(8)
    layers, bs, seq, hidden, heads, ffn = 2, 2, 16, 32, 2, 64
    per = hidden * 3 * hidden + hidden * hidden + 2 * hidden * ffn
    weights = _rand16(g, (layers * per,), 0.1)
    h = _rand16(g, (bs * seq, hidden))
    lens = np.array([16, 5], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    want = _torch_encoder(h, weights, lens, layers, bs, seq, hidden, heads, ffn, gelu)
    # unrounded intermediates: agrees with the torch fp64 graph to fp32 precision
    pure = oracle.bert_encoder(h, weights, cu, layers, bs, seq, hidden, heads, ffn, gelu_form=gelu,
                               round_intermediates=False)
    for b in range(bs):
        assert np.abs(pure[b, :lens[b]] - want[b, :lens[b]]).max() < 2e-5
    # fp16 rounding at every stored tensor: a few 1e-3 after two layers
    out32 = oracle.bert_encoder(h, weights, cu, layers, bs, seq, hidden, heads, ffn, gelu_form=gelu)
    for b in range(bs):
        err = np.abs(out32[b, :lens[b]] - want[b, :lens[b]]).max()
        assert 1e-5 < err < 2e-2
