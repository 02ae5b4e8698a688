"""Seeded synthetic inputs for the benchmark / parity configurations.

Config numbering follows the workload list: 1 GEMM+bias+GELU (FFN1 shape),
2 residual add + layer norm, 3 packed-QKV attention, 4 BERT-base encoder,
5 BERT-large encoder and the skinny split-K GEMM.  Every tensor comes from
numpy's PCG64 seeded with SEED_BASE + config, drawn in the order listed, in
fp32 and then rounded to fp16 (round to nearest even).
"""
import numpy as np

SEED_BASE = 0x484F4D00


def rng(config):
    return np.random.Generator(np.random.PCG64(SEED_BASE + config))


def normal16(g, shape, std=1.0, mean=0.0):
    return (g.standard_normal(shape, dtype=np.float32) * std + mean).astype(np.float16)


def gemm_bias_gelu(M=1024, K=768, N=3072, config=1):
    g = rng(config)
    return {"A": normal16(g, (1, M, K)), "B": normal16(g, (1, K, N), 0.02),
            "bias": normal16(g, (1, 1, N), 0.02)}


def add_layernorm(rows=1024, hidden=768, config=2):
    g = rng(config)
    return {"x": normal16(g, (rows, hidden)), "res": normal16(g, (rows, hidden)),
            "gamma": normal16(g, (hidden,), 0.02, 1.0), "beta": normal16(g, (hidden,), 0.02),
            "eps": 1e-12}


def seq_lengths(g, bs, seq, lo=32):
    lo = min(lo, seq)
    return g.integers(lo, seq + 1, size=bs).astype(np.int32)


def mask_from_lengths(lens, seq):
    return (np.arange(seq)[None, :] < np.asarray(lens)[:, None]).astype(np.int64)


def attention(bs=8, seq=128, heads=12, d=64, config=3):
    g = rng(config)
    qkv = normal16(g, (bs, seq, 3 * heads * d))
    lens = seq_lengths(g, bs, seq)
    return {"qkv": qkv, "lens": lens, "mask": mask_from_lengths(lens, seq),
            "scale": 1.0 / np.sqrt(d), "heads": heads}


def bert_encoder(layers=12, hidden=768, heads=12, ffn=3072, bs=8, seq=128, vocab=30522,
                 config=4):
    """Random-init encoder: W ~ N(0, 0.02) fp16, [K, N] row-major per GEMM."""
    g = rng(config)
    weights = []
    for _ in range(layers):
        weights.append({
            "wqkv": normal16(g, (hidden, 3 * hidden), 0.02),
            "wo": normal16(g, (hidden, hidden), 0.02),
            "w1": normal16(g, (hidden, ffn), 0.02),
            "w2": normal16(g, (ffn, hidden), 0.02),
        })
    word = normal16(g, (vocab, hidden), 0.02)
    pos_type = normal16(g, (seq, hidden), 0.02)
    ids = g.integers(0, vocab, size=(bs, seq)).astype(np.int64)
    lens = seq_lengths(g, bs, seq)
    # masked-LM head: transform dense [H, H]; the decoder is tied to `word` (drawn last so that the
    # tensors above do not depend on it)
    w_transform = normal16(g, (hidden, hidden), 0.02)
    return {"weights": weights, "word": word, "pos_type": pos_type, "ids": ids, "lens": lens,
            "w_transform": w_transform,
            "mask": mask_from_lengths(lens, seq),
            "dims": dict(layers=layers, hidden=hidden, heads=heads, ffn=ffn, bs=bs, seq=seq,
                         vocab=vocab)}


def skinny_gemm(M=64, K=4096, N=1024, config=5):
    g = rng(config)
    return {"A": normal16(g, (1, M, K)), "B": normal16(g, (1, K, N), 0.02)}
