"""Seeded synthetic inputs for the five benchmark configurations (numpy, PCG64).

One generator, one rule: tensor `name` of configuration `cfg` is drawn from
numpy.random.default_rng([cfg, crc32(name), index]).  Value distributions follow
the configuration text: MXFP4 nibbles uniform 0..15 with e8m0 bytes uniform
118..130, q8_0 int8 uniform -127..127 with scales |N(0, 0.02)| / 127 stored as
f16, activations N(0, 1).
"""
import zlib

import numpy as np

D_MODEL = 7168
D_INTER = 2048
VOCAB = 163840
N_EXPERTS = 256
TOP_K = 8
MLA_HEADS = 128
MLA_LATENT = 512
MLA_ROPE = 64
MLA_SCALE = float(np.float32(1.0) / np.sqrt(np.float32(192.0)))


def rng(cfg, name, index=0):
    return np.random.default_rng([cfg, zlib.crc32(name.encode()), index])


def mxfp4_matrix(cfg, name, rows, cols, index=0):
    """(packed [rows, cols/2] u8, scales [rows, cols/32] u8)."""
    g = rng(cfg, name, index)
    packed = g.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    scales = g.integers(118, 131, (rows, cols // 32), dtype=np.uint8)
    return packed, scales


def normal(cfg, name, shape, index=0):
    return rng(cfg, name, index).standard_normal(shape, dtype=np.float32)


def config0(rows=2048, cols=D_MODEL, index=0):
    """Single MXFP4 GEMV: weight + activation."""
    p, s = mxfp4_matrix(0, "w", rows, cols, index)
    return p, s, normal(0, "x", cols, index)


def config1(rows=VOCAB, cols=D_MODEL, batch=8):
    """q8_0 lm_head: int8 rows, f16 scales, `batch` activation rows."""
    g = rng(1, "w")
    q = g.integers(-127, 128, (rows, cols), dtype=np.int8)
    s = (np.abs(g.standard_normal((rows, cols // 32), dtype=np.float32)) * np.float32(0.02) / np.float32(127.0)).astype(np.float16)
    return q, s, normal(1, "x", (batch, cols))


def config2_expert(e, d=D_MODEL, inter=D_INTER):
    """Expert e of the MoE layer: (w1, w3, w2), each (packed, scales); e == N_EXPERTS is the shared expert."""
    return (mxfp4_matrix(2, "w1", inter, d, e), mxfp4_matrix(2, "w3", inter, d, e), mxfp4_matrix(2, "w2", d, inter, e))


def config2_tokens(batch, d=D_MODEL, n_experts=N_EXPERTS):
    """(router logits [B, n_experts], hidden [B, d])."""
    return normal(2, "logits", (batch, n_experts), batch), normal(2, "hidden", (batch, d), batch)


def config3_raw(ctx, L=MLA_LATENT, R=MLA_ROPE, nh=MLA_HEADS):
    """(latent [ctx, L], rope [ctx, R], query [nh, L+R]) before quantization."""
    return normal(3, "latent", (ctx, L), ctx), normal(3, "rope", (ctx, R), ctx), normal(3, "q", (nh, L + R), ctx)


def q8_0_rows(x):
    """q8_0 of the rows of x with the reference rule (src/q8.rs:57-68: dx = max/127 in f32, q = roundf(x / dx) clamped
    to +-127, zero block -> scale 0), scales stored as f16.  The f32 quotient is rounded half away from zero in f64,
    where |r| + 0.5 is exact, so that r = 0.49999997 gives 0 as roundf does."""
    x = np.ascontiguousarray(x, np.float32)
    n, w = x.shape
    b = x.reshape(n, w // 32, 32)
    dx = (np.abs(b).max(axis=2) / np.float32(127.0)).astype(np.float32)
    safe = np.where(dx == 0, np.float32(1), dx)
    r = (b / safe[..., None]).astype(np.float32).astype(np.float64)
    q = np.clip(np.sign(r) * np.floor(np.abs(r) + 0.5), -127, 127)
    q = np.where(dx[..., None] == 0, 0, q).astype(np.int8).reshape(n, w)
    return q, dx.astype(np.float16)


def config4_tokens(n_tokens=512, d=D_MODEL, n_experts=N_EXPERTS):
    """(router logits [T, n_experts], activations [T, d] rounded to bf16 values)."""
    logits = normal(4, "logits", (n_tokens, n_experts))
    x = normal(4, "x", (n_tokens, d))
    xb = (x.view(np.uint32) + 0x7FFF + ((x.view(np.uint32) >> 16) & 1)) & 0xFFFF0000  # round to nearest even bf16
    return logits, xb.astype(np.uint32).view(np.float32)
