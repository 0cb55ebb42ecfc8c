"""Seeded synthetic tensors of the shapes and distributions the benchmark
configurations name (random Q8_0 / Q4_K weights, N(0,1) activations).

Pure numpy; the same bytes feed the GPU path, the CPU checker and the CPU
baseline.  Block layouts follow the reference's readers:
Q8_0 = [f16 d][32 x int8] (src/ops/kernel/q8_0/scalar.rs:42-48),
Q4_K = [f16 d][f16 dmin][12 B scales][128 B nibbles] (src/ops/quant/mod.rs:219-222),
Q6_K = [128 B low nibbles][64 B high bit pairs][16 x int8 scales][f16 d] (src/ops/quant/mod.rs:530-541).
"""
import numpy as np

Q8_0_BLOCK = 34
Q4_0_BLOCK = 18
Q4_K_BLOCK = 144
Q6_K_BLOCK = 210

# Qwen3-0.6B projection set: (name, n_out, n_in) per layer, then lm_head.
QWEN3_0_6B_LAYER = [
    ("attn_q", 2048, 1024),
    ("attn_k", 1024, 1024),
    ("attn_v", 1024, 1024),
    ("attn_output", 1024, 2048),
    ("ffn_gate", 3072, 1024),
    ("ffn_up", 3072, 1024),
    ("ffn_down", 1024, 3072),
]
QWEN3_0_6B_LAYERS = 28
QWEN3_0_6B_LM_HEAD = ("lm_head", 151936, 1024)


def seed_for(config_id, tensor_id):
    return 0x5EED0000 + config_id * 0x100000 + tensor_id


def q8_0_weight(seed, n_out, n_in, scale_sigma=0.02):
    """Quants uniform in [-127,127]; per-block scale f16(|N(0,sigma)|/127)."""
    rng = np.random.default_rng(seed)
    nb = n_in // 32
    w = np.empty((n_out, nb, Q8_0_BLOCK), np.uint8)
    d = (np.abs(rng.normal(0.0, scale_sigma, (n_out, nb))) / 127.0).astype(np.float16)
    w[:, :, 0:2] = d.view(np.uint8).reshape(n_out, nb, 2)
    w[:, :, 2:] = rng.integers(-127, 128, (n_out, nb, 32), dtype=np.int8).view(np.uint8)
    return w.reshape(-1)


def q4_0_weight(seed, n_out, n_in, scale_sigma=0.02):
    """Nibbles uniform in [0,15] (values -8..7); per-block scale f16(|N(0,sigma)|/8)
    (block layout: src/ops/kernel/q4_0/scalar.rs:24-47)."""
    rng = np.random.default_rng(seed)
    nb = n_in // 32
    w = rng.integers(0, 256, (n_out, nb, Q4_0_BLOCK), dtype=np.uint8)
    d = (np.abs(rng.normal(0.0, scale_sigma, (n_out, nb))) / 8.0).astype(np.float16)
    w[:, :, 0:2] = d.view(np.uint8).reshape(n_out, nb, 2)
    return w.reshape(-1)


def q4_k_weight(seed, n_out, n_in, sigma=0.01):
    """Nibbles uniform in [0,15], 12 scale bytes uniform, d/dmin f16(|N(0,sigma)|)."""
    rng = np.random.default_rng(seed)
    nb = n_in // 256
    w = rng.integers(0, 256, (n_out, nb, Q4_K_BLOCK), dtype=np.uint8)
    dd = np.abs(rng.normal(0.0, sigma, (n_out, nb, 2))).astype(np.float16)
    w[:, :, 0:4] = dd.view(np.uint8).reshape(n_out, nb, 4)
    return w.reshape(-1)


def q6_k_weight(seed, n_out, n_in, sigma=0.01):
    """6-bit quants and int8 sub-block scales uniform, d f16(|N(0,sigma)|/32)."""
    rng = np.random.default_rng(seed)
    nb = n_in // 256
    w = rng.integers(0, 256, (n_out, nb, Q6_K_BLOCK), dtype=np.uint8)
    dd = (np.abs(rng.normal(0.0, sigma, (n_out, nb, 1))) / 32.0).astype(np.float16)
    w[:, :, 208:210] = dd.view(np.uint8).reshape(n_out, nb, 2)
    return w.reshape(-1)


def activations(seed, n_tokens, n_in):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((n_tokens, n_in), dtype=np.float32)


def q8_0_weight_bytes(n_out, n_in):
    return n_out * (n_in // 32) * Q8_0_BLOCK


def q8_0_gemv_bytes(n_out, n_in, batch=1):
    """Algorithmic bytes of one Q8_0 GEMV: 34-byte source blocks, int8 + f32
    per-block-scale activations, f32 outputs."""
    return q8_0_weight_bytes(n_out, n_in) + batch * (n_in + 4 * (n_in // 32)) + batch * 4 * n_out


def q4_k_gemv_bytes(n_out, n_in, batch=1):
    return n_out * (n_in // 256) * Q4_K_BLOCK + batch * (n_in // 256) * 292 + batch * 4 * n_out


def q6_k_gemv_bytes(n_out, n_in, batch=1):
    return n_out * (n_in // 256) * Q6_K_BLOCK + batch * (n_in // 256) * 292 + batch * 4 * n_out


def q4_0_gemv_bytes(n_out, n_in, batch=1):
    return n_out * (n_in // 32) * Q4_0_BLOCK + batch * (n_in + 4 * (n_in // 32)) + batch * 4 * n_out
