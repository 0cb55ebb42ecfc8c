"""Deterministic generators restated from the reference's own tests, so that
the parity tests here run on the inputs the reference's tests use."""
import numpy as np


def f16_bits(v):
    return int(np.float32(v).astype(np.float16).view(np.uint16))


def q8_0_uniform_row(value, scale, n_blocks=1):
    """src/ops/kernel/q8_0/mod.rs:64-72: every quant = value, scale f16(scale)."""
    blk = np.zeros(34, np.uint8)
    blk[0:2] = np.array([f16_bits(scale)], np.uint16).view(np.uint8)
    blk[2:] = np.uint8(np.int8(value).view(np.uint8))
    return np.tile(blk, n_blocks)


def make_q8_0_weight(n_rows, n_cols, row_offset):
    """tests/q8_0_parallel_matmul.rs:26-42."""
    nb = n_cols // 32
    r = np.arange(n_rows, dtype=np.int64)[:, None, None]
    b = np.arange(nb, dtype=np.int64)[None, :, None]
    j = np.arange(32, dtype=np.int64)[None, None, :]
    v = (row_offset + r + b + j // 4).astype(np.int8)  # `as i8` wraps
    scale = (np.float32(0.5) + np.float32(0.01) * np.arange(n_rows, dtype=np.float32)).astype(np.float16)
    w = np.empty((n_rows, nb, 34), np.uint8)
    w[:, :, 0:2] = np.broadcast_to(scale.view(np.uint8).reshape(n_rows, 1, 2), (n_rows, nb, 2))
    w[:, :, 2:] = v.view(np.uint8)
    return w.reshape(-1)


def valid_q8_weights(n_in, n_out):
    """src/ops/matmul_tests.rs:511-526."""
    nb = n_in // 32
    row = np.arange(n_out, dtype=np.int64)[:, None, None]
    blk = np.arange(nb, dtype=np.int64)[None, :, None]
    lane = np.arange(32, dtype=np.int64)[None, None, :]
    q = (((row * 17 + blk * 13 + lane * 7) % 255) - 127).astype(np.int8)
    scale = (np.float32(0.01) + (row + blk)[:, :, 0].astype(np.float32) * np.float32(0.0001)).astype(np.float16)
    w = np.empty((n_out, nb, 34), np.uint8)
    w[:, :, 0:2] = scale.view(np.uint8).reshape(n_out, nb, 2)
    w[:, :, 2:] = q.view(np.uint8)
    return w.reshape(-1)


def make_qk_weight(total_bytes, row_bytes, seed):
    """tests/fused_ffn_matmul_parity.rs:163-172: byte = seed + row + col (u8 wrap)."""
    n_rows = total_bytes // row_bytes
    r = np.arange(n_rows, dtype=np.int64)[:, None]
    j = np.arange(row_bytes, dtype=np.int64)[None, :]
    return ((seed + r + j) & 0xFF).astype(np.uint8).reshape(-1)


def ramp_input(n):
    """`(i as f32 * 0.013) - 4.0`, in f32 arithmetic."""
    return np.arange(n, dtype=np.float32) * np.float32(0.013) - np.float32(4.0)
