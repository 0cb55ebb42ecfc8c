"""Pins the CPU checker's Q6_K functions: the reference's known-answer vector,
its two statements of the element layout against each other, integer sums by
brute force, f64 dequantised dots, and the intrinsics twin.  CPU only."""
import numpy as np
import pytest

import gen
from conftest import bits

S, A = 0, 1


def _elements(blk):
    """Independent numpy statement of the 256 signed 6-bit values of one super-block
    (the aux8 unpack of src/ops/quant/mod.rs:653-673)."""
    ql, qh = blk[0:128].astype(np.int64), blk[128:192].astype(np.int64)
    a = np.zeros(256, np.int64)
    for j in range(2):
        lo0, lo1, h = ql[64 * j:64 * j + 32], ql[64 * j + 32:64 * j + 64], qh[32 * j:32 * j + 32]
        a[128 * j + 0:128 * j + 32] = ((lo0 & 0xF) | ((h & 3) << 4)) - 32
        a[128 * j + 32:128 * j + 64] = ((lo1 & 0xF) | (((h >> 2) & 3) << 4)) - 32
        a[128 * j + 64:128 * j + 96] = ((lo0 >> 4) | (((h >> 4) & 3) << 4)) - 32
        a[128 * j + 96:128 * j + 128] = ((lo1 >> 4) | (((h >> 6) & 3) << 4)) - 32
    return a


def _dequant_f64(row, nb):
    out = np.zeros(nb * 256)
    for b in range(nb):
        blk = row[b * 210:(b + 1) * 210]
        d = float(blk[208:210].copy().view(np.float16)[0])
        sc = blk[192:208].view(np.int8).astype(np.float64)
        out[b * 256:(b + 1) * 256] = d * np.repeat(sc, 16) * _elements(blk)
    return out


def test_q6_k_kernel_multiplies_uniform_block(oracle):
    """tests/quantized_inference.rs:252-263: ql 0x11, qh 0xaa, scales 1, d 1.0, x = 1 -> 256."""
    w = np.full(210, 0x11, np.uint8)
    w[128:192] = 0xAA
    w[192:208] = 1
    w[208:210] = np.array([gen.f16_bits(1.0)], np.uint16).view(np.uint8)
    out = np.zeros(1, np.float32)
    oracle.q6k_forward_prequantized(w, np.ones(256, np.uint8), np.ones(8, np.float32), out, 256, 1)
    assert out[0] == 256.0
    assert np.array_equal(oracle.dequantize_row_q6_k(w, 256), np.ones(256, np.float32))
    d, qs, bs = oracle.quantize_row_q8_k(np.ones(256, np.float32), S)
    for variant in (S, A):
        assert abs(oracle.vec_dot_q6k_q8k(w, d, qs, bs, variant) - 256.0) < 1e-3


def test_dequantize_row_q6_k_layout(oracle, rmi):
    """The row decoder (src/ops/quant/mod.rs:530-569) against the dot's own unpack (:653-673),
    on the byte pattern of tests/quantized_inference.rs:132-139 and on random blocks."""
    rows = ((np.arange(420) * 37 + 11) & 0xFF).astype(np.uint8)
    rows[208:210] = np.array([gen.f16_bits(0.03125)], np.uint16).view(np.uint8)
    rows[418:420] = np.array([gen.f16_bits(-0.0625)], np.uint16).view(np.uint8)
    got = oracle.dequantize_row_q6_k(rows, 512)
    want = _dequant_f64(rows, 2)
    assert np.array_equal(got.astype(np.float64), want)  # d is a power of two: every product is exact
    w = rmi.synth.q6_k_weight(3, 4, 512).reshape(4, -1)
    for r in range(4):
        assert np.allclose(oracle.dequantize_row_q6_k(w[r], 512), _dequant_f64(w[r], 2), rtol=3e-7, atol=0)


def test_q6k_ints_by_brute_force(oracle, rmi):
    rng = np.random.default_rng(8)
    row = rmi.synth.q6_k_weight(9, 1, 1024)
    x = rng.standard_normal(1024).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    isum = oracle.q6k_q8k_block_ints(row, qs)
    lanes = oracle.q6k_q8k_lane_ints(row, qs, bs)
    for b in range(4):
        blk = row[b * 210:(b + 1) * 210]
        el = _elements(blk)
        sc = np.repeat(blk[192:208].view(np.int8).astype(np.int64), 16)
        q8 = qs[b * 256:(b + 1) * 256].astype(np.int64)
        assert isum[b] == int((sc * el * q8).sum())
        # lane m of the AVX2 kernel: unsigned quants of elements 4m..4m+3 of every 32-group,
        # minus 32 * the two (bsums x scale) products 2m, 2m+1 (src/ops/quant/mod.rs:996-1055)
        u = el + 32
        s16 = blk[192:208].view(np.int8).astype(np.int64)
        b16 = bs[b * 16:(b + 1) * 16].astype(np.int64)
        for m in range(8):
            idx = (np.arange(8)[:, None] * 32 + 4 * m + np.arange(4)[None, :]).reshape(-1)
            want = int((sc[idx] * u[idx] * q8[idx]).sum()) - 32 * int(b16[2 * m] * s16[2 * m] + b16[2 * m + 1] * s16[2 * m + 1])
            assert lanes[b, m] == want
        assert int(lanes[b].sum()) == isum[b]


@pytest.mark.parametrize("variant", [S, A])
def test_vec_dot_q6k_q8k_against_f64(oracle, rmi, variant):
    rng = np.random.default_rng(10)
    n_in = 2048
    w = rmi.synth.q6_k_weight(11, 8, n_in).reshape(8, -1)
    x = rng.standard_normal(n_in).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, variant)
    xd = qs.astype(np.float64) * np.repeat(d.astype(np.float64), 256)
    for r in range(8):
        y = oracle.vec_dot_q6k_q8k(w[r], d, qs, bs, variant)
        wd = _dequant_f64(w[r], n_in // 256)
        assert abs(y - wd @ xd) <= 2e-6 * (np.abs(wd) @ np.abs(xd))
        isum = oracle.q6k_q8k_block_ints(w[r], qs)
        dd = w[r].reshape(-1, 210)[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
        assert abs(y - float((dd * isum * d.astype(np.float64)).sum())) <= 2e-6 * (np.abs(wd) @ np.abs(xd))


def test_q6k_avx2_order_matches_twin_and_scalar_tolerance(oracle, rmi):
    """src/ops/quant/mod.rs:1165-1211: AVX2 vs scalar within rel 1e-3; the plain-C
    AVX2 order equals the kernel written with the reference's intrinsics bit for bit."""
    rng = np.random.default_rng(12)
    n_in = 3584
    w = rmi.synth.q6_k_weight(13, 16, n_in).reshape(16, -1)
    x = rng.standard_normal(n_in).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    for r in range(16):
        ya = oracle.vec_dot_q6k_q8k(w[r], d, qs, bs, A)
        ys = oracle.vec_dot_q6k_q8k(w[r], d, qs, bs, S)
        assert abs(ya - ys) <= 1e-3 * max(abs(ys), 1.0)
        if oracle.have_avx2():
            yt = oracle.x86_vec_dot_q6k_q8k(w[r], d, qs, bs)
            assert bits(np.array([ya]))[0] == bits(np.array([yt]))[0]


def test_q6k_twin_on_reference_inputs(oracle):
    """Inputs of src/ops/quant/mod.rs:1165-1211 (one block and four blocks) and the byte
    pattern of tests/quantized_inference.rs:213-231; the emulation equals the intrinsics."""
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")

    def blk(ql, qh, scales, d):
        v = np.zeros(210, np.uint8)
        v[0:128], v[128:192] = ql, qh
        v[192:208] = np.array(scales, np.int8).view(np.uint8)
        v[208:210] = np.array([gen.f16_bits(d)], np.uint16).view(np.uint8)
        return v

    cases = []
    w1 = blk([i % 4 for i in range(128)], [i * 5 % 4 for i in range(64)], [i - 4 for i in range(16)], 0.5)
    cases.append((w1, np.array([(i - 128.0) * 0.01 for i in range(256)], np.float32)))
    w4 = np.concatenate([blk([(i * 11 + j * 3) % 4 for j in range(128)], [(i + j * 7) % 4 for j in range(64)],
                             [i * 5 + k - 6 for k in range(16)], np.float32(0.01) + np.float32(i) * np.float32(0.1))
                         for i in range(4)])
    cases.append((w4, np.array([(i - 512.0) * 0.01 for i in range(1024)], np.float32)))
    w = ((np.arange(210) * 17 + 3) & 0xFF).astype(np.uint8)
    w[208:210] = np.array([gen.f16_bits(0.015625)], np.uint16).view(np.uint8)
    cases.append((w, np.array([((i % 19) - 9) / 5.0 for i in range(256)], np.float32)))
    for w, x in cases:
        d, qs, bs = oracle.quantize_row_q8_k(x, A)
        a = np.array([oracle.vec_dot_q6k_q8k(w, d, qs, bs, A)], np.float32)
        t = np.array([oracle.x86_vec_dot_q6k_q8k(w, d, qs, bs)], np.float32)
        s = oracle.vec_dot_q6k_q8k(w, d, qs, bs, S)
        assert bits(a)[0] == bits(t)[0]
        assert abs(a[0] - s) <= 1e-3 * max(abs(s), 1e-3)


def test_q6k_partition_and_fusion_bit_exact(oracle):
    """tests/fused_ffn_matmul_parity.rs:232-300, 296-299 (Q6_K case, n_in 1024, rows cut to 448 per side)."""
    n_in, n_per = 1024, 448
    row_bytes = n_in // 256 * 210
    gate = gen.make_qk_weight(n_per * row_bytes, row_bytes, 0)
    up = gen.make_qk_weight(n_per * row_bytes, row_bytes, 17)
    d, qs, bs = oracle.quantize_row_q8_k(gen.ramp_input(n_in), S)

    def run(w, rows, nth):
        out = np.zeros(rows, np.float32)
        for ith in range(nth):
            oracle.q6k_forward_prepared(w, d, qs, bs, out, n_in, rows, ith, nth, S)
        return out

    def same(a, b):
        return np.array_equal(bits(a)[~np.isnan(a)], bits(b)[~np.isnan(b)]) and np.array_equal(np.isnan(a), np.isnan(b))

    g1, u1 = run(gate, n_per, 1), run(up, n_per, 1)
    assert same(g1, run(gate, n_per, 8)) and same(u1, run(up, n_per, 5))
    fused, rows = oracle.fuse_vstack(gate, n_per, up, n_per)
    f8 = run(fused, rows, 8)
    assert same(f8[:n_per], g1) and same(f8[n_per:], u1)


def test_q6k_dequant_path_against_f64(oracle, rmi):
    rng = np.random.default_rng(14)
    n_in, n_out = 2048, 12
    w = rmi.synth.q6_k_weight(15, n_out, n_in)
    x = rng.standard_normal(n_in).astype(np.float32)
    q8, sc = oracle.quantize_q8_0(x, A)
    out = np.zeros(n_out, np.float32)
    oracle.q6k_forward_prequantized(w, q8, sc, out, n_in, n_out)
    xq = q8.view(np.int8).astype(np.float64) * np.repeat(sc.astype(np.float64), 32)
    for r in range(n_out):
        wd = _dequant_f64(w.reshape(n_out, -1)[r], n_in // 256)
        assert abs(out[r] - wd @ xq) <= 1e-5 * (np.abs(wd) @ np.abs(xq))
    part = np.zeros(n_out, np.float32)
    oracle.q6k_forward_prequantized(w, q8, sc, part, n_in, n_out, 1, 4)
    assert np.array_equal(bits(part[3:6]), bits(out[3:6])) and not part[:3].any() and not part[6:].any()
