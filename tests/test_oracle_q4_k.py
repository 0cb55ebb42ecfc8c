"""Pins the CPU checker's Q8_K / Q4_K functions: reference known-answer vectors,
the reference's two scale-unpack formulations against each other, integer sums
by brute force, f64 dequantised dots, and the intrinsics twin.  CPU only."""
import numpy as np
import pytest

import gen
from conftest import bits

S, A = 0, 1


def _synth(rmi):
    return rmi.synth


def test_block_sizes():
    """src/core/tensor.rs:61-87: (32,34), (256,144), (256,292)."""
    assert 2 + 32 == 34 and 2 + 2 + 12 + 128 == 144 and 4 + 256 + 16 * 2 == 292


@pytest.mark.parametrize("variant", [S, A])
def test_q8_k_quantizer_uses_nearest_even_rounding(oracle, variant):
    """tests/quantized_inference.rs:170-186."""
    x = np.zeros(256, np.float32)
    x[:5] = [-127.0, 0.5, 1.5, 2.5, -0.5]
    d, qs, bs = oracle.quantize_row_q8_k(x, variant)
    assert list(qs[:5]) == [-127, 0, 2, 2, 0]
    assert d[0] == np.float32(1.0)


@pytest.mark.parametrize("variant", [S, A])
def test_q8_k_quantizer_returns_one_complete_block(oracle, variant):
    """tests/quantized_inference.rs:152-168."""
    x = np.array([(i - 127) * 0.03125 for i in range(256)], np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, variant)
    assert d.size == 1 and int(bs.astype(np.int32).sum()) == int(qs.astype(np.int32).sum())
    assert np.array_equal(bs, qs.astype(np.int32).reshape(16, 16).sum(axis=1).astype(np.int16))


def test_q8_k_scalar_avx2_and_twin_agree(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(256 * 64) * rng.choice([1e-4, 1.0, 300.0], 256 * 64)).astype(np.float32)
    x[:256] = 0
    x[256:512] = -x[256:512].__abs__()  # negative extreme element
    ds, qs, bs = oracle.quantize_row_q8_k(x, S)
    da, qa, ba = oracle.quantize_row_q8_k(x, A)
    assert np.array_equal(bits(ds), bits(da)) and np.array_equal(qs, qa) and np.array_equal(bs, ba)
    assert ds[0] == 0 and not qs[:256].any()
    # largest-magnitude element maps to -127 and d reproduces it
    blk = x[256:512]
    k = np.argmax(np.abs(blk))
    assert qs[256 + k] == -127 and np.isclose(ds[1] * -127, blk[k], rtol=1e-6)
    if oracle.have_avx2():
        dt, qt, bt = oracle.x86_quantize_row_q8_k(x)
        assert np.array_equal(bits(dt), bits(da)) and np.array_equal(qt, qa) and np.array_equal(bt, ba)


def test_scale_min_k4_equals_kmask_unpack(oracle):
    """src/ops/quant/mod.rs:25-33 against :237-258, two formulations of one unpack."""
    rng = np.random.default_rng(6)
    cases = [rng.integers(0, 256, 12, dtype=np.uint8) for _ in range(2000)]
    cases += [np.full(12, v, np.uint8) for v in (0, 0xFF, 0x3F, 0xC0, 0x0F, 0xF0)]
    for s in cases:
        u = oracle.unpack_scales_kmask(s)
        for j in range(8):
            sc, mn = oracle.get_scale_min_k4(j, s)
            assert (sc, mn) == (int(u[j]), int(u[8 + j])) and sc < 64 and mn < 64


def _dequant_f64(row, nb):
    """Independent numpy statement of the Q4_K element formula (f64)."""
    out = np.zeros(nb * 256)
    for b in range(nb):
        blk = row[b * 144:(b + 1) * 144]
        d = float(blk[0:2].copy().view(np.float16)[0])
        dmin = float(blk[2:4].copy().view(np.float16)[0])
        s = blk[4:16].astype(np.int64)
        q = blk[16:144]
        for j in range(8):
            if j < 4:
                sc, mn = s[j] & 63, s[j + 4] & 63
            else:
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            nib = q[(j // 2) * 32:(j // 2) * 32 + 32]
            v = (nib & 0xF) if j % 2 == 0 else (nib >> 4)
            out[b * 256 + j * 32:b * 256 + j * 32 + 32] = d * sc * v.astype(np.float64) - dmin * mn
    return out


def test_dequantize_row_q4_k(oracle, rmi):
    w = rmi.synth.q4_k_weight(7, 3, 512).reshape(3, -1)
    for r in range(3):
        got = oracle.dequantize_row_q4_k(w[r], 512)
        want = _dequant_f64(w[r], 2)
        assert np.allclose(got, want, rtol=3e-7, atol=1e-9)


def test_q4_k_kernel_multiplies_uniform_block(oracle):
    """tests/quantized_inference.rs:233-249: d=1, dmin=0, scales -> 1, nibbles 0x11, x=1 -> 256."""
    w = np.zeros(144, np.uint8)
    w[0:2] = np.array([gen.f16_bits(1.0)], np.uint16).view(np.uint8)
    w[4:16] = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
    w[16:] = 0x11
    out = np.zeros(1, np.float32)
    oracle.q4k_forward_prequantized(w, np.ones(256, np.uint8), np.ones(8, np.float32), out, 256, 1)
    assert out[0] == 256.0
    assert oracle.quantized_linear_forward(w, np.ones(256, np.float32), 256, 1)[0] == 256.0
    # the integer path on the same block: x = 1.0 quantises to -(-127)... d*q = 1
    d, qs, bs = oracle.quantize_row_q8_k(np.ones(256, np.float32), S)
    for variant in (S, A):
        y = oracle.vec_dot_q4k_q8k(w, d, qs, bs, variant)
        assert abs(y - 256.0) < 1e-3


def test_q4k_block_ints_by_brute_force(oracle, rmi):
    rng = np.random.default_rng(8)
    row = rmi.synth.q4_k_weight(9, 1, 1024)
    x = rng.standard_normal(1024).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    isum, msum = oracle.q4k_q8k_block_ints(row, qs, bs)
    for b in range(4):
        blk = row[b * 144:(b + 1) * 144]
        u = oracle.unpack_scales_kmask(blk[4:16]).astype(np.int64)
        q = blk[16:144].astype(np.int64)
        el = np.zeros(256, np.int64)
        for g in range(4):
            el[64 * g:64 * g + 32] = q[32 * g:32 * g + 32] & 0xF
            el[64 * g + 32:64 * g + 64] = q[32 * g:32 * g + 32] >> 4
        q8 = qs[b * 256:(b + 1) * 256].astype(np.int64)
        want_i = sum(int(u[j]) * int((el[32 * j:32 * j + 32] * q8[32 * j:32 * j + 32]).sum()) for j in range(8))
        want_m = sum(int(u[8 + j]) * int(q8[32 * j:32 * j + 32].sum()) for j in range(8))
        assert isum[b] == want_i and msum[b] == want_m


@pytest.mark.parametrize("variant", [S, A])
def test_vec_dot_q4k_q8k_against_f64_and_ints(oracle, rmi, variant):
    rng = np.random.default_rng(10)
    n_in = 2048
    w = rmi.synth.q4_k_weight(11, 8, n_in).reshape(8, -1)
    x = rng.standard_normal(n_in).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, variant)
    xd = qs.astype(np.float64) * np.repeat(d.astype(np.float64), 256)
    for r in range(8):
        y = oracle.vec_dot_q4k_q8k(w[r], d, qs, bs, variant)
        wd = _dequant_f64(w[r], n_in // 256)
        want = wd @ xd
        assert abs(y - want) <= 2e-6 * (np.abs(wd) @ np.abs(xd))
        # same number rebuilt from the exact per-block integers
        isum, msum = oracle.q4k_q8k_block_ints(w[r], qs, bs)
        blocks = w[r].reshape(-1, 144)
        dd = blocks[:, 0:2].copy().view(np.float16).astype(np.float64)[:, 0]
        dm = blocks[:, 2:4].copy().view(np.float16).astype(np.float64)[:, 0]
        rebuilt = float(((dd * isum - dm * msum) * d.astype(np.float64)).sum())
        assert abs(y - rebuilt) <= 2e-6 * (np.abs(wd) @ np.abs(xd))


def test_q4k_avx2_emulation_matches_twin_and_scalar_tolerance(oracle, rmi):
    """src/ops/quant/mod.rs:1112-1162: AVX2 vs scalar within rel 1e-3."""
    rng = np.random.default_rng(12)
    n_in = 6144
    w = rmi.synth.q4_k_weight(13, 16, n_in).reshape(16, -1)
    x = rng.standard_normal(n_in).astype(np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    for r in range(16):
        ya = oracle.vec_dot_q4k_q8k(w[r], d, qs, bs, A)
        ys = oracle.vec_dot_q4k_q8k(w[r], d, qs, bs, S)
        assert abs(ya - ys) <= 1e-3 * max(abs(ys), 1.0)
        if oracle.have_avx2():
            yt = oracle.x86_vec_dot_q4k_q8k(w[r], d, qs, bs)
            assert bits(np.array([ya]))[0] == bits(np.array([yt]))[0]


def test_q4k_twin_on_reference_byte_pattern(oracle):
    """Weight bytes of tests/quantized_inference.rs:188-198 (index*29+7) and of
    make_qk_weight; d/dmin may decode to inf/nan there, so compare bit patterns."""
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    w = ((np.arange(144) * 29 + 7) & 0xFF).astype(np.uint8)
    x = np.array([((i % 23) - 11) / 7.0 for i in range(256)], np.float32)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    a = np.array([oracle.vec_dot_q4k_q8k(w, d, qs, bs, A)], np.float32)
    t = np.array([oracle.x86_vec_dot_q4k_q8k(w, d, qs, bs)], np.float32)
    assert (np.isnan(a[0]) and np.isnan(t[0])) or bits(a)[0] == bits(t)[0]


def test_kk_partition_and_fusion_bit_exact(oracle):
    """tests/fused_ffn_matmul_parity.rs:232-300 (Q4_K case, rows cut to 512 per side)."""
    n_in, n_per = 1024, 512
    nb = n_in // 256
    row_bytes = nb * 144
    gate = gen.make_qk_weight(n_per * row_bytes, row_bytes, 0)
    up = gen.make_qk_weight(n_per * row_bytes, row_bytes, 17)
    d, qs, bs = oracle.quantize_row_q8_k(gen.ramp_input(n_in), S)

    def run(w, rows, nth):
        out = np.zeros(rows, np.float32)
        for ith in range(nth):
            oracle.q4k_forward_prepared(w, d, qs, bs, out, n_in, rows, ith, nth, S)
        return out

    def same(a, b):
        return np.array_equal(bits(a)[~np.isnan(a)], bits(b)[~np.isnan(b)]) and np.array_equal(np.isnan(a), np.isnan(b))

    g1, u1 = run(gate, n_per, 1), run(up, n_per, 1)
    assert same(g1, run(gate, n_per, 8)) and same(u1, run(up, n_per, 8))
    fused, rows = oracle.fuse_vstack(gate, n_per, up, n_per)
    f8 = run(fused, rows, 8)
    assert same(f8[:n_per], g1) and same(f8[n_per:], u1)


def test_dequant_path_against_f64(oracle, rmi):
    rng = np.random.default_rng(14)
    n_in, n_out = 2048, 12
    w = rmi.synth.q4_k_weight(15, n_out, n_in)
    x = rng.standard_normal(n_in).astype(np.float32)
    y = oracle.quantized_linear_forward(w, x, n_in, n_out)
    q8, sc = oracle.quantize_q8_0(x, A)
    out = np.zeros(n_out, np.float32)
    oracle.q4k_forward_prequantized(w, q8, sc, out, n_in, n_out)
    xq = q8.view(np.int8).astype(np.float64) * np.repeat(sc.astype(np.float64), 32)
    for r in range(n_out):
        wd = _dequant_f64(w.reshape(n_out, -1)[r], n_in // 256)
        assert abs(y[r] - wd @ x.astype(np.float64)) <= 1e-5 * (np.abs(wd) @ np.abs(x))
        assert abs(out[r] - wd @ xq) <= 1e-5 * (np.abs(wd) @ np.abs(xq))
    # row partition writes only its slice
    part = np.zeros(n_out, np.float32)
    oracle.q4k_forward_prequantized(w, q8, sc, part, n_in, n_out, 1, 4)
    assert np.array_equal(bits(part[3:6]), bits(out[3:6])) and not part[:3].any() and not part[6:].any()


def test_block_ints_matrix_is_the_per_row_function_row_by_row(oracle):
    rng = np.random.default_rng(77)
    n_out, n_in = 9, 768
    w = rng.integers(0, 256, n_out * (n_in // 256) * 144, dtype=np.uint8)
    qs = rng.integers(-127, 128, n_in, dtype=np.int8)
    bs = qs.reshape(-1, 16).astype(np.int32).sum(axis=1).astype(np.int16)
    ints = oracle.q4k_q8k_block_ints_matrix(w, n_out, qs, bs)
    wr = w.reshape(n_out, -1)
    for r in range(n_out):
        isum, msum = oracle.q4k_q8k_block_ints(wr[r], qs, bs)
        assert np.array_equal(ints[r, :, 0], isum) and np.array_equal(ints[r, :, 1], msum)
