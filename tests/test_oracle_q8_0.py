"""Pins the CPU checker's Q8_0 functions against the known-answer vectors the
reference's own tests hold and against independent formulations (numpy.float16,
brute-force integer dots, f64 dequantised dots, the intrinsics twin).  CPU only."""
import numpy as np
import pytest

import gen
from conftest import bits

S, A, N = 0, 1, 2  # SCALAR, AVX2, NEON


# ---------------------------------------------------------------- f16

def test_f16_to_f32_all_patterns(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(b)) for b in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])


def test_f32_to_f16_round_to_nearest_even(oracle):
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-8, 2.9802322e-8, 2.98023224e-8 * 1.0001,
                  6.1035156e-5, 6.0975552e-5, np.inf, -np.inf, 1.0, 1.00048828125, 1.0009765625, 1.00146484375],
                 np.float32),
        # exact ties between adjacent f16 values
        (np.arange(1024, 3000, dtype=np.uint16).view(np.float16).astype(np.float32)
         + np.arange(1025, 3001, dtype=np.uint16).view(np.float16).astype(np.float32)) / np.float32(2),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(v) for v in vals], np.uint16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------ quantizer

def test_q8_quantization_stores_f16_scale_without_requantizing_values(oracle):
    """src/ops/matmul_tests.rs:558-571 (arch independent: holds for every variant)."""
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    x[1] = np.array([0x3D11213E], np.uint32).view(np.float32)[0]
    for variant in (S, A, N):
        q8, sc = oracle.quantize_q8_0(x, variant)
        assert q8.view(np.int8)[0] == 127 and q8.view(np.int8)[1] == 4
        assert int(bits(sc)[0]) == 0x3C010000


def test_scalar_quantizer_rounds_half_away(oracle):
    """tests/quantized_inference.rs:57-66."""
    x = np.zeros(32, np.float32)
    x[:3] = [127.0, 0.5, -0.5]
    q8, _ = oracle.quantize_q8_0(x, S)
    assert list(q8.view(np.int8)[:3]) == [127, 1, -1]


def test_simd_quantizers_round_ties_to_even(oracle):
    """src/ops/matmul_tests.rs:546-556 (NEON); the AVX2 variant uses the same rule."""
    x = np.zeros(32, np.float32)
    x[0], x[1] = 127.0, 34.5
    for variant in (A, N):
        q8, _ = oracle.quantize_q8_0(x, variant)
        assert q8.view(np.int8)[1] == 34
    q8, _ = oracle.quantize_q8_0(x, S)
    assert q8.view(np.int8)[1] == 35


def test_neon_quantization_matches_scalar_on_reference_input(oracle):
    """src/ops/matmul_tests.rs:528-544."""
    x = np.array([((i % 17) - 8) * 0.125 for i in range(64)], np.float32)
    qs, ss = oracle.quantize_q8_0(x, S)
    qn, sn = oracle.quantize_q8_0(x, N)
    assert np.array_equal(qs, qn) and np.array_equal(bits(ss), bits(sn))


def test_quantizer_zero_block_and_dequant_error(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(4096).astype(np.float32)
    x[64:96] = 0.0
    for variant in (S, A, N):
        q8, sc = oracle.quantize_q8_0(x, variant)
        assert sc[2] == 0.0 and not q8[64:96].any()
        deq = q8.view(np.int8).astype(np.float32) * np.repeat(sc, 32)
        amax = np.abs(x.reshape(-1, 32)).max(axis=1)
        # half a quantisation step plus the f16 rounding of the scale
        assert np.all(np.abs(deq - x).reshape(-1, 32).max(axis=1) <= amax / 127 * 0.5 + amax * 2.0 ** -11 + 1e-12)


def test_avx2_quantizer_twin_matches_emulation(oracle):
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(32 * 2000) * rng.choice([1e-3, 1.0, 50.0], 32 * 2000)).astype(np.float32)
    x[:32] = 0
    x[32:64] = np.arange(32) + 0.5  # many exact ties
    q1, s1 = oracle.quantize_q8_0(x, A)
    q2, s2 = oracle.x86_quantize_q8_0(x)
    assert np.array_equal(q1, q2) and np.array_equal(bits(s1), bits(s2))


# ----------------------------------------------------------------- GEMV

@pytest.mark.parametrize("variant", [S, A, N])
def test_q8_kernel_closed_forms(oracle, variant):
    """src/ops/kernel/q8_0/mod.rs:74-156."""
    ones_q = np.ones(32, np.uint8)
    one_s = np.ones(1, np.float32)
    w = gen.q8_0_uniform_row(1, 1.0)
    assert list(oracle.matmul_q8_0_quantized(w, ones_q, one_s, 32, 1, variant)) == [32.0]
    w2 = np.concatenate([w, w])
    assert list(oracle.matmul_q8_0_quantized(w2, ones_q, one_s, 32, 2, variant)) == [32.0, 32.0]
    assert list(oracle.matmul_q8_0_quantized(gen.q8_0_uniform_row(1, 0.5), ones_q, one_s, 32, 1, variant)) == [16.0]
    w4 = np.tile(w, 4)
    out_a = np.zeros(4, np.float32)
    oracle.matmul_q8_0_quantized_parallel_rows(w4, ones_q, one_s, out_a, 32, 4, 0, 2, variant)
    out_b = np.zeros(4, np.float32)
    oracle.matmul_q8_0_quantized_parallel_rows(w4, ones_q, one_s, out_b, 32, 4, 1, 2, variant)
    assert list(out_a) == [32.0, 32.0, 0.0, 0.0] and list(out_b) == [0.0, 0.0, 32.0, 32.0]


@pytest.mark.parametrize("variant", [S, A, N])
def test_forward_with_f32_ones(oracle, variant):
    """src/app/embedding.rs:817-835: f16(1/127) * 127 * 32 = 31.998047."""
    w = gen.q8_0_uniform_row(1, 1.0)
    y = oracle.q8_0_forward_batched(w, np.ones(32, np.float32), 32, 1, variant)
    assert y[0, 0] == np.float32(31.998047)


def test_neon_order_bit_pin(oracle):
    """src/ops/matmul_tests.rs:288-306: sum = fma(dot, wd*s, sum) gives 0x3d1cc57d."""
    blk = np.zeros(34, np.uint8)
    blk[0:2] = np.array([0x1800], np.uint16).view(np.uint8)
    blk[2] = 127
    w = np.concatenate([blk, blk])
    q8 = np.zeros(64, np.uint8)
    q8[0] = np.int8(-127).view(np.uint8)
    q8[32] = 127
    sc = np.array([oracle.f16_to_f32(0x1800), oracle.f16_to_f32(0x1A7D)], np.float32)
    y = oracle.matmul_q8_0_quantized(w, q8, sc, 64, 1, N)
    assert int(bits(y)[0]) == 0x3D1CC57D
    # the unfused scalar order rounds the second product first and lands elsewhere
    # or on the same bits; both must stay within one ulp of the fused result
    ys = oracle.matmul_q8_0_quantized(w, q8, sc, 64, 1, S)
    assert abs(int(bits(ys)[0]) - 0x3D1CC57D) <= 1


def test_q8_0_quantize_and_matmul_256_ones(oracle):
    """src/models/qwen35.rs:1134-1152."""
    rows = []
    for v in (1, -2):
        blk = np.zeros(34, np.uint8)
        blk[0:2] = [0x00, 0x3C]
        blk[2:] = np.int8(v).view(np.uint8)
        rows.append(np.tile(blk, 8))
    w = np.concatenate(rows)
    for variant in (S, A, N):
        y = oracle.q8_0_forward_batched(w, np.ones(256, np.float32), 256, 2, variant)[0]
        assert abs(y[0] - 256.0) < 0.05 and abs(y[1] + 512.0) < 0.05


def _random_case(seed, n_out, n_in, rmi_synth=None):
    rng = np.random.default_rng(seed)
    nb = n_in // 32
    w = np.empty((n_out, nb, 34), np.uint8)
    w[:, :, 0:2] = (np.abs(rng.normal(0, 0.02, (n_out, nb))) / 127).astype(np.float16).view(np.uint8).reshape(n_out, nb, 2)
    w[:, :, 2:] = rng.integers(-127, 128, (n_out, nb, 32), dtype=np.int8).view(np.uint8)
    x = rng.standard_normal(n_in).astype(np.float32)
    return w.reshape(-1), x


def _dequant_f64(w, n_out, n_in):
    blocks = w.reshape(n_out, n_in // 32, 34)
    d = blocks[:, :, 0:2].copy().view(np.float16).astype(np.float64)
    q = blocks[:, :, 2:].view(np.int8).astype(np.float64)
    return (q * d).reshape(n_out, n_in)


def test_block_dots_are_plain_int32_sums(oracle):
    w, x = _random_case(11, 64, 256)
    q8, _ = oracle.quantize_q8_0(x, A)
    got = oracle.block_dots_q8_0(w, q8, 256, 64)
    qw = w.reshape(64, 8, 34)[:, :, 2:].view(np.int8).astype(np.int64)
    qx = q8.view(np.int8).astype(np.int64).reshape(8, 32)
    want = np.einsum("rbk,bk->rb", qw, qx)
    assert np.array_equal(got, want.astype(np.int32))


@pytest.mark.parametrize("variant", [S, A, N])
def test_gemv_against_f64_dequantised_dot(oracle, variant):
    n_out, n_in = 96, 1024
    w, x = _random_case(12, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x, variant)
    y = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, variant)
    xd = q8.view(np.int8).astype(np.float64) * np.repeat(sc.astype(np.float64), 32)
    want = _dequant_f64(w, n_out, n_in) @ xd
    terms = np.abs(_dequant_f64(w, n_out, n_in)) @ np.abs(xd)
    assert np.all(np.abs(y - want) <= 1e-6 * terms)


def test_three_orders_agree_within_reference_tolerance(oracle):
    """src/bin/micro_bench.rs:112-120: tol = 1e-4 + 1e-4*|ref|."""
    n_out, n_in = 128, 3072
    w, x = _random_case(13, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x, A)
    ys = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, S)
    for variant in (A, N):
        yv = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, variant)
        assert np.all(np.abs(yv - ys) <= 1e-4 + 1e-4 * np.abs(ys))


def test_avx2_order_emulation_matches_intrinsics_twin(oracle):
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    for seed, n_out, n_in in [(20, 131, 1024), (21, 7, 3072), (22, 64, 32)]:
        w, x = _random_case(seed, n_out, n_in)
        q8, sc = oracle.quantize_q8_0(x, A)
        a = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
        b = oracle.x86_matmul_q8_0_range(w, q8, sc, n_in, 0, n_out)
        assert np.array_equal(bits(a), bits(b))
        # tile rows and tail rows take different code in the twin: a shifted range
        # moves every row to another tile slot and must not change a bit
        c = oracle.x86_matmul_q8_0_range(w, q8, sc, n_in, 1, n_out)
        assert np.array_equal(bits(a[1:]), bits(c))
    # extreme quants, including the -128 weight the sign trick must survive
    w = gen.valid_q8_weights(256, 16).copy()
    w.reshape(16, 8, 34)[3, 2, 2:] = np.int8(-128).view(np.uint8)
    q8 = np.full(256, 127, np.uint8)
    sc = np.full(8, 0.25, np.float32)
    assert np.array_equal(bits(oracle.matmul_q8_0_quantized(w, q8, sc, 256, 16, A)),
                          bits(oracle.x86_matmul_q8_0_range(w, q8, sc, 256, 0, 16)))


@pytest.mark.parametrize("n_threads", [1, 2, 4, 8])
def test_parallel_rows_match_single_thread_bit_exact(oracle, n_threads):
    """tests/q8_0_parallel_matmul.rs:82-145 (n_out 7168 shortened rows kept: 1024 cols)."""
    n_in, n_out = 1024, 7168
    w = gen.make_q8_0_weight(n_out, n_in, 7)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    out = np.zeros(n_out, np.float32)
    for ith in range(n_threads):
        oracle.matmul_q8_0_quantized_parallel_rows(w, q8, sc, out, n_in, n_out, ith, n_threads, A)
    assert np.array_equal(bits(out), bits(ref))


def test_fused_vstack_equals_separate(oracle):
    """tests/fused_ffn_matmul_parity.rs:92-127, src/ops/quant/fuse.rs:102-184."""
    n_in, n_per = 1024, 3584
    gate = gen.make_q8_0_weight(n_per, n_in, 0)
    up = gen.make_q8_0_weight(n_per, n_in, 17)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    fused, rows = oracle.fuse_vstack(gate, n_per, up, n_per)
    assert rows == 2 * n_per and np.array_equal(fused, np.concatenate([gate, up]))
    yf = oracle.matmul_q8_0_quantized(fused, q8, sc, n_in, rows, A)
    assert np.array_equal(bits(yf[:n_per]), bits(oracle.matmul_q8_0_quantized(gate, q8, sc, n_in, n_per, A)))
    assert np.array_equal(bits(yf[n_per:]), bits(oracle.matmul_q8_0_quantized(up, q8, sc, n_in, n_per, A)))
    # mismatched row byte lengths -> None
    assert oracle.fuse_vstack(gate[: 34 * 32], 1, up[: 34 * 16], 1) is None


def test_pool_matches_single_thread(oracle):
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    n_in, n_out = 1024, 3001
    w, x = _random_case(30, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x, A)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    pool = oracle.Pool(4)
    out = np.zeros(n_out, np.float32)
    for _ in range(3):
        out[:] = 0
        pool.matmul_q8_0(w, q8, sc, out, n_in, n_out)
        assert np.array_equal(bits(out), bits(ref))
    pool.close()


def test_legacy_f32_matmul_against_f64(oracle):
    """`ops::matmul_q8_0` (f32 activations, no activation quantisation)."""
    n_out, n_in = 64, 512
    w, x = _random_case(31, n_out, n_in)
    want = _dequant_f64(w, n_out, n_in) @ x.astype(np.float64)
    terms = np.abs(_dequant_f64(w, n_out, n_in)) @ np.abs(x.astype(np.float64))
    for variant in (S, A):
        y = oracle.matmul_q8_0_f32(w, x, n_in, n_out, variant)
        assert np.all(np.abs(y - want) <= 2e-6 * terms)


def test_expf_restatement_equals_host_libm(oracle):
    """The formula the GPU kernels use for exp (glibc's expf, FMA build) against this host's expf: every 64th
    float bit pattern (67 M inputs, all exponents, both signs, NaN/inf) plus the dense range softmax and
    SiLU live in.  On all 2^32 patterns the count is 0 as well (a minute of CPU time, not run here)."""
    assert oracle.lib.rmi_ref_expf_mismatches(0, 64, 1 << 26) == 0
    lo = int(np.float32(-20.0).view(np.uint32))
    assert oracle.lib.rmi_ref_expf_mismatches(lo - (1 << 22), 1, 1 << 22) == 0   # (-20, -10]
    assert oracle.lib.rmi_ref_expf_mismatches(int(np.float32(1.0).view(np.uint32)), 1, 1 << 22) == 0  # [1, 1.5)
    assert oracle.expf_restated(0.0) == 1.0 and oracle.expf_restated(-np.inf) == 0.0
    assert np.isnan(oracle.expf_restated(np.nan)) and oracle.expf_restated(89.0) == np.inf


def test_neon_split_chain_is_the_neon_chain_for_one_part_and_within_tolerance_for_more(oracle):
    """The checker's statement of the split-K GEMM: one run is the aarch64 chain bit for bit; several runs stay
    within the reference's tolerance of every reference order and differ from the single chain somewhere (the
    split is real)."""
    n_out, n_in = 64, 3072
    w = gen.q8_0_weight(4242, n_out, n_in) if hasattr(gen, "q8_0_weight") else None
    if w is None:
        rng = np.random.default_rng(4242)
        blocks = np.zeros((n_out * n_in // 32, 34), np.uint8)
        blocks[:, :2] = (np.abs(rng.normal(0, 0.02, (n_out * n_in // 32, 1))) / 127).astype(np.float16).view(np.uint8).reshape(-1, 2)
        blocks[:, 2:] = rng.integers(-127, 128, (n_out * n_in // 32, 32), dtype=np.int8).view(np.uint8)
        w = blocks.reshape(-1)
    x = np.random.default_rng(4243).normal(0, 1, n_in).astype(np.float32)
    q8, sc = oracle.quantize_q8_0(x, oracle.AVX2)
    neon = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, oracle.NEON)
    assert np.array_equal(bits(oracle.matmul_q8_0_neon_split(w, q8, sc, n_in, n_out, 24)), bits(neon))
    avx2 = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, oracle.AVX2)
    differs = False
    for per in (1, 2, 3, 5, 12, 23):
        y = oracle.matmul_q8_0_neon_split(w, q8, sc, n_in, n_out, per)
        for ref in (neon, avx2):
            assert np.all(np.abs(y - ref) <= 1e-4 + 1e-4 * np.abs(ref))
        differs |= not np.array_equal(bits(y), bits(neon))
    assert differs
    assert np.array_equal(bits(oracle.matmul_q8_0_neon_interleaved(w, q8, sc, n_in, n_out, 1)), bits(neon))
    for groups in (2, 4):
        y = oracle.matmul_q8_0_neon_interleaved(w, q8, sc, n_in, n_out, groups)
        for ref in (neon, avx2):
            assert np.all(np.abs(y - ref) <= 1e-4 + 1e-4 * np.abs(ref))
        assert not np.array_equal(bits(y), bits(neon))
