"""GPU parity of the Q8_0 path, through the C ABI, against the CPU checker.

Bars: per-block int32 dots bit-exact; GEMV f32 bit-exact against the restated
x86-64 production kernel (AVX2 order); MFMA GEMM f32 bit-exact against the
restated fused sequential (NEON) order and within 1e-4 + 1e-4*|ref| of the AVX2
order (the reference's own cross-backend tolerance, src/bin/micro_bench.rs:112-120).
"""
import threading

import numpy as np
import pytest

import gen
from conftest import bits

pytestmark = pytest.mark.gpu

S, A, N = 0, 1, 2
TOL = lambda ref: 1e-4 + 1e-4 * np.abs(ref)  # noqa: E731


def _case(rmi, seed, n_out, n_in, n_tokens=1):
    w = rmi.synth.q8_0_weight(seed, n_out, n_in)
    x = rmi.synth.activations(seed + 1, n_tokens, n_in)
    return w, x


def _quantize_rows(oracle, x, variant=A):
    q8 = np.zeros(x.shape, np.uint8)
    sc = np.zeros((x.shape[0], x.shape[1] // 32), np.float32)
    for t in range(x.shape[0]):
        q8[t], sc[t] = oracle.quantize_q8_0(x[t], variant)
    return q8, sc


# ------------------------------------------------------------ reference's unit tests

def test_q8_kernel_closed_forms(hip):
    """src/ops/kernel/q8_0/mod.rs:74-156, through the mirrored Kernel interface."""
    K = hip.kernel
    ones_q, one_s = np.ones(32, np.uint8), np.ones(1, np.float32)
    out = np.zeros(1, np.float32)
    K.Q8Kernel(gen.q8_0_uniform_row(1, 1.0), 32, 1).forward_prequantized(ones_q, one_s, out, 32, 1, 0, 1)
    assert list(out) == [32.0]
    out = np.zeros(2, np.float32)
    K.Q8Kernel(np.tile(gen.q8_0_uniform_row(1, 1.0), 2), 32, 2).forward_prequantized(ones_q, one_s, out, 32, 2, 0, 1)
    assert list(out) == [32.0, 32.0]
    out = np.zeros(1, np.float32)
    K.Q8Kernel(gen.q8_0_uniform_row(1, 0.5), 32, 1).forward_prequantized(ones_q, one_s, out, 32, 1, 0, 1)
    assert list(out) == [16.0]
    out = np.zeros(1, np.float32)
    K.Q8Kernel(gen.q8_0_uniform_row(1, 1.0), 32, 1).forward(np.ones(32, np.float32), out, 32, 1)
    assert abs(out[0] - 32.0) < 5e-3 and out[0] == np.float32(31.998047)  # src/app/embedding.rs:817-835
    kernel = K.Q8Kernel(np.tile(gen.q8_0_uniform_row(1, 1.0), 4), 32, 4)
    out_a, out_b = np.zeros(4, np.float32), np.zeros(4, np.float32)
    kernel.forward_prequantized(ones_q, one_s, out_a, 32, 4, 0, 2)
    kernel.forward_prequantized(ones_q, one_s, out_b, 32, 4, 1, 2)
    assert list(out_a) == [32.0, 32.0, 0.0, 0.0] and list(out_b) == [0.0, 0.0, 32.0, 32.0]


def test_q8_0_256_ones(hip):
    """src/models/qwen35.rs:1134-1152."""
    rows = []
    for v in (1, -2):
        blk = np.zeros(34, np.uint8)
        blk[0:2] = [0x00, 0x3C]
        blk[2:] = np.int8(v).view(np.uint8)
        rows.append(np.tile(blk, 8))
    out = np.zeros(2, np.float32)
    hip.kernel.Q8Kernel(np.concatenate(rows), 256, 2).forward(np.ones(256, np.float32), out, 256, 2)
    assert abs(out[0] - 256.0) < 0.05 and abs(out[1] + 512.0) < 0.05


# ------------------------------------------------------------------ integer dots

@pytest.mark.parametrize("n_out,n_in", [(3072, 1024), (1, 32), (13, 96), (5, 160), (64, 2048), (9, 288)])
def test_block_dots_bit_exact(hip, oracle, n_out, n_in):
    w, x = _case(hip, 100 + n_out, n_out, n_in)
    q8, _ = oracle.quantize_q8_0(x[0], A)
    got = hip.kernel.Q8Kernel(w, n_in, n_out).block_dots(q8)
    assert np.array_equal(got, oracle.block_dots_q8_0(w, q8, n_in, n_out))


def test_block_dots_extreme_quants(hip, oracle):
    """+-127/-128 everywhere: the largest dots the format can hold."""
    n_out, n_in = 16, 256
    w = gen.valid_q8_weights(n_in, n_out).copy()
    w.reshape(n_out, 8, 34)[::2, :, 2:] = np.int8(-128).view(np.uint8)
    w.reshape(n_out, 8, 34)[1::2, :, 2:] = 127
    q8 = np.full(n_in, 127, np.uint8)
    q8[::3] = np.int8(-128).view(np.uint8)
    assert np.array_equal(hip.kernel.Q8Kernel(w, n_in, n_out).block_dots(q8), oracle.block_dots_q8_0(w, q8, n_in, n_out))


def test_activation_quants_of_minus_128_follow_the_exact_integer_dot(hip, oracle):
    """Prequantized input that holds -128: the device sums the exact products (the scalar kernel,
    src/ops/kernel/q8_0/scalar.rs:49-53).  The x86-64 kernel negates the activation byte where the weight is
    negative, which wraps -(-128) to -128, and saturates pair sums to i16 (avx2.rs:128-147): it is wrong on every
    row that meets such a quant with a negative weight, and the device does not follow it there."""
    n_out, n_in = 16, 64
    w = hip.synth.q8_0_weight(431, n_out, n_in).reshape(n_out, 2, 34).copy()
    hot = [(0, 0), (0, 1), (1, 7)]  # (block, element) of the activation quants set to -128
    for b, k in hot:
        w[2:8, b, 2 + k] = np.abs(w[2:8, b, 2 + k].view(np.int8)).view(np.uint8)  # rows 2..7: weights >= 0 there
    w[0, 0, 2:4] = 0x80      # row 0: a -128 weight pair against the -128 activation pair
    w[1, 1, 2 + 7] = 0x85    # row 1: one negative weight against a -128
    w = np.ascontiguousarray(w).reshape(-1)
    q8 = np.random.default_rng(432).integers(-127, 128, n_in, dtype=np.int8)
    for b, k in hot:
        q8[32 * b + k] = -128
    sc = np.array([0.5, 0.25], np.float32)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    dots = kernel.block_dots(q8.view(np.uint8))
    assert np.array_equal(dots, oracle.block_dots_q8_0(w, q8.view(np.uint8), n_in, n_out))
    wq = w.reshape(n_out, 2, 34)[:, :, 2:].view(np.int8).astype(np.int64)
    assert np.array_equal(dots, np.einsum("rbk,bk->rb", wq, q8.reshape(2, 32).astype(np.int64)))
    out = np.zeros(n_out, np.float32)
    kernel.forward_prequantized(q8.view(np.uint8), sc, out, n_in, n_out, 0, 1)
    ref_s = oracle.matmul_q8_0_quantized(w, q8.view(np.uint8), sc, n_in, n_out, S)
    ref_a = oracle.matmul_q8_0_quantized(w, q8.view(np.uint8), sc, n_in, n_out, A)
    assert np.all(np.abs(out - ref_s) <= TOL(ref_s))
    assert np.array_equal(bits(out[2:8]), bits(ref_a[2:8]))  # no negative weight meets a -128: the x86-64 bits
    assert not np.all(np.abs(ref_a[:2] - ref_s[:2]) <= TOL(ref_s[:2]))  # the x86-64 kernel is off on rows 0, 1


# ------------------------------------------------------------------------- GEMV

QWEN_SHAPES = [(3072, 1024), (2048, 1024), (1024, 1024), (1024, 2048), (1024, 3072)]


@pytest.mark.parametrize("n_out,n_in", QWEN_SHAPES + [(1, 32), (7, 64), (13, 96), (100, 160), (33, 4096), (8, 8192)])
def test_gemv_bit_exact_vs_avx2_order(hip, oracle, n_out, n_in):
    w, x = _case(hip, 200 + n_out + n_in, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x[0], A)
    out = np.zeros(n_out, np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    assert np.array_equal(bits(out), bits(ref))
    # and within the stated tolerance of the other two reference kernels
    for variant in (S, N):
        other = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, variant)
        assert np.all(np.abs(out - other) <= TOL(other))


def test_gemv_lm_head_rows(hip, oracle):
    """151936 x 1024 (tied lm_head): checker on a strided sample of rows, all rows
    by the linearity-free invariant that a row's bits do not depend on its tile."""
    n_out, n_in = 151936, 1024
    w, x = _case(hip, 300, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x[0], A)
    out = np.zeros(n_out, np.float32)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    kernel.forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
    wr = w.reshape(n_out, -1)
    rows = np.unique(np.concatenate([np.arange(0, n_out, 997), np.arange(n_out - 64, n_out), np.arange(64)]))
    ref = oracle.matmul_q8_0_quantized(np.ascontiguousarray(wr[rows]).reshape(-1), q8, sc, n_in, rows.size, A)
    assert np.array_equal(bits(out[rows]), bits(ref))
    # a second pass over a shifted row range must reproduce every row bit for bit
    part = np.zeros(n_out - 3, np.float32)
    kernel.matmul_q8_0_quantized_range(q8, sc, part, n_in, 3, n_out)
    assert np.array_equal(bits(part), bits(out[3:]))


def test_gemv_reference_generators(hip, oracle):
    """Inputs of tests/q8_0_parallel_matmul.rs (large magnitudes, y ~ 1e5)."""
    n_in, n_out = 1024, 7168
    w = gen.make_q8_0_weight(n_out, n_in, 7)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    out = np.zeros(n_out, np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
    assert np.array_equal(bits(out), bits(oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)))


def test_gemv_tiny_and_huge_scales(hip, oracle):
    """f16 subnormal weight scales, f32 products far below the f16 range, and large ones."""
    n_out, n_in = 24, 512
    w = hip.synth.q8_0_weight(400, n_out, n_in).reshape(n_out, -1, 34).copy()
    w[:8, :, 0:2] = np.array([0x0001, 0x03FF, 0x0400, 0x8001] * 4, np.uint16).view(np.uint8).reshape(16, 2)
    w[8:16, :, 0:2] = np.array([0x7BFF], np.uint16).view(np.uint8)
    w = w.reshape(-1)
    q8 = np.random.default_rng(401).integers(-127, 128, n_in, dtype=np.int8).view(np.uint8)
    for s in (1e-30, 6e-8, 1.0, 3e4):
        sc = np.full(n_in // 32, s, np.float32)
        out = np.zeros(n_out, np.float32)
        hip.kernel.Q8Kernel(w, n_in, n_out).forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
        ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
        assert np.array_equal(bits(out), bits(ref)), s


@pytest.mark.parametrize("n_tokens", [2, 3, 4, 5, 7, 8])
def test_gemv_batched_tiny_and_huge_scales(hip, oracle, n_tokens):
    """Several tokens a launch share their scale products between lanes: weight scales that are zero, f16
    subnormals, the largest f16, inf and NaN against token scales from f32 subnormals to large, a different one per
    token and block, must give the single-token kernel's bits for every token."""
    n_out, n_in = 8 * 5 + 3, 768
    rng = np.random.default_rng(4100 + n_tokens)
    w = hip.synth.q8_0_weight(410, n_out, n_in).reshape(n_out, -1, 34).copy()
    special = np.array([0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x8001, 0x7BFF, 0xFBFF, 0x7C00, 0x7E00], np.uint16)
    pick = special[rng.integers(0, special.size, (n_out, n_in // 32))]
    keep = rng.random((n_out, n_in // 32)) < 0.6
    own = w[:, :, :2].copy().view(np.uint16)[:, :, 0]
    w[:, :, :2] = np.where(keep, own, pick).astype(np.uint16)[:, :, None].view(np.uint8)
    w = np.ascontiguousarray(w).reshape(-1)
    q8 = rng.integers(-127, 128, (n_tokens, n_in), dtype=np.int8)
    sc = rng.choice(np.array([0.0, 1e-41, 1e-30, 6e-8, 1.0, 3e4, 2e38], np.float32), (n_tokens, n_in // 32)).astype(np.float32)
    H = hip.hip
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    d_q8, d_sc = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)
    d_y = H.DeviceBuffer(n_tokens * n_out * 4)
    H.check(H.lib.rmi_hip_gemv_q8_0_dev(kernel.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, n_out, 0, n_out, None))
    H.check(H.lib.rmi_hip_synchronize())
    out = d_y.to_array(np.float32, (n_tokens, n_out))
    with np.errstate(all="ignore"):
        ref = np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, A) for t in range(n_tokens)])
    nan_o, nan_r = np.isnan(out), np.isnan(ref)
    assert np.array_equal(nan_o, nan_r) and nan_r.any() and not nan_r.all()
    assert np.array_equal(bits(out)[~nan_o], bits(ref)[~nan_r])
    # products below the normal range were exercised
    wd = np.where(keep, own, pick).astype(np.uint16).view(np.float16).astype(np.float32)
    with np.errstate(all="ignore"):
        prod = wd[:, None, :] * sc[None, :, :]
    assert np.count_nonzero((prod != 0) & (np.abs(prod) < 1.17549435e-38)) > 100


@pytest.mark.parametrize("n_out,n_in", [(1021, 2048), (517, 3072), (40, 1984), (99, 2944), (8, 1824), (3, 2848), (2048, 3072), (2056, 2048)])
def test_gemv_with_a_tile_on_four_waves(hip, oracle, n_out, n_in):
    """Rows of 8 or 12 octets (1793 to 2048 and 2817 to 3072 elements) in matrices of up to 256 tiles: a tile's
    octets are multiplied by four waves and summed in block order by the first (the last shape is one tile beyond).  Row lengths that end inside the
    last octet, row counts that end inside a tile, and (ith, nth) slices that begin and end inside tiles."""
    w, x = _case(hip, 900 + n_out + n_in, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x[0], A)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    out = np.zeros(n_out, np.float32)
    kernel.forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
    assert np.array_equal(bits(out), bits(ref))
    nth = 3
    for ith in range(nth):
        single = np.full(n_out, -1.0, np.float32)
        kernel.forward_prequantized(q8, sc, single, n_in, n_out, ith, nth)
        per = -(-n_out // nth)
        lo, hi = min(ith * per, n_out), min(ith * per + per, n_out)
        assert np.all(single[:lo] == -1.0) and np.all(single[hi:] == -1.0)
        assert np.array_equal(bits(single[lo:hi]), bits(ref[lo:hi]))


@pytest.mark.parametrize("nth", [1, 2, 3, 4, 8, 16])
def test_thread_partition_bit_exact(hip, oracle, nth):
    """tests/q8_0_parallel_matmul.rs:82-145: every (ith, nth) slice of the full output."""
    n_in, n_out = 1024, 3584
    w = gen.make_q8_0_weight(n_out, n_in, 7)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    out = np.zeros(n_out, np.float32)
    for ith in range(nth):
        single = np.full(n_out, -1.0, np.float32)
        kernel.forward_prequantized(q8, sc, single, n_in, n_out, ith, nth)
        per = -(-n_out // nth)
        lo, hi = min(ith * per, n_out), min(ith * per + per, n_out)
        assert np.all(single[:lo] == -1.0) and np.all(single[hi:] == -1.0)  # writes only its slice
        out[lo:hi] = single[lo:hi]
    assert np.array_equal(bits(out), bits(ref))


def test_concurrent_pool_threads(hip, oracle):
    """Kernel is Send + Sync: 8 host threads call with the same full output at once."""
    n_in, n_out, nth = 1024, 7168, 8
    w = gen.make_q8_0_weight(n_out, n_in, 7)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, A)
    for _ in range(3):
        out = np.zeros(n_out, np.float32)
        errs = []

        def work(ith):
            try:
                kernel.forward_prequantized(q8, sc, out, n_in, n_out, ith, nth)
            except Exception as e:  # pragma: no cover
                errs.append(e)

        threads = [threading.Thread(target=work, args=(i,)) for i in range(nth)]
        [t.start() for t in threads]
        [t.join() for t in threads]
        assert not errs and np.array_equal(bits(out), bits(ref))


def test_pre_sliced_range_convention(hip, oracle):
    """dispatch.rs:36: output[0] is row_start."""
    n_in, n_out = 2048, 100
    w, x = _case(hip, 500, n_out, n_in)
    q8, sc = oracle.quantize_q8_0(x[0], A)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    for lo, hi in [(0, 100), (3, 50), (8, 16), (97, 100), (41, 42), (7, 7)]:
        out = np.zeros(hi - lo, np.float32)
        kernel.matmul_q8_0_quantized_range(q8, sc, out, n_in, lo, hi)
        assert np.array_equal(bits(out), bits(oracle.matmul_q8_0_quantized_range(w, q8, sc, n_in, lo, hi, A)))


def test_fused_vstack_matches_separate(hip, oracle):
    """tests/fused_ffn_matmul_parity.rs:92-127 (gate offset 0, up offset 17), plus ragged row counts."""
    K = hip.kernel
    n_in = 1024
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    for n_a, n_b in [(3584, 3584), (13, 5), (8, 3), (1, 1)]:
        gate, up = gen.make_q8_0_weight(n_a, n_in, 0), gen.make_q8_0_weight(n_b, n_in, 17)
        kg, ku = K.Q8Kernel(gate, n_in, n_a), K.Q8Kernel(up, n_in, n_b)
        fused = K.fuse_vstack(kg, ku)
        assert fused is not None and fused.w.n_out == n_a + n_b
        of = np.zeros(n_a + n_b, np.float32)
        fused.forward_prequantized(q8, sc, of, n_in, n_a + n_b, 0, 1)
        og, ou = np.zeros(n_a, np.float32), np.zeros(n_b, np.float32)
        kg.forward_prequantized(q8, sc, og, n_in, n_a, 0, 1)
        ku.forward_prequantized(q8, sc, ou, n_in, n_b, 0, 1)
        assert np.array_equal(bits(of[:n_a]), bits(og)) and np.array_equal(bits(of[n_a:]), bits(ou))
        ref, rows = oracle.fuse_vstack(gate, n_a, up, n_b)
        assert np.array_equal(bits(of), bits(oracle.matmul_q8_0_quantized(ref, q8, sc, n_in, rows, A)))
    # different n_in -> None, as the reference
    assert K.fuse_vstack(K.Q8Kernel(gen.make_q8_0_weight(4, 64, 0), 64, 4),
                         K.Q8Kernel(gen.make_q8_0_weight(4, 32, 0), 32, 4)) is None


# -------------------------------------------------------------------- quantizer

@pytest.mark.parametrize("rounding,variant", [(1, A), (0, S), (2, N)])
def test_device_quantizer_bit_exact(hip, oracle, rounding, variant):
    rng = np.random.default_rng(600)
    x = (rng.standard_normal(32 * 4096) * rng.choice([1e-6, 1e-3, 1.0, 50.0, 3e4], 32 * 4096)).astype(np.float32)
    x[:32] = 0
    x[32:64] = np.arange(32) + 0.5
    x[64:96] = -(np.arange(32) + 0.5)
    x[96:128] = 1e-41  # f32 subnormals
    x[128] = 127.0
    x[129] = 34.5
    q8, sc = hip.kernel.quantize_q8_0(x, x.size, rounding)
    rq, rs = oracle.quantize_q8_0(x, variant)
    assert np.array_equal(q8, rq) and np.array_equal(bits(sc), bits(rs))


def test_device_quantizer_reference_kats(hip):
    """src/ops/matmul_tests.rs:558-571 and :546-556, tests/quantized_inference.rs:57-66."""
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    x[1] = np.array([0x3D11213E], np.uint32).view(np.float32)[0]
    for rounding in (0, 1, 2):
        q8, sc = hip.kernel.quantize_q8_0(x, 32, rounding)
        assert list(q8.view(np.int8)[:2]) == [127, 4] and int(bits(sc)[0]) == 0x3C010000
    x = np.zeros(32, np.float32)
    x[:3] = [127.0, 0.5, -0.5]
    assert list(hip.kernel.quantize_q8_0(x, 32, 0)[0].view(np.int8)[:3]) == [127, 1, -1]
    x[1] = 34.5
    assert hip.kernel.quantize_q8_0(x, 32, 1)[0].view(np.int8)[1] == 34
    assert hip.kernel.quantize_q8_0(x, 32, 2)[0].view(np.int8)[1] == 34  # src/ops/matmul_tests.rs:546-556
    # src/ops/matmul_tests.rs:528-544: the NEON quantizer equals the scalar one on this input
    x = np.array([((i % 17) - 8) * 0.125 for i in range(64)], np.float32)
    qs, ss = hip.kernel.quantize_q8_0(x, 64, 0)
    qn, sn = hip.kernel.quantize_q8_0(x, 64, 2)
    assert np.array_equal(qs, qn) and np.array_equal(bits(ss), bits(sn))


def test_device_quantizer_neon_clamps_and_non_finite(hip, oracle):
    """The aarch64 quantizer never emits -128 and turns a block with a NaN or an infinity into zeros (vmaxq hands
    the NaN on, 1/scale becomes 0 or the product NaN, vcvtnq of NaN is 0); the x86-64 one can emit -128."""
    x = hip.synth.activations(5, 1, 32 * 64)[0]
    x[40] = np.nan
    x[70] = np.inf
    x[100] = -np.inf
    q8, sc = hip.kernel.quantize_q8_0(x, x.size, 2)
    rq, rs = oracle.quantize_q8_0(x, N)
    assert np.array_equal(q8, rq)
    ok = np.isfinite(rs)
    assert np.array_equal(bits(sc)[ok], bits(rs)[ok]) and np.array_equal(np.isnan(sc), np.isnan(rs))
    assert not q8[32:64].any() and not q8[64:128].any() and np.isnan(sc[1]) and np.isinf(sc[2])
    assert q8.view(np.int8).min() >= -127
    assert hip.hip.lib.rmi_hip_quantize_q8_0(hip.hip.ptr(x, hip.hip._f32p), 32, hip.hip.ptr(q8, hip.hip._u8p),
                                             hip.hip.ptr(sc, hip.hip._f32p), 7) == -1


# ------------------------------------------------------------- batches and GEMM

@pytest.mark.parametrize("n_tokens", [1, 2, 3, 5, 8, 11])
def test_prequantized_batch_bit_exact(hip, oracle, n_tokens):
    n_out, n_in = 1024, 3072
    w, x = _case(hip, 700 + n_tokens, n_out, n_in, n_tokens)
    q8, sc = _quantize_rows(oracle, x)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).matmul_q8_0_quantized_batch(q8, sc, out, n_in, n_out, n_tokens)
    for t in range(n_tokens):
        assert np.array_equal(bits(out[t]), bits(oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, A))), t


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(4, 1030, 1024), (5, 77, 2048), (6, 264, 3072), (7, 8, 6144), (8, 515, 6144),
                                                  (8, 9, 7168), (5, 130, 7168), (4, 136, 7424), (8, 520, 1056)])
def test_batches_of_four_to_eight_on_both_kernels(hip, oracle, n_tokens, n_out, n_in):
    """From four tokens on the x86-64-order GEMV computes its 4-byte dots on the matrix cores; rows too long for that
    kernel's LDS staging (7168 and 7424 elements here) keep the kernel with the dots on the vector ALU.  Both against
    the checker's AVX2 order, every row and token, with row counts that are not multiples of eight and a row length
    that is not a whole octet (1056)."""
    w, x = _case(hip, 7700 + n_tokens + n_in, n_out, n_in, n_tokens)
    q8, sc = _quantize_rows(oracle, x)
    out = np.full((n_tokens, n_out), np.nan, np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).matmul_q8_0_quantized_batch(q8, sc, out, n_in, n_out, n_tokens)
    for t in range(n_tokens):
        assert np.array_equal(bits(out[t]), bits(oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, A))), t


@pytest.mark.parametrize("n_tokens", [1, 4, 8])
def test_forward_batched_small_is_gemv_order(hip, oracle, n_tokens):
    """Kernel::forward_batched up to 8 tokens: device quantizer + GEMV in the AVX2 order, bit-exact."""
    n_out, n_in = 512, 1024
    w, x = _case(hip, 800 + n_tokens, n_out, n_in, n_tokens)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out)
    assert np.array_equal(bits(out), bits(oracle.q8_0_forward_batched(w, x, n_in, n_out, A)))


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(64, 3072, 1024), (64, 1024, 3072), (512, 256, 1024), (16, 32, 32),
                                                  (37, 45, 96), (100, 1000, 160), (65, 33, 2048)])
def test_gemm_mfma_parity(hip, oracle, n_tokens, n_out, n_in):
    """Prefill GEMM = n_tokens independent GEMVs (trait_.rs:78-109).  Bit-exact against
    the fused sequential (NEON) order; within tolerance of the x86-64 (AVX2) order."""
    w, x = _case(hip, 900 + n_tokens + n_out, n_out, n_in, n_tokens)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out, matrix_cores=True)
    q8, sc = _quantize_rows(oracle, x)
    ref_n = np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, N) for t in range(n_tokens)])
    assert np.array_equal(bits(out), bits(ref_n))
    ref_a = oracle.q8_0_forward_batched(w, x, n_in, n_out, A)
    assert np.all(np.abs(out - ref_a) <= TOL(ref_a))


@pytest.mark.parametrize("f16_token_scales", [False, True])
def test_gemm_special_scales(hip, oracle, f16_token_scales):
    """Weight scales that are zero, negative zero, f16 subnormals, the largest f16, inf and NaN, against token
    scales down to f32 subnormals (the f32 outer product on the matrix cores) or token scales that are f16 values,
    as every quantizer of the reference writes them, down to f16 subnormals (the f16 one): either way the scale
    products must round like the f32 multiply."""
    n_tokens, n_out, n_in = 96, 160, 320
    rng = np.random.default_rng(77)
    w = hip.synth.q8_0_weight(1234, n_out, n_in).reshape(n_out, n_in // 32, 34).copy()
    special = np.array([0x0000, 0x8000, 0x0001, 0x83ff, 0x7bff, 0xfbff, 0x7c00, 0xfc00, 0x7e00, 0x0400, 0x3c00],
                       np.uint16)
    pick = rng.integers(0, special.size, (n_out, n_in // 32))
    keep = rng.random((n_out, n_in // 32)) < 0.5
    scales = w[:, :, :2].copy().view(np.uint16)[:, :, 0]
    scales = np.where(keep, scales, special[pick]).astype(np.uint16)
    w[:, :, :2] = scales[:, :, None].view(np.uint8)
    w = np.ascontiguousarray(w).reshape(-1)
    q8 = rng.integers(-127, 128, (n_tokens, n_in), dtype=np.int8)
    sc = (rng.random((n_tokens, n_in // 32), dtype=np.float32) + 0.5) * \
        np.float32(10.0) ** rng.integers(-44, 3, (n_tokens, n_in // 32)).astype(np.float32)
    sc[rng.random(sc.shape) < 0.05] = 0.0
    sc = sc.astype(np.float32)
    if f16_token_scales:
        sc = (rng.random(sc.shape, dtype=np.float32) + 0.5) * np.float32(10.0) ** rng.integers(-8, 7, sc.shape).astype(np.float32)
        sc[rng.random(sc.shape) < 0.05] = 0.0
        with np.errstate(over="ignore"):
            sc = sc.astype(np.float16).astype(np.float32)  # incl. f16 subnormals, zeros and inf
        assert np.isinf(sc).any() and (np.abs(sc[sc != 0]) < 6.1e-5).any()
    H = hip.hip
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    d_q8, d_sc = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)
    d_y = H.DeviceBuffer(n_tokens * n_out * 4)
    H.check(H.lib.rmi_hip_gemm_q8_0_dev(kernel.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, n_out, None))
    H.check(H.lib.rmi_hip_synchronize())
    out = d_y.to_array(np.float32, (n_tokens, n_out))
    with np.errstate(all="ignore"):
        ref = np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, N) for t in range(n_tokens)])
    nan_o, nan_r = np.isnan(out), np.isnan(ref)
    assert np.array_equal(nan_o, nan_r) and nan_r.any() and not nan_r.all()
    assert np.array_equal(bits(out)[~nan_o], bits(ref)[~nan_r])
    # subnormal scale products were exercised (f16 subnormal weight scale x tiny token scale)
    wd = scales.view(np.float16).astype(np.float32)
    with np.errstate(all="ignore"):
        prod = wd[:, None, :] * sc[None, :, :]
    if not f16_token_scales:
        assert np.count_nonzero((prod != 0) & (np.abs(prod) < 1.17549435e-38)) > 1000


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(2048, 3072, 1024), (2048, 1024, 3072), (512, 3072, 1024),
                                                  (512, 1024, 3072)])
def test_gemm_full_size_properties(hip, oracle, n_tokens, n_out, n_in):
    """The prefill configuration at its stated sizes (M = 512 and 2048, the FFN up and down shapes): token rows
    sampled against the checker's NEON order, bit for bit, and within tolerance of the x86-64 order; every token
    row equals the same token run through a 64-token call (tile position must not change bits)."""
    w, x = _case(hip, 1000 + n_tokens + n_in, n_out, n_in, n_tokens)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    out = np.zeros((n_tokens, n_out), np.float32)
    kernel.forward_batched(x, out, n_in, n_out, matrix_cores=True)
    sample = [0, 1, 63, 64, n_tokens // 2 - 1, n_tokens - 1]
    q8, sc = _quantize_rows(oracle, x[sample])
    for i, t in enumerate(sample):
        assert np.array_equal(bits(out[t]), bits(oracle.matmul_q8_0_quantized(w, q8[i], sc[i], n_in, n_out, N)))
        ref_a = oracle.matmul_q8_0_quantized(w, q8[i], sc[i], n_in, n_out, A)
        assert np.all(np.abs(out[t] - ref_a) <= TOL(ref_a))
    lo = n_tokens // 2 - 24
    part = np.zeros((64, n_out), np.float32)
    kernel.forward_batched(x[lo:lo + 64], part, n_in, n_out, matrix_cores=True)
    assert np.array_equal(bits(part), bits(out[lo:lo + 64]))


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(512, 768, 512), (256, 1536, 256), (130, 200, 320)])
def test_gemm_tile_to_xcd_assignment_changes_no_bit(hip, oracle, monkeypatch, n_tokens, n_out, n_in):
    """Which XCD takes which tile of the prefill GEMM (one-dimensional renumbering, 2 x 4 or 4 x 2 grids of XCDs) is a
    matter of cache traffic: forced each way, where the tile grid allows it and where it does not, every output has the
    same bits, and those of the checker's NEON order."""
    w, x = _case(hip, 3000 + n_tokens, n_out, n_in, n_tokens)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    outs = []
    for split in (None, "0", "2", "4"):
        if split is None:
            monkeypatch.delenv("RMI_GEMM_XCD_SPLIT", raising=False)
        else:
            monkeypatch.setenv("RMI_GEMM_XCD_SPLIT", split)
        out = np.full((n_tokens, n_out), np.nan, np.float32)
        kernel.forward_batched(x, out, n_in, n_out, matrix_cores=True)
        outs.append(out)
    for o in outs[1:]:
        assert np.array_equal(bits(o), bits(outs[0]))
    sample = [0, n_tokens // 3, n_tokens - 1]
    q8, sc = _quantize_rows(oracle, x[sample])
    for i, t in enumerate(sample):
        assert np.array_equal(bits(outs[0][t]), bits(oracle.matmul_q8_0_quantized(w, q8[i], sc[i], n_in, n_out, N)))


@pytest.mark.parametrize("n_tokens", [9, 16, 17, 40])
def test_forward_batched_does_not_depend_on_the_batch(hip, oracle, n_tokens):
    """trait_.rs:78-109: every token goes through the same quantizer and kernel, so forward_batched(x)[t] ==
    forward(x[t]) bit for bit, and both are the x86-64 kernel's result, for any token count."""
    n_out, n_in = 520, 1024
    w, x = _case(hip, 1900 + n_tokens, n_out, n_in, n_tokens)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    out = np.zeros((n_tokens, n_out), np.float32)
    kernel.forward_batched(x, out, n_in, n_out)
    for t in range(n_tokens):
        one = np.zeros(n_out, np.float32)
        kernel.forward(x[t], one, n_in, n_out)
        assert np.array_equal(bits(out[t]), bits(one)), t
    assert np.array_equal(bits(out), bits(oracle.q8_0_forward_batched(w, x, n_in, n_out, A)))
    # the matrix-core path is batch-independent too, in its own (aarch64) order
    mc = np.zeros((n_tokens, n_out), np.float32)
    kernel.forward_batched(x, mc, n_in, n_out, matrix_cores=True)
    one = np.zeros((1, n_out), np.float32)
    kernel.forward_batched(x[n_tokens - 1], one, n_in, n_out, matrix_cores=True)
    assert np.array_equal(bits(mc[n_tokens - 1]), bits(one[0]))


@pytest.mark.parametrize("n_tokens", [1, 5, 16, 33, 100])
def test_aarch64_host_end_to_end(hip, oracle, n_tokens):
    """What an aarch64 host computes: its own quantizer (1/d, ties to even, clamp to [-127, 127],
    src/ops/quant/q8_0.rs:75-164) and its kernel's order (neon.rs:49-73), for any token count."""
    n_out, n_in = 264, 1024
    w, x = _case(hip, 1950 + n_tokens, n_out, n_in, n_tokens)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out, rounding=hip.hip.ROUND_NEON,
                                                        matrix_cores=True)
    assert np.array_equal(bits(out), bits(oracle.q8_0_forward_batched(w, x, n_in, n_out, N)))


def test_batch_8_on_the_lm_head(hip, oracle):
    """Decode batch 8 on the 151 936-row head: rows sampled against the checker's x86-64 order."""
    n_tokens, n_out, n_in = 8, 151936, 1024
    w, x = _case(hip, 1990, n_out, n_in, n_tokens)
    q8, sc = _quantize_rows(oracle, x)
    out = np.zeros((n_tokens, n_out), np.float32)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    kernel.matmul_q8_0_quantized_batch(q8, sc, out, n_in, n_out, n_tokens)
    rows = np.unique(np.concatenate([np.arange(0, 24), np.arange(n_out - 24, n_out),
                                     np.random.default_rng(5).integers(0, n_out, 2000)]))
    wr = np.ascontiguousarray(w.reshape(n_out, -1)[rows]).reshape(-1)
    for t in range(n_tokens):
        ref = oracle.matmul_q8_0_quantized(wr, q8[t], sc[t], n_in, rows.size, A)
        assert np.array_equal(bits(out[t, rows]), bits(ref)), t
    assert np.isfinite(out).all()


# -------------------------------------------------------------- device-resident

def test_grouped_launch_equals_single_launches(hip, oracle):
    """One launch over a list of independent GEMVs (two Qwen3 layers' worth + a wide head)."""
    H, K = hip.hip, hip.kernel
    shapes = hip.synth.QWEN3_0_6B_LAYER * 2 + [("head", 4099, 1024)]
    for n_tokens in (1, 3, 8):
        kernels, xq, xs, ys, refs = [], [], [], [], []
        for i, (_, n_out, n_in) in enumerate(shapes):
            w, x = _case(hip, 1100 + i, n_out, n_in, n_tokens)
            q8, sc = _quantize_rows(oracle, x)
            kernels.append(K.Q8Kernel(w, n_in, n_out))
            xq.append(H.DeviceBuffer.from_array(q8))
            xs.append(H.DeviceBuffer.from_array(sc))
            ys.append(H.DeviceBuffer(n_tokens * n_out * 4))
            refs.append(np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, A)
                                  for t in range(n_tokens)]))
        n = len(shapes)
        arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
        g = H.lib.rmi_hip_gemv_group_create(n, arr([k.w.handle for k in kernels]), arr([b.ptr for b in xq]),
                                            arr([b.ptr for b in xs]), arr([b.ptr for b in ys]), n_tokens)
        assert g, H.last_error()
        H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))
        H.check(H.lib.rmi_hip_synchronize())
        for i, (_, n_out, _) in enumerate(shapes):
            got = ys[i].to_array(np.float32, (n_tokens, n_out))
            assert np.array_equal(bits(got), bits(refs[i])), (n_tokens, i)
        H.lib.rmi_hip_gemv_group_destroy(g)


def test_device_entry_points_roundtrip(hip, oracle):
    """quantize_dev -> gemv_dev with activations that never leave HBM."""
    H = hip.hip
    n_tokens, n_out, n_in = 4, 2048, 1024
    w, x = _case(hip, 1200, n_out, n_in, n_tokens)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    d_x = H.DeviceBuffer.from_array(x)
    d_q8, d_sc, d_y = H.DeviceBuffer(x.size), H.DeviceBuffer(x.size // 32 * 4), H.DeviceBuffer(n_tokens * n_out * 4)
    H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q8.ptr, d_sc.ptr, n_tokens, n_in, 1, None))
    H.check(H.lib.rmi_hip_gemv_q8_0_dev(kernel.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, n_out, 0, n_out, None))
    H.check(H.lib.rmi_hip_synchronize())
    got = d_y.to_array(np.float32, (n_tokens, n_out))
    assert np.array_equal(bits(got), bits(oracle.q8_0_forward_batched(w, x, n_in, n_out, A)))


# ------------------------------------------------------------------ legacy + errors

def test_legacy_f32_matmul_bit_exact(hip, oracle):
    """`ops::matmul_q8_0`: f32 activations, AVX2 accumulation order (avx2.rs:180-217)."""
    for n_out, n_in in [(64, 512), (13, 96), (1024, 1024)]:
        w, x = _case(hip, 1300 + n_out, n_out, n_in)
        out = np.zeros(n_out, np.float32)
        hip.kernel.Q8Kernel(w, n_in, n_out).matmul_q8_0(x[0], out, n_in, n_out)
        assert np.array_equal(bits(out), bits(oracle.matmul_q8_0_f32(w, x[0], n_in, n_out, A)))


def test_legacy_f32_matmul_scalar_order_bit_exact(hip, oracle):
    """`matmul_q8_0_fallback_range` (scalar.rs:3-29): one f32 chain per row, products and sums rounded separately;
    whole matrices, ragged shapes, and row ranges that start and end inside a tile."""
    for n_out, n_in in [(64, 512), (13, 96), (1024, 1024), (203, 3072)]:
        w, x = _case(hip, 1350 + n_out, n_out, n_in)
        kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
        ref = oracle.matmul_q8_0_f32(w, x[0], n_in, n_out, S)
        out = np.zeros(n_out, np.float32)
        kernel.matmul_q8_0_fallback_range(x[0], out, n_in, 0, n_out)
        assert np.array_equal(bits(out), bits(ref))
        # not the AVX2 order's bits (the two differ in the last places on data like this)
        assert not np.array_equal(bits(out), bits(oracle.matmul_q8_0_f32(w, x[0], n_in, n_out, A)))
        for lo, hi in [(3, n_out - 2), (n_out // 2, n_out // 2), (0, 1)]:
            part = np.full(max(hi - lo, 1), np.nan, np.float32)
            kernel.matmul_q8_0_fallback_range(x[0], part, n_in, lo, hi)
            assert np.array_equal(bits(part[:hi - lo]), bits(ref[lo:hi]))
    H = hip.hip
    kernel = hip.kernel.Q8Kernel(*_case(hip, 1360, 16, 64)[:1], 64, 16)
    out = np.zeros(16, np.float32)
    with pytest.raises(H.RmiHipError):
        kernel.matmul_q8_0_fallback_range(np.zeros(64, np.float32), out, 64, 4, 17)


def test_legacy_via_q8_and_batch(hip, oracle):
    """`matmul_q8_0_via_q8` (legacy.rs:27-83) quantizes into the caller's scratch and runs the prequantized
    GEMV; `matmul_q8_0_batch` (batch.rs:32-79) runs a list of f32-activation matmuls."""
    K = hip.kernel
    n_out, n_in = 200, 768
    w, x = _case(hip, 1400, n_out, n_in)
    kernel = K.Q8Kernel(w, n_in, n_out)
    out = np.zeros(n_out, np.float32)
    q8_buf, scale_buf = np.zeros(n_in, np.uint8), np.zeros(n_in // 32, np.float32)
    kernel.matmul_q8_0_via_q8(x[0], out, n_in, n_out, q8_buf, scale_buf)
    ref_q8, ref_sc = oracle.quantize_q8_0(x[0], A)
    assert np.array_equal(q8_buf.view(np.int8), np.asarray(ref_q8).view(np.int8).reshape(-1))
    assert np.array_equal(bits(scale_buf), bits(ref_sc))
    assert np.array_equal(bits(out), bits(oracle.q8_0_forward_batched(w, x, n_in, n_out, A)[0]))
    tasks, refs = [], []
    for i, (no, ni) in enumerate([(64, 512), (130, 96), (257, 1024)]):
        wi, xi = _case(hip, 1410 + i, no, ni)
        tasks.append(K.MatmulTask(K.Q8Kernel(wi, ni, no), xi[0], np.zeros(no, np.float32), ni, no))
        refs.append(oracle.matmul_q8_0_f32(wi, xi[0], ni, no, A))
    K.matmul_q8_0_batch(tasks)
    for t, r in zip(tasks, refs):
        assert np.array_equal(bits(t.output), bits(r))


def test_error_codes(hip):
    H, K = hip.hip, hip.kernel
    kernel = K.Q8Kernel(gen.make_q8_0_weight(4, 64, 0), 64, 4)
    out = np.zeros(4, np.float32)
    with pytest.raises(H.RmiHipError) as e:
        kernel.forward_prequantized(np.zeros(32, np.uint8), np.zeros(1, np.float32), out, 32, 4, 0, 1)
    assert e.value.code == -1 and "64" in str(e.value)
    with pytest.raises(H.RmiHipError):  # slice shorter than n_out x n_in
        K.Q8Kernel(np.zeros(33, np.uint8), 32, 1)
    with pytest.raises(H.RmiHipError):  # n_in not a multiple of 32
        K.Q8Kernel(np.zeros(340, np.uint8), 40, 8)
    # ith beyond the last slice writes nothing and is not an error (parallel.rs:127-129)
    out[:] = 7
    kernel.forward_prequantized(np.zeros(64, np.uint8), np.zeros(2, np.float32), out, 64, 4, 5, 3)
    assert np.all(out == 7)
    # zero rows
    K.Q8Kernel(np.zeros(0, np.uint8), 64, 0).forward_prequantized(np.zeros(64, np.uint8), np.zeros(2, np.float32),
                                                                 out, 64, 0, 0, 1)


def test_misaligned_device_pointers_are_refused(hip):
    """The staging kernels read activation quants 16 bytes at a time and the rest 4 bytes at a time: a device
    pointer that is not so aligned is an argument error, reported before anything is launched."""
    H, K = hip.hip, hip.kernel
    q8 = K.Q8Kernel(gen.make_q8_0_weight(16, 256, 3), 256, 16)
    q4k = K.Q4_KKernel(hip.synth.q4_k_weight(5, 16, 256), 256, 16)
    buf, y = H.DeviceBuffer(4096), H.DeviceBuffer(4096)
    ok = H.lib.rmi_hip_gemv_q8_0_dev(q8.w.handle, buf.ptr, buf.ptr + 1024, y.ptr, 1, 16, 0, 16, None)
    assert ok == 0, H.last_error()
    for dq, ds, dy in ((4, 0, 0), (0, 2, 0), (0, 0, 2)):
        rc = H.lib.rmi_hip_gemv_q8_0_dev(q8.w.handle, buf.ptr + dq, buf.ptr + 1024 + ds, y.ptr + dy, 1, 16, 0, 16, None)
        assert rc == -1 and "aligned" in H.last_error(), (dq, ds, dy)
        rc = H.lib.rmi_hip_gemm_q8_0_dev(q8.w.handle, buf.ptr + dq, buf.ptr + 1024 + ds, y.ptr + dy, 1, 16, None)
        assert rc == -1 and "aligned" in H.last_error(), (dq, ds, dy)
    rc = H.lib.rmi_hip_gemv_q4_k_q8k_dev(q4k.w.handle, buf.ptr, buf.ptr + 1024 + 8, buf.ptr + 2048, y.ptr, 1, 16, 0, 16, None)
    assert rc == -1 and "aligned" in H.last_error()
    rc = H.lib.rmi_hip_gemv_q4_k_q8k_dev(q4k.w.handle, buf.ptr, buf.ptr + 1024, buf.ptr + 2048 + 2, y.ptr, 1, 16, 0, 16, None)
    assert rc == -1 and "aligned" in H.last_error()
    H.check(H.lib.rmi_hip_synchronize())
