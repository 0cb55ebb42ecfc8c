"""GPU parity of the Q6_K path (Q6_KKernel), through the C ABI.

Bars: the eight int32 accumulator lanes per super-block bit-exact; Q6_K x Q8_K
GEMV f32 bit-exact against the restated x86-64 kernel (vec_dot_q6k_q8k_avx2
order) and within rel 1e-3 of the scalar one (the reference's own bound,
src/ops/quant/mod.rs:1165-1211); the dequantise-and-dot path bit-exact against
the restated sequential f32 sum.
"""
import numpy as np
import pytest

import gen
from conftest import bits

pytestmark = pytest.mark.gpu

S, A = 0, 1


def _same(a, b):
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(bits(a)[~na], bits(b)[~nb])


def _q8k_blocks(K, d, qs, bs):
    return [K.BlockQ8K(float(d[i]), qs[i * 256:(i + 1) * 256], bs[i * 16:(i + 1) * 16]) for i in range(d.size)]


def test_q6_k_kernel_multiplies_uniform_block(hip):
    """tests/quantized_inference.rs:252-263."""
    w = np.full(210, 0x11, np.uint8)
    w[128:192] = 0xAA
    w[192:208] = 1
    w[208:210] = np.array([gen.f16_bits(1.0)], np.uint16).view(np.uint8)
    out = np.zeros(1, np.float32)
    hip.kernel.Q6_KKernel(w, 256, 1).forward_prequantized(np.ones(256, np.uint8), np.ones(8, np.float32), out, 256, 1,
                                                         0, 1)
    assert list(out) == [256.0]


def test_q6_k_prepared_path_on_reference_bytes(hip, oracle):
    """tests/quantized_inference.rs:213-231: byte pattern index*17+3, d = 2^-6, q8_k = None."""
    K = hip.kernel
    w = ((np.arange(210) * 17 + 3) & 0xFF).astype(np.uint8)
    w[208:210] = np.array([gen.f16_bits(0.015625)], np.uint16).view(np.uint8)
    x = np.array([((i % 19) - 9) / 5.0 for i in range(256)], np.float32)
    out = np.zeros(1, np.float32)
    K.Q6_KKernel(w, 256, 1).forward_prepared(x, None, None, None, out, 256, 1, 0, 1)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    assert bits(out)[0] == bits(np.array([oracle.vec_dot_q6k_q8k(w, d, qs, bs, A)]))[0]
    # one super-block: eight lanes, one product each; the scalar order differs by rounding only
    assert abs(out[0] - oracle.vec_dot_q6k_q8k(w, d, qs, bs, S)) <= 1e-5 * abs(out[0])


@pytest.mark.parametrize("n_out,n_in", [(6144, 2048), (2048, 6144), (1, 256), (13, 512), (100, 1024), (151, 3584)])
def test_q6k_q8k_gemv_bit_exact(hip, oracle, n_out, n_in):
    K = hip.kernel
    w = hip.synth.q6_k_weight(60 + n_out, n_out, n_in)
    x = hip.synth.activations(61 + n_in, 1, n_in)[0]
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    kernel = K.Q6_KKernel(w, n_in, n_out)
    out = np.zeros(n_out, np.float32)
    kernel.forward_prepared(x, None, None, _q8k_blocks(K, d, qs, bs), out, n_in, n_out, 0, 1)
    ref = np.zeros(n_out, np.float32)
    oracle.q6k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
    assert np.array_equal(bits(out), bits(ref))
    refs = np.zeros(n_out, np.float32)
    oracle.q6k_forward_prepared(w, d, qs, bs, refs, n_in, n_out, 0, 1, S)
    assert np.all(np.abs(out - refs) <= 1e-3 * np.maximum(np.abs(refs), 1.0))
    # exact lane integers per super-block, read back from the repacked HBM copy
    lanes = kernel.block_lanes(_q8k_blocks(K, d, qs, bs))
    wr = w.reshape(n_out, -1)
    for r in np.unique(np.linspace(0, n_out - 1, min(n_out, 40)).astype(int)):
        assert np.array_equal(lanes[r], oracle.q6k_q8k_lane_ints(wr[r], qs, bs)), r
        assert np.array_equal(lanes[r].sum(axis=1), oracle.q6k_q8k_block_ints(wr[r], qs)), r
    # q8_k = None: the kernel quantizes input_f32 itself (q6_k.rs:63-69)
    out2 = np.zeros(n_out, np.float32)
    kernel.forward_prepared(x, None, None, None, out2, n_in, n_out, 0, 1)
    assert np.array_equal(bits(out2), bits(out))


def test_q6k_extreme_values_bit_exact(hip, oracle):
    """Scales -128/127, quants 0/63, activations +-127: the largest lane integers (beyond 2^24)."""
    K = hip.kernel
    n_out, n_in = 16, 1024
    rng = np.random.default_rng(7)
    w = np.zeros((n_out, n_in // 256, 210), np.uint8)
    w[:, :, 0:192] = rng.choice(np.array([0x00, 0xFF], np.uint8), (n_out, n_in // 256, 192))
    w[:, :, 192:208] = rng.choice(np.array([0x80, 0x7F], np.uint8), (n_out, n_in // 256, 16))
    w[:, :, 208:210] = np.array([gen.f16_bits(0.001)], np.uint16).view(np.uint8)
    w[0, :, 0:192] = 0xFF
    w[0, :, 192:208] = 0x7F
    w[1, :, 0:192] = 0x00
    w[1, :, 192:208] = 0x80
    w = w.reshape(-1)
    x = rng.choice(np.array([-3.0, 3.0], np.float32), n_in)
    x[:256] = 3.0
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    assert set(np.unique(qs)) <= {-127, 127}
    kernel = K.Q6_KKernel(w, n_in, n_out)
    blocks = _q8k_blocks(K, d, qs, bs)
    lanes = kernel.block_lanes(blocks)
    wr = w.reshape(n_out, -1)
    for r in range(n_out):
        assert np.array_equal(lanes[r], oracle.q6k_q8k_lane_ints(wr[r], qs, bs)), r
    assert np.abs(lanes).max() > 1 << 24
    out, ref = np.zeros(n_out, np.float32), np.zeros(n_out, np.float32)
    kernel.forward_prepared(x, None, None, blocks, out, n_in, n_out, 0, 1)
    oracle.q6k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
    assert np.array_equal(bits(out), bits(ref))


def test_q6k_partition_and_fusion(hip, oracle):
    """tests/fused_ffn_matmul_parity.rs:232-300, 296-299 on make_qk_weight bytes (d may be inf/nan)."""
    K = hip.kernel
    n_in, n_per = 1024, 3584
    row_bytes = n_in // 256 * 210
    gate = gen.make_qk_weight(n_per * row_bytes, row_bytes, 0)
    up = gen.make_qk_weight(n_per * row_bytes, row_bytes, 17)
    d, qs, bs = oracle.quantize_row_q8_k(gen.ramp_input(n_in), A)
    blocks = _q8k_blocks(K, d, qs, bs)
    kg, ku = K.Q6_KKernel(gate, n_in, n_per), K.Q6_KKernel(up, n_in, n_per)

    def run(kernel, rows, nth):
        out = np.zeros(rows, np.float32)
        for ith in range(nth):
            kernel.forward_prepared(None, None, None, blocks, out, n_in, rows, ith, nth)
        return out

    g1, u1 = run(kg, n_per, 1), run(ku, n_per, 1)
    rg, ru = np.zeros(n_per, np.float32), np.zeros(n_per, np.float32)
    oracle.q6k_forward_prepared(gate, d, qs, bs, rg, n_in, n_per, 0, 1, A)
    oracle.q6k_forward_prepared(up, d, qs, bs, ru, n_in, n_per, 0, 1, A)
    assert _same(g1, rg) and _same(u1, ru)
    assert _same(run(kg, n_per, 8), g1) and _same(run(ku, n_per, 3), u1)
    fused = K.fuse_vstack(kg, ku)
    f8 = run(fused, 2 * n_per, 8)
    assert _same(f8[:n_per], g1) and _same(f8[n_per:], u1)
    # a second weight that starts inside a tile (ragged first part)
    ka = K.Q6_KKernel(gate[:13 * row_bytes], n_in, 13)
    f2 = run(K.fuse_vstack(ka, ku), 13 + n_per, 4)
    assert _same(f2[:13], g1[:13]) and _same(f2[13:], u1)
    assert K.fuse_vstack(kg, K.Q4_KKernel(np.zeros(4 * 4 * 144, np.uint8), n_in, 4)) is None


@pytest.mark.parametrize("n_tokens", [1, 3, 8, 12])
def test_q6k_forward_batched(hip, oracle, n_tokens):
    n_out, n_in = 512, 2048
    w = hip.synth.q6_k_weight(70, n_out, n_in)
    x = hip.synth.activations(71, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q6_KKernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out)
    for t in range(n_tokens):
        d, qs, bs = oracle.quantize_row_q8_k(x[t], A)
        ref = np.zeros(n_out, np.float32)
        oracle.q6k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
        assert np.array_equal(bits(out[t]), bits(ref)), t


def test_q6k_grouped_launch_bit_exact(hip, oracle):
    """One launch over a list of independent Q6_K x Q8_K GEMVs of mixed shapes, 1, 3 and 8 tokens."""
    H, K = hip.hip, hip.kernel
    shapes = [(1536, 1024), (1024, 1536), (37, 256), (6144, 2048), (2048, 6144), (9, 512)]
    for n_tokens in (1, 3, 8):
        kernels, bufs, refs = [], [], []
        for i, (n_out, n_in) in enumerate(shapes):
            w = hip.synth.q6_k_weight(300 + i, n_out, n_in)
            x = hip.synth.activations(320 + 10 * n_tokens + i, n_tokens, n_in)
            q = [oracle.quantize_row_q8_k(x[t], A) for t in range(n_tokens)]
            ref = np.zeros((n_tokens, n_out), np.float32)
            for t, (d, qs, bs) in enumerate(q):
                oracle.q6k_forward_prepared(w, d, qs, bs, ref[t], n_in, n_out, 0, 1, A)
            refs.append(ref)
            kernels.append(K.Q6_KKernel(w, n_in, n_out))
            bufs.append((H.DeviceBuffer.from_array(np.stack([t[0] for t in q])),
                         H.DeviceBuffer.from_array(np.stack([t[1] for t in q])),
                         H.DeviceBuffer.from_array(np.stack([t[2] for t in q])),
                         H.DeviceBuffer(n_tokens * n_out * 4)))
        n = len(shapes)
        arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
        g = H.lib.rmi_hip_gemv_group_create_q6_k(n, arr([k.w.handle for k in kernels]), arr([b[0].ptr for b in bufs]),
                                                 arr([b[1].ptr for b in bufs]), arr([b[2].ptr for b in bufs]),
                                                 arr([b[3].ptr for b in bufs]), n_tokens)
        assert g, H.last_error()
        for _ in range(2):
            H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))
        H.check(H.lib.rmi_hip_synchronize())
        for i, (n_out, _) in enumerate(shapes):
            got = bufs[i][3].to_array(np.float32, (n_tokens, n_out))
            assert np.array_equal(bits(got), bits(refs[i])), (n_tokens, i)
        H.lib.rmi_hip_gemv_group_destroy(g)
    # a Q4_K handle in a Q6_K group is refused
    k4 = K.Q4_KKernel(np.zeros(4 * 144, np.uint8), 256, 4)
    one = lambda v: (H.C.c_void_p * 1)(v)  # noqa: E731
    p = bufs[0]
    assert not H.lib.rmi_hip_gemv_group_create_q6_k(1, one(k4.w.handle), one(p[0].ptr), one(p[1].ptr), one(p[2].ptr),
                                                    one(p[3].ptr), 1)
    assert "bad weight handle" in H.last_error()


# the last two: an activation that needs more than 64 KiB of LDS beside the products, and one beyond the
# workgroup's LDS altogether (the one-lane-per-row kernel takes it)
@pytest.mark.parametrize("n_out,n_in", [(1024, 2048), (2048, 6144), (5, 256), (77, 768), (41, 12288), (19, 36864)])
def test_q6k_dequant_dot_path_bit_exact(hip, oracle, n_out, n_in):
    """Q6_KKernel::forward_prequantized = matmul_q6_k_scalar_range (q6_k.rs:83-119), (ith, nth) slices."""
    K = hip.kernel
    w = hip.synth.q6_k_weight(80 + n_out, n_out, n_in)
    x = hip.synth.activations(81 + n_in, 1, n_in)[0]
    q8, sc = oracle.quantize_q8_0(x, A)
    ref = np.zeros(n_out, np.float32)
    oracle.q6k_forward_prequantized(w, q8, sc, ref, n_in, n_out, 0, 1)
    got = np.zeros(n_out, np.float32)
    kernel = K.Q6_KKernel(w, n_in, n_out)
    for ith in range(3):
        kernel.forward_prequantized(q8, sc, got, n_in, n_out, ith, 3)
    assert np.array_equal(bits(got), bits(ref))
    # the factory picks the Q6_K kernel for the Q6_K type tag
    k2 = K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q6_K, w, n_in, n_out).into_kernel()
    assert isinstance(k2, K.Q6_KKernel) and k2.w.dtype == hip.hip.DTYPE_Q6_K


def test_q6k_errors(hip):
    H, K = hip.hip, hip.kernel
    with pytest.raises(H.RmiHipError):
        K.Q6_KKernel(np.zeros(210, np.uint8), 128, 1)  # n_in not a multiple of 256
    with pytest.raises(H.RmiHipError):
        K.Q6_KKernel(np.zeros(209, np.uint8), 256, 1)  # slice too short
    kernel = K.Q6_KKernel(np.zeros(210 * 2, np.uint8), 256, 2)
    with pytest.raises(H.RmiHipError):
        kernel.forward_prequantized(np.zeros(512, np.uint8), np.zeros(16, np.float32), np.zeros(2, np.float32), 512, 2,
                                    0, 1)
    # a Q6_K handle passed to a Q4_K entry point is refused
    with pytest.raises(H.RmiHipError):
        H.check(H.lib.rmi_hip_q4_k_forward_batched(kernel.w.handle, H.ptr(np.zeros(256, np.float32), H._f32p),
                                                   H.ptr(np.zeros(2, np.float32), H._f32p), 256, 2, 1))
