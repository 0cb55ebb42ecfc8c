"""GPU parity of the Q4_K path (Q4_KKernel, QuantizedLinear), through the C ABI.

Bars: Q8_K quantizer and per-super-block integers bit-exact; Q4_K x Q8_K GEMV
f32 bit-exact against the restated x86-64 kernel (vec_dot_q4k_q8k_avx2 order)
and within rel 1e-3 of the scalar one (the reference's own bound,
src/ops/quant/mod.rs:1112-1162); dequantise-and-dot paths bit-exact against the
restated sequential f32 sums.
"""
import numpy as np
import pytest

import gen
from conftest import bits

pytestmark = pytest.mark.gpu

S, A = 0, 1


def _same(a, b):
    """Bit equality, with NaNs only required to coincide in position."""
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(bits(a)[~na], bits(b)[~nb])


def _q8k_blocks(K, d, qs, bs):
    return [K.BlockQ8K(float(d[i]), qs[i * 256:(i + 1) * 256], bs[i * 16:(i + 1) * 16]) for i in range(d.size)]


# ------------------------------------------------------------------ Q8_K quantizer

def test_q8_k_quantizer_reference_kats(hip):
    """tests/quantized_inference.rs:152-186."""
    x = np.zeros(256, np.float32)
    x[:5] = [-127.0, 0.5, 1.5, 2.5, -0.5]
    blocks = hip.kernel.quantize_row_q8_k(x)
    assert list(blocks[0].qs[:5]) == [-127, 0, 2, 2, 0]
    x = np.array([(i - 127) * 0.03125 for i in range(256)], np.float32)
    blocks = hip.kernel.quantize_row_q8_k(x)
    assert len(blocks) == 1
    assert int(blocks[0].bsums.astype(np.int32).sum()) == int(blocks[0].qs.astype(np.int32).sum())


def test_q8_k_quantizer_bit_exact(hip, oracle):
    rng = np.random.default_rng(50)
    x = (rng.standard_normal(256 * 96) * rng.choice([1e-5, 1.0, 300.0], 256 * 96)).astype(np.float32)
    x[:256] = 0
    x[256:512] = -np.abs(x[256:512])
    x[512:768] = 1.0                      # every element ties for the maximum: the first wins
    x[768:1024] = np.tile([2.0, -2.0], 128)  # +max before -max
    x[1024:1280] = np.tile([-2.0, 2.0], 128)  # -max before +max
    x[1280:1536] = np.arange(256) - 127.5
    H = hip.hip
    d = np.zeros(x.size // 256, np.float32)
    qs = np.zeros(x.size, np.int8)
    bs = np.zeros(x.size // 16, np.int16)
    H.check(H.lib.rmi_hip_quantize_row_q8_k(H.ptr(x, H._f32p), x.size, H.ptr(d, H._f32p), H.ptr(qs, H._i8p),
                                            H.ptr(bs, H._i16p)))
    for variant in (S, A):
        rd, rq, rb = oracle.quantize_row_q8_k(x, variant)
        assert np.array_equal(bits(d), bits(rd)) and np.array_equal(qs, rq) and np.array_equal(bs, rb)


# ------------------------------------------------------------------ integer path

@pytest.mark.parametrize("n_out,n_in", [(6144, 2048), (2048, 6144), (1, 256), (13, 512), (100, 1024)])
def test_q4k_q8k_gemv_bit_exact(hip, oracle, n_out, n_in):
    K = hip.kernel
    w = hip.synth.q4_k_weight(60 + n_out, n_out, n_in)
    x = hip.synth.activations(61 + n_in, 1, n_in)[0]
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    kernel = K.Q4_KKernel(w, n_in, n_out)
    out = np.zeros(n_out, np.float32)
    kernel.forward_prepared(x, None, None, _q8k_blocks(K, d, qs, bs), out, n_in, n_out, 0, 1)
    ref = np.zeros(n_out, np.float32)
    oracle.q4k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
    assert np.array_equal(bits(out), bits(ref))
    refs = np.zeros(n_out, np.float32)
    oracle.q4k_forward_prepared(w, d, qs, bs, refs, n_in, n_out, 0, 1, S)
    assert np.all(np.abs(out - refs) <= 1e-3 * np.maximum(np.abs(refs), 1.0))
    # exact integers per super-block, read back from the repacked HBM copy
    isum, msum = kernel.block_ints(_q8k_blocks(K, d, qs, bs))
    rows = np.unique(np.linspace(0, n_out - 1, min(n_out, 40)).astype(int))
    wr = w.reshape(n_out, -1)
    for r in rows:
        ri, rm = oracle.q4k_q8k_block_ints(wr[r], qs, bs)
        assert np.array_equal(isum[r], ri) and np.array_equal(msum[r], rm)
    # q8_k = None: the kernel quantizes input_f32 itself (q4_k.rs:77-84)
    out2 = np.zeros(n_out, np.float32)
    kernel.forward_prepared(x, None, None, None, out2, n_in, n_out, 0, 1)
    assert np.array_equal(bits(out2), bits(out))


def test_q4k_partition_and_fusion(hip, oracle):
    """tests/fused_ffn_matmul_parity.rs:232-300 on make_qk_weight bytes (d/dmin may be inf/nan)."""
    K = hip.kernel
    n_in, n_per = 1024, 3584
    row_bytes = n_in // 256 * 144
    gate = gen.make_qk_weight(n_per * row_bytes, row_bytes, 0)
    up = gen.make_qk_weight(n_per * row_bytes, row_bytes, 17)
    d, qs, bs = oracle.quantize_row_q8_k(gen.ramp_input(n_in), A)
    blocks = _q8k_blocks(K, d, qs, bs)
    kg, ku = K.Q4_KKernel(gate, n_in, n_per), K.Q4_KKernel(up, n_in, n_per)

    def run(kernel, rows, nth):
        out = np.zeros(rows, np.float32)
        for ith in range(nth):
            kernel.forward_prepared(None, None, None, blocks, out, n_in, rows, ith, nth)
        return out

    g1, u1 = run(kg, n_per, 1), run(ku, n_per, 1)
    rg, ru = np.zeros(n_per, np.float32), np.zeros(n_per, np.float32)
    oracle.q4k_forward_prepared(gate, d, qs, bs, rg, n_in, n_per, 0, 1, A)
    oracle.q4k_forward_prepared(up, d, qs, bs, ru, n_in, n_per, 0, 1, A)
    assert _same(g1, rg) and _same(u1, ru)
    assert _same(run(kg, n_per, 8), g1) and _same(run(ku, n_per, 3), u1)
    fused = K.fuse_vstack(kg, ku)
    f8 = run(fused, 2 * n_per, 8)
    assert _same(f8[:n_per], g1) and _same(f8[n_per:], u1)
    assert K.fuse_vstack(kg, K.Q8Kernel(gen.make_q8_0_weight(4, n_in, 0), n_in, 4)) is None


@pytest.mark.parametrize("n_tokens", [1, 3, 8, 12, 16, 40])
def test_q4k_forward_batched(hip, oracle, n_tokens):
    n_out, n_in = 512, 2048
    w = hip.synth.q4_k_weight(70, n_out, n_in)
    x = hip.synth.activations(71, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q4_KKernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out)
    for t in range(n_tokens):
        d, qs, bs = oracle.quantize_row_q8_k(x[t], A)
        ref = np.zeros(n_out, np.float32)
        oracle.q4k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
        assert np.array_equal(bits(out[t]), bits(ref)), t


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(64, 1000, 512), (37, 45, 256), (130, 6144, 2048), (300, 200, 6144),
                                                  (16, 8, 256), (512, 6144, 2048), (512, 2048, 6144)])
def test_q4k_gemm_mfma_parity(hip, oracle, n_tokens, n_out, n_in):
    """Prefill (>= 16 tokens) goes through the matrix cores: the integers are exact, the f32 sums run in one
    chain per output instead of the AVX2 kernel's lane chains.  Within 1e-4 + 1e-4*|ref| of the AVX2-order
    result, within the reference's own 1e-3 of the scalar one, and within 2e-6 relative of the f64 sum over
    the exact per-super-block integers."""
    w = hip.synth.q4_k_weight(80 + n_tokens, n_out, n_in)
    x = hip.synth.activations(81 + n_out, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q4_KKernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out, matrix_cores=True)
    wr = w.reshape(n_out, -1, 144)
    wd = wr[:, :, 0:2].copy().view(np.float16)[:, :, 0].astype(np.float64)
    wdmin = wr[:, :, 2:4].copy().view(np.float16)[:, :, 0].astype(np.float64)
    rows = np.unique(np.linspace(0, n_out - 1, min(n_out, 24)).astype(int))
    for t in np.unique(np.linspace(0, n_tokens - 1, min(n_tokens, 12)).astype(int)):
        d, qs, bs = oracle.quantize_row_q8_k(x[t], A)
        ref = np.zeros(n_out, np.float32)
        oracle.q4k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
        assert np.all(np.abs(out[t] - ref) <= 1e-4 + 1e-4 * np.abs(ref)), t
        refs = np.zeros(n_out, np.float32)
        oracle.q4k_forward_prepared(w, d, qs, bs, refs, n_in, n_out, 0, 1, S)
        assert np.all(np.abs(out[t] - refs) <= 1e-3 * np.maximum(np.abs(refs), 1.0)), t
        for r in rows:
            isum, msum = oracle.q4k_q8k_block_ints(wr[r].reshape(-1), qs, bs)
            exact = np.sum(wd[r] * d.astype(np.float64) * isum - wdmin[r] * d.astype(np.float64) * msum)
            scale = np.sum(np.abs(wd[r] * d * isum) + np.abs(wdmin[r] * d * msum))
            assert abs(float(out[t, r]) - exact) <= 2e-6 * scale + 1e-30, (t, r)


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(70, 300, 768), (33, 129, 256), (200, 1024, 2048)])
def test_q4k_gemm_both_token_tile_widths(hip, oracle, monkeypatch, n_tokens, n_out, n_in):
    """The GEMM has a 32-token and a 64-token tile; the launcher picks by problem size.  Forced either way the
    integers are the same and the f32 chain is the same, so the two agree bit for bit with each other and to
    rounding with the AVX2-order result; ragged row and token tiles included."""
    w = hip.synth.q4_k_weight(90 + n_tokens, n_out, n_in)
    x = hip.synth.activations(91 + n_out, n_tokens, n_in)
    kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
    outs = {}
    for tile in ("1", "2"):
        monkeypatch.setenv("RMI_Q4K_GEMM_TTW", tile)
        out = np.full((n_tokens, n_out), np.nan, np.float32)
        kernel.forward_batched(x, out, n_in, n_out, matrix_cores=True)
        outs[tile] = out
    assert np.array_equal(bits(outs["1"]), bits(outs["2"]))
    out = outs["1"]
    for t in np.unique(np.linspace(0, n_tokens - 1, 9).astype(int)):
        d, qs, bs = oracle.quantize_row_q8_k(x[t], A)
        ref = np.zeros(n_out, np.float32)
        oracle.q4k_forward_prepared(w, d, qs, bs, ref, n_in, n_out, 0, 1, A)
        assert np.all(np.abs(out[t] - ref) <= 1e-4 + 1e-4 * np.abs(ref)), t


def test_q4k_gemm_ragged_shapes_both_widths(hip, oracle, monkeypatch):
    """Row counts around the 8-row tile and the 128-row workgroup, token counts around the 32- and 64-token tiles,
    one to three super-blocks: both tile widths against the AVX2-order result, every output."""
    shapes = [(17, 1, 256), (31, 7, 256), (32, 8, 512), (33, 9, 256), (63, 127, 256), (64, 128, 768), (65, 129, 512),
              (96, 136, 256), (127, 250, 512), (129, 64, 256)]
    for i, (n_tokens, n_out, n_in) in enumerate(shapes):
        w = hip.synth.q4_k_weight(400 + i, n_out, n_in)
        x = hip.synth.activations(420 + i, n_tokens, n_in)
        kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
        ref = np.zeros((n_tokens, n_out), np.float32)
        for t in range(n_tokens):
            d, qs, bs = oracle.quantize_row_q8_k(x[t], A)
            oracle.q4k_forward_prepared(w, d, qs, bs, ref[t], n_in, n_out, 0, 1, A)
        outs = []
        for tile in ("1", "2"):
            monkeypatch.setenv("RMI_Q4K_GEMM_TTW", tile)
            out = np.full((n_tokens + 1, n_out), np.nan, np.float32)  # one row more: nothing may be written past the end
            kernel.forward_batched(x, out[:n_tokens], n_in, n_out, matrix_cores=True)
            assert np.all(np.isnan(out[n_tokens])), (n_tokens, n_out, n_in, tile)
            assert np.all(np.abs(out[:n_tokens] - ref) <= 1e-4 + 1e-4 * np.abs(ref)), (n_tokens, n_out, n_in, tile)
            outs.append(out[:n_tokens].copy())
        assert np.array_equal(bits(outs[0]), bits(outs[1])), (n_tokens, n_out, n_in)


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(256, 1024, 512), (128, 512, 256), (70, 300, 768)])
def test_q4k_gemm_tile_to_xcd_assignment_changes_no_bit(hip, oracle, monkeypatch, n_tokens, n_out, n_in):
    """The Q4_K prefill GEMM with the assignment of tiles to XCDs forced each way: the same bits."""
    w = hip.synth.q4_k_weight(500 + n_tokens, n_out, n_in)
    x = hip.synth.activations(501 + n_out, n_tokens, n_in)
    kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
    outs = []
    for split in (None, "0", "2", "4"):
        if split is None:
            monkeypatch.delenv("RMI_GEMM_XCD_SPLIT", raising=False)
        else:
            monkeypatch.setenv("RMI_GEMM_XCD_SPLIT", split)
        out = np.full((n_tokens, n_out), np.nan, np.float32)
        kernel.forward_batched(x, out, n_in, n_out, matrix_cores=True)
        outs.append(out)
    assert not np.any(np.isnan(outs[0]))
    for o in outs[1:]:
        assert np.array_equal(bits(o), bits(outs[0]))


# ----------------------------------------------------------------- dequant paths

def test_q4k_grouped_launch_bit_exact(hip, oracle):
    """One launch over a list of independent Q4_K x Q8_K GEMVs of mixed shapes, 1, 3 and 8 tokens."""
    H, K = hip.hip, hip.kernel
    shapes = [(1536, 1024), (1024, 1536), (37, 256), (6144, 2048), (2048, 6144), (9, 512)]
    for n_tokens in (1, 3, 8):
        kernels, bufs, refs = [], [], []
        for i, (n_out, n_in) in enumerate(shapes):
            w = hip.synth.q4_k_weight(300 + i, n_out, n_in)
            x = hip.synth.activations(320 + 10 * n_tokens + i, n_tokens, n_in)
            q = [oracle.quantize_row_q8_k(x[t], A) for t in range(n_tokens)]
            ref = np.zeros((n_tokens, n_out), np.float32)
            for t, (d, qs, bs) in enumerate(q):
                oracle.q4k_forward_prepared(w, d, qs, bs, ref[t], n_in, n_out, 0, 1, A)
            refs.append(ref)
            kernels.append(K.Q4_KKernel(w, n_in, n_out))
            bufs.append((H.DeviceBuffer.from_array(np.stack([t[0] for t in q])),
                         H.DeviceBuffer.from_array(np.stack([t[1] for t in q])),
                         H.DeviceBuffer.from_array(np.stack([t[2] for t in q])),
                         H.DeviceBuffer(n_tokens * n_out * 4)))
        n = len(shapes)
        arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
        g = H.lib.rmi_hip_gemv_group_create_q4_k(n, arr([k.w.handle for k in kernels]), arr([b[0].ptr for b in bufs]),
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
    # a Q8_0 handle in a Q4_K group is refused
    k8 = K.Q8Kernel(gen.make_q8_0_weight(4, 256, 0), 256, 4)
    one = lambda v: (H.C.c_void_p * 1)(v)  # noqa: E731
    p = bufs[0]
    assert not H.lib.rmi_hip_gemv_group_create_q4_k(1, one(k8.w.handle), one(p[0].ptr), one(p[1].ptr), one(p[2].ptr),
                                                    one(p[3].ptr), 1)
    assert "bad weight handle" in H.last_error()


def test_q4_k_kernel_multiplies_uniform_block(hip):
    """tests/quantized_inference.rs:233-249."""
    w = np.zeros(144, np.uint8)
    w[0:2] = np.array([gen.f16_bits(1.0)], np.uint16).view(np.uint8)
    w[4:16] = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
    w[16:] = 0x11
    out = np.zeros(1, np.float32)
    hip.kernel.Q4_KKernel(w, 256, 1).forward_prequantized(np.ones(256, np.uint8), np.ones(8, np.float32), out, 256, 1,
                                                         0, 1)
    assert list(out) == [256.0]


# the last two: an activation that needs more than 64 KiB of LDS beside the products, and one beyond the
# workgroup's LDS altogether (the one-lane-per-row kernel takes it)
@pytest.mark.parametrize("n_out,n_in", [(6144, 2048), (2048, 6144), (5, 256), (77, 768), (41, 12288), (19, 36864)])
def test_dequant_dot_paths_bit_exact(hip, oracle, n_out, n_in):
    K = hip.kernel
    w = hip.synth.q4_k_weight(80 + n_out, n_out, n_in)
    x = hip.synth.activations(81 + n_in, 1, n_in)[0]
    # QuantizedLinear::forward through the Layer interface
    layer = K.QuantizedLinear.from_weight_slice(w, None, n_in, n_out, "ffn")
    assert (layer.input_dim(), layer.output_dim(), layer.name()) == (n_in, n_out, "ffn")
    out = np.zeros(n_out, np.float32)
    layer.forward(x, out, K.ExecContext(scratch=np.zeros(0, np.float32)))
    assert np.array_equal(bits(out), bits(oracle.quantized_linear_forward(w, x, n_in, n_out)))
    # Q4_KKernel::forward_prequantized with a (ith, nth) slice
    q8, sc = oracle.quantize_q8_0(x, A)
    ref = np.zeros(n_out, np.float32)
    oracle.q4k_forward_prequantized(w, q8, sc, ref, n_in, n_out, 0, 1)
    got = np.zeros(n_out, np.float32)
    for ith in range(3):
        layer.kernel.forward_prequantized(q8, sc, got, n_in, n_out, ith, 3)
    assert np.array_equal(bits(got), bits(ref))


def test_model_graph_two_layers(hip, oracle):
    """ModelGraph::forward_all ping-pong (src/core/model.rs:123-152)."""
    K = hip.kernel
    w1 = hip.synth.q4_k_weight(90, 512, 256)
    w2 = hip.synth.q4_k_weight(91, 256, 512)
    x = hip.synth.activations(92, 1, 256)[0]
    graph = K.ModelGraph()
    graph.add_layer(K.QuantizedLinear.from_weight_slice(w1, None, 256, 512, "a"))
    graph.add_layer(K.QuantizedLinear.from_weight_slice(w2, None, 512, 256, "b"))
    out = np.zeros(256, np.float32)
    graph.forward_all(x, out, np.zeros(1024, np.float32), K.ExecContext(scratch=np.zeros(0, np.float32)))
    h = oracle.quantized_linear_forward(w1, x, 256, 512)
    assert np.array_equal(bits(out), bits(oracle.quantized_linear_forward(w2, h, 512, 256)))


def test_q4k_errors(hip):
    H, K = hip.hip, hip.kernel
    with pytest.raises(H.RmiHipError):
        K.Q4_KKernel(np.zeros(144, np.uint8), 128, 1)  # n_in not a multiple of 256
    kernel = K.Q4_KKernel(np.zeros(144 * 2, np.uint8), 256, 2)
    with pytest.raises(H.RmiHipError):
        kernel.forward_prequantized(np.zeros(512, np.uint8), np.zeros(16, np.float32), np.zeros(2, np.float32), 512, 2,
                                    0, 1)


def _gemm_block_ints(hip, kernel, x, n_tokens, n_in, n_out):
    """Q8_K-quantizes x on the device and returns what the GEMM's matrix-core chains deliver per super-block,
    int32[n_tokens][n_out][n_in/256][2], plus the quantized activation."""
    H = hip.hip
    d_x = H.DeviceBuffer.from_array(H.as_f32(x))
    d_d, d_q, d_b = H.DeviceBuffer(n_tokens * n_in // 256 * 4), H.DeviceBuffer(n_tokens * n_in), H.DeviceBuffer(n_tokens * n_in // 16 * 2)
    H.check(H.lib.rmi_hip_quantize_row_q8_k_dev(d_x.ptr, d_d.ptr, d_q.ptr, d_b.ptr, n_tokens, n_in, None))
    d_i = H.DeviceBuffer.from_array(np.full(n_tokens * n_out * (n_in // 256) * 2, -1, np.int32))
    H.check(H.lib.rmi_hip_gemm_block_ints_q4_k_dev(kernel.w.handle, d_d.ptr, d_q.ptr, d_b.ptr, d_i.ptr, n_tokens, None))
    H.check(H.lib.rmi_hip_synchronize())
    ints = d_i.to_array(np.int32, (n_tokens, n_out, n_in // 256, 2))
    qs = d_q.to_array(np.int8, (n_tokens, n_in))
    bs = d_b.to_array(np.int16, (n_tokens, n_in // 16))
    for b in (d_x, d_d, d_q, d_b, d_i):
        b.free()
    return ints, qs, bs


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(512, 6144, 2048), (512, 2048, 6144)])
def test_q4k_gemm_block_ints_bit_exact_full_size(hip, oracle, n_tokens, n_out, n_in):
    """The per-super-block integers of the prefill GEMM (8 * D_hi + D_lo from the two int8 MFMA chains, the min
    term from the f16 MFMA) against the checker's scalar integers (quant/mod.rs:210-289), every token, row and
    super-block of the 1.7B-class FFN shapes at M = 512."""
    from concurrent.futures import ThreadPoolExecutor

    print(f"q4k gemm block ints: {n_tokens} tokens, {n_out}x{n_in}", flush=True)
    w = hip.synth.q4_k_weight(300 + n_out, n_out, n_in)
    x = hip.synth.activations(301 + n_in, n_tokens, n_in)
    kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
    ints, qs, bs = _gemm_block_ints(hip, kernel, x, n_tokens, n_in, n_out)

    def bad(t):
        return int(np.count_nonzero(ints[t] != oracle.q4k_q8k_block_ints_matrix(w, n_out, qs[t], bs[t])))

    with ThreadPoolExecutor(8) as ex:
        assert sum(ex.map(bad, range(n_tokens))) == 0
    assert np.abs(ints[..., 0]).max() > 10_000  # integers of the size a rounding tolerance would hide an error in


@pytest.mark.parametrize("ttw", ["1", "2"])
def test_q4k_gemm_block_ints_both_tile_widths_ragged_and_extreme(hip, oracle, monkeypatch, ttw):
    """Both token tile widths on ragged row and token tiles; and the largest integers the format allows (all
    nibbles 15, all scales and mins 63, all quants +-127), where 8 * D_hi + D_lo reaches 256 * 15 * 63 * 127."""
    monkeypatch.setenv("RMI_Q4K_GEMM_TTW", ttw)
    n_tokens, n_out, n_in = 70, 300, 768
    w = hip.synth.q4_k_weight(310, n_out, n_in)
    x = hip.synth.activations(311, n_tokens, n_in)
    kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
    ints, qs, bs = _gemm_block_ints(hip, kernel, x, n_tokens, n_in, n_out)
    for t in range(n_tokens):
        assert np.array_equal(ints[t], oracle.q4k_q8k_block_ints_matrix(w, n_out, qs[t], bs[t])), t
    # extremes: header = d, dmin, then twelve 0xff bytes (every 6-bit scale and min 63), nibbles all 15
    n_out, n_in, n_tokens = 40, 512, 33
    wx = np.full((n_out, n_in // 256, 144), 0xFF, np.uint8)
    wx[:, :, 0:4] = np.array([0x00, 0x3C, 0x00, 0x3C], np.uint8)  # d = dmin = 1.0
    # constant rows quantize to -127 everywhere (Q8_K's scale takes the sign of the largest element); every
    # third token alternates the sign from element to element instead
    xx = np.ones((n_tokens, n_in), np.float32)
    xx[::3, 1::2] = -1.0
    kx = hip.kernel.Q4_KKernel(wx.reshape(-1), n_in, n_out)
    ints, qs, bs = _gemm_block_ints(hip, kx, xx, n_tokens, n_in, n_out)
    assert set(np.unique(qs).tolist()) == {-127, 127}
    for t in range(n_tokens):
        assert np.array_equal(ints[t], oracle.q4k_q8k_block_ints_matrix(wx.reshape(-1), n_out, qs[t], bs[t])), t
    assert np.abs(ints[..., 0]).max() == 256 * 15 * 63 * 127


@pytest.mark.parametrize("groups", ["1", "2"])
def test_q4k_gemm_groups_of_waves_on_alternate_super_blocks(hip, oracle, monkeypatch, groups):
    """Long rows with few tiles run two groups of waves per tile, on the even and the odd super-blocks; forced either
    way the per-super-block integers are the checker's, every output is within 1e-4 + 1e-4 |ref| of the AVX2-order
    result and within 2e-6 of the f64 sum over the exact integers; ragged row and token tiles included."""
    monkeypatch.setenv("RMI_Q4K_GEMM_GROUPS", groups)
    for n_tokens, n_out, n_in in [(70, 300, 4096), (512, 2048, 6144)]:
        print(f"q4k gemm groups={groups}: {n_tokens} tokens, {n_out}x{n_in}", flush=True)
        w = hip.synth.q4_k_weight(320 + n_tokens, n_out, n_in)
        x = hip.synth.activations(321 + n_tokens, n_tokens, n_in)
        kernel = hip.kernel.Q4_KKernel(w, n_in, n_out)
        out = np.zeros((n_tokens, n_out), np.float32)
        kernel.forward_batched(x, out, n_in, n_out, matrix_cores=True)
        ints, qs, bs = _gemm_block_ints(hip, kernel, x, n_tokens, n_in, n_out)
        wr = w.reshape(n_out, -1, 144)
        wd = wr[:, :, 0:2].copy().view(np.float16)[:, :, 0].astype(np.float64)
        wdmin = wr[:, :, 2:4].copy().view(np.float16)[:, :, 0].astype(np.float64)
        for t in np.unique(np.linspace(0, n_tokens - 1, 6).astype(int)):
            d, rq, rb = oracle.quantize_row_q8_k(x[t], A)
            assert np.array_equal(rq, qs[t]) and np.array_equal(rb, bs[t])
            want = oracle.q4k_q8k_block_ints_matrix(w, n_out, qs[t], bs[t])
            assert np.array_equal(ints[t], want), t
            ref = np.zeros(n_out, np.float32)
            oracle.q4k_forward_prepared(w, d, qs[t], bs[t], ref, n_in, n_out, 0, 1, A)
            assert np.all(np.abs(out[t] - ref) <= 1e-4 + 1e-4 * np.abs(ref)), t
            exact = np.sum(wd * d.astype(np.float64)[None, :] * want[:, :, 0] - wdmin * d.astype(np.float64)[None, :] * want[:, :, 1], axis=1)
            scale = np.sum(np.abs(wd * d[None, :] * want[:, :, 0]) + np.abs(wdmin * d[None, :] * want[:, :, 1]), axis=1)
            assert np.all(np.abs(out[t].astype(np.float64) - exact) <= 2e-6 * scale + 1e-30), t
