"""GPU parity of the Q4_0 path (Q4_0Kernel), through the C ABI.

Bars: per-block int32 dots bit-exact; f32 outputs bit-exact against the restated scalar kernel
(src/ops/kernel/q4_0/scalar.rs:13-52), which the reference's AVX2 kernel equals bit for bit.
"""
import numpy as np
import pytest

import gen
from conftest import bits
from test_oracle_q4_0 import Q8_INPUTS, build_block

pytestmark = pytest.mark.gpu

A = 1


def _same(a, b):
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(bits(a)[~na], bits(b)[~nb])


def _ref(oracle, w, q8, sc, n_in, n_out):
    out = np.zeros(n_out, np.float32)
    oracle.matmul_q4_0_scalar_range(w, q8, sc, out, n_in, n_out)
    return out


@pytest.mark.parametrize("low,hi,inp,scale,xs,want", [
    (0, 0, "zero", 1.0, 1.0, 0.0), (15, 15, "zero", 1.0, 1.0, 0.0), (0, 0, "max", 1.0, 1.0, -32512.0),
    (0, 0, "min", 1.0, 1.0, 32768.0), (15, 15, "max", 1.0, 1.0, 28448.0)])
def test_q4_0_reference_closed_forms(hip, low, hi, inp, scale, xs, want):
    """src/ops/kernel/q4_0/avx2.rs:243-303."""
    k = hip.kernel.Q4_0Kernel(build_block(scale, low, hi), 32, 1)
    out = np.zeros(1, np.float32)
    k.forward_prequantized(Q8_INPUTS[inp], np.array([xs], np.float32), out, 32, 1, 0, 1)
    assert out[0] == np.float32(want)
    assert k.block_dots(Q8_INPUTS[inp])[0, 0] == int(want)


def test_q4_0_reference_mixed_cases(hip, oracle):
    """src/ops/kernel/q4_0/avx2.rs:305-329."""
    for w, q8, sc in [(build_block(0.7, 0, 15), Q8_INPUTS["linspace"], np.array([1.3], np.float32)),
                      (build_block(2.5, 8, 3), Q8_INPUTS["alt"], np.array([0.42], np.float32))]:
        out = np.zeros(1, np.float32)
        hip.kernel.Q4_0Kernel(w, 32, 1).forward_prequantized(q8, sc, out, 32, 1, 0, 1)
        assert np.array_equal(bits(out), bits(_ref(oracle, w, q8, sc, 32, 1)))


@pytest.mark.parametrize("n_out,n_in", [(3072, 1024), (1024, 3072), (1, 32), (13, 96), (100, 1056), (2048, 2048), (151, 4096)])
def test_q4_0_gemv_bit_exact(hip, oracle, n_out, n_in):
    K = hip.kernel
    w = hip.synth.q4_0_weight(500 + n_out, n_out, n_in)
    x = hip.synth.activations(501 + n_in, 1, n_in)[0] * np.float32(3.0)
    q8, sc = oracle.quantize_q8_0(x, A)
    kernel = K.Q4_0Kernel(w, n_in, n_out)
    ref = _ref(oracle, w, q8, sc, n_in, n_out)
    out = np.zeros(n_out, np.float32)
    for ith in range(3):
        kernel.forward_prequantized(q8, sc, out, n_in, n_out, ith, 3)
    assert np.array_equal(bits(out), bits(ref))
    if oracle.have_avx2():
        assert np.array_equal(bits(out), bits(oracle.x86_matmul_q4_0_range(w, q8, sc, n_in, 0, n_out)))
    dots = kernel.block_dots(q8)
    assert np.array_equal(dots, oracle.block_dots_q4_0(w, q8, n_in, n_out))
    # f32 input: the device quantizer, then the same product (Kernel::forward)
    out2 = np.zeros(n_out, np.float32)
    kernel.forward(x, out2, n_in, n_out)
    assert np.array_equal(bits(out2), bits(out))


@pytest.mark.parametrize("n_tokens", [1, 2, 5, 8, 11])
def test_q4_0_forward_batched(hip, oracle, n_tokens):
    n_out, n_in = 520, 1024
    w = hip.synth.q4_0_weight(510, n_out, n_in)
    x = hip.synth.activations(511, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q4_0Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out)
    for t in range(n_tokens):
        q8, sc = oracle.quantize_q8_0(x[t], A)
        assert np.array_equal(bits(out[t]), bits(_ref(oracle, w, q8, sc, n_in, n_out))), t


def test_q4_0_sign_of_zero_and_special_scales(hip, oracle):
    """All-zero activations, negative zero products, inf/nan block scales: same bits as the scalar kernel."""
    n_out, n_in = 24, 96  # three blocks per row: the octet is padded with five empty blocks
    rng = np.random.default_rng(3)
    w = hip.synth.q4_0_weight(520, n_out, n_in).reshape(n_out, 3, 18)
    w[0, :, 0:2] = np.array([0x8000], np.uint16).view(np.uint8)   # d = -0
    w[1, 1, 0:2] = np.array([0x7C00], np.uint16).view(np.uint8)   # d = +inf
    w[2, 2, 0:2] = np.array([0x7E00], np.uint16).view(np.uint8)   # d = nan
    w = w.reshape(-1)
    kernel = hip.kernel.Q4_0Kernel(w, n_in, n_out)
    for q8, sc in [(np.zeros(n_in, np.uint8), np.zeros(3, np.float32)),
                   (rng.integers(-127, 128, n_in, dtype=np.int8).view(np.uint8), np.array([0.5, 0.0, 0.25], np.float32)),
                   (rng.integers(-127, 128, n_in, dtype=np.int8).view(np.uint8), np.array([-0.0, 1.0, 2.0], np.float32))]:
        out = np.zeros(n_out, np.float32)
        kernel.forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
        assert _same(out, _ref(oracle, w, q8, sc, n_in, n_out))


def test_q4_0_fusion_and_errors(hip, oracle):
    H, K = hip.hip, hip.kernel
    n_in = 1024
    a = hip.synth.q4_0_weight(530, 1000, n_in)
    b = hip.synth.q4_0_weight(531, 37, n_in)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(n_in), A)
    ka, kb = K.Q4_0Kernel(a, n_in, 1000), K.Q4_0Kernel(b, n_in, 37)
    fused = K.fuse_vstack(kb, ka)  # the second weight starts inside a tile
    out = np.zeros(1037, np.float32)
    fused.forward_prequantized(q8, sc, out, n_in, 1037, 0, 1)
    assert np.array_equal(bits(out[:37]), bits(_ref(oracle, b, q8, sc, n_in, 37)))
    assert np.array_equal(bits(out[37:]), bits(_ref(oracle, a, q8, sc, n_in, 1000)))
    assert K.fuse_vstack(ka, K.Q8Kernel(gen.make_q8_0_weight(4, n_in, 0), n_in, 4)) is None
    with pytest.raises(H.RmiHipError):
        K.Q4_0Kernel(np.zeros(18, np.uint8), 48, 1)  # n_in not a multiple of 32
    with pytest.raises(H.RmiHipError):
        K.Q4_0Kernel(np.zeros(17, np.uint8), 32, 1)  # slice too short
    with pytest.raises(H.RmiHipError):  # a Q4_0 handle passed to a Q8_0 entry point is refused
        H.check(H.lib.rmi_hip_q8_0_forward_prequantized(ka.w.handle, H.ptr(q8, H._u8p), H.ptr(sc, H._f32p),
                                                        H.ptr(out, H._f32p), n_in, 1000, 0, 1))
    k2 = K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q4_0, a, n_in, 1000).into_kernel()
    assert isinstance(k2, K.Q4_0Kernel) and k2.w.dtype == H.DTYPE_Q4_0


def test_q4_0_grouped_launch_equals_the_scalar_kernel(hip, oracle):
    """One launch over a list of independent Q4_0 GEMVs of different shapes (a ragged row count, a partly filled
    octet, a wide head); mixing weight types in one group is refused."""
    H, K = hip.hip, hip.kernel
    shapes = [(2048, 1024), (1024, 1024), (1024, 2048), (3072, 1024), (1024, 3072), (4099, 1024), (13, 96), (520, 288)]
    for n_tokens in (1, 3, 8):
        kernels, xq, xs, ys, refs = [], [], [], [], []
        for i, (n_out, n_in) in enumerate(shapes):
            w = hip.synth.q4_0_weight(1300 + i, n_out, n_in)
            x = hip.synth.activations(1400 + i, n_tokens, n_in)
            qs = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
            q8, sc = np.stack([q for q, _ in qs]), np.stack([s for _, s in qs])
            kernels.append(K.Q4_0Kernel(w, n_in, n_out))
            xq.append(H.DeviceBuffer.from_array(q8))
            xs.append(H.DeviceBuffer.from_array(sc))
            ys.append(H.DeviceBuffer(n_tokens * n_out * 4))
            refs.append(np.stack([_ref(oracle, w, q8[t], sc[t], n_in, n_out) for t in range(n_tokens)]))
        n = len(shapes)
        arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
        g = H.lib.rmi_hip_gemv_group_create(n, arr([k.w.handle for k in kernels]), arr([b.ptr for b in xq]),
                                            arr([b.ptr for b in xs]), arr([b.ptr for b in ys]), n_tokens)
        assert g, H.last_error()
        H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))
        H.check(H.lib.rmi_hip_synchronize())
        for i, (n_out, _) in enumerate(shapes):
            got = ys[i].to_array(np.float32, (n_tokens, n_out))
            assert np.array_equal(bits(got), bits(refs[i])), (n_tokens, i)
        H.lib.rmi_hip_gemv_group_destroy(g)
    q8k = K.Q8Kernel(hip.synth.q8_0_weight(5, 64, 1024), 1024, 64)
    two = lambda a, b: (H.C.c_void_p * 2)(a, b)  # noqa: E731
    g = H.lib.rmi_hip_gemv_group_create(2, two(kernels[0].w.handle, q8k.w.handle), two(xq[0].ptr, xq[0].ptr),
                                        two(xs[0].ptr, xs[0].ptr), two(ys[0].ptr, ys[0].ptr), 1)
    assert not g and "bad weight handle" in H.last_error()
