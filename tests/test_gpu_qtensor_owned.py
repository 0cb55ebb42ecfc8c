"""`QTensorOwned` over the device kernels: the reference's own tests of the type
(src/ops/kernel/qtensor_owned.rs:640-745) and `quantize_and_matmul_with_scratch` (:533-589) against the checker."""
import numpy as np
import pytest

import gen
from conftest import bits

pytestmark = pytest.mark.gpu

A = 1


def test_from_bytes_owned_shape_and_type(hip):
    K = hip.kernel
    owned = K.QTensorOwned.from_bytes_owned(gen.make_q8_0_weight(4, 64, 0), K.GGML_TYPE_Q8_0, 64, 4)
    assert owned.ggml_type() == K.GGML_TYPE_Q8_0 and owned.n_in() == 64 and owned.n_cols() == 64 and owned.n_rows() == 4
    assert K.QTensorOwned.from_bytes_owned(np.zeros(16, np.uint8), "F16", 4, 2) is None
    q = K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q8_0, gen.make_q8_0_weight(4, 64, 0), 64, 4)
    assert K.QTensorOwned.from_quantized(q).n_rows() == 4
    with pytest.raises(ValueError):
        K.QTensorOwned.from_quantized(K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q4_0, np.zeros(36, np.uint8), 64, 1))


def test_owned_kernel_matches_borrowed_kernel_bit_exact(hip, oracle):
    """qtensor_owned.rs:663-684."""
    K = hip.kernel
    data = gen.make_q8_0_weight(8, 64, 3)
    owned = K.QTensorOwned.from_bytes_owned(data, K.GGML_TYPE_Q8_0, 64, 8)
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(64), A)
    out_owned, out_borrowed = np.zeros(8, np.float32), np.zeros(8, np.float32)
    owned.forward_prequantized(q8, sc, out_owned, 64, 8, 0, 1)
    K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q8_0, data, 64, 8).into_kernel().forward_prequantized(
        q8, sc, out_borrowed, 64, 8, 0, 1)
    assert np.array_equal(bits(out_owned), bits(out_borrowed))
    assert np.array_equal(bits(out_owned), bits(oracle.matmul_q8_0_quantized(data, q8, sc, 64, 8, A)))
    out_prepared = np.zeros(8, np.float32)
    owned.forward_prepared(gen.ramp_input(64), q8, sc, None, out_prepared, 64, 8, 0, 1)  # Q8_0 ignores q8_k
    assert np.array_equal(bits(out_prepared), bits(out_owned))


def test_fuse_vstack_layout_mismatch_and_dispatch(hip, oracle):
    """qtensor_owned.rs:686-745: rows of `a` then rows of `b`; None on a column mismatch; the fused kernel's
    output is the two kernels' outputs one after the other."""
    K = hip.kernel
    gate, up = gen.make_q8_0_weight(4, 64, 0), gen.make_q8_0_weight(6, 64, 17)
    fused = K.QTensorOwned.fuse_vstack(K.QTensorOwned.from_bytes_owned(gate, K.GGML_TYPE_Q8_0, 64, 4),
                                       K.QTensorOwned.from_bytes_owned(up, K.GGML_TYPE_Q8_0, 64, 6))
    assert fused.n_rows() == 10 and fused.n_in() == 64
    a = K.QTensorOwned.from_bytes_owned(gen.make_q8_0_weight(2, 64, 0), K.GGML_TYPE_Q8_0, 64, 2)
    b = K.QTensorOwned.from_bytes_owned(gen.make_q8_0_weight(2, 32, 0), K.GGML_TYPE_Q8_0, 32, 2)
    assert K.QTensorOwned.fuse_vstack(a, b) is None
    k4 = K.QTensorOwned.from_bytes_owned(hip.synth.q4_k_weight(1, 2, 256), K.GGML_TYPE_Q4_K, 256, 2)
    k8 = K.QTensorOwned.from_bytes_owned(gen.make_q8_0_weight(2, 256, 0), K.GGML_TYPE_Q8_0, 256, 2)
    assert K.QTensorOwned.fuse_vstack(k4, k8) is None
    q8, sc = oracle.quantize_q8_0(gen.ramp_input(64), A)
    out = np.zeros(10, np.float32)
    fused.forward_prequantized(q8, sc, out, 64, 10, 0, 1)
    assert np.array_equal(bits(out[:4]), bits(oracle.matmul_q8_0_quantized(gate, q8, sc, 64, 4, A)))
    assert np.array_equal(bits(out[4:]), bits(oracle.matmul_q8_0_quantized(up, q8, sc, 64, 6, A)))


def test_quantize_and_matmul_with_scratch_q8_0(hip, oracle):
    """Q8_0 arm (qtensor_owned.rs:551-572): quantize_q8_0_into the scratch, then the row-parallel GEMV."""
    K = hip.kernel
    n_rows, n_cols = 1024, 2048
    w = hip.synth.q8_0_weight(3100, n_rows, n_cols)
    x = hip.synth.activations(3101, 1, n_cols)[0]
    owned = K.QTensorOwned.from_bytes_owned(w, K.GGML_TYPE_Q8_0, n_cols, n_rows)
    q8_buf, scale_buf, buf = np.zeros(n_cols + 64, np.uint8), np.zeros(n_cols // 32 + 2, np.float32), np.zeros(n_rows, np.float32)
    owned.quantize_and_matmul_with_scratch(x, [], q8_buf, scale_buf, buf, None)
    rq, rs = oracle.quantize_q8_0(x, A)
    assert np.array_equal(q8_buf[:n_cols], rq) and np.array_equal(bits(scale_buf[:n_cols // 32]), bits(rs))
    assert not q8_buf[n_cols:].any() and not scale_buf[n_cols // 32:].any()  # nothing written past the used part
    assert np.array_equal(bits(buf), bits(oracle.matmul_q8_0_quantized(w, rq, rs, n_cols, n_rows, A)))
    buf2 = np.zeros(n_rows, np.float32)
    owned.quantize_and_matmul(x, [], buf2)
    assert np.array_equal(bits(buf2), bits(buf))


@pytest.mark.parametrize("kind", ["Q4_K", "Q6_K"])
def test_quantize_and_matmul_with_scratch_k_quants(hip, oracle, kind):
    """K-quant arm (qtensor_owned.rs:543-550): quantize_row_q8_k_into the scratch blocks, then the Q8_K dot of
    every row (the AVX2 kernels on an x86-64 host)."""
    K = hip.kernel
    n_rows, n_cols = 300, 1024
    w = hip.synth.q4_k_weight(3200, n_rows, n_cols) if kind == "Q4_K" else hip.synth.q6_k_weight(3200, n_rows, n_cols)
    x = hip.synth.activations(3201, 1, n_cols)[0]
    owned = K.QTensorOwned.from_bytes_owned(w, kind, n_cols, n_rows)
    q8k_buf, buf = [None] * (n_cols // 256 + 1), np.zeros(n_rows, np.float32)
    owned.quantize_and_matmul_with_scratch(x, q8k_buf, None, None, buf, None)
    d, qs, bs = oracle.quantize_row_q8_k(x, A)
    assert q8k_buf[-1] is None and all(b is not None for b in q8k_buf[:-1])
    assert np.array_equal(np.concatenate([b.qs for b in q8k_buf[:-1]]), qs)
    assert np.array_equal(bits(np.array([b.d for b in q8k_buf[:-1]], np.float32)), bits(d))
    ref = np.zeros(n_rows, np.float32)
    (oracle.q4k_forward_prepared if kind == "Q4_K" else oracle.q6k_forward_prepared)(w, d, qs, bs, ref, n_cols, n_rows, 0, 1, A)
    assert np.array_equal(bits(buf), bits(ref))
    # the Q8_K helpers on the same blocks, whole and sliced
    blocks = q8k_buf[:-1]
    assert np.array_equal(bits(owned.matmul_with_q8k(blocks)), bits(ref))
    part = np.zeros(50, np.float32)
    owned.matmul_into_with_q8k(blocks, part, 100, 150)
    assert np.array_equal(bits(part), bits(ref[100:150]))
    assert np.array_equal(bits(owned.matmul(x)), bits(ref))
    with pytest.raises(ValueError):
        K.QTensorOwned.from_bytes_owned(gen.make_q8_0_weight(2, 256, 0), K.GGML_TYPE_Q8_0, 256, 2).matmul_with_q8k(blocks)
