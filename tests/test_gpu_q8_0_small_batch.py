"""The small-batch Q8_0 kernel on the matrix cores (1..64 tokens, weights streamed once): every output must have
the bits of the reference's NEON kernel, sum = fma(float(dot_b), f32(w.d_b) * x_scale_b, sum) block after block
(src/ops/kernel/q8_0/neon.rs:49-73; the order is pinned by the reference's own vector, src/ops/matmul_tests.rs:
288-306, in test_oracle_q8_0.py), and lie within 1e-4 + 1e-4*|ref| of the AVX2 kernel's."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu

A, N = 1, 2  # the checker's AVX2-order and NEON-order variants


def TOL(ref):
    return 1e-4 + 1e-4 * np.abs(ref)


def _acts(hip, oracle, seed, n_tokens, n_in):
    x = hip.synth.activations(seed, n_tokens, n_in)
    per = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
    return np.stack([p[0] for p in per]), np.stack([p[1] for p in per])


def _ref(oracle, w, q8, sc, n_in, n_out, variant=N):
    return np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, variant) for t in range(q8.shape[0])])


def _run(hip, oracle, seed, n_out, n_in, n_tokens, r0=0, r1=None, extra_stride=0):
    H = hip.hip
    r1 = n_out if r1 is None else r1
    stride = n_out + extra_stride
    w = hip.synth.q8_0_weight(seed, n_out, n_in)
    k = hip.kernel.Q8Kernel(w, n_in, n_out)
    q8, sc = _acts(hip, oracle, seed + 5, n_tokens, n_in)
    d_q8, d_sc = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)
    sentinel = np.full((n_tokens, stride), np.float32(-3.75))
    d_y = H.DeviceBuffer.from_array(sentinel)
    H.check(H.lib.rmi_hip_gemv_q8_0_neon_dev(k.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, stride, r0, r1, None))
    H.check(H.lib.rmi_hip_synchronize())
    got = d_y.to_array(np.float32, (n_tokens, stride))
    ref = _ref(oracle, w, q8, sc, n_in, n_out)
    assert np.array_equal(bits(got[:, r0:r1]), bits(ref[:, r0:r1])), (n_out, n_in, n_tokens, r0, r1)
    assert np.all(got[:, :r0] == sentinel[:, :r0]) and np.all(got[:, r1:] == sentinel[:, r1:]), "outside the row range"
    ref_a = _ref(oracle, w, q8, sc, n_in, n_out, A)
    assert np.all(np.abs(got[:, r0:r1] - ref_a[:, r0:r1]) <= TOL(ref_a[:, r0:r1]))


@pytest.mark.parametrize("n_tokens", [1, 2, 7, 8, 15, 16, 17, 31, 32, 33, 48, 64])
def test_token_counts(hip, oracle, n_tokens):
    """Every count of sixteens and the ragged ones between; a matrix of an odd number of tiles with a last tile of 5 rows."""
    _run(hip, oracle, 300 + n_tokens, 8 * 9 + 5, 512, n_tokens)


@pytest.mark.parametrize("n_out,n_in", [(1, 32), (9, 32), (24, 96), (61, 256), (64, 288), (1024, 3072), (2048, 1024),
                                        (1000, 2048), (8 * 2048 * 4 + 8 * 3 + 1, 256), (8 * 2048 * 2 + 3, 768)])
def test_shapes(hip, oracle, n_out, n_in):
    """Rows that are not whole octets (n_in = 32, 96, 288), one tile, runs of one pair, and launches large enough
    for runs of many pairs with a last run that is shorter and ends on a single tile."""
    for n_tokens in (3, 16, 20):
        _run(hip, oracle, 400 + n_in // 32 + n_tokens, n_out, n_in, n_tokens)


def test_row_ranges_and_stride(hip, oracle):
    n_out, n_in = 8 * 300 + 6, 1024
    _run(hip, oracle, 500, n_out, n_in, 5, r0=13, r1=n_out - 5, extra_stride=3)
    _run(hip, oracle, 501, n_out, n_in, 18, r0=8 * 100 + 7, r1=8 * 100 + 9)
    _run(hip, oracle, 502, n_out, n_in, 2, r0=8 * 17, r1=8 * 18)  # one whole tile, an odd one
    _run(hip, oracle, 503, n_out, n_in, 4, r0=500, r1=500)  # empty: nothing is written


def test_output_store_paths(hip, oracle):
    """The kernel stores a lane's four neighbouring rows as one 16-byte piece where y allows it (base 16-byte
    aligned, stride a multiple of four floats, the four rows inside the row range) and row by row elsewhere: a
    row range that cuts groups of four at both ends on an aligned stride, the same on a base that is 4 bytes off,
    and an odd number of tile pairs so that the last stores hold one pair."""
    H = hip.hip
    n_out, n_in, n_tokens = 8 * 37, 512, 11
    w = hip.synth.q8_0_weight(610, n_out, n_in)
    k = hip.kernel.Q8Kernel(w, n_in, n_out)
    q8, sc = _acts(hip, oracle, 611, n_tokens, n_in)
    d_q8, d_sc = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)
    ref = _ref(oracle, w, q8, sc, n_in, n_out)
    for stride, shift, r0, r1 in ((n_out + 8, 0, 13, n_out - 5), (n_out + 8, 1, 13, n_out - 5), (n_out, 0, 0, n_out),
                                  (n_out + 4, 1, 0, n_out), (n_out + 8, 0, 4, 8)):
        sentinel = np.full(n_tokens * stride + 4, np.float32(-3.75))
        d_y = H.DeviceBuffer.from_array(sentinel)
        H.check(H.lib.rmi_hip_gemv_q8_0_neon_dev(k.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr + 4 * shift, n_tokens, stride,
                                                 r0, r1, None))
        H.check(H.lib.rmi_hip_synchronize())
        flat = d_y.to_array(np.float32, (n_tokens * stride + 4,))
        got = flat[shift:shift + n_tokens * stride].reshape(n_tokens, stride)
        assert np.array_equal(bits(got[:, r0:r1]), bits(ref[:, r0:r1])), (stride, shift, r0, r1)
        keep = np.ones(flat.shape, bool)
        keep[shift:shift + n_tokens * stride].reshape(n_tokens, stride)[:, r0:r1] = False
        assert np.all(flat[keep] == np.float32(-3.75)), ("outside the row range", stride, shift, r0, r1)


@pytest.mark.parametrize("seed", [1, 2])
def test_grouped_launch(hip, oracle, seed):
    """One launch over a list of matrices of unlike widths and heights, 3 / 16 / 40 tokens."""
    H = hip.hip
    rng = np.random.default_rng(900 + seed)
    for n_tokens in (3, 16, 40):
        shapes = [(int(rng.integers(1, 700)), int(rng.integers(1, 14)) * 32) for _ in range(int(rng.integers(3, 10)))]
        shapes.append((int(rng.integers(30000, 50000)), 256 * int(rng.integers(1, 4))))
        ks, acts, ys, refs = [], [], [], []
        for i, (n_out, n_in) in enumerate(shapes):
            w = hip.synth.q8_0_weight(9000 + 100 * seed + i, n_out, n_in)
            ks.append(hip.kernel.Q8Kernel(w, n_in, n_out))
            q8, sc = _acts(hip, oracle, 9500 + 100 * seed + i, n_tokens, n_in)
            acts.append((H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)))
            ys.append(H.DeviceBuffer.from_array(np.full((n_tokens, n_out), np.float32(2.5))))
            refs.append(_ref(oracle, w, q8, sc, n_in, n_out))
        n = len(ks)
        arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
        g = H.lib.rmi_hip_gemv_group_create_neon(n, arr([k.w.handle for k in ks]), arr([a[0].ptr for a in acts]),
                                                 arr([a[1].ptr for a in acts]), arr([y.ptr for y in ys]), n_tokens)
        assert g, H.last_error()
        for _ in range(2):  # a group is launched many times
            H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))
        H.check(H.lib.rmi_hip_synchronize())
        for i, (n_out, n_in) in enumerate(shapes):
            got = ys[i].to_array(np.float32, (n_tokens, n_out))
            assert np.array_equal(bits(got), bits(refs[i])), (seed, n_tokens, i, n_out, n_in)
        H.lib.rmi_hip_gemv_group_destroy(g)


def test_special_scales(hip, oracle):
    """Zero, negative zero, subnormal, largest, infinite and NaN weight scales against token scales down to f32
    subnormals: the scale product must round like the f32 multiply, and NaN must appear where the CPU gives NaN."""
    H = hip.hip
    n_tokens, n_out, n_in = 21, 72, 320
    rng = np.random.default_rng(78)
    w = hip.synth.q8_0_weight(4321, n_out, n_in).reshape(n_out, n_in // 32, 34).copy()
    special = np.array([0x0000, 0x8000, 0x0001, 0x83ff, 0x7bff, 0xfbff, 0x7c00, 0xfc00, 0x7e00, 0x0400, 0x3c00], np.uint16)
    pick = rng.integers(0, special.size, (n_out, n_in // 32))
    keep = rng.random((n_out, n_in // 32)) < 0.5
    scales = w[:, :, :2].copy().view(np.uint16)[:, :, 0]
    scales = np.where(keep, scales, special[pick]).astype(np.uint16)
    w[:, :, :2] = scales[:, :, None].view(np.uint8)
    w = np.ascontiguousarray(w).reshape(-1)
    q8 = rng.integers(-127, 128, (n_tokens, n_in), dtype=np.int8)
    sc = ((rng.random((n_tokens, n_in // 32), dtype=np.float32) + 0.5) *
          np.float32(10.0) ** rng.integers(-44, 3, (n_tokens, n_in // 32)).astype(np.float32)).astype(np.float32)
    sc[rng.random(sc.shape) < 0.05] = 0.0
    k = hip.kernel.Q8Kernel(w, n_in, n_out)
    d_q8, d_sc, d_y = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc), H.DeviceBuffer(n_tokens * n_out * 4)
    H.check(H.lib.rmi_hip_gemv_q8_0_neon_dev(k.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, n_out, 0, n_out, None))
    H.check(H.lib.rmi_hip_synchronize())
    out = d_y.to_array(np.float32, (n_tokens, n_out))
    with np.errstate(all="ignore"):
        ref = _ref(oracle, w, q8.view(np.uint8), sc, n_in, n_out)
    nan_o, nan_r = np.isnan(out), np.isnan(ref)
    assert np.array_equal(nan_o, nan_r) and nan_r.any() and not nan_r.all()
    assert np.array_equal(bits(out)[~nan_o], bits(ref)[~nan_r])


@pytest.mark.parametrize("n_tokens", [9, 15, 16, 40, 64])
def test_forward_batched_takes_this_path(hip, oracle, n_tokens):
    """The matrix-core variant of Kernel::forward_batched is in the NEON order, whichever kernel runs."""
    n_out, n_in = 520, 1024
    w = hip.synth.q8_0_weight(600 + n_tokens, n_out, n_in)
    x = hip.synth.activations(610 + n_tokens, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out, matrix_cores=True)
    per = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
    ref = np.stack([oracle.matmul_q8_0_quantized(w, per[t][0], per[t][1], n_in, n_out, N) for t in range(n_tokens)])
    assert np.array_equal(bits(out), bits(ref))


def test_forward_batched_wide_rows_stay_in_this_order(hip, oracle):
    """11 tokens of 16384 elements do not fit the staging at once (and are too few for the tiled GEMM): they go
    through the same kernel a few at a time, so the order does not depend on the width."""
    n_tokens, n_out, n_in = 11, 24, 16384
    w = hip.synth.q8_0_weight(700, n_out, n_in)
    x = hip.synth.activations(701, n_tokens, n_in)
    out = np.zeros((n_tokens, n_out), np.float32)
    hip.kernel.Q8Kernel(w, n_in, n_out).forward_batched(x, out, n_in, n_out, matrix_cores=True)
    per = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
    ref = np.stack([oracle.matmul_q8_0_quantized(w, per[t][0], per[t][1], n_in, n_out, N) for t in range(n_tokens)])
    assert np.array_equal(bits(out), bits(ref))


def test_limits(hip):
    H = hip.hip
    k = hip.kernel.Q8Kernel(hip.synth.q8_0_weight(1, 16, 256), 256, 16)
    buf, y = H.DeviceBuffer(65 * 256 * 2), H.DeviceBuffer(65 * 16 * 4)
    rc = H.lib.rmi_hip_gemv_q8_0_neon_dev(k.w.handle, buf.ptr, buf.ptr + 65 * 256, y.ptr, 65, 16, 0, 16, None)
    assert rc == -1 and "tokens" in H.last_error()
    wide = hip.kernel.Q8Kernel(hip.synth.q8_0_weight(2, 8, 32768), 32768, 8)  # 16 tokens x 32768 do not fit 159 KiB
    big = H.DeviceBuffer(16 * 32768 * 2)
    rc = H.lib.rmi_hip_gemv_q8_0_neon_dev(wide.w.handle, big.ptr, big.ptr + 16 * 32768, y.ptr, 16, 8, 0, 8, None)
    assert rc == -1 and "fit" in H.last_error()
    H.check(H.lib.rmi_hip_synchronize())
