"""The Q8_0 prefill GEMM for few tokens (rmi_hip_gemm_q8_0_ksplit_dev): one 32 x 32 tile per workgroup, the blocks
of a row split over its waves, through the C ABI.  Semantics: Kernel::forward_batched
(src/ops/kernel/trait_.rs:78-109), every token an independent GEMV.  The bar: the reference's tolerance against both
CPU accumulation orders (their per-block integer dots are the same exact integers), and, bit for bit, the checker's
statement of the split chain (runs of whole quads summed from zero in block order, the runs' sums added in run
order), which makes the result deterministic and independent of the batch."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu

S, A, N = 0, 1, 2


def TOL(ref):
    return 1e-4 + 1e-4 * np.abs(ref)


def _run(hip, kernel, q8, sc, n_tokens, n_out, y_stride=None):
    H = hip.hip
    y_stride = y_stride or n_out
    d_q8, d_sc = H.DeviceBuffer.from_array(q8), H.DeviceBuffer.from_array(sc)
    d_y = H.DeviceBuffer.from_array(np.full(n_tokens * y_stride, np.nan, np.float32))  # every output must be written
    H.check(H.lib.rmi_hip_gemm_q8_0_ksplit_dev(kernel.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, y_stride, None))
    H.check(H.lib.rmi_hip_synchronize())
    out = d_y.to_array(np.float32, (n_tokens, y_stride))
    for b in (d_q8, d_sc, d_y):
        b.free()
    return out


def _case(hip, oracle, seed, n_tokens, n_out, n_in):
    w = hip.synth.q8_0_weight(seed, n_out, n_in)
    x = hip.synth.activations(seed + 1, n_tokens, n_in)
    pairs = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
    q8 = np.stack([np.asarray(p[0]).view(np.uint8).reshape(-1) for p in pairs])
    sc = np.stack([np.asarray(p[1], np.float32).reshape(-1) for p in pairs])
    return w, q8, sc


@pytest.mark.parametrize("n_tokens", [64, 128])
@pytest.mark.parametrize("n_out,n_in", [(3072, 1024), (1024, 3072)])
def test_ksplit_ffn_shapes(hip, oracle, n_tokens, n_out, n_in):
    """Both FFN shapes of the prefill configuration at M = 64 and 128: every output within 1e-4 + 1e-4 |ref| of the
    aarch64-order and of the x86-64-order result, and equal, bit for bit, to the checker's chain cut into the runs
    the library says it uses for this row length."""
    print(f"ksplit: {n_tokens} tokens, {n_out}x{n_in}", flush=True)
    H = hip.hip
    w, q8, sc = _case(hip, oracle, 5000 + n_tokens + n_in, n_tokens, n_out, n_in)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    per = H.lib.rmi_hip_gemm_q8_0_ksplit_quads_per_part(n_in)
    assert per == (1 if n_in == 1024 else 2)
    got = _run(hip, kernel, q8, sc, n_tokens, n_out)
    want = np.stack([oracle.matmul_q8_0_neon_split(w, q8[t], sc[t], n_in, n_out, per) for t in range(n_tokens)])
    assert np.array_equal(bits(got), bits(want))
    for variant in (N, A):
        ref = np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, variant) for t in range(n_tokens)])
        assert np.all(np.abs(got - ref) <= TOL(ref))
    # the split is real: somewhere the bits differ from the single chain
    assert not np.array_equal(bits(got), bits(ref))


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(70, 200, 1120), (33, 65, 640), (1, 8, 256), (130, 300, 2048), (5, 40, 32),
                                                  (40, 33, 6144), (3, 16, 16384)])
def test_ksplit_ragged_tiles_rows_and_long_rows(hip, oracle, n_tokens, n_out, n_in):
    """Row and token counts that end inside a tile, row lengths whose last quad is partly padding (n_in / 32 not a
    multiple of 4), a single block, rows long enough for several quads a wave (6144: 3, 16384: 8), and an output
    stride wider than the row count."""
    H = hip.hip
    w, q8, sc = _case(hip, oracle, 5100 + n_tokens, n_tokens, n_out, n_in)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    per = H.lib.rmi_hip_gemm_q8_0_ksplit_quads_per_part(n_in)
    got = _run(hip, kernel, q8, sc, n_tokens, n_out, y_stride=n_out + 5)
    assert np.isnan(got[:, n_out:]).all()  # nothing written beside the rows
    got = got[:, :n_out]
    want = np.stack([oracle.matmul_q8_0_neon_split(w, q8[t], sc[t], n_in, n_out, per) for t in range(n_tokens)])
    assert np.array_equal(bits(got), bits(want))
    ref = np.stack([oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, A) for t in range(n_tokens)])
    assert np.all(np.abs(got - ref) <= TOL(ref))


def test_ksplit_does_not_depend_on_the_batch(hip, oracle):
    """A token's outputs are the same bits whether it arrives alone, in a batch of 64 or at another position."""
    n_out, n_in = 520, 1024
    w, q8, sc = _case(hip, oracle, 5200, 64, n_out, n_in)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    full = _run(hip, kernel, q8, sc, 64, n_out)
    for t in (0, 31, 32, 63):
        assert np.array_equal(bits(_run(hip, kernel, q8[t:t + 1], sc[t:t + 1], 1, n_out)[0]), bits(full[t]))
    assert np.array_equal(bits(_run(hip, kernel, q8[17:50], sc[17:50], 33, n_out)), bits(full[17:50]))


def test_ksplit_special_scales(hip, oracle):
    """Weight scales that are zero, negative zero, f16 subnormals, the largest f16, inf and NaN against token scales
    down to f32 subnormals and zero: every scale product must round like the f32 multiply, NaN for NaN."""
    n_tokens, n_out, n_in = 40, 96, 352  # 11 blocks: the last quad is partly padding
    rng = np.random.default_rng(78)
    w = hip.synth.q8_0_weight(1235, n_out, n_in).reshape(n_out, n_in // 32, 34).copy()
    special = np.array([0x0000, 0x8000, 0x0001, 0x83ff, 0x7bff, 0xfbff, 0x7c00, 0xfc00, 0x7e00, 0x0400, 0x3c00], np.uint16)
    pick = rng.integers(0, special.size, (n_out, n_in // 32))
    keep = rng.random((n_out, n_in // 32)) < 0.5
    scales = w[:, :, :2].copy().view(np.uint16)[:, :, 0]
    scales = np.where(keep, scales, special[pick]).astype(np.uint16)
    w[:, :, :2] = scales[:, :, None].view(np.uint8)
    w = np.ascontiguousarray(w).reshape(-1)
    q8 = rng.integers(-127, 128, (n_tokens, n_in), dtype=np.int8).view(np.uint8)
    sc = (rng.random((n_tokens, n_in // 32), dtype=np.float32) + 0.5) * \
        np.float32(10.0) ** rng.integers(-44, 3, (n_tokens, n_in // 32)).astype(np.float32)
    sc[rng.random(sc.shape) < 0.05] = 0.0
    sc = sc.astype(np.float32)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    per = hip.hip.lib.rmi_hip_gemm_q8_0_ksplit_quads_per_part(n_in)
    got = _run(hip, kernel, q8, sc, n_tokens, n_out)
    with np.errstate(all="ignore"):
        want = np.stack([oracle.matmul_q8_0_neon_split(w, q8[t], sc[t], n_in, n_out, per) for t in range(n_tokens)])
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    assert np.array_equal(nan_g, nan_w) and nan_w.any() and not nan_w.all()
    assert np.array_equal(bits(got)[~nan_g], bits(want)[~nan_w])


@pytest.mark.parametrize("n_tokens,n_out,n_in", [(64, 1024, 3072), (512, 3072, 1024), (512, 1024, 3072), (256, 1024, 3072),
                                                  (2048, 3072, 1024), (2048, 1024, 3072), (300, 520, 1024), (200, 260, 1120)])
def test_fast_entry_follows_its_plan(hip, oracle, n_tokens, n_out, n_in):
    """rmi_hip_gemm_q8_0_fast_dev picks a kernel per product and rmi_hip_gemm_q8_0_fast_plan names it: sampled token
    rows equal, bit for bit, the checker's statement of that plan (the single chain, the chain cut into runs of quads,
    or interleaved groups of quads), every sampled row is within tolerance of both CPU orders, and a second call
    gives the same bits."""
    import ctypes as C
    H = hip.hip
    w = hip.synth.q8_0_weight(5300 + n_tokens, n_out, n_in)
    x = hip.synth.activations(5301 + n_tokens, n_tokens, n_in)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    d_x = H.DeviceBuffer.from_array(H.as_f32(x))
    d_q8, d_sc = H.DeviceBuffer(n_tokens * n_in), H.DeviceBuffer(n_tokens * (n_in // 32) * 4)
    H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q8.ptr, d_sc.ptr, n_tokens, n_in, H.ROUND_TIES_EVEN, None))
    param = C.c_uint32(0)
    plan = H.lib.rmi_hip_gemm_q8_0_fast_plan(kernel.w.handle, n_tokens, C.byref(param))
    print(f"fast plan for {n_tokens} x {n_out}x{n_in}: kind {plan}, param {param.value}", flush=True)
    outs = []
    for _ in range(2):
        d_y = H.DeviceBuffer.from_array(np.full(n_tokens * n_out, np.nan, np.float32))
        H.check(H.lib.rmi_hip_gemm_q8_0_fast_dev(kernel.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, n_tokens, n_out, None))
        H.check(H.lib.rmi_hip_synchronize())
        outs.append(d_y.to_array(np.float32, (n_tokens, n_out)))
        d_y.free()
    assert np.array_equal(bits(outs[0]), bits(outs[1])) and not np.isnan(outs[0]).any()
    q8 = d_q8.to_array(np.uint8, (n_tokens, n_in))
    sc = d_sc.to_array(np.float32, (n_tokens, n_in // 32))
    for t in sorted({0, 1, 31, 32, 63, min(64, n_tokens - 1), n_tokens // 2, n_tokens - 2, n_tokens - 1}):
        if plan == 2:
            want = oracle.matmul_q8_0_neon_split(w, q8[t], sc[t], n_in, n_out, param.value)
        elif plan == 1:
            want = oracle.matmul_q8_0_neon_interleaved(w, q8[t], sc[t], n_in, n_out, param.value)
        else:
            want = oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, N)
        assert np.array_equal(bits(outs[0][t]), bits(want)), t
        for variant in (A, N):
            ref = oracle.matmul_q8_0_quantized(w, q8[t], sc[t], n_in, n_out, variant)
            assert np.all(np.abs(outs[0][t] - ref) <= TOL(ref)), (variant, t)
    for b in (d_x, d_q8, d_sc):
        b.free()


def test_forward_batched_mode_selects_the_path_without_touching_call_sites(hip, oracle):
    """rmi_hip_set_forward_batched_mode: the same Kernel::forward_batched call gives the x86-64 order's bits by
    default, the aarch64 order's bits in AARCH64_ORDER, and in FAST the x86-64 bits up to 8 tokens and a result within
    tolerance beyond; an unknown mode is refused and changes nothing; Q4_K follows the same switch."""
    H, K = hip.hip, hip.kernel
    n_out, n_in = 520, 1024
    w = hip.synth.q8_0_weight(5400, n_out, n_in)
    kernel = K.Q8Kernel(w, n_in, n_out)
    assert H.lib.rmi_hip_get_forward_batched_mode() == H.BATCHED_X86_ORDER
    try:
        for n_tokens in (3, 8, 40, 200):
            x = hip.synth.activations(5401 + n_tokens, n_tokens, n_in)
            pairs = [oracle.quantize_q8_0(x[t], A) for t in range(n_tokens)]
            ref = {v: np.stack([oracle.matmul_q8_0_quantized(w, p[0], p[1], n_in, n_out, v) for p in pairs]) for v in (A, N)}
            outs = {}
            for mode in (H.BATCHED_X86_ORDER, H.BATCHED_AARCH64_ORDER, H.BATCHED_FAST):
                K.set_forward_batched_mode(mode)
                outs[mode] = np.zeros((n_tokens, n_out), np.float32)
                kernel.forward_batched(x, outs[mode], n_in, n_out)
            assert np.array_equal(bits(outs[H.BATCHED_X86_ORDER]), bits(ref[A]))
            assert np.array_equal(bits(outs[H.BATCHED_AARCH64_ORDER]), bits(ref[N]))
            if n_tokens <= 8:
                assert np.array_equal(bits(outs[H.BATCHED_FAST]), bits(ref[A]))
            assert np.all(np.abs(outs[H.BATCHED_FAST] - ref[A]) <= TOL(ref[A]))
        assert H.lib.rmi_hip_set_forward_batched_mode(7) == -1 and H.lib.rmi_hip_get_forward_batched_mode() == H.BATCHED_FAST
        # Q4_K: X86_ORDER is the GEMV for every token (AVX2 order, bit for bit), the other two the GEMM from 16 tokens on
        n_out, n_in, n_tokens = 300, 1024, 48
        wk = hip.synth.q4_k_weight(5410, n_out, n_in)
        xk = hip.synth.activations(5411, n_tokens, n_in)
        kk = K.Q4_KKernel(wk, n_in, n_out)
        want = np.zeros((n_tokens, n_out), np.float32)
        for t in range(n_tokens):
            d, qs, bs = oracle.quantize_row_q8_k(xk[t], A)
            oracle.q4k_forward_prepared(wk, d, qs, bs, want[t], n_in, n_out, 0, 1, A)
        got = {}
        for mode in (H.BATCHED_X86_ORDER, H.BATCHED_FAST):
            K.set_forward_batched_mode(mode)
            got[mode] = np.zeros((n_tokens, n_out), np.float32)
            kk.forward_batched(xk, got[mode], n_in, n_out)
        assert np.array_equal(bits(got[H.BATCHED_X86_ORDER]), bits(want))
        assert np.all(np.abs(got[H.BATCHED_FAST] - want) <= TOL(want))
        assert not np.array_equal(bits(got[H.BATCHED_FAST]), bits(want))  # the matrix-core path did run
    finally:
        K.set_forward_batched_mode(H.BATCHED_X86_ORDER)
