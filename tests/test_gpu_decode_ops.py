"""Per-kernel parity of the device-resident decode step, through the C ABI, bit for bit against the
restated CPU pieces of Qwen3Session::generate_inner (rms_norm + quantizer, q/k norm + RoPE + f16
rounding, F16-cache attention + quantizer, SiLU*up + quantizer).  Many random draws each: what can go
wrong here is rare (a rounding tie, a last-bit difference before a rounding to int8 or f16)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

A = 1  # AVX2 rounding of the activation quantizer, as the x86-64 reference build


def _quant(oracle, v):
    q8, sc = oracle.quantize_q8_0(np.ascontiguousarray(v, np.float32), A)
    return q8.view(np.int8), sc


def _dev(H, a):
    return H.DeviceBuffer.from_array(np.ascontiguousarray(a))


@pytest.mark.parametrize("n", [1024, 512, 3072, 96])
def test_rms_norm_quantize(hip, oracle, n):
    H = hip.hip
    rng = np.random.default_rng(n)
    for trial in range(60):
        x = (rng.normal(0, 1, n) * rng.choice([1e-3, 1.0, 30.0])).astype(np.float32)
        x[rng.integers(0, n, 3)] *= 50.0  # outliers, as residual streams have
        r = rng.normal(0, 0.5, n).astype(np.float32) if trial % 2 else None
        w = (1.0 + 0.1 * rng.normal(0, 1, n)).astype(np.float32)
        d_x, d_w = _dev(H, x), _dev(H, w)
        d_r = _dev(H, r) if r is not None else None
        d_q, d_s = H.DeviceBuffer(n), H.DeviceBuffer(n // 32 * 4)
        H.check(H.lib.rmi_hip_rms_norm_quantize_q8_0_dev(d_x.ptr, d_r.ptr if d_r else None, d_w.ptr, n, 1e-6, d_q.ptr,
                                                         d_s.ptr, A, None))
        H.check(H.lib.rmi_hip_synchronize())
        xs = x + r if r is not None else x
        assert np.array_equal(d_x.to_array(np.float32, (n,)).view(np.uint32), xs.view(np.uint32))
        q_ref, s_ref = _quant(oracle, oracle.rms_norm(xs, w, 1e-6))
        assert np.array_equal(d_q.to_array(np.int8, (n,)), q_ref), trial
        assert np.array_equal(d_s.to_array(np.float32, (n // 32,)).view(np.uint32), s_ref.view(np.uint32)), trial
        for b in (d_x, d_w, d_q, d_s) + ((d_r,) if d_r else ()):
            b.free()


@pytest.mark.parametrize("n_in,n_out", [(1024, 4096), (1024, 6144), (256, 13), (2048, 1000), (1024, 8320), (1536, 520)])
def test_rms_norm_gemv_fused(hip, oracle, n_in, n_out):
    """add + rms_norm + quantize folded into the Q8_0 product (src/models/qwen3.rs:719-774): the same bits
    as the three restated steps followed by the restated AVX2 matmul.  (Rows of 4 or 8 octets in up to 512 tiles
    take a tile on four waves, the others a wave a tile.)"""
    H, K = hip.hip, hip.kernel
    rng = np.random.default_rng(n_in + n_out)
    w = hip.synth.q8_0_weight(900 + n_out, n_out, n_in)
    kernel = K.Q8Kernel(w, n_in, n_out)
    for trial in range(12):
        x = (rng.normal(0, 1, n_in) * rng.choice([1e-3, 1.0, 30.0])).astype(np.float32)
        x[rng.integers(0, n_in, 3)] *= 50.0
        r = rng.normal(0, 0.5, n_in).astype(np.float32) if trial % 2 else None
        nw = (1.0 + 0.1 * rng.normal(0, 1, n_in)).astype(np.float32)
        d_x, d_w = _dev(H, x), _dev(H, nw)
        d_r = _dev(H, r) if r is not None else None
        d_xo, d_y = H.DeviceBuffer(n_in * 4), H.DeviceBuffer(n_out * 4)
        H.check(H.lib.rmi_hip_rms_norm_gemv_q8_0_dev(kernel.w.handle, d_x.ptr, d_r.ptr if d_r else None, d_w.ptr, 1e-6, A,
                                                     d_xo.ptr, d_y.ptr, None))
        H.check(H.lib.rmi_hip_synchronize())
        xs = x + r if r is not None else x
        assert np.array_equal(d_xo.to_array(np.float32, (n_in,)).view(np.uint32), xs.view(np.uint32))
        assert np.array_equal(d_x.to_array(np.float32, (n_in,)).view(np.uint32), x.view(np.uint32))  # input untouched
        q_ref, s_ref = oracle.quantize_q8_0(oracle.rms_norm(xs, nw, 1e-6), A)
        y_ref = oracle.matmul_q8_0_quantized(w, q_ref, s_ref, n_in, n_out, A)
        assert np.array_equal(d_y.to_array(np.float32, (n_out,)).view(np.uint32), y_ref.view(np.uint32)), trial
        for b in (d_x, d_w, d_xo, d_y) + ((d_r,) if d_r else ()):
            b.free()
    # shapes the fused kernel does not cover are refused, not mis-computed
    big = K.Q8Kernel(hip.synth.q8_0_weight(1, 8, 4096), 4096, 8)
    d = H.DeviceBuffer(4096 * 4)
    assert H.lib.rmi_hip_rms_norm_gemv_q8_0_dev(big.w.handle, d.ptr, None, d.ptr, 1e-6, A, d_y.ptr, d_y.ptr, None) != 0


@pytest.mark.parametrize("n_in,n_ff", [(1024, 3072), (2048, 6144), (256, 32), (512, 96)])
def test_rms_norm_ffn_gate_up_fused(hip, oracle, n_in, n_ff):
    """norm + gate/up products + SiLU*up + quantizer in one launch (src/models/qwen3.rs:1016-1027): the same
    bits as the restated steps one after the other."""
    H, K = hip.hip, hip.kernel
    rng = np.random.default_rng(n_in + n_ff)
    wg = hip.synth.q8_0_weight(910 + n_ff, n_ff, n_in, scale_sigma=0.05)
    wu = hip.synth.q8_0_weight(911 + n_ff, n_ff, n_in, scale_sigma=0.05)
    fused = K.fuse_vstack(K.Q8Kernel(wg, n_in, n_ff), K.Q8Kernel(wu, n_in, n_ff))
    for trial in range(10):
        x = (rng.normal(0, 1, n_in) * rng.choice([0.1, 1.0, 30.0])).astype(np.float32)
        r = rng.normal(0, 0.5, n_in).astype(np.float32) if trial % 2 else None
        nw = (1.0 + 0.1 * rng.normal(0, 1, n_in)).astype(np.float32)
        d_x, d_w = _dev(H, x), _dev(H, nw)
        d_r = _dev(H, r) if r is not None else None
        d_xo, d_q, d_s = H.DeviceBuffer(n_in * 4), H.DeviceBuffer(n_ff), H.DeviceBuffer(n_ff // 32 * 4)
        H.check(H.lib.rmi_hip_rms_norm_ffn_gate_up_q8_0_dev(fused.w.handle, d_x.ptr, d_r.ptr if d_r else None, d_w.ptr,
                                                            1e-6, A, d_xo.ptr, d_q.ptr, d_s.ptr, None))
        H.check(H.lib.rmi_hip_synchronize())
        xs = x + r if r is not None else x
        assert np.array_equal(d_xo.to_array(np.float32, (n_in,)).view(np.uint32), xs.view(np.uint32))
        q_in, s_in = oracle.quantize_q8_0(oracle.rms_norm(xs, nw, 1e-6), A)
        g = oracle.matmul_q8_0_quantized(wg, q_in, s_in, n_in, n_ff, A)
        u = oracle.matmul_q8_0_quantized(wu, q_in, s_in, n_in, n_ff, A)
        q_ref, s_ref = _quant(oracle, oracle.silu_mul(g, u))
        assert np.array_equal(d_q.to_array(np.int8, (n_ff,)), q_ref), trial
        assert np.array_equal(d_s.to_array(np.float32, (n_ff // 32,)).view(np.uint32), s_ref.view(np.uint32)), trial
        for b in (d_x, d_w, d_xo, d_q, d_s) + ((d_r,) if d_r else ()):
            b.free()


def test_silu_mul_quantize(hip, oracle):
    H = hip.hip
    rng = np.random.default_rng(3)
    n_ff = 3072
    for trial in range(40):
        gu = (rng.normal(0, 1, 2 * n_ff) * rng.choice([0.05, 1.0, 8.0, 40.0])).astype(np.float32)
        d_gu, d_q, d_s = _dev(H, gu), H.DeviceBuffer(n_ff), H.DeviceBuffer(n_ff // 32 * 4)
        H.check(H.lib.rmi_hip_silu_mul_quantize_q8_0_dev(d_gu.ptr, n_ff, d_q.ptr, d_s.ptr, A, None))
        H.check(H.lib.rmi_hip_synchronize())
        q_ref, s_ref = _quant(oracle, oracle.silu_mul(gu[:n_ff], gu[n_ff:]))
        assert np.array_equal(d_q.to_array(np.int8, (n_ff,)), q_ref), trial
        assert np.array_equal(d_s.to_array(np.float32, (n_ff // 32,)).view(np.uint32), s_ref.view(np.uint32)), trial
        for b in (d_gu, d_q, d_s):
            b.free()


@pytest.mark.parametrize("hk", [128, 64])
def test_qk_norm_rope_f16(hip, oracle, hk):
    H = hip.hip
    rng = np.random.default_rng(hk)
    n_head, n_kv, hv = 16, 8, hk
    n_q, n_k, n_v = n_head * hk, n_kv * hk, n_kv * hv
    for trial in range(40):
        pos = int(rng.integers(0, 4000))
        qkv = (rng.normal(0, 1, n_q + n_k + n_v) * rng.choice([0.1, 1.0, 20.0])).astype(np.float32)
        qn = (1.0 + 0.2 * rng.normal(0, 1, hk)).astype(np.float32)
        kn = (1.0 + 0.2 * rng.normal(0, 1, hk)).astype(np.float32)
        with_norm = trial % 3 != 0
        c, s = oracle.rope_angles(pos, hk, 1e6)
        d = [_dev(H, a) for a in (qkv, qn, kn, c, s)]
        d_q16, d_k, d_v = H.DeviceBuffer(n_q * 2), H.DeviceBuffer(n_k * 2), H.DeviceBuffer(n_v * 2)
        H.check(H.lib.rmi_hip_qk_norm_rope_f16_dev(d[0].ptr, d[1].ptr if with_norm else None,
                                                   d[2].ptr if with_norm else None, d[3].ptr, d[4].ptr, d_q16.ptr,
                                                   d_k.ptr, d_v.ptr, n_head, n_kv, hk, hv, 1e-6, None))
        H.check(H.lib.rmi_hip_synchronize())

        def ref_heads(vec, n, w):
            out = []
            for h in range(n):
                x = vec[h * hk:(h + 1) * hk]
                if with_norm:
                    x = oracle.rms_norm(x, w, 1e-6)
                out.append(oracle.rope_neox(x, pos, 1e6))
            return np.concatenate(out).astype(np.float16).view(np.uint16)

        assert np.array_equal(d_q16.to_array(np.uint16, (n_q,)), ref_heads(qkv[:n_q], n_head, qn)), trial
        assert np.array_equal(d_k.to_array(np.uint16, (n_k,)), ref_heads(qkv[n_q:n_q + n_k], n_kv, kn)), trial
        assert np.array_equal(d_v.to_array(np.uint16, (n_v,)), qkv[n_q + n_k:].astype(np.float16).view(np.uint16))
        for b in d + [d_q16, d_k, d_v]:
            b.free()


@pytest.mark.parametrize("n_in,n_head,n_kv", [(1024, 16, 8), (512, 4, 4), (256, 3, 1)])
def test_rms_norm_qkv_rope_fused(hip, oracle, n_in, n_head, n_kv):
    """norm + q/k/v products + head norms + rotation + f16 rounding in one launch (src/models/qwen3.rs:719-874):
    the same bits as the restated steps one after the other."""
    H, K = hip.hip, hip.kernel
    rng = np.random.default_rng(n_in + n_head)
    hk = 128
    n_q, n_k = n_head * hk, n_kv * hk
    wq = hip.synth.q8_0_weight(920, n_q, n_in, scale_sigma=0.05)
    wk = hip.synth.q8_0_weight(921, n_k, n_in, scale_sigma=0.05)
    wv = hip.synth.q8_0_weight(922, n_k, n_in, scale_sigma=0.05)
    fused = K.fuse_vstack(K.fuse_vstack(K.Q8Kernel(wq, n_in, n_q), K.Q8Kernel(wk, n_in, n_k)), K.Q8Kernel(wv, n_in, n_k))
    for trial in range(10):
        pos = int(rng.integers(0, 4000))
        x = (rng.normal(0, 1, n_in) * rng.choice([0.1, 1.0, 30.0])).astype(np.float32)
        r = rng.normal(0, 0.5, n_in).astype(np.float32) if trial % 2 else None
        nw = (1.0 + 0.1 * rng.normal(0, 1, n_in)).astype(np.float32)
        qn = (1.0 + 0.2 * rng.normal(0, 1, hk)).astype(np.float32)
        kn = (1.0 + 0.2 * rng.normal(0, 1, hk)).astype(np.float32)
        with_norm = trial % 3 != 0
        c, s = oracle.rope_angles(pos, hk, 1e6)
        d = [_dev(H, a) for a in (x, nw, qn, kn, c, s)]
        d_r = _dev(H, r) if r is not None else None
        d_xo, d_q16, d_k, d_v = H.DeviceBuffer(n_in * 4), H.DeviceBuffer(n_q * 2), H.DeviceBuffer(n_k * 2), H.DeviceBuffer(n_k * 2)
        H.check(H.lib.rmi_hip_rms_norm_qkv_rope_q8_0_dev(fused.w.handle, d[0].ptr, d_r.ptr if d_r else None, d[1].ptr, 1e-6,
                                                         A, d_xo.ptr, d[2].ptr if with_norm else None,
                                                         d[3].ptr if with_norm else None, d[4].ptr, d[5].ptr, d_q16.ptr,
                                                         d_k.ptr, d_v.ptr, n_head, n_kv, None))
        H.check(H.lib.rmi_hip_synchronize())
        xs = x + r if r is not None else x
        assert np.array_equal(d_xo.to_array(np.float32, (n_in,)).view(np.uint32), xs.view(np.uint32))
        q_in, s_in = oracle.quantize_q8_0(oracle.rms_norm(xs, nw, 1e-6), A)
        qv = oracle.matmul_q8_0_quantized(wq, q_in, s_in, n_in, n_q, A)
        kv = oracle.matmul_q8_0_quantized(wk, q_in, s_in, n_in, n_k, A)
        vv = oracle.matmul_q8_0_quantized(wv, q_in, s_in, n_in, n_k, A)

        def ref_heads(vec, n, w):
            out = []
            for h in range(n):
                hx = vec[h * hk:(h + 1) * hk]
                if with_norm:
                    hx = oracle.rms_norm(hx, w, 1e-6)
                out.append(oracle.rope_neox(hx, pos, 1e6))
            return np.concatenate(out).astype(np.float16).view(np.uint16)

        assert np.array_equal(d_q16.to_array(np.uint16, (n_q,)), ref_heads(qv, n_head, qn)), trial
        assert np.array_equal(d_k.to_array(np.uint16, (n_k,)), ref_heads(kv, n_kv, kn)), trial
        assert np.array_equal(d_v.to_array(np.uint16, (n_k,)), vv.astype(np.float16).view(np.uint16)), trial
        for b in d + [d_xo, d_q16, d_k, d_v] + ([d_r] if d_r else []):
            b.free()


@pytest.mark.parametrize("hk,n_head,n_kv", [(128, 16, 8), (64, 8, 4)])
def test_attention_f16_quantize(hip, oracle, hk, n_head, n_kv):
    H = hip.hip
    rng = np.random.default_rng(hk + 1)
    hv = hk
    kv_stride = n_kv * hk
    # 5000 and 12000 keys take more than the default 64 KiB of LDS per workgroup; from 1280 keys on, head dimension
    # 128 goes through the launches that split a head's keys over workgroups (5 to 16 parts of whole 64-key groups);
    # from 64 keys up to there a head is four workgroups of one launch, whose key slices outgrow their prefetch at 768
    for n_keys in [1, 2, 7, 8, 9, 36, 63, 64, 255, 256, 257, 383, 640, 767, 768, 769, 833, 1025, 1279, 1280, 1281, 2048, 4097, 5000, 12000]:
        for trial in range(3 if n_keys < 1000 else 1):
            scale = rng.choice([0.3, 1.0, 3.0])
            q = (rng.normal(0, 1, n_head * hk) * scale).astype(np.float32)
            kc = (rng.normal(0, 1, (n_keys, kv_stride)) * scale).astype(np.float16).view(np.uint16)
            vc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
            d_q, d_k, d_v = _dev(H, q.astype(np.float16).view(np.uint16)), _dev(H, kc), _dev(H, vc)
            d_o, d_s = H.DeviceBuffer(n_head * hv), H.DeviceBuffer(n_head * hv // 32 * 4)
            H.check(H.lib.rmi_hip_attention_f16_quantize_q8_0_dev(d_q.ptr, d_k.ptr, d_v.ptr, n_keys, kv_stride, n_head,
                                                                  n_kv, hk, hv, d_o.ptr, d_s.ptr, A, None))
            H.check(H.lib.rmi_hip_synchronize())
            ref = oracle.attention_f16(q, kc, vc, n_keys - 1, kv_stride, n_head, n_kv, hk, hv)
            q_ref, s_ref = _quant(oracle, ref)
            assert np.array_equal(d_o.to_array(np.int8, (n_head * hv,)), q_ref), (n_keys, trial)
            assert np.array_equal(d_s.to_array(np.float32, (n_head * hv // 32,)).view(np.uint32),
                                  s_ref.view(np.uint32)), (n_keys, trial)
            for b in (d_q, d_k, d_v, d_o, d_s):
                b.free()


def test_attention_split_mixed_head_counts(hip, oracle):
    """Head dimension 128 from 1280 keys on: launches with different head counts and key counts in turn share the
    calling thread's scratch region (partial sums, arrival counters); every result has the checker's bits."""
    H = hip.hip
    rng = np.random.default_rng(77)
    hk = hv = 128
    for n_head, n_kv, n_keys in [(32, 8, 4097), (6, 2, 1500), (16, 8, 1281), (32, 4, 1280), (6, 6, 2300), (16, 8, 640), (32, 8, 1024), (8, 8, 1344)]:
        kv_stride = n_kv * hk
        q = rng.normal(0, 1, n_head * hk).astype(np.float32)
        kc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        vc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        d_q, d_k, d_v = _dev(H, q.astype(np.float16).view(np.uint16)), _dev(H, kc), _dev(H, vc)
        d_o, d_s = H.DeviceBuffer(n_head * hv), H.DeviceBuffer(n_head * hv // 32 * 4)
        for _ in range(2):  # the second call meets the counters as the first left them
            H.check(H.lib.rmi_hip_attention_f16_quantize_q8_0_dev(d_q.ptr, d_k.ptr, d_v.ptr, n_keys, kv_stride, n_head,
                                                                  n_kv, hk, hv, d_o.ptr, d_s.ptr, A, None))
        H.check(H.lib.rmi_hip_synchronize())
        ref = oracle.attention_f16(q, kc, vc, n_keys - 1, kv_stride, n_head, n_kv, hk, hv)
        q_ref, s_ref = _quant(oracle, ref)
        assert np.array_equal(d_o.to_array(np.int8, (n_head * hv,)), q_ref), (n_head, n_kv, n_keys)
        assert np.array_equal(d_s.to_array(np.float32, (n_head * hv // 32,)).view(np.uint32), s_ref.view(np.uint32)), (n_head, n_kv, n_keys)
        for b in (d_q, d_k, d_v, d_o, d_s):
            b.free()


def test_attention_reserve_then_calls_allocate_nothing(hip, oracle):
    """rmi_hip_attention_reserve makes the calling thread's scratch for the two-launch attention ahead of time: a call
    over 1024 keys from a thread that reserved first leaves the device's free memory as it was (the HIP runtime is the
    meter), and has the checker's bits.  Between the 13 000 keys one workgroup holds and the 16 384 the two launches
    hold, the call is accepted as well (the LDS figure that is checked is that of the path taken)."""
    import ctypes
    import threading

    H = hip.hip
    rt = ctypes.CDLL("libamdhip64.so")
    rt.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    rng = np.random.default_rng(91)
    hk = hv = 128
    for n_head, n_kv, n_keys in [(16, 8, 1024), (2, 1, 14000)]:
        kv_stride = n_kv * hk
        q = rng.normal(0, 1, n_head * hk).astype(np.float32)
        kc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        vc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        d_q, d_k, d_v = _dev(H, q.astype(np.float16).view(np.uint16)), _dev(H, kc), _dev(H, vc)
        d_o, d_s = H.DeviceBuffer(n_head * hv), H.DeviceBuffer(n_head * hv // 32 * 4)
        H.check(H.lib.rmi_hip_synchronize())
        seen = {}

        def call():
            seen["reserve"] = H.lib.rmi_hip_attention_reserve(n_head, n_keys)
            seen["free_before"] = free_bytes()
            seen["rc"] = H.lib.rmi_hip_attention_f16_quantize_q8_0_dev(d_q.ptr, d_k.ptr, d_v.ptr, n_keys, kv_stride, n_head,
                                                                      n_kv, hk, hv, d_o.ptr, d_s.ptr, A, None)
            seen["free_after"] = free_bytes()
            seen["sync"] = H.lib.rmi_hip_synchronize()  # before the thread, and with it its scratch, goes away

        t = threading.Thread(target=call)
        t.start()
        t.join()
        assert seen["reserve"] == 0 and seen["rc"] == 0 and seen["sync"] == 0, (seen, H.last_error())
        assert seen["free_after"] == seen["free_before"], (n_head, n_keys)
        ref = oracle.attention_f16(q, kc, vc, n_keys - 1, kv_stride, n_head, n_kv, hk, hv)
        q_ref, s_ref = _quant(oracle, ref)
        assert np.array_equal(d_o.to_array(np.int8, (n_head * hv,)), q_ref), (n_head, n_keys)
        assert np.array_equal(d_s.to_array(np.float32, (n_head * hv // 32,)).view(np.uint32), s_ref.view(np.uint32))
        for b in (d_q, d_k, d_v, d_o, d_s):
            b.free()
    assert H.lib.rmi_hip_attention_reserve(0, 1024) != 0


@pytest.mark.parametrize("n_head,n_kv,with_norm", [(16, 8, True), (16, 8, False), (6, 6, True), (32, 4, True)])
def test_qkv_attention_in_one_launch_equals_the_two_calls(hip, oracle, n_head, n_kv, with_norm):
    """rmi_hip_qkv_attention_f16_quantize_q8_0_dev against rmi_hip_qk_norm_rope_f16_dev followed by
    rmi_hip_attention_f16_quantize_q8_0_dev: the quantized output, its scales and the two cache rows of the new
    position, bit for bit, from the first position (no cached key) to several hundred; the other cache rows
    untouched.  The two calls are held to the checker elsewhere in this file."""
    H = hip.hip
    rng = np.random.default_rng(n_head * 31 + n_kv)
    hd = 128
    kv_stride = n_kv * hd + 8  # rows wider than the heads: the stride is not the width
    for n_keys in [1, 2, 3, 16, 17, 33, 127, 128, 129, 257, 512, 640, 767, 769, 1024, 1279]:
        scale = rng.choice([0.3, 1.0, 3.0])
        qkv = (rng.normal(0, 1, (n_head + 2 * n_kv) * hd) * scale).astype(np.float32)
        qn = rng.normal(1, 0.2, hd).astype(np.float32)
        kn = rng.normal(1, 0.2, hd).astype(np.float32)
        ang = rng.uniform(-3, 3, 64)
        cs, sn = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        kc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        vc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
        kc[-1] = 0x7e00  # the new position's rows hold NaN until the call fills them
        vc[-1] = 0x7e00
        d_qkv, d_qn, d_kn, d_cs, d_sn = (_dev(H, a) for a in (qkv, qn, kn, cs, sn))
        outs = []
        for fused in (False, True):
            d_k, d_v = _dev(H, kc), _dev(H, vc)
            d_o, d_s = H.DeviceBuffer(n_head * hd), H.DeviceBuffer(n_head * hd // 32 * 4)
            row = (n_keys - 1) * kv_stride * 2
            if fused:
                H.check(H.lib.rmi_hip_qkv_attention_f16_quantize_q8_0_dev(
                    d_qkv.ptr, d_qn.ptr if with_norm else None, d_kn.ptr if with_norm else None, d_cs.ptr, d_sn.ptr, d_k.ptr,
                    d_v.ptr, n_keys, kv_stride, n_head, n_kv, 1e-6, d_o.ptr, d_s.ptr, A, None))
            else:
                d_q16 = H.DeviceBuffer(n_head * hd * 2)
                H.check(H.lib.rmi_hip_qk_norm_rope_f16_dev(d_qkv.ptr, d_qn.ptr if with_norm else None,
                                                          d_kn.ptr if with_norm else None, d_cs.ptr, d_sn.ptr, d_q16.ptr,
                                                          d_k.ptr + row, d_v.ptr + row, n_head, n_kv, hd, hd, 1e-6, None))
                H.check(H.lib.rmi_hip_attention_f16_quantize_q8_0_dev(d_q16.ptr, d_k.ptr, d_v.ptr, n_keys, kv_stride, n_head,
                                                                      n_kv, hd, hd, d_o.ptr, d_s.ptr, A, None))
            H.check(H.lib.rmi_hip_synchronize())
            outs.append((d_o.to_array(np.int8, (n_head * hd,)), d_s.to_array(np.uint32, (n_head * hd // 32,)),
                         d_k.to_array(np.uint16, (n_keys, kv_stride)), d_v.to_array(np.uint16, (n_keys, kv_stride))))
            for b in (d_k, d_v, d_o, d_s):
                b.free()
        (o0, s0, k0, v0), (o1, s1, k1, v1) = outs
        assert np.array_equal(k0, k1) and np.array_equal(v0, v1), n_keys
        assert np.array_equal(k1[:-1], kc[:-1]) and np.array_equal(v1[:-1], vc[:-1]), n_keys
        assert not (k1[-1, :n_kv * hd] == 0x7e00).any() and np.all(k1[-1, n_kv * hd:] == 0x7e00), n_keys
        assert np.array_equal(o0, o1) and np.array_equal(s0, s1), n_keys
        for b in (d_qkv, d_qn, d_kn, d_cs, d_sn):
            b.free()
    # beyond what it holds: refused with the way out named
    d = H.DeviceBuffer(64)
    rc = H.lib.rmi_hip_qkv_attention_f16_quantize_q8_0_dev(d.ptr, None, None, d.ptr, d.ptr, d.ptr, d.ptr, 5000, 1024, 16, 8,
                                                           1e-6, d.ptr, d.ptr, A, None)
    assert rc == -1 and "rmi_hip_qk_norm_rope_f16_dev" in H.last_error()
