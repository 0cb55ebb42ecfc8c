"""The entry point that allocates nothing, rmi_hip_q8_0_forward_noalloc_dev, against the entry point it is a
variant of (rmi_hip_q8_0_forward_batched), bit for bit, through the C ABI: two calls in a row that share the
library's fixed scratch array, the second with a smaller input; then the size limit."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu


def _both(hip, seed, n_out, n_in, n_tokens, rounding):
    H = hip.hip
    w = hip.synth.q8_0_weight(seed, n_out, n_in)
    x = hip.synth.activations(seed + 1, n_tokens, n_in)
    kernel = hip.kernel.Q8Kernel(w, n_in, n_out)
    want = np.zeros((n_tokens, n_out), np.float32)
    H.check(H.lib.rmi_hip_q8_0_forward_batched(kernel.w.handle, H.ptr(H.as_f32(x), H._f32p), H.ptr(want, H._f32p), n_in,
                                               n_out, n_tokens, rounding))
    d_x = H.DeviceBuffer.from_array(H.as_f32(x))
    d_y = H.DeviceBuffer.from_array(np.full((n_tokens, n_out), np.nan, np.float32))
    H.check(H.lib.rmi_hip_q8_0_forward_noalloc_dev(kernel.w.handle, d_x.ptr, d_y.ptr, n_tokens, n_out, rounding, None))
    H.check(H.lib.rmi_hip_synchronize())
    got = d_y.to_array(np.float32, (n_tokens, n_out))
    d_x.free()
    d_y.free()
    return got, want


def test_noalloc_equals_forward_batched_twice_second_smaller(hip):
    H = hip.hip
    print("noalloc case 1: 3072x1024, 8 tokens, ties-even", flush=True)
    got, want = _both(hip, 910, 3072, 1024, 8, H.ROUND_TIES_EVEN)
    assert np.array_equal(bits(got), bits(want))
    assert np.isfinite(got).all() and np.abs(got).max() > 0
    # the second call finds the first call's quants in the scratch array and must not read past its own
    print("noalloc case 2: 203x512, 3 tokens, half-away", flush=True)
    got, want = _both(hip, 920, 203, 512, 3, H.ROUND_HALF_AWAY)
    assert np.array_equal(bits(got), bits(want))
    print("noalloc case 3: 1024x3072, 1 token", flush=True)
    got, want = _both(hip, 930, 1024, 3072, 1, H.ROUND_TIES_EVEN)
    assert np.array_equal(bits(got), bits(want))


def test_noalloc_rejects_sizes_beyond_the_scratch(hip):
    H = hip.hip
    n_in, n_out = 1024, 64
    kernel = hip.kernel.Q8Kernel(hip.synth.q8_0_weight(940, n_out, n_in), n_in, n_out)
    n_tokens = H.NOALLOC_MAX_ELEMS // n_in + 1
    d_x = H.DeviceBuffer(n_tokens * n_in * 4)
    d_y = H.DeviceBuffer(n_tokens * n_out * 4)
    rc = H.lib.rmi_hip_q8_0_forward_noalloc_dev(kernel.w.handle, d_x.ptr, d_y.ptr, n_tokens, n_out, H.ROUND_TIES_EVEN, None)
    assert rc == -1 and "exceed the fixed scratch" in H.last_error()
    # the limit itself is accepted
    H.check(H.lib.rmi_hip_q8_0_forward_noalloc_dev(kernel.w.handle, d_x.ptr, d_y.ptr, n_tokens - 1, n_out,
                                                   H.ROUND_TIES_EVEN, None))
    H.check(H.lib.rmi_hip_synchronize())
    d_x.free()
    d_y.free()


def test_shutdown_then_init_rebuilds_the_calling_threads_stream(hip, oracle):
    """After rmi_hip_shutdown and a new rmi_hip_init the same host thread gets a fresh stream and staging instead of
    running on the emptied ones; threads that come and go reuse each other's contexts.  (Here, in the file that
    runs last, because shutdown frees every thread's staging.)"""
    import threading

    H = hip.hip
    n_out, n_in = 264, 512
    w = hip.synth.q8_0_weight(950, n_out, n_in)
    x = hip.synth.activations(951, 1, n_in)[0]
    q8, sc = oracle.quantize_q8_0(x, 1)
    ref = oracle.matmul_q8_0_quantized(w, q8, sc, n_in, n_out, 1)

    def run():
        out = np.zeros(n_out, np.float32)
        hip.kernel.Q8Kernel(w, n_in, n_out).forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
        return np.array_equal(bits(out), bits(ref))

    assert run()
    H.lib.rmi_hip_shutdown()
    assert H.lib.rmi_hip_synchronize() == -3
    H.init(0)
    assert run() and run()
    before = H.lib.rmi_hip_thread_context_count()
    results = []
    for _ in range(6):  # six threads one after the other: at most one more context than before
        t = threading.Thread(target=lambda: results.append(run()))
        t.start()
        t.join()
    assert results == [True] * 6
    assert H.lib.rmi_hip_thread_context_count() <= before + 1
