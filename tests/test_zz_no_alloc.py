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


def test_noalloc_allocates_nothing_and_builds_no_thread_context(hip):
    """The property the entry point is named for: across a call made from a host thread that has never called the
    library (so it owns no stream and no staging), the device's free memory and the number of thread contexts are
    what they were.  The buffers are made before the first reading; the HIP runtime's own calls are the meter."""
    import ctypes
    import threading

    H = hip.hip
    rt = ctypes.CDLL("libamdhip64.so")
    rt.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    n_out, n_in, n_tokens = 1024, 2048, 8
    kernel = hip.kernel.Q8Kernel(hip.synth.q8_0_weight(960, n_out, n_in), n_in, n_out)
    x = hip.synth.activations(961, n_tokens, n_in)
    d_x = H.DeviceBuffer.from_array(H.as_f32(x))
    d_y = H.DeviceBuffer.from_array(np.zeros((n_tokens, n_out), np.float32))
    H.check(H.lib.rmi_hip_synchronize())
    seen = {}

    def call():
        seen["ctx_before"] = H.lib.rmi_hip_thread_context_count()
        seen["free_before"] = free_bytes()
        seen["rc"] = H.lib.rmi_hip_q8_0_forward_noalloc_dev(kernel.w.handle, d_x.ptr, d_y.ptr, n_tokens, n_out,
                                                            H.ROUND_TIES_EVEN, None)
        seen["free_after"] = free_bytes()
        seen["ctx_after"] = H.lib.rmi_hip_thread_context_count()

    t = threading.Thread(target=call)
    t.start()
    t.join()
    H.check(H.lib.rmi_hip_synchronize())
    assert seen["rc"] == 0
    assert seen["free_after"] == seen["free_before"]
    assert seen["ctx_after"] == seen["ctx_before"]
    assert np.abs(d_y.to_array(np.float32, (n_tokens, n_out))).max() > 0
    d_x.free()
    d_y.free()


def test_noalloc_refuses_a_row_too_long_for_the_staging_before_it_enqueues_anything(hip):
    H = hip.hip
    n_in, n_out = 65536, 8  # 256 octets: beyond what the GEMV stages in LDS, within the scratch array's size
    kernel = hip.kernel.Q8Kernel(hip.synth.q8_0_weight(970, n_out, n_in), n_in, n_out)
    d_x = H.DeviceBuffer(n_in * 4)
    d_y = H.DeviceBuffer(n_out * 4)
    rc = H.lib.rmi_hip_q8_0_forward_noalloc_dev(kernel.w.handle, d_x.ptr, d_y.ptr, 1, n_out, H.ROUND_TIES_EVEN, None)
    assert rc == -1 and "too long for the GEMV staging" in H.last_error()
    d_x.free()
    d_y.free()
