"""rmi_hip_shutdown followed by rmi_hip_init, in a file of its own that pytest collects last: shutdown frees every
thread's staging, so a failure here must not be able to hide behind, or in front of, any other test."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu


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
