"""Device-resident decode (rmi_hip_qwen3_*): the whole token step in HBM.

Compared with the restated Qwen3Session::generate_inner on the CPU (CPU matmuls):
greedy tokens and the argmax of every step identical, the dumped logits
bit-identical.  The GPU step keeps every rounding point of the CPU path, exp has
the bits of the host libm, and only the f64 sums of rms_norm are summed in a tree
(which can change a result about once in 2^29 norms); one quant flipped by a last-bit
difference would move logits by 1e-2, so a tolerance would say little here.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _write_model(rmi, tmp_path, **kw):
    path = os.path.join(str(tmp_path), "synthetic-qwen3-q8_0.gguf")
    rmi.gguf.write_synthetic_qwen3(path, seed=4, **kw)
    return rmi.gguf.GGUFFile(path)


def _tensors(f):
    return {name: t[2] for name, t in f.tensors.items()}


def _compare(cpu, gpu, what):
    assert np.array_equal(cpu["argmax"], gpu["argmax"]), what
    assert np.array_equal(cpu["tokens"], gpu["tokens"]), what
    assert np.array_equal(cpu["top2"].view(np.uint32), gpu["top2"].view(np.uint32)), what  # two largest logits, all steps
    ref, got = cpu["dump"], gpu["dump"]
    err = np.abs(ref - got) / (1e-4 + 1e-4 * np.abs(ref))
    same_rows = int(np.sum(np.all(ref.view(np.uint32) == got.view(np.uint32), axis=1)))
    assert same_rows == ref.shape[0], (what, same_rows, float(err.max()))
    return float(err.max()), same_rows


def test_device_expf_has_the_bits_of_the_host_libm(hip, oracle):
    H = hip.hip
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.integers(0, 1 << 32, 1 << 21, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        rng.uniform(-30.0, 0.0, 1 << 21).astype(np.float32),
                        rng.normal(0.0, 4.0, 1 << 21).astype(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.0, 88.72, 88.73, -87.4, -103.9, -104.0,
                                  -103.97, 1e-30, -1e-30], np.float32)])
    d_x, d_y = H.DeviceBuffer.from_array(x), H.DeviceBuffer(x.size * 4)
    H.check(H.lib.rmi_hip_expf_dev(d_x.ptr, d_y.ptr, x.size, None))
    H.check(H.lib.rmi_hip_synchronize())
    got = d_y.to_array(np.float32, (x.size,))
    with np.errstate(all="ignore"):
        ref = oracle.expf_array(x)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])


def test_small_model_device_decode_matches_cpu(hip, oracle, tmp_path):
    kw = dict(n_layer=3, n_embd=512, n_head=8, n_head_kv=4, head_dim=64, n_ff=1024, vocab=5000, n_ctx=4096)
    f = _write_model(hip, tmp_path, **kw)
    pool = oracle.Pool(8)
    prompt = np.random.default_rng(6).integers(0, 5000, 40, dtype=np.uint32)
    steps = list(range(63))
    cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 24, dump_steps=steps)
    sess = hip.decode.Qwen3Session(f.metadata, _tensors(f), capacity=64)
    gpu = sess.generate(prompt, 24, dump_steps=steps)
    worst, same = _compare(cpu, gpu, "small")
    print(f"\nsmall model: {same}/63 steps bit-identical, worst error {worst:.3g} of tolerance")
    # a second generation on the same session starts from a clean cache position 0 and repeats the first
    again = sess.generate(prompt, 24, dump_steps=steps)
    assert np.array_equal(again["dump"].view(np.uint32), gpu["dump"].view(np.uint32))
    # capacity and vocabulary are checked on the host
    with pytest.raises(hip.hip.RmiHipError):
        sess.generate(prompt, 30)
    with pytest.raises(hip.hip.RmiHipError):
        sess.generate(np.array([5000], np.uint32), 1)
    sess.close()
    pool.close()


def test_stop_ids_end_the_generation_before_the_stop_token(hip, tmp_path):
    """generate_inner breaks at EOS / im_end before pushing the token (src/models/qwen3.rs:1123-1130)."""
    kw = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, vocab=1000, n_ctx=4096)
    f = _write_model(hip, tmp_path, **kw)
    sess = hip.decode.Qwen3Session(f.metadata, _tensors(f), capacity=128)
    prompt = np.random.default_rng(8).integers(0, 1000, 10, dtype=np.uint32)
    full = sess.generate(prompt, 100)
    assert full["tokens"].size == 100
    for cut in (0, 5, 31, 32, 70):  # before, on and after a host check boundary
        stop = int(full["tokens"][cut])
        first = int(np.flatnonzero(full["tokens"] == stop)[0])
        sess.set_stop_ids([stop, 999999])
        got = sess.generate(prompt, 100)
        assert got["tokens"].size == first and np.array_equal(got["tokens"], full["tokens"][:first]), cut
    sess.set_stop_ids([])
    assert np.array_equal(sess.generate(prompt, 100)["tokens"], full["tokens"])
    sess.close()


def test_create_rejects_null_and_overflowing_shapes(hip):
    import ctypes as C

    H = hip.hip
    c = H.Qwen3Config()
    c.n_embd, c.n_layer, c.n_head, c.n_head_kv, c.head_dim_k, c.head_dim_v = 64, 2, 2, 1, 32, 32
    c.n_ff, c.vocab, c.capacity, c.eps, c.freq_base, c.has_qk_norm, c.rounding = 64, 10, 16, 1e-6, 1e6, 1, 1
    w = H.Qwen3Weights()
    embd, norm = np.zeros(10 * 2 * 34, np.uint8), np.ones(64, np.float32)
    w.token_embd, w.output_norm = H.ptr(embd, H._u8p), H.ptr(norm, H._f32p)
    assert not H.lib.rmi_hip_qwen3_create(C.byref(c), C.byref(w)) and "per-layer" in H.last_error()
    mats = (H._u8p * 2)(H.ptr(np.zeros(64 * 2 * 34, np.uint8), H._u8p), None)
    norms = (H._f32p * 2)(H.ptr(norm, H._f32p), H.ptr(norm, H._f32p))
    for field in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
        setattr(w, field, mats)
    for field in ("attn_norm", "ffn_norm", "q_norm", "k_norm"):
        setattr(w, field, norms)
    assert not H.lib.rmi_hip_qwen3_create(C.byref(c), C.byref(w)) and "layer 1" in H.last_error()
    c.n_head, c.n_head_kv, c.head_dim_k, c.head_dim_v, c.n_layer = 1 << 24, 1 << 24, 1024, 1024, 1
    assert not H.lib.rmi_hip_qwen3_create(C.byref(c), C.byref(w)) and "overflow" in H.last_error()


def test_long_context_device_decode_crosses_the_attention_split(hip, oracle, tmp_path):
    """From 1280 cached positions on, the head-dimension-128 attention of the device-resident step runs as two
    launches with a head's keys split over workgroups; logits before, at and after the switch equal the CPU loop's."""
    kw = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=128, n_ff=512, vocab=2000, n_ctx=4096)
    f = _write_model(hip, tmp_path, **kw)
    pool = oracle.Pool(8)
    prompt = np.random.default_rng(9).integers(0, 2000, 1210, dtype=np.uint32)
    steps = [0, 1209, 1277, 1278, 1279, 1280, 1281, 1344, 1345, 1409]
    cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 201, dump_steps=steps)
    sess = hip.decode.Qwen3Session(f.metadata, _tensors(f), capacity=1411)
    gpu = sess.generate(prompt, 201, dump_steps=steps)
    assert gpu["steps"] == 1410
    worst, same = _compare(cpu, gpu, "long context")
    print(f"\nlong context: {same}/{len(steps)} dumped steps bit-identical, worst error {worst:.3g} of tolerance")
    again = sess.generate(prompt, 201, dump_steps=steps)  # the split's arrival counters were left at zero
    assert np.array_equal(again["dump"].view(np.uint32), gpu["dump"].view(np.uint32))
    sess.close()
    pool.close()


def test_prompt_passes_change_no_bit(hip, oracle, tmp_path):
    """Prompt positions 128 (or 7, 8, 16, 32) to a pass against every position its own step: tokens, every step's
    argmax and top-2 logits and every dumped step's logits identical, for prompts that end inside a pass, on a pass
    boundary and before the first pass is full; and equal to the CPU loop's."""
    kw = dict(n_layer=3, n_embd=512, n_head=8, n_head_kv=4, head_dim=128, n_ff=1024, vocab=5000, n_ctx=4096)
    f = _write_model(hip, tmp_path, **kw)
    pool = oracle.Pool(8)
    sess = hip.decode.Qwen3Session(f.metadata, _tensors(f), capacity=96)
    for n_prompt, per_pass in ((1, True), (5, True), (8, 8), (9, 8), (32, 32), (33, 32), (40, 16), (43, 7), (70, True), (75, 32)):
        prompt = np.random.default_rng(60 + n_prompt).integers(0, 5000, n_prompt, dtype=np.uint32)
        steps = list(range(n_prompt + 11))
        sess.set_prompt_passes(per_pass)
        fast = sess.generate(prompt, 12, dump_steps=steps)
        sess.set_prompt_passes(False)
        slow = sess.generate(prompt, 12, dump_steps=steps)
        assert np.array_equal(fast["tokens"], slow["tokens"]), n_prompt
        assert np.array_equal(fast["argmax"], slow["argmax"]) and np.array_equal(fast["top2"].view(np.uint32), slow["top2"].view(np.uint32))
        assert np.array_equal(fast["dump"].view(np.uint32), slow["dump"].view(np.uint32)), n_prompt
        if n_prompt in (9, 43, 75):
            cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 12, dump_steps=steps)
            _compare(cpu, fast, f"prompt passes, {n_prompt} prompt tokens")
    sess.set_prompt_passes(True)
    sess.close()
    pool.close()


def test_full_qwen3_0_6b_device_decode_512_plus_128(hip, oracle, tmp_path):
    """512 prompt tokens + 128 greedy tokens = 639 steps of a random-init Qwen3-0.6B-architecture Q8_0 GGUF."""
    f = _write_model(hip, tmp_path)  # 28 layers, 1024 wide, vocab 151936
    pool = oracle.Pool(16)
    prompt = np.random.default_rng(7).integers(0, 151936, 512, dtype=np.uint32)
    steps = [0, 1, 100, 511, 512, 600, 638]
    sess = hip.decode.Qwen3Session(f.metadata, _tensors(f), capacity=640)
    gpu = sess.generate(prompt, 128, dump_steps=steps)
    cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 128, dump_steps=steps)
    assert gpu["steps"] == 639 and gpu["tokens"].size == 128
    worst, same = _compare(cpu, gpu, "qwen3-0.6b")
    margin = (cpu["top2"][:, 0] - cpu["top2"][:, 1]).min()
    print(f"\n639 steps on the device: {gpu['seconds']:.3f} s = {639 / gpu['seconds']:.0f} token-steps/s "
          f"(CPU path, {pool.n_threads} threads: {cpu['seconds']:.1f} s = {639 / cpu['seconds']:.0f}/s); "
          f"{same}/{len(steps)} dumped steps bit-identical, worst logit error {worst:.3g} of tolerance, "
          f"smallest top-1 margin {margin:.3e}")
    sess.close()
    pool.close()
