"""Pins the CPU checker's Q4_0 functions: the closed forms of the reference's own tests, integer dots by
brute force, f64 dequantised dots, and the intrinsics twin (which the reference holds to the scalar kernel
bit for bit, src/ops/kernel/q4_0/avx2.rs:226-241).  CPU only."""
import numpy as np
import pytest

import gen
from conftest import bits


def build_block(scale, low, hi):
    """src/ops/kernel/q4_0/avx2.rs:196-205"""
    v = np.zeros(18, np.uint8)
    v[0:2] = np.array([gen.f16_bits(scale)], np.uint16).view(np.uint8)
    v[2:] = (hi << 4) | low
    return v


Q8_INPUTS = {
    "zero": np.zeros(32, np.uint8),
    "max": np.full(32, 0x7F, np.uint8),
    "min": np.full(32, 0x80, np.uint8),
    "linspace": np.arange(32, dtype=np.int8).view(np.uint8),
    "alt": np.array([0x7F if i % 2 == 0 else 0x80 for i in range(32)], np.uint8),
}


def _run(oracle, w, q8, sc, n_in, n_out):
    out = np.zeros(n_out, np.float32)
    oracle.matmul_q4_0_scalar_range(w, q8, sc, out, n_in, n_out)
    return out


@pytest.mark.parametrize("low,hi,inp,scale,xs,want", [
    (0, 0, "zero", 1.0, 1.0, 0.0),          # avx2.rs:243-253
    (15, 15, "zero", 1.0, 1.0, 0.0),        # :255-265
    (0, 0, "max", 1.0, 1.0, -32512.0),      # :267-279: -8 * 32 * 127
    (0, 0, "min", 1.0, 1.0, 32768.0),       # :281-291: -8 * 32 * -128
    (15, 15, "max", 1.0, 1.0, 28448.0),     # :293-303: 7 * 32 * 127
])
def test_q4_0_closed_forms(oracle, low, hi, inp, scale, xs, want):
    w = build_block(scale, low, hi)
    out = _run(oracle, w, Q8_INPUTS[inp], np.array([xs], np.float32), 32, 1)
    assert out[0] == np.float32(want)
    assert oracle.block_dots_q4_0(w, Q8_INPUTS[inp], 32, 1)[0, 0] == int(want)


def test_q4_0_twin_on_reference_cases(oracle):
    """The mixed cases of avx2.rs:305-363: scalar restatement == kernel written with the reference's intrinsics."""
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    cases = [(build_block(0.7, 0, 15), Q8_INPUTS["linspace"], np.array([1.3], np.float32)),
             (build_block(2.5, 8, 3), Q8_INPUTS["alt"], np.array([0.42], np.float32))]
    # parity_many_blocks_random: 4 rows x 16 blocks from the reference's LCG
    state, w = 0xDEADBEEF12345678, []
    mask = (1 << 64) - 1
    for _ in range(4):
        for _ in range(16):
            state = (state * 6364136223846793005 + 1442695040888963407) & mask
            d = np.float32(0.01) + np.float32(state >> 33) / np.float32(0xFFFFFFFF)
            w += list(np.array([gen.f16_bits(d)], np.uint16).view(np.uint8))
            for _ in range(16):
                state = (state * 6364136223846793005 + 1442695040888963407) & mask
                w.append((state >> 33) & 0xFF)
    q8 = np.array([((i % 31) - 15) for i in range(512)], np.int8).view(np.uint8)
    sc = (np.float32(0.01) + np.arange(16, dtype=np.float32) * np.float32(0.001)).astype(np.float32)
    cases.append((np.array(w, np.uint8), q8, sc))
    for w, q8, sc in cases:
        n_in = q8.size
        n_out = w.size // (n_in // 32 * 18)
        a = _run(oracle, w, q8, sc, n_in, n_out)
        t = oracle.x86_matmul_q4_0_range(w, q8, sc, n_in, 0, n_out)
        assert np.array_equal(bits(a), bits(t))


def test_q4_0_dots_brute_force_and_f64(oracle, rmi):
    rng = np.random.default_rng(40)
    n_in, n_out = 1024, 9
    w = rmi.synth.q4_0_weight(41, n_out, n_in)
    x = rng.standard_normal(n_in).astype(np.float32)
    q8, sc = oracle.quantize_q8_0(x, 1)
    dots = oracle.block_dots_q4_0(w, q8, n_in, n_out)
    y = _run(oracle, w, q8, sc, n_in, n_out)
    blocks = w.reshape(n_out, n_in // 32, 18)
    nib = blocks[:, :, 2:].astype(np.int64)
    vals = np.concatenate([(nib & 0xF) - 8, (nib >> 4) - 8], axis=2)          # [row][block][32]
    yq = q8.view(np.int8).astype(np.int64).reshape(n_in // 32, 32)
    want = (vals * yq[None, :, :]).sum(axis=2)
    assert np.array_equal(dots, want.astype(np.int32))
    d = blocks[:, :, 0:2].copy().view(np.float16)[:, :, 0].astype(np.float64)
    exact = (want * d * sc.astype(np.float64)[None, :]).sum(axis=1)
    scale = (np.abs(want) * d * sc.astype(np.float64)[None, :]).sum(axis=1)
    assert np.all(np.abs(y - exact) <= 1e-5 * scale)
    if oracle.have_avx2():
        assert np.array_equal(bits(y), bits(oracle.x86_matmul_q4_0_range(w, q8, sc, n_in, 0, n_out)))
    # row partition writes only its slice of the full output (scalar.rs:26-33)
    part = np.zeros(n_out, np.float32)
    oracle.matmul_q4_0_scalar_range(w, q8, sc, part, n_in, n_out, 1, 4)
    assert np.array_equal(bits(part[3:6]), bits(y[3:6])) and not part[:3].any() and not part[6:].any()
