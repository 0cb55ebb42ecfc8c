"""Every path of the four-deep walk a GEMV wave takes over its run of the tile stream, for the four block
formats: runs of 1..3 units (the prefetch loads duplicates), of 4..7 (no steady loop, an epilogue of 0..3
units), longer ones whose length leaves every remainder, runs of several tiles whose results leave eight at a
time, workgroups whose last waves have no run, row ranges that start and end inside a tile, 1 / 3 / 8 tokens.
Outputs must equal the CPU kernels bit for bit; rows outside the range must stay untouched."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu

A = 1  # the AVX2-order variants of the checker


class _Q8_0:
    unit = 256  # elements per unit of the walk (an octet of blocks)

    @staticmethod
    def weight(rmi, seed, n_out, n_in):
        return rmi.synth.q8_0_weight(seed, n_out, n_in), rmi.kernel.Q8Kernel

    @staticmethod
    def quantize(oracle, x):
        return oracle.quantize_q8_0(x, A)

    @staticmethod
    def gemv(H, k, acts, y, n_tokens, stride, r0, r1):
        return H.lib.rmi_hip_gemv_q8_0_dev(k.w.handle, acts[0].ptr, acts[1].ptr, y.ptr, n_tokens, stride, r0, r1, None)

    @staticmethod
    def ref(oracle, w, act, n_in, n_out):
        return oracle.matmul_q8_0_quantized(w, act[0], act[1], n_in, n_out, A)


class _Q4_0(_Q8_0):
    @staticmethod
    def weight(rmi, seed, n_out, n_in):
        return rmi.synth.q4_0_weight(seed, n_out, n_in), rmi.kernel.Q4_0Kernel

    @staticmethod
    def gemv(H, k, acts, y, n_tokens, stride, r0, r1):
        return H.lib.rmi_hip_gemv_q4_0_dev(k.w.handle, acts[0].ptr, acts[1].ptr, y.ptr, n_tokens, stride, r0, r1, None)

    @staticmethod
    def ref(oracle, w, act, n_in, n_out):
        out = np.zeros(n_out, np.float32)
        oracle.matmul_q4_0_scalar_range(w, act[0], act[1], out, n_in, n_out)
        return out


class _Q4_K:
    unit = 256

    @staticmethod
    def weight(rmi, seed, n_out, n_in):
        return rmi.synth.q4_k_weight(seed, n_out, n_in), rmi.kernel.Q4_KKernel

    @staticmethod
    def quantize(oracle, x):
        return oracle.quantize_row_q8_k(x, A)

    @staticmethod
    def gemv(H, k, acts, y, n_tokens, stride, r0, r1):
        return H.lib.rmi_hip_gemv_q4_k_q8k_dev(k.w.handle, acts[0].ptr, acts[1].ptr, acts[2].ptr, y.ptr, n_tokens, stride,
                                               r0, r1, None)

    @staticmethod
    def ref(oracle, w, act, n_in, n_out):
        out = np.zeros(n_out, np.float32)
        oracle.q4k_forward_prepared(w, act[0], act[1], act[2], out, n_in, n_out, 0, 1, A)
        return out


class _Q6_K(_Q4_K):
    @staticmethod
    def weight(rmi, seed, n_out, n_in):
        return rmi.synth.q6_k_weight(seed, n_out, n_in), rmi.kernel.Q6_KKernel

    @staticmethod
    def gemv(H, k, acts, y, n_tokens, stride, r0, r1):
        return H.lib.rmi_hip_gemv_q6_k_q8k_dev(k.w.handle, acts[0].ptr, acts[1].ptr, acts[2].ptr, y.ptr, n_tokens, stride,
                                               r0, r1, None)

    @staticmethod
    def ref(oracle, w, act, n_in, n_out):
        out = np.zeros(n_out, np.float32)
        oracle.q6k_forward_prepared(w, act[0], act[1], act[2], out, n_in, n_out, 0, 1, A)
        return out


FORMATS = {"q8_0": _Q8_0, "q4_0": _Q4_0, "q4_k": _Q4_K, "q6_k": _Q6_K}


def _run(hip, oracle, fmt, seed, n_out, n_units, n_tokens, r0=0, r1=None):
    H, F = hip.hip, FORMATS[fmt]
    n_in = n_units * F.unit
    r1 = n_out if r1 is None else r1
    w, kernel_cls = F.weight(hip, seed, n_out, n_in)
    k = kernel_cls(w, n_in, n_out)
    x = hip.synth.activations(seed + 7, n_tokens, n_in)
    per_token = [F.quantize(oracle, x[t]) for t in range(n_tokens)]
    acts = [H.DeviceBuffer.from_array(np.stack([a[i] for a in per_token])) for i in range(len(per_token[0]))]
    sentinel = np.full((n_tokens, n_out), np.float32(-7.25))
    y = H.DeviceBuffer.from_array(sentinel)
    H.check(F.gemv(H, k, acts, y, n_tokens, n_out, r0, r1))
    H.check(H.lib.rmi_hip_synchronize())
    got = y.to_array(np.float32, (n_tokens, n_out))
    for t in range(n_tokens):
        ref = F.ref(oracle, w, per_token[t], n_in, n_out)
        assert np.array_equal(bits(got[t, r0:r1]), bits(ref[r0:r1])), (fmt, n_out, n_units, n_tokens, t)
        assert np.all(got[t, :r0] == sentinel[t, :r0]) and np.all(got[t, r1:] == sentinel[t, r1:]), "rows outside the range"


@pytest.mark.parametrize("fmt", list(FORMATS))
@pytest.mark.parametrize("n_units", [1, 2, 3, 4, 5, 6, 7, 8, 9, 11, 13])
def test_short_runs_one_tile_per_wave(hip, oracle, fmt, n_units):
    """Small launches give every wave one tile: the run is n_units long."""
    for n_tokens, n_out in ((1, 61), (3, 24), (8, 9)):
        _run(hip, oracle, fmt, 40 + n_units, n_out, n_units, n_tokens)


@pytest.mark.parametrize("fmt", list(FORMATS))
@pytest.mark.parametrize("n_units,n_out", [(1, 8 * 2048 * 16 + 5), (2, 8 * 2048 * 8 + 8 * 3 + 1), (3, 8 * 2048 * 5 + 8 * 2),
                                           (5, 8 * 2048 * 3 + 8 * 1 + 7), (7, 8 * 2048 * 2 + 3)])
def test_long_runs_of_several_tiles(hip, oracle, fmt, n_units, n_out):
    """Launches large enough for runs of 16, 8, 5, 3 and 2 tiles (16, 16, 15, 15 and 14 units): the steady loop,
    every epilogue length, sixteen tiles leaving in two groups of eight, a last run shorter than the others and
    (with several waves per workgroup) waves without a run."""
    _run(hip, oracle, fmt, 90 + n_units, n_out, n_units, 1)


@pytest.mark.parametrize("fmt", list(FORMATS))
def test_row_ranges_and_batches_over_long_runs(hip, oracle, fmt):
    n_units, n_out = 2, 8 * 2048 * 8 + 77
    _run(hip, oracle, fmt, 130, n_out, n_units, 3)
    _run(hip, oracle, fmt, 131, n_out, n_units, 1, r0=13, r1=n_out - 5)
    _run(hip, oracle, fmt, 132, n_out, n_units, 2, r0=8 * 1000 + 7, r1=8 * 1000 + 9)
    _run(hip, oracle, fmt, 133, n_out, n_units, 1, r0=40000, r1=40000)  # empty range: nothing is written


def _group_create(H, fmt, kernels, acts, ys, n_tokens):
    n = len(kernels)
    arr = lambda vals: (H.C.c_void_p * n)(*vals)  # noqa: E731
    handles = arr([k.w.handle for k in kernels])
    outs = arr([y.ptr for y in ys])
    if fmt in ("q8_0", "q4_0"):
        return H.lib.rmi_hip_gemv_group_create(n, handles, arr([a[0].ptr for a in acts]), arr([a[1].ptr for a in acts]), outs,
                                               n_tokens)
    create = H.lib.rmi_hip_gemv_group_create_q4_k if fmt == "q4_k" else H.lib.rmi_hip_gemv_group_create_q6_k
    return create(n, handles, arr([a[0].ptr for a in acts]), arr([a[1].ptr for a in acts]), arr([a[2].ptr for a in acts]),
                  outs, n_tokens)


@pytest.mark.parametrize("fmt", list(FORMATS))
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_grouped_launches(hip, oracle, fmt, seed):
    """One launch over a random list of matrices of unlike widths and heights (so the runs of one workgroup's
    waves, their lengths and the padding runs differ from launch to launch), 1 / 2 / 5 / 8 tokens."""
    H, F = hip.hip, FORMATS[fmt]
    rng = np.random.default_rng(1000 * seed + len(fmt))
    for n_tokens in (1, 2, 5, 8):
        shapes = [(int(rng.integers(1, 700)), int(rng.integers(1, 14))) for _ in range(int(rng.integers(3, 12)))]
        shapes.append((int(rng.integers(30000, 50000)), int(rng.integers(1, 4))))  # one tall matrix: runs of many tiles
        kernels, acts, ys, refs = [], [], [], []
        for i, (n_out, n_units) in enumerate(shapes):
            n_in = n_units * F.unit
            w, kernel_cls = F.weight(hip, 7000 + 100 * seed + i, n_out, n_in)
            kernels.append(kernel_cls(w, n_in, n_out))
            x = hip.synth.activations(8000 + 100 * seed + i, n_tokens, n_in)
            per_token = [F.quantize(oracle, x[t]) for t in range(n_tokens)]
            acts.append([H.DeviceBuffer.from_array(np.stack([a[j] for a in per_token])) for j in range(len(per_token[0]))])
            ys.append(H.DeviceBuffer.from_array(np.full((n_tokens, n_out), np.float32(3.5))))
            refs.append(np.stack([F.ref(oracle, w, per_token[t], n_in, n_out) for t in range(n_tokens)]))
        g = _group_create(H, fmt, kernels, acts, ys, n_tokens)
        assert g, H.last_error()
        H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))
        H.check(H.lib.rmi_hip_synchronize())
        for i, (n_out, n_units) in enumerate(shapes):
            got = ys[i].to_array(np.float32, (n_tokens, n_out))
            assert np.array_equal(bits(got), bits(refs[i])), (fmt, seed, n_tokens, i, n_out, n_units)
        H.lib.rmi_hip_gemv_group_destroy(g)


@pytest.mark.parametrize("n_units,n_out,n_tokens", [(1, 8 * 2048 * 16 + 5, 8), (2, 8 * 2048 * 8 + 8 * 3 + 1, 4), (3, 8 * 2048 * 5 + 8 * 2, 5),
                                                    (5, 8 * 2048 * 3 + 8 * 1 + 7, 8), (7, 8 * 2048 * 2 + 3, 6)])
def test_long_runs_with_four_to_eight_tokens(hip, oracle, n_units, n_out, n_tokens):
    """The Q8_0 kernel for four tokens and more (its dots on the matrix cores, its results parked in LDS and leaving
    eight tiles at a time) over the same run lengths, and over row ranges that start and end inside a tile."""
    _run(hip, oracle, "q8_0", 170 + n_units, n_out, n_units, n_tokens)
    _run(hip, oracle, "q8_0", 180 + n_units, n_out, n_units, n_tokens, r0=8 * 517 + 3, r1=n_out - 8 * 11 - 6)
    _run(hip, oracle, "q8_0", 190 + n_units, n_out, n_units, n_tokens, r0=8 * 1000 + 7, r1=8 * 1000 + 9)
