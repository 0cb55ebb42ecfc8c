"""ctypes/numpy front end of the CPU checker ``librmi_oracle.so``.

TEST INFRASTRUCTURE ONLY.  Importable from ``tests/``, from
``__graft_entry__.smoke()`` and from the ``cpu_baseline`` leg of ``bench.py``;
the GPU product path never imports this module.

Each wrapper mirrors one reference function (cited in ``rmi_oracle.h``) and
takes/returns numpy arrays.  ``variant`` selects which of the reference's three
f32 accumulation orders is restated: SCALAR, AVX2 (x86-64 production) or NEON.
"""
import ctypes as C
import os
import subprocess

import numpy as np

SCALAR, AVX2, NEON = 0, 1, 2
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librmi_oracle.so")

_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_i16p = C.POINTER(C.c_int16)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_sz = C.c_size_t


def build(force=False):
    """Compile the checker with gcc (a few seconds)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    sig = {
        "rmi_ref_f16_to_f32": (C.c_float, [C.c_uint16]),
        "rmi_ref_f32_to_f16": (C.c_uint16, [C.c_float]),
        "rmi_ref_quantize_q8_0": (None, [_f32p, _sz, _u8p, _f32p, C.c_int]),
        "rmi_ref_matmul_q8_0_quantized_range": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_matmul_q8_0_quantized_parallel_rows": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_block_dots_q8_0": (None, [_u8p, _u8p, _i32p, _sz, _sz]),
        "rmi_ref_matmul_q8_0_f32": (None, [_u8p, _f32p, _f32p, _sz, _sz, C.c_int]),
        "rmi_ref_q8_0_forward_batched": (None, [_u8p, _f32p, _f32p, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_fuse_vstack": (_sz, [_u8p, _sz, _sz, _u8p, _sz, _sz, _u8p]),
        "rmi_ref_quantize_row_q8_k": (None, [_f32p, _sz, _f32p, _i8p, _i16p, C.c_int]),
        "rmi_ref_get_scale_min_k4": (None, [C.c_int, _u8p, _u8p, _u8p]),
        "rmi_ref_unpack_scales_kmask": (None, [_u8p, _u8p]),
        "rmi_ref_vec_dot_q4k_q8k": (C.c_float, [_u8p, _sz, _f32p, _i8p, _i16p, C.c_int]),
        "rmi_ref_q4k_q8k_block_ints": (None, [_u8p, _sz, _i8p, _i16p, _i32p, _i32p]),
        "rmi_ref_dequantize_row_q4_k": (None, [_u8p, _f32p, _sz]),
        "rmi_ref_q4k_forward_prepared": (None, [_u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_q4k_forward_prequantized": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, _sz]),
        "rmi_ref_quantized_linear_forward": (None, [_u8p, _f32p, _f32p, _sz, _sz]),
        "rmi_ref_have_avx2": (C.c_int, []),
        "rmi_ref_x86_quantize_q8_0": (None, [_f32p, _sz, _u8p, _f32p]),
        "rmi_ref_x86_matmul_q8_0_range": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz]),
        "rmi_ref_x86_vec_dot_q4k_q8k": (C.c_float, [_u8p, _sz, _f32p, _i8p, _i16p]),
        "rmi_ref_x86_quantize_row_q8_k": (None, [_f32p, _sz, _f32p, _i8p, _i16p]),
        "rmi_ref_pool_create": (C.c_void_p, [C.c_int]),
        "rmi_ref_pool_destroy": (None, [C.c_void_p]),
        "rmi_ref_pool_threads": (C.c_int, [C.c_void_p]),
        "rmi_ref_pool_matmul_q8_0": (None, [C.c_void_p, _u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz]),
        "rmi_ref_pool_matmul_q4k_q8k": (None, [C.c_void_p, _u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a, ty):
    return a.ctypes.data_as(ty)


def _u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype in (np.uint8, np.int8)
    return a.view(np.uint8)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def have_avx2():
    return bool(lib.rmi_ref_have_avx2())


def f16_to_f32(bits):
    return float(lib.rmi_ref_f16_to_f32(int(bits)))


def f32_to_f16(v):
    return int(lib.rmi_ref_f32_to_f16(float(v)))


def quantize_q8_0(x, variant=AVX2):
    """`quantize_q8_0_into`: returns (q8 uint8[n], scales f32[n/32])."""
    x = _f32(x)
    n = x.size
    q8 = np.zeros(n, np.uint8)
    sc = np.zeros(n // 32, np.float32)
    lib.rmi_ref_quantize_q8_0(_p(x, _f32p), n, _p(q8, _u8p), _p(sc, _f32p), variant)
    return q8, sc


def matmul_q8_0_quantized_range(w, q8, sc, n_in, row_start, row_end, variant=AVX2):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    out = np.zeros(row_end - row_start, np.float32)
    lib.rmi_ref_matmul_q8_0_quantized_range(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in,
                                            row_start, row_end, variant)
    return out


def matmul_q8_0_quantized_parallel_rows(w, q8, sc, out, n_in, n_out, ith, nth, variant=AVX2):
    """Writes rows of thread `ith` of `nth` into the full-length `out` in place."""
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    assert out.dtype == np.float32 and out.size >= n_out and out.flags.c_contiguous
    lib.rmi_ref_matmul_q8_0_quantized_parallel_rows(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in,
                                                    n_out, ith, nth, variant)
    return out


def matmul_q8_0_quantized(w, q8, sc, n_in, n_out, variant=AVX2):
    return matmul_q8_0_quantized_range(w, q8, sc, n_in, 0, n_out, variant)


def block_dots_q8_0(w, q8, n_in, n_out):
    w, q8 = _u8(w), _u8(q8)
    dots = np.zeros((n_out, n_in // 32), np.int32)
    lib.rmi_ref_block_dots_q8_0(_p(w, _u8p), _p(q8, _u8p), _p(dots, _i32p), n_in, n_out)
    return dots


def matmul_q8_0_f32(w, x, n_in, n_out, variant=AVX2):
    w, x = _u8(w), _f32(x)
    out = np.zeros(n_out, np.float32)
    lib.rmi_ref_matmul_q8_0_f32(_p(w, _u8p), _p(x, _f32p), _p(out, _f32p), n_in, n_out, variant)
    return out


def q8_0_forward_batched(w, x, n_in, n_out, variant=AVX2):
    """`Kernel::forward_batched` for a Q8_0 weight: x[n_tokens, n_in] -> y[n_tokens, n_out]."""
    w, x = _u8(w), _f32(x)
    n_tokens = x.size // n_in
    out = np.zeros((n_tokens, n_out), np.float32)
    lib.rmi_ref_q8_0_forward_batched(_p(w, _u8p), _p(x, _f32p), _p(out, _f32p), n_in, n_out, n_tokens, variant)
    return out


def fuse_vstack(a, a_rows, b, b_rows):
    """Returns (fused bytes, rows) or None when the row byte lengths differ."""
    a, b = _u8(a), _u8(b)
    fused = np.zeros(a.size + b.size, np.uint8)
    rows = lib.rmi_ref_fuse_vstack(_p(a, _u8p), a.size, a_rows, _p(b, _u8p), b.size, b_rows, _p(fused, _u8p))
    return (fused, rows) if rows else None


def quantize_row_q8_k(x, variant=AVX2):
    """Returns (d f32[n/256], qs int8[n], bsums int16[n/16])."""
    x = _f32(x)
    n = x.size
    d = np.zeros(n // 256, np.float32)
    qs = np.zeros(n, np.int8)
    bs = np.zeros(n // 16, np.int16)
    lib.rmi_ref_quantize_row_q8_k(_p(x, _f32p), n, _p(d, _f32p), _p(qs, _i8p), _p(bs, _i16p), variant)
    return d, qs, bs


def get_scale_min_k4(j, scales12):
    s = _u8(scales12)
    sc, mn = C.c_uint8(), C.c_uint8()
    lib.rmi_ref_get_scale_min_k4(j, _p(s, _u8p), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


def unpack_scales_kmask(scales12):
    s = _u8(scales12)
    out = np.zeros(16, np.uint8)
    lib.rmi_ref_unpack_scales_kmask(_p(s, _u8p), _p(out, _u8p))
    return out


def vec_dot_q4k_q8k(row, d, qs, bsums, variant=AVX2):
    row, d = _u8(row), _f32(d)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    return np.float32(lib.rmi_ref_vec_dot_q4k_q8k(_p(row, _u8p), d.size, _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p),
                                                  variant))


def q4k_q8k_block_ints(row, qs, bsums):
    row = _u8(row)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    nb = qs.size // 256
    isum = np.zeros(nb, np.int32)
    msum = np.zeros(nb, np.int32)
    lib.rmi_ref_q4k_q8k_block_ints(_p(row, _u8p), nb, _p(qs, _i8p), _p(bsums, _i16p), _p(isum, _i32p), _p(msum, _i32p))
    return isum, msum


def dequantize_row_q4_k(blocks, n):
    blocks = _u8(blocks)
    out = np.zeros(n, np.float32)
    lib.rmi_ref_dequantize_row_q4_k(_p(blocks, _u8p), _p(out, _f32p), n)
    return out


def q4k_forward_prepared(w, d, qs, bsums, out, n_in, n_out, ith=0, nth=1, variant=AVX2):
    w, d = _u8(w), _f32(d)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    lib.rmi_ref_q4k_forward_prepared(_p(w, _u8p), _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p), _p(out, _f32p), n_in,
                                     n_out, ith, nth, variant)
    return out


def q4k_forward_prequantized(w, q8, sc, out, n_in, n_out, ith=0, nth=1):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    lib.rmi_ref_q4k_forward_prequantized(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out, ith,
                                         nth)
    return out


def quantized_linear_forward(w, x, in_features, out_features):
    w, x = _u8(w), _f32(x)
    out = np.zeros(out_features, np.float32)
    lib.rmi_ref_quantized_linear_forward(_p(w, _u8p), _p(x, _f32p), _p(out, _f32p), in_features, out_features)
    return out


# ---- intrinsics twin (x86-64 hosts with AVX2+FMA+F16C only) ----

def x86_quantize_q8_0(x):
    x = _f32(x)
    q8 = np.zeros(x.size, np.uint8)
    sc = np.zeros(x.size // 32, np.float32)
    lib.rmi_ref_x86_quantize_q8_0(_p(x, _f32p), x.size, _p(q8, _u8p), _p(sc, _f32p))
    return q8, sc


def x86_matmul_q8_0_range(w, q8, sc, n_in, row_start, row_end):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    out = np.zeros(row_end - row_start, np.float32)
    lib.rmi_ref_x86_matmul_q8_0_range(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, row_start,
                                      row_end)
    return out


def x86_vec_dot_q4k_q8k(row, d, qs, bsums):
    row, d = _u8(row), _f32(d)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    return np.float32(lib.rmi_ref_x86_vec_dot_q4k_q8k(_p(row, _u8p), d.size, _p(d, _f32p), _p(qs, _i8p),
                                                      _p(bsums, _i16p)))


def x86_quantize_row_q8_k(x):
    x = _f32(x)
    n = x.size
    d = np.zeros(n // 256, np.float32)
    qs = np.zeros(n, np.int8)
    bs = np.zeros(n // 16, np.int16)
    lib.rmi_ref_x86_quantize_row_q8_k(_p(x, _f32p), n, _p(d, _f32p), _p(qs, _i8p), _p(bs, _i16p))
    return d, qs, bs


class Pool:
    """Persistent-thread (ith, nth) row partition: the timed CPU baseline."""

    def __init__(self, n_threads):
        self._h = lib.rmi_ref_pool_create(n_threads)
        self.n_threads = lib.rmi_ref_pool_threads(self._h)

    def matmul_q8_0(self, w, q8, sc, out, n_in, n_out, n_tokens=1):
        lib.rmi_ref_pool_matmul_q8_0(self._h, _p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out,
                                     n_tokens)
        return out

    def matmul_q4k_q8k(self, w, d, qs, bsums, out, n_in, n_out):
        lib.rmi_ref_pool_matmul_q4k_q8k(self._h, _p(w, _u8p), _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p),
                                        _p(out, _f32p), n_in, n_out)
        return out

    def close(self):
        if self._h:
            lib.rmi_ref_pool_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()
