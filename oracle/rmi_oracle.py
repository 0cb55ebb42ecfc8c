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
        "rmi_ref_matmul_q8_0_neon_split": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz]),
        "rmi_ref_matmul_q8_0_neon_interleaved": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz]),
        "rmi_ref_q4k_q8k_block_ints": (None, [_u8p, _sz, _i8p, _i16p, _i32p, _i32p]),
        "rmi_ref_q4k_q8k_block_ints_matrix": (None, [_u8p, _sz, _sz, _i8p, _i16p, _i32p]),
        "rmi_ref_dequantize_row_q4_k": (None, [_u8p, _f32p, _sz]),
        "rmi_ref_q4k_forward_prepared": (None, [_u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_q4k_forward_prequantized": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, _sz]),
        "rmi_ref_quantized_linear_forward": (None, [_u8p, _f32p, _f32p, _sz, _sz]),
        "rmi_ref_matmul_q4_0_scalar_range": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, _sz]),
        "rmi_ref_block_dots_q4_0": (None, [_u8p, _u8p, _i32p, _sz, _sz]),
        "rmi_ref_x86_matmul_q4_0_range": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz]),
        "rmi_ref_dequantize_row_q6_k": (None, [_u8p, _f32p, _sz]),
        "rmi_ref_vec_dot_q6k_q8k": (C.c_float, [_u8p, _sz, _f32p, _i8p, _i16p, C.c_int]),
        "rmi_ref_q6k_q8k_block_ints": (None, [_u8p, _sz, _i8p, _i32p]),
        "rmi_ref_q6k_q8k_lane_ints": (None, [_u8p, _sz, _i8p, _i16p, _i32p]),
        "rmi_ref_q6k_forward_prepared": (None, [_u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz, _sz, _sz, C.c_int]),
        "rmi_ref_q6k_forward_prequantized": (None, [_u8p, _u8p, _f32p, _f32p, _sz, _sz, _sz, _sz]),
        "rmi_ref_x86_vec_dot_q6k_q8k": (C.c_float, [_u8p, _sz, _f32p, _i8p, _i16p]),
        "rmi_ref_x86_q6k_forward_prepared": (None, [_u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz, _sz, _sz]),
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
        "rmi_ref_pool_matmul_q4_0": (None, [C.c_void_p, _u8p, _u8p, _f32p, _f32p, _sz, _sz]),
        "rmi_ref_pool_matmul_q6k_q8k": (None, [C.c_void_p, _u8p, _f32p, _i8p, _i16p, _f32p, _sz, _sz]),
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


lib.rmi_ref_expf_restated.restype = C.c_float
lib.rmi_ref_expf_restated.argtypes = [C.c_float]
lib.rmi_ref_expf_mismatches.restype = C.c_uint64
lib.rmi_ref_expf_mismatches.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64]


def rms_norm(x, weight, eps):
    x, weight = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(weight, np.float32)
    out = np.empty_like(x)
    lib.rmi_ref_rms_norm(_p(x, _f32p), _p(weight, _f32p), _p(out, _f32p), C.c_size_t(x.size), C.c_float(eps))
    return out


def rope_neox(x, pos, freq_base):
    x = np.array(x, np.float32)
    lib.rmi_ref_rope_neox(_p(x, _f32p), C.c_size_t(pos), C.c_size_t(x.size), C.c_float(freq_base))
    return x


def rope_angles(pos, head_dim, freq_base):
    c, s = np.empty(head_dim // 2, np.float32), np.empty(head_dim // 2, np.float32)
    lib.rmi_ref_rope_angles(C.c_size_t(pos), C.c_size_t(head_dim), C.c_float(freq_base), _p(c, _f32p), _p(s, _f32p))
    return c, s


def silu_mul(gate_out, up_out):
    g, u = np.ascontiguousarray(gate_out, np.float32), np.array(up_out, np.float32)
    lib.rmi_ref_silu_mul(_p(g, _f32p), _p(u, _f32p), C.c_size_t(g.size))
    return u


def attention_f16(q, k_cache, v_cache, step, kv_stride, n_head, n_head_kv, hk, hv):
    q = np.ascontiguousarray(q, np.float32)
    k_cache, v_cache = np.ascontiguousarray(k_cache, np.uint16), np.ascontiguousarray(v_cache, np.uint16)
    out = np.zeros(n_head * hv, np.float32)
    u16p = C.POINTER(C.c_uint16)
    lib.rmi_ref_attention_f16(_p(q, _f32p), k_cache.ctypes.data_as(u16p), v_cache.ctypes.data_as(u16p),
                              C.c_size_t(step), C.c_size_t(kv_stride), C.c_size_t(n_head), C.c_size_t(n_head_kv),
                              C.c_size_t(hk), C.c_size_t(hv), _p(out, _f32p))
    return out


def softmax(x):
    x = np.array(x, np.float32)
    lib.rmi_ref_softmax(_p(x, _f32p), C.c_size_t(x.size))
    return x


lib.rmi_ref_dot_f16.restype = C.c_float


def dot_f16(a, b):
    a, b = np.ascontiguousarray(a, np.uint16), np.ascontiguousarray(b, np.uint16)
    u16p = C.POINTER(C.c_uint16)
    return np.float32(lib.rmi_ref_dot_f16(a.ctypes.data_as(u16p), b.ctypes.data_as(u16p), C.c_size_t(min(a.size, b.size))))


def embedding_lookup_q8_0(weight, token_id, n_embd):
    weight = np.ascontiguousarray(weight, np.uint8)
    out = np.zeros(n_embd, np.float32)
    lib.rmi_ref_embedding_lookup_q8_0(_p(weight, _u8p), C.c_uint32(token_id), C.c_size_t(n_embd), _p(out, _f32p))
    return out


lib.rmi_ref_greedy_token.restype = C.c_int


def greedy_token(logits):
    """Token id of the first strict maximum; None for empty or non-finite logits (the reference's Err)."""
    logits = np.ascontiguousarray(logits, np.float32)
    tid = C.c_uint32(0)
    rc = lib.rmi_ref_greedy_token(_p(logits, _f32p), C.c_size_t(logits.size), C.byref(tid))
    return None if rc != 0 else int(tid.value)


def expf_array(x, restated=False):
    """exp of an f32 array through the host libm's expf, or through the restated formula"""
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    lib.rmi_ref_expf_array(_p(x, _f32p), _p(y, _f32p), C.c_size_t(x.size), int(restated))
    return y


def expf_restated(x):
    return float(lib.rmi_ref_expf_restated(float(x)))


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


def matmul_q8_0_neon_split(w, q8, sc, n_in, n_out, quads_per_part):
    """The aarch64 kernel's chain cut into runs of `quads_per_part` whole quads (128 elements), each summed from zero in
    block order, the runs' sums added in run order: what the device's split-K GEMM computes (not a function of the
    reference)."""
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    out = np.zeros(n_out, np.float32)
    lib.rmi_ref_matmul_q8_0_neon_split(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out, quads_per_part)
    return out


def matmul_q8_0_neon_interleaved(w, q8, sc, n_in, n_out, n_groups):
    """The aarch64 kernel's chain as `n_groups` interleaved chains (group g: quads g, g + n_groups, ...), the groups'
    sums added in group order: what the device's tiled GEMM computes with groups of waves (not a function of the
    reference)."""
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    out = np.zeros(n_out, np.float32)
    lib.rmi_ref_matmul_q8_0_neon_interleaved(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out, n_groups)
    return out


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


def q4k_q8k_block_ints_matrix(w, n_out, qs, bsums):
    """`q4k_q8k_block_ints` for every row of a weight against one token: int32[n_out][n_in/256][2] = {isum, msum}."""
    w = _u8(w)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    nb = qs.size // 256
    ints = np.zeros((n_out, nb, 2), np.int32)
    lib.rmi_ref_q4k_q8k_block_ints_matrix(_p(w, _u8p), n_out, nb, _p(qs, _i8p), _p(bsums, _i16p), _p(ints, _i32p))
    return ints


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


# ---- Q4_0 ----

def matmul_q4_0_scalar_range(w, q8, sc, out, n_in, n_out, ith=0, nth=1):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    lib.rmi_ref_matmul_q4_0_scalar_range(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out, ith, nth)
    return out


def block_dots_q4_0(w, q8, n_in, n_out):
    w, q8 = _u8(w), _u8(q8)
    dots = np.zeros((n_out, n_in // 32), np.int32)
    lib.rmi_ref_block_dots_q4_0(_p(w, _u8p), _p(q8, _u8p), _p(dots, _i32p), n_in, n_out)
    return dots


def x86_matmul_q4_0_range(w, q8, sc, n_in, row_start, row_end):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    out = np.zeros(max(row_end - row_start, 0), np.float32)
    lib.rmi_ref_x86_matmul_q4_0_range(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, row_start, row_end)
    return out


# ---- Q6_K ----

def dequantize_row_q6_k(blocks, n):
    blocks = _u8(blocks)
    out = np.zeros(n, np.float32)
    lib.rmi_ref_dequantize_row_q6_k(_p(blocks, _u8p), _p(out, _f32p), n)
    return out


def _q8k_args(d, qs, bsums):
    return _f32(d), np.ascontiguousarray(qs, np.int8), np.ascontiguousarray(bsums, np.int16)


def vec_dot_q6k_q8k(row, d, qs, bsums, variant=AVX2):
    row = _u8(row)
    d, qs, bsums = _q8k_args(d, qs, bsums)
    return np.float32(lib.rmi_ref_vec_dot_q6k_q8k(_p(row, _u8p), d.size, _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p),
                                                  variant))


def q6k_q8k_block_ints(row, qs):
    row = _u8(row)
    qs = np.ascontiguousarray(qs, np.int8)
    isum = np.zeros(qs.size // 256, np.int32)
    lib.rmi_ref_q6k_q8k_block_ints(_p(row, _u8p), isum.size, _p(qs, _i8p), _p(isum, _i32p))
    return isum


def q6k_q8k_lane_ints(row, qs, bsums):
    row = _u8(row)
    qs = np.ascontiguousarray(qs, np.int8)
    bsums = np.ascontiguousarray(bsums, np.int16)
    lanes = np.zeros((qs.size // 256, 8), np.int32)
    lib.rmi_ref_q6k_q8k_lane_ints(_p(row, _u8p), lanes.shape[0], _p(qs, _i8p), _p(bsums, _i16p), _p(lanes, _i32p))
    return lanes


def q6k_forward_prepared(w, d, qs, bsums, out, n_in, n_out, ith=0, nth=1, variant=AVX2):
    w = _u8(w)
    d, qs, bsums = _q8k_args(d, qs, bsums)
    lib.rmi_ref_q6k_forward_prepared(_p(w, _u8p), _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p), _p(out, _f32p), n_in,
                                     n_out, ith, nth, variant)
    return out


def q6k_forward_prequantized(w, q8, sc, out, n_in, n_out, ith=0, nth=1):
    w, q8, sc = _u8(w), _u8(q8), _f32(sc)
    lib.rmi_ref_q6k_forward_prequantized(_p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out, ith,
                                         nth)
    return out


def x86_vec_dot_q6k_q8k(row, d, qs, bsums):
    row = _u8(row)
    d, qs, bsums = _q8k_args(d, qs, bsums)
    return np.float32(lib.rmi_ref_x86_vec_dot_q6k_q8k(_p(row, _u8p), d.size, _p(d, _f32p), _p(qs, _i8p),
                                                      _p(bsums, _i16p)))


def x86_q6k_forward_prepared(w, d, qs, bsums, out, n_in, n_out, ith=0, nth=1):
    w = _u8(w)
    d, qs, bsums = _q8k_args(d, qs, bsums)
    lib.rmi_ref_x86_q6k_forward_prepared(_p(w, _u8p), _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p), _p(out, _f32p),
                                         n_in, n_out, ith, nth)
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

    def matmul_q4_0(self, w, q8, sc, out, n_in, n_out):
        lib.rmi_ref_pool_matmul_q4_0(self._h, _p(w, _u8p), _p(q8, _u8p), _p(sc, _f32p), _p(out, _f32p), n_in, n_out)
        return out

    def matmul_q6k_q8k(self, w, d, qs, bsums, out, n_in, n_out):
        lib.rmi_ref_pool_matmul_q6k_q8k(self._h, _p(w, _u8p), _p(d, _f32p), _p(qs, _i8p), _p(bsums, _i16p),
                                        _p(out, _f32p), n_in, n_out)
        return out

    def close(self):
        if self._h:
            lib.rmi_ref_pool_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()


# ---- restated Qwen3 decode loop with a pluggable matmul (rmi_qwen3.c) ----

MATMUL_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, _u8p, _f32p, _f32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32)
_fpp = C.POINTER(_f32p)
_vpp = C.POINTER(C.c_void_p)


class Qwen3ModelStruct(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_embd", "n_layer", "n_head", "n_head_kv", "head_dim_k", "head_dim_v",
                                          "n_ff", "vocab", "n_ctx")] + [
        ("eps", C.c_float), ("freq_base", C.c_float), ("has_qk_norm", C.c_int32), ("quant_variant", C.c_int32),
        ("token_embd", C.c_void_p), ("output_norm", _f32p), ("output", C.c_void_p),
        ("attn_norm", _fpp), ("ffn_norm", _fpp), ("q_norm", _fpp), ("k_norm", _fpp),
        ("wq", _vpp), ("wk", _vpp), ("wv", _vpp), ("wo", _vpp), ("w_gate", _vpp), ("w_up", _vpp), ("w_down", _vpp)]


class CpuWeight(C.Structure):
    _fields_ = [("blocks", C.c_void_p), ("pool", C.c_void_p)]


lib.rmi_ref_cpu_matmul.restype = C.c_int
lib.rmi_ref_qwen3_generate.restype = C.c_int
lib.rmi_ref_qwen3_generate.argtypes = [C.POINTER(Qwen3ModelStruct), C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32),
                                       C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64),
                                       C.POINTER(C.c_uint32), _f32p, C.POINTER(C.c_uint32), C.c_uint32, _f32p,
                                       C.POINTER(C.c_double), C.POINTER(C.c_double)]

_MATMUL_NAMES = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
_FIELD_OF = dict(zip(_MATMUL_NAMES, ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")))


class Qwen3Decoder:
    """The restated `Qwen3Session` over a GGUF-like tensor dict.

    `weight_handle(name, bytes, n_in, n_out)` turns each Q8_0 matrix into the opaque
    first argument of `matmul_fn` (a C function pointer with the signature of
    Kernel::forward_prequantized).  With the defaults both are the restated CPU kernels.
    """

    def __init__(self, metadata, tensors, pool, matmul_fn=None, weight_handle=None, quant_variant=AVX2):
        g = lambda k: int(metadata[f"qwen3.{k}"])  # noqa: E731
        self.pool = pool
        self._keep = []
        m = Qwen3ModelStruct()
        m.n_embd, m.n_layer, m.n_head, m.n_head_kv = g("embedding_length"), g("block_count"), g(
            "attention.head_count"), g("attention.head_count_kv")
        m.head_dim_k = int(metadata.get("qwen3.attention.key_length", m.n_embd // m.n_head))
        m.head_dim_v = int(metadata.get("qwen3.attention.value_length", m.n_embd // m.n_head))
        m.n_ff, m.n_ctx = g("feed_forward_length"), g("context_length")
        m.vocab = int(metadata["qwen3.vocab_size"])
        m.eps = float(metadata["qwen3.attention.layer_norm_rms_epsilon"])
        m.freq_base = float(metadata.get("qwen3.rope.freq_base", 1e6))
        m.has_qk_norm, m.quant_variant = 1, quant_variant
        if weight_handle is None:
            def weight_handle(name, data, n_in, n_out):
                cw = CpuWeight(data.ctypes.data, pool._h)
                self._keep.append(cw)
                return C.addressof(cw)
            matmul_fn = C.cast(lib.rmi_ref_cpu_matmul, C.c_void_p).value
        self.matmul_fn = matmul_fn

        def f32(name):
            a = np.ascontiguousarray(tensors[name].view(np.float32))
            self._keep.append(a)
            return a.ctypes.data_as(_f32p)

        def raw(name):
            a = np.ascontiguousarray(tensors[name])
            self._keep.append(a)
            return a

        embd = raw("token_embd.weight")
        m.token_embd = embd.ctypes.data
        m.output_norm = f32("output_norm.weight")
        q_dim, kv_dim = m.n_head * m.head_dim_k, m.n_head_kv * m.head_dim_k
        shapes = {"attn_q": (m.n_embd, q_dim), "attn_k": (m.n_embd, kv_dim), "attn_v": (m.n_embd, kv_dim),
                  "attn_output": (m.n_head * m.head_dim_v, m.n_embd), "ffn_gate": (m.n_embd, m.n_ff),
                  "ffn_up": (m.n_embd, m.n_ff), "ffn_down": (m.n_ff, m.n_embd)}
        # tied lm_head: the embedding table is also the output matrix (qwen3.rs:283-287)
        out_name = "output.weight" if "output.weight" in tensors else "token_embd.weight"
        m.output = weight_handle(out_name, raw(out_name), m.n_embd, m.vocab)
        for field in ("attn_norm", "ffn_norm", "q_norm", "k_norm"):
            gname = {"attn_norm": "attn_norm", "ffn_norm": "ffn_norm", "q_norm": "attn_q_norm", "k_norm": "attn_k_norm"}[field]
            arr = (_f32p * m.n_layer)(*[f32(f"blk.{layer}.{gname}.weight") for layer in range(m.n_layer)])
            self._keep.append(arr)
            setattr(m, field, arr)
        for name in _MATMUL_NAMES:
            n_in, n_out = shapes[name]
            arr = (C.c_void_p * m.n_layer)(*[weight_handle(f"blk.{layer}.{name}.weight",
                                                           raw(f"blk.{layer}.{name}.weight"), n_in, n_out)
                                             for layer in range(m.n_layer)])
            self._keep.append(arr)
            setattr(m, _FIELD_OF[name], arr)
        self.model = m

    def generate(self, prompt, max_new, dump_steps=()):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        steps = prompt.size + max_new - 1
        gen = np.zeros(max_new, np.uint32)
        hashes = np.zeros(steps, np.uint64)
        argmax = np.zeros(steps, np.uint32)
        top2 = np.zeros((steps, 2), np.float32)
        dump_steps = np.ascontiguousarray(dump_steps, np.uint32)
        dump = np.zeros((max(dump_steps.size, 1), self.model.vocab), np.float32)
        t_total, t_mm = C.c_double(), C.c_double()
        u32p = C.POINTER(C.c_uint32)
        n = lib.rmi_ref_qwen3_generate(C.byref(self.model), self.matmul_fn, self.pool._h, prompt.ctypes.data_as(u32p),
                                       prompt.size, max_new, gen.ctypes.data_as(u32p),
                                       hashes.ctypes.data_as(C.POINTER(C.c_uint64)), argmax.ctypes.data_as(u32p),
                                       _p(top2, _f32p), dump_steps.ctypes.data_as(u32p), dump_steps.size,
                                       _p(dump, _f32p), C.byref(t_total), C.byref(t_mm))
        if n < 0:
            raise RuntimeError("qwen3_generate failed (non-finite logits, capacity, or a failing matmul)")
        return dict(tokens=gen[:n], hashes=hashes, argmax=argmax, top2=top2, dump=dump[:dump_steps.size],
                    seconds=t_total.value, seconds_matmul=t_mm.value, steps=steps)
