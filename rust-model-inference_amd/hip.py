"""ctypes binding of ``librmi_hip.so`` (the C ABI declared in ``include/rmi_hip.h``).

This is the only way Python reaches the GPU path: there is no CPU fallback, and
loading fails loudly when the library has not been built.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librmi_hip.so")

DTYPE_Q4_0 = 2
DTYPE_Q8_0 = 8
DTYPE_Q4_K = 12
DTYPE_Q6_K = 14
BATCHED_X86_ORDER, BATCHED_AARCH64_ORDER, BATCHED_FAST = 0, 1, 2
ROUND_HALF_AWAY = 0
ROUND_TIES_EVEN = 1
ROUND_NEON = 2
NOALLOC_MAX_ELEMS = 262144

_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_i16p = C.POINTER(C.c_int16)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_vp = C.c_void_p
_u32 = C.c_uint32
_u64 = C.c_uint64
_sz = C.c_size_t

_u32p = C.POINTER(C.c_uint32)
_f32pp = C.POINTER(_f32p)
_u8pp = C.POINTER(_u8p)


class Qwen3Config(C.Structure):
    """rmi_hip_qwen3_config"""
    _fields_ = [(n, C.c_uint32) for n in ("n_embd", "n_layer", "n_head", "n_head_kv", "head_dim_k", "head_dim_v", "n_ff",
                                          "vocab", "capacity")] + [
        ("eps", C.c_float), ("freq_base", C.c_float), ("has_qk_norm", C.c_int32), ("rounding", C.c_int32)]


class Qwen3Weights(C.Structure):
    """rmi_hip_qwen3_weights"""
    _fields_ = [("token_embd", _u8p), ("output", _u8p), ("output_norm", _f32p),
                ("attn_norm", _f32pp), ("ffn_norm", _f32pp), ("q_norm", _f32pp), ("k_norm", _f32pp),
                ("wq", _u8pp), ("wk", _u8pp), ("wv", _u8pp), ("wo", _u8pp), ("w_gate", _u8pp), ("w_up", _u8pp),
                ("w_down", _u8pp)]


# name -> (restype, argtypes); must list every symbol of include/rmi_hip.h
SIGNATURES = {
    "rmi_hip_init": (C.c_int, [C.c_int]),
    "rmi_hip_shutdown": (None, []),
    "rmi_hip_last_error": (C.c_char_p, []),
    "rmi_hip_thread_context_count": (_sz, []),
    "rmi_hip_attention_reserve": (C.c_int, [_u32, _u32]),
    "rmi_hip_set_forward_batched_mode": (C.c_int, [C.c_int]),
    "rmi_hip_get_forward_batched_mode": (C.c_int, []),
    "rmi_hip_device_info": (C.c_int, [C.c_char_p, _sz, C.POINTER(C.c_int), C.POINTER(_sz)]),
    "rmi_hip_upload_q8_0": (_vp, [_u8p, _sz, _u32, _u32]),
    "rmi_hip_upload_q4_k": (_vp, [_u8p, _sz, _u32, _u32]),
    "rmi_hip_upload_q4_0": (_vp, [_u8p, _sz, _u32, _u32]),
    "rmi_hip_upload_q6_k": (_vp, [_u8p, _sz, _u32, _u32]),
    "rmi_hip_fuse_vstack": (_vp, [_vp, _vp]),
    "rmi_hip_free_weight": (None, [_vp]),
    "rmi_hip_weight_n_in": (_u32, [_vp]),
    "rmi_hip_weight_n_out": (_u32, [_vp]),
    "rmi_hip_weight_dtype": (C.c_int, [_vp]),
    "rmi_hip_weight_device_bytes": (_sz, [_vp]),
    "rmi_hip_weight_device_data": (_vp, [_vp]),
    "rmi_hip_q8_0_forward_prequantized": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_matmul_q8_0_quantized_range": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_matmul_q8_0_quantized_batch": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_q8_0_forward_batched": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32, C.c_int]),
    "rmi_hip_q8_0_forward_batched_neon": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32, C.c_int]),
    "rmi_hip_quantize_q8_0": (C.c_int, [_f32p, _u32, _u8p, _f32p, C.c_int]),
    "rmi_hip_block_dots_q8_0": (C.c_int, [_vp, _u8p, _i32p]),
    "rmi_hip_matmul_q8_0_f32": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32]),
    "rmi_hip_matmul_q8_0_fallback_range": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_q4_k_forward_prepared": (C.c_int, [_vp, _f32p, _i8p, _i16p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_q4_k_forward_batched": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_q4_k_forward_batched_mfma": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_quantize_row_q8_k": (C.c_int, [_f32p, _u32, _f32p, _i8p, _i16p]),
    "rmi_hip_q4_k_forward_prequantized": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_quantized_linear_forward": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32]),
    "rmi_hip_quantized_linear_forward_dev": (C.c_int, [_vp, _vp, _vp, _vp]),
    "rmi_hip_block_ints_q4_k": (C.c_int, [_vp, _i8p, _i16p, _i32p, _i32p]),
    "rmi_hip_q4_0_forward_prequantized": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_q4_0_forward_batched": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32, C.c_int]),
    "rmi_hip_block_dots_q4_0": (C.c_int, [_vp, _u8p, _i32p]),
    "rmi_hip_q6_k_forward_prepared": (C.c_int, [_vp, _f32p, _i8p, _i16p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_q6_k_forward_batched": (C.c_int, [_vp, _f32p, _f32p, _u32, _u32, _u32]),
    "rmi_hip_q6_k_forward_prequantized": (C.c_int, [_vp, _u8p, _f32p, _f32p, _u32, _u32, _u32, _u32]),
    "rmi_hip_block_lanes_q6_k": (C.c_int, [_vp, _i8p, _i16p, _i32p]),
    "rmi_hip_malloc": (_vp, [_sz]),
    "rmi_hip_free": (None, [_vp]),
    "rmi_hip_memcpy_h2d": (C.c_int, [_vp, _vp, _sz]),
    "rmi_hip_memcpy_d2h": (C.c_int, [_vp, _vp, _sz]),
    "rmi_hip_synchronize": (C.c_int, []),
    "rmi_hip_copy_dev": (C.c_int, [_vp, _vp, _sz, _vp]),
    "rmi_hip_gemv_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rmi_hip_q8_0_forward_noalloc_dev": (C.c_int, [_vp, _vp, _vp, _u32, _u32, C.c_int, _vp]),
    "rmi_hip_quantize_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _u32, _u32, C.c_int, _vp]),
    "rmi_hip_gemm_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_gemv_q4_k_q8k_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rmi_hip_gemm_q4_k_q8k_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_gemm_q8_0_ksplit_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_gemm_q8_0_fast_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_gemm_q8_0_fast_plan": (C.c_int, [_vp, _u32, C.POINTER(_u32)]),
    "rmi_hip_gemm_q8_0_ksplit_quads_per_part": (_u32, [_u32]),
    "rmi_hip_gemm_block_ints_q4_k_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u32, _vp]),
    "rmi_hip_gemv_q4_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rmi_hip_gemv_q6_k_q8k_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rmi_hip_quantize_row_q8_k_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_gemv_group_create": (_vp, [_u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _u32]),
    "rmi_hip_gemv_group_create_neon": (_vp, [_u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _u32]),
    "rmi_hip_gemv_q8_0_neon_dev": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "rmi_hip_gemv_group_create_q4_k": (_vp, [_u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                             C.POINTER(_vp), _u32]),
    "rmi_hip_gemv_group_create_q6_k": (_vp, [_u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                             C.POINTER(_vp), _u32]),
    "rmi_hip_expf_dev": (C.c_int, [_vp, _vp, _sz, _vp]),
    "rmi_hip_rms_norm_quantize_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _u32, C.c_float, _vp, _vp, C.c_int, _vp]),
    "rmi_hip_rms_norm_gemv_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, C.c_float, C.c_int, _vp, _vp, _vp]),
    "rmi_hip_rms_norm_qkv_rope_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, C.c_float, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp,
                                                     _vp, _vp, _u32, _u32, _vp]),
    "rmi_hip_rms_norm_ffn_gate_up_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, C.c_float, C.c_int, _vp, _vp, _vp, _vp]),
    "rmi_hip_silu_mul_quantize_q8_0_dev": (C.c_int, [_vp, _u32, _vp, _vp, C.c_int, _vp]),
    "rmi_hip_qk_norm_rope_f16_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32,
                                               C.c_float, _vp]),
    "rmi_hip_qkv_attention_f16_quantize_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, C.c_float,
                                                              _vp, _vp, C.c_int, _vp]),
    "rmi_hip_attention_f16_quantize_q8_0_dev": (C.c_int, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _vp, _vp,
                                                          C.c_int, _vp]),
    "rmi_hip_qwen3_create": (_vp, [C.POINTER(Qwen3Config), C.POINTER(Qwen3Weights)]),
    "rmi_hip_qwen3_destroy": (None, [_vp]),
    "rmi_hip_qwen3_set_stop_ids": (C.c_int, [_vp, _u32p, _u32]),
    "rmi_hip_qwen3_set_prompt_passes": (C.c_int, [_vp, C.c_int]),
    "rmi_hip_qwen3_generate": (C.c_int, [_vp, _u32p, _u32, _u32, _u32p, _u32p, _f32p, _u32p, _u32, _f32p,
                                         C.POINTER(C.c_double)]),
    "rmi_hip_gguf_open": (_vp, [C.c_char_p]),
    "rmi_hip_gguf_close": (None, [_vp]),
    "rmi_hip_gguf_version": (_u32, [_vp]),
    "rmi_hip_gguf_alignment": (_u64, [_vp]),
    "rmi_hip_gguf_data_offset": (_u64, [_vp]),
    "rmi_hip_gguf_n_tensors": (_u64, [_vp]),
    "rmi_hip_gguf_n_kv": (_u64, [_vp]),
    "rmi_hip_gguf_kv_key": (C.c_char_p, [_vp, _u64]),
    "rmi_hip_gguf_meta_type": (C.c_int, [_vp, C.c_char_p]),
    "rmi_hip_gguf_meta_u64": (C.c_int, [_vp, C.c_char_p, C.POINTER(_u64)]),
    "rmi_hip_gguf_meta_f64": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_double)]),
    "rmi_hip_gguf_meta_bool": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_int)]),
    "rmi_hip_gguf_meta_str": (C.c_int64, [_vp, C.c_char_p, C.c_char_p, _sz]),
    "rmi_hip_gguf_meta_array_len": (C.c_int64, [_vp, C.c_char_p, C.POINTER(C.c_int)]),
    "rmi_hip_gguf_meta_array_u64": (C.c_int, [_vp, C.c_char_p, _u64, C.POINTER(_u64)]),
    "rmi_hip_gguf_find_tensor": (C.c_int64, [_vp, C.c_char_p]),
    "rmi_hip_gguf_tensor_info": (C.c_int, [_vp, _u64, C.POINTER(C.c_char_p), C.POINTER(_u32), C.POINTER(_u64), _u32,
                                           C.POINTER(C.c_int), C.POINTER(_u64), C.POINTER(_u64)]),
    "rmi_hip_gguf_tensor_data": (_vp, [_vp, _u64]),
    "rmi_hip_gguf_upload": (_vp, [_vp, C.c_char_p]),
    "rmi_hip_gguf_upload_stack": (_vp, [_vp, C.POINTER(C.c_char_p), C.c_int]),
    "rmi_hip_gguf_qwen3_config": (C.c_int, [_vp, _u32, C.c_int, C.POINTER(Qwen3Config)]),
    "rmi_hip_qwen3_create_from_gguf": (_vp, [_vp, _u32, C.c_int]),
    "rmi_hip_gemv_group_shape": (C.c_int, [_vp, C.POINTER(_u32), C.POINTER(_u32)]),
    "rmi_hip_gemv_group_destroy": (None, [_vp]),
    "rmi_hip_gemv_group_run_dev": (C.c_int, [_vp, _vp]),
}


class RmiHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"rmi_hip error {code}: {message}")
        self.code = code


def load_library():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc, gfx950); there is no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names a missing export
        fn.restype = res
        fn.argtypes = args
    return lib


lib = load_library()


def last_error():
    return (lib.rmi_hip_last_error() or b"").decode()


def check(rc):
    if rc != 0:
        raise RmiHipError(rc, last_error())


def init(device=0):
    check(lib.rmi_hip_init(device))


def device_info():
    name = C.create_string_buffer(128)
    cus, hbm = C.c_int(), _sz()
    check(lib.rmi_hip_device_info(name, 128, C.byref(cus), C.byref(hbm)))
    return name.value.decode(), cus.value, hbm.value


def ptr(a, ty):
    return a.ctypes.data_as(ty)


def as_u8(a):
    a = np.ascontiguousarray(a)
    if a.dtype not in (np.uint8, np.int8):
        raise TypeError("expected a byte array")
    return a.view(np.uint8)


def as_f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class DeviceBuffer:
    """A raw HBM allocation (for the device-resident entry points)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = lib.rmi_hip_malloc(self.nbytes)
        if not self.ptr:
            raise RmiHipError(-2, last_error())

    @classmethod
    def from_array(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        check(lib.rmi_hip_memcpy_h2d(buf.ptr, a.ctypes.data, a.nbytes))
        return buf

    def to_array(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib.rmi_hip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            lib.rmi_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
