"""Host-side mirror of the reference's operator interface for the quantized
matmul path, over the C ABI.  Names, argument order and argument meaning follow
the Rust traits so that tests read like the reference's own:

  Kernel                 src/ops/kernel/trait_.rs:15-110
  Q8Kernel               src/ops/kernel/q8_0/mod.rs:21-56
  Q4_0Kernel             src/ops/kernel/q4_0/mod.rs:18-123
  Q4_KKernel             src/ops/kernel/q4_k.rs:7-93
  Q6_KKernel             src/ops/kernel/q6_k.rs:7-80
  QuantizedTensor        src/ops/kernel/quantized_tensor.rs:32-190  (from_bytes / into_kernel)
  QTensorOwned           src/ops/kernel/qtensor_owned.rs:34-164 (constructors, fuse_vstack), :167-255 (Kernel),
                         :374-471 (Q8_K matmuls), :533-589 (quantize_and_matmul_with_scratch)
  QuantizedLinear, Layer, ExecContext   src/core/model.rs:12-104, src/core/traits.rs:45-74
  quantize_q8_0_into, quantize_row_q8_k  src/ops/quant/q8_0.rs:3-24, src/ops/quant/mod.rs:42-59

Outputs are numpy arrays written in place, as the `&mut [f32]` slices are.
Weights are uploaded to HBM when the kernel object is made; every call then
runs on the GPU.  A failing call raises (the reference panics on a failed GPU
call, src/ops/kernel/q8_0/dispatch.rs:45-48).
"""
from dataclasses import dataclass

import numpy as np

from . import hip
from .hip import C, _f32p, _i8p, _i16p, _i32p, _u8p, as_f32, as_u8, check, lib, ptr

GGML_TYPE_Q8_0 = "Q8_0"
GGML_TYPE_Q4_0 = "Q4_0"
GGML_TYPE_Q4_K = "Q4_K"
GGML_TYPE_Q6_K = "Q6_K"


@dataclass
class BlockQ8K:
    """src/ops/quant/mod.rs:35-40"""
    d: float
    qs: np.ndarray     # int8[256]
    bsums: np.ndarray  # int16[16]


def _q8k_arrays(q8_k):
    d = np.array([b.d for b in q8_k], np.float32)
    qs = np.ascontiguousarray(np.concatenate([np.asarray(b.qs, np.int8) for b in q8_k]))
    bs = np.ascontiguousarray(np.concatenate([np.asarray(b.bsums, np.int16) for b in q8_k]))
    return d, qs, bs


def _out(output, n):
    if not (isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous):
        raise TypeError("output must be a contiguous float32 numpy array")
    if output.size < n:
        raise ValueError(f"output holds {output.size} values, {n} needed")
    return output


def quantize_q8_0_into(input, n, q8, scales, rounding=hip.ROUND_TIES_EVEN):
    """`quantize_q8_0_into(input, n, q8, scales)` on the device.  `rounding`
    selects the reference's per-architecture variant (x86-64 default: ties-even)."""
    x = as_f32(input)
    check(lib.rmi_hip_quantize_q8_0(ptr(x, _f32p), n, ptr(q8, _u8p), ptr(scales, _f32p), rounding))


def quantize_q8_0(input, n, rounding=hip.ROUND_TIES_EVEN):
    q8 = np.zeros(n, np.uint8)
    scales = np.zeros(n // 32, np.float32)
    quantize_q8_0_into(input, n, q8, scales, rounding)
    return q8, scales


def quantize_row_q8_k(x):
    """`quantize_row_q8_k(x) -> Vec<BlockQ8K>` on the device."""
    x = as_f32(x)
    n = x.size
    d = np.zeros(n // 256, np.float32)
    qs = np.zeros(n, np.int8)
    bs = np.zeros(n // 16, np.int16)
    check(lib.rmi_hip_quantize_row_q8_k(ptr(x, _f32p), n, ptr(d, _f32p), ptr(qs, _i8p), ptr(bs, _i16p)))
    return [BlockQ8K(float(d[i]), qs[i * 256:(i + 1) * 256].copy(), bs[i * 16:(i + 1) * 16].copy())
            for i in range(n // 256)]


class Kernel:
    """`pub trait Kernel: Send + Sync` with its default methods."""

    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        raise NotImplementedError

    def forward_prepared(self, input_f32, input_q8, input_scales, q8_k, output, n_in, n_out, ith, nth):
        self.forward_prequantized(input_q8, input_scales, output, n_in, n_out, ith, nth)

    def forward(self, input, output, n_in, n_out):
        q8, scales = quantize_q8_0(np.asarray(input, np.float32)[:n_in], n_in)
        self.forward_prepared(input, q8, scales, None, output, n_in, n_out, 0, 1)

    def forward_batched(self, input, output, n_in, n_out):
        x = as_f32(input).reshape(-1)
        n_tokens = x.size // n_in
        assert x.size == n_tokens * n_in and output.size == n_tokens * n_out
        out = output.reshape(n_tokens, n_out)
        for t in range(n_tokens):
            self.forward(x[t * n_in:(t + 1) * n_in], out[t], n_in, n_out)


def set_forward_batched_mode(mode):
    """How `Kernel::forward_batched` of the Q8_0 and Q4_K kernels multiplies a batch, for the whole process:
    `hip.BATCHED_X86_ORDER` (default: the x86-64 kernels' bits for every token), `hip.BATCHED_AARCH64_ORDER` or
    `hip.BATCHED_FAST` (the fastest kernel per product, within the reference's tolerance).  Returns the mode it
    replaces."""
    old = lib.rmi_hip_get_forward_batched_mode()
    check(lib.rmi_hip_set_forward_batched_mode(mode))
    return old


class _DeviceWeight:
    def __init__(self, handle):
        if not handle:
            raise hip.RmiHipError(-1, hip.last_error())
        self.handle = handle

    @property
    def n_in(self):
        return lib.rmi_hip_weight_n_in(self.handle)

    @property
    def n_out(self):
        return lib.rmi_hip_weight_n_out(self.handle)

    @property
    def dtype(self):
        return lib.rmi_hip_weight_dtype(self.handle)

    @property
    def device_bytes(self):
        return lib.rmi_hip_weight_device_bytes(self.handle)

    def free(self):
        if self.handle:
            lib.rmi_hip_free_weight(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Q8Kernel(Kernel):
    """Q8_0 weight in HBM; `forward_prequantized` is the hot path."""

    def __init__(self, weight, n_in, n_out, _handle=None):
        if _handle is None:
            w = as_u8(weight)
            _handle = lib.rmi_hip_upload_q8_0(ptr(w, _u8p), w.size, n_in, n_out)
        self.w = _DeviceWeight(_handle)

    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_q8_0_forward_prequantized(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                    ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward(self, input, output, n_in, n_out, rounding=hip.ROUND_TIES_EVEN):
        x = as_f32(input)[:n_in]
        check(lib.rmi_hip_q8_0_forward_batched(self.w.handle, ptr(x, _f32p), ptr(_out(output, n_out), _f32p), n_in,
                                               n_out, 1, rounding))

    def forward_batched(self, input, output, n_in, n_out, rounding=hip.ROUND_TIES_EVEN, matrix_cores=False):
        """`Kernel::forward_batched`.  By default every token goes through the x86-64-order GEMV, so
        `forward_batched(x)[t] == forward(x[t])` bit for bit as in the reference; `matrix_cores=True` asks for
        the aarch64 kernel's order on int8 MFMA (the prefill path), equally batch-independent."""
        x = as_f32(input).reshape(-1)
        n_tokens = x.size // n_in
        assert x.size == n_tokens * n_in
        fn = lib.rmi_hip_q8_0_forward_batched_neon if matrix_cores else lib.rmi_hip_q8_0_forward_batched
        check(fn(self.w.handle, ptr(x, _f32p), ptr(_out(output, n_tokens * n_out), _f32p), n_in, n_out, n_tokens,
                 rounding))

    # free functions of the reference that take the weight slice as first argument
    def matmul_q8_0_quantized_range(self, input_q8, input_scales, output, n_in, row_start, row_end):
        """`matmul_q8_0_quantized_range`: `output` is pre-sliced (index 0 = row_start)."""
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_matmul_q8_0_quantized_range(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                      ptr(_out(output, max(row_end - row_start, 0)), _f32p), n_in,
                                                      row_start, row_end))

    def matmul_q8_0_quantized_batch(self, input_q8, input_scales, output, n_in, n_out, n_tokens):
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_matmul_q8_0_quantized_batch(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                      ptr(_out(output, n_tokens * n_out), _f32p), n_in, n_out,
                                                      n_tokens))

    def matmul_q8_0(self, input, output, n_in, n_out):
        """`ops::matmul_q8_0`: f32 activations, no activation quantisation."""
        x = as_f32(input)
        check(lib.rmi_hip_matmul_q8_0_f32(self.w.handle, ptr(x, _f32p), ptr(_out(output, n_out), _f32p), n_in, n_out))

    def matmul_q8_0_fallback_range(self, input, output, n_in, row_start, row_end):
        """`matmul_q8_0_fallback_range` (src/ops/kernel/q8_0/scalar.rs:3-29): the f32-activation product in the
        scalar kernel's order, rows [row_start, row_end) into `output[0 .. row_end - row_start)`."""
        x = as_f32(input)
        check(lib.rmi_hip_matmul_q8_0_fallback_range(self.w.handle, ptr(x, _f32p),
                                                     ptr(_out(output, row_end - row_start), _f32p), n_in, row_start,
                                                     row_end))

    def matmul_q8_0_via_q8(self, input, output, n_in, n_out, q8_buf, scale_buf, rounding=hip.ROUND_TIES_EVEN):
        """`matmul_q8_0_via_q8` (src/ops/kernel/q8_0/legacy.rs:27-83): quantize the f32 input into the caller's
        scratch (which keeps the quants and scales afterwards, as in the reference), then the prequantized GEMV."""
        quantize_q8_0_into(input, n_in, q8_buf, scale_buf, rounding)
        self.forward_prequantized(q8_buf, scale_buf, output, n_in, n_out, 0, 1)

    def block_dots(self, input_q8):
        q8 = as_u8(input_q8)
        dots = np.zeros((self.w.n_out, self.w.n_in // 32), np.int32)
        check(lib.rmi_hip_block_dots_q8_0(self.w.handle, ptr(q8, _u8p), ptr(dots, _i32p)))
        return dots


class MatmulTask:
    """One f32-input matmul of a batch (`MatmulTask`, src/ops/kernel/q8_0/batch.rs:20-26); `weight` is a Q8Kernel."""

    def __init__(self, weight, input, output, n_in, n_out):
        self.weight, self.input, self.output, self.n_in, self.n_out = weight, input, output, n_in, n_out


def matmul_q8_0_batch(tasks):
    """`matmul_q8_0_batch` (batch.rs:32-79): every task is the f32-activation matmul over all of its rows; the
    reference's 128-row chunks are a scheduling detail and leave each row's result unchanged."""
    for t in tasks:
        t.weight.matmul_q8_0(t.input, t.output, t.n_in, t.n_out)


class Q4_0Kernel(Kernel):
    def __init__(self, data, n_in, n_out, _handle=None):
        if _handle is None:
            w = as_u8(data)
            _handle = lib.rmi_hip_upload_q4_0(ptr(w, _u8p), w.size, n_in, n_out)
        self.w = _DeviceWeight(_handle)

    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_q4_0_forward_prequantized(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                    ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward(self, input, output, n_in, n_out, rounding=hip.ROUND_TIES_EVEN):
        self.forward_batched(as_f32(input)[:n_in], output, n_in, n_out, rounding)

    def forward_batched(self, input, output, n_in, n_out, rounding=hip.ROUND_TIES_EVEN):
        x = as_f32(input).reshape(-1)
        n_tokens = x.size // n_in
        check(lib.rmi_hip_q4_0_forward_batched(self.w.handle, ptr(x, _f32p),
                                               ptr(_out(output, n_tokens * n_out), _f32p), n_in, n_out, n_tokens,
                                               rounding))

    def block_dots(self, input_q8):
        q8 = as_u8(input_q8)
        dots = np.zeros((self.w.n_out, self.w.n_in // 32), np.int32)
        check(lib.rmi_hip_block_dots_q4_0(self.w.handle, ptr(q8, _u8p), ptr(dots, _i32p)))
        return dots


class Q4_KKernel(Kernel):
    def __init__(self, data, n_in, n_out, _handle=None):
        if _handle is None:
            w = as_u8(data)
            _handle = lib.rmi_hip_upload_q4_k(ptr(w, _u8p), w.size, n_in, n_out)
        self.w = _DeviceWeight(_handle)

    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_q4_k_forward_prequantized(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                    ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward_prepared(self, input_f32, input_q8, input_scales, q8_k, output, n_in, n_out, ith, nth):
        if q8_k is None:  # q4_k.rs:77-84: the kernel quantizes input_f32[..n_in] itself
            q8_k = quantize_row_q8_k(as_f32(input_f32)[:n_in])
        d, qs, bs = _q8k_arrays(q8_k)
        check(lib.rmi_hip_q4_k_forward_prepared(self.w.handle, ptr(d, _f32p), ptr(qs, _i8p), ptr(bs, _i16p),
                                                ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward_batched(self, input, output, n_in, n_out, matrix_cores=False):
        """Every token through the x86-64-order GEMV (bit-exact, batch-independent); `matrix_cores=True` takes
        the int8 MFMA GEMM from 16 tokens on (exact integers, f32 within 1e-4 + 1e-4 |ref|)."""
        x = as_f32(input).reshape(-1)
        n_tokens = x.size // n_in
        fn = lib.rmi_hip_q4_k_forward_batched_mfma if matrix_cores else lib.rmi_hip_q4_k_forward_batched
        check(fn(self.w.handle, ptr(x, _f32p), ptr(_out(output, n_tokens * n_out), _f32p), n_in, n_out, n_tokens))

    def block_ints(self, q8_k):
        _, qs, bs = _q8k_arrays(q8_k)
        shape = (self.w.n_out, self.w.n_in // 256)
        isum, msum = np.zeros(shape, np.int32), np.zeros(shape, np.int32)
        check(lib.rmi_hip_block_ints_q4_k(self.w.handle, ptr(qs, _i8p), ptr(bs, _i16p), ptr(isum, _i32p),
                                          ptr(msum, _i32p)))
        return isum, msum


class Q6_KKernel(Kernel):
    def __init__(self, data, n_in, n_out, _handle=None):
        if _handle is None:
            w = as_u8(data)
            _handle = lib.rmi_hip_upload_q6_k(ptr(w, _u8p), w.size, n_in, n_out)
        self.w = _DeviceWeight(_handle)

    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        q8, sc = as_u8(input_q8), as_f32(input_scales)
        check(lib.rmi_hip_q6_k_forward_prequantized(self.w.handle, ptr(q8, _u8p), ptr(sc, _f32p),
                                                    ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward_prepared(self, input_f32, input_q8, input_scales, q8_k, output, n_in, n_out, ith, nth):
        if q8_k is None:  # q6_k.rs:63-69: the kernel quantizes input_f32[..n_in] itself
            q8_k = quantize_row_q8_k(as_f32(input_f32)[:n_in])
        d, qs, bs = _q8k_arrays(q8_k)
        check(lib.rmi_hip_q6_k_forward_prepared(self.w.handle, ptr(d, _f32p), ptr(qs, _i8p), ptr(bs, _i16p),
                                                ptr(_out(output, n_out), _f32p), n_in, n_out, ith, nth))

    def forward_batched(self, input, output, n_in, n_out):
        x = as_f32(input).reshape(-1)
        n_tokens = x.size // n_in
        check(lib.rmi_hip_q6_k_forward_batched(self.w.handle, ptr(x, _f32p),
                                               ptr(_out(output, n_tokens * n_out), _f32p), n_in, n_out, n_tokens))

    def block_lanes(self, q8_k):
        """The eight int32 accumulator lanes per (row, super-block)."""
        _, qs, bs = _q8k_arrays(q8_k)
        lanes = np.zeros((self.w.n_out, self.w.n_in // 256, 8), np.int32)
        check(lib.rmi_hip_block_lanes_q6_k(self.w.handle, ptr(qs, _i8p), ptr(bs, _i16p), ptr(lanes, _i32p)))
        return lanes


class QuantizedTensor:
    """`QuantizedTensor::from_bytes(..).into_kernel()`: the factory the `hip`
    back end hooks (quantized_tensor.rs:120-138, 167-190)."""

    def __init__(self, ggml_type, data, n_in, n_out):
        self.ggml_type, self.data, self._n_in, self._n_out = ggml_type, data, n_in, n_out

    @classmethod
    def from_bytes(cls, ggml_type, data, n_in, n_out):
        if ggml_type not in (GGML_TYPE_Q8_0, GGML_TYPE_Q4_0, GGML_TYPE_Q4_K, GGML_TYPE_Q6_K):
            return None  # other dtypes stay on the reference's CPU kernels
        return cls(ggml_type, data, n_in, n_out)

    def n_in(self):
        return self._n_in

    def n_out(self):
        return self._n_out

    def into_kernel(self):
        if self.ggml_type == GGML_TYPE_Q8_0:
            return Q8Kernel(self.data, self._n_in, self._n_out)
        if self.ggml_type == GGML_TYPE_Q6_K:
            return Q6_KKernel(self.data, self._n_in, self._n_out)
        if self.ggml_type == GGML_TYPE_Q4_0:
            return Q4_0Kernel(self.data, self._n_in, self._n_out)
        return Q4_KKernel(self.data, self._n_in, self._n_out)


def fuse_vstack(a, b):
    """`QTensorOwned::fuse_vstack(a, b) -> Option<Self>` on device-resident weights."""
    if type(a) is not type(b):
        return None
    handle = lib.rmi_hip_fuse_vstack(a.w.handle, b.w.handle)
    if not handle:
        return None
    return type(a)(None, a.w.n_in, a.w.n_out + b.w.n_out, _handle=handle)


class QTensorOwned(Kernel):
    """`QTensorOwned` (src/ops/kernel/qtensor_owned.rs): the owned weight of the Qwen3.5 path.  Here every weight
    is owned by construction (the bytes are copied to HBM), so this is the same device kernel behind the owned
    type's method names.  Q8_0, Q4_K and Q6_K are offered; F32 / F16 / Q5_K stay on the host crate's CPU kernels
    (`from_bytes_owned` returns None for them, which is the caller's signal to keep its own)."""

    _KERNELS = {GGML_TYPE_Q8_0: Q8Kernel, GGML_TYPE_Q4_K: Q4_KKernel, GGML_TYPE_Q6_K: Q6_KKernel}

    def __init__(self, ggml_type, kernel):
        self._type, self.kernel = ggml_type, kernel

    @classmethod
    def from_bytes_owned(cls, data, ggml_type, n_cols, n_rows):
        if ggml_type not in cls._KERNELS:
            return None
        return cls(ggml_type, cls._KERNELS[ggml_type](data, n_cols, n_rows))

    @classmethod
    def from_quantized(cls, q):
        """`from_quantized(QuantizedTensor)`; Q4_0 is not modelled by the owned type (qtensor_owned.rs:129-133)."""
        if q.ggml_type == GGML_TYPE_Q4_0:
            raise ValueError("Q4_0 / Q4_1 not yet supported in QTensorOwned")
        return cls.from_bytes_owned(q.data, q.ggml_type, q.n_in(), q.n_out())

    def n_in(self):
        return self.kernel.w.n_in

    n_cols = n_in

    def n_rows(self):
        return self.kernel.w.n_out

    def ggml_type(self):
        return self._type

    @staticmethod
    def fuse_vstack(a, b):
        """None when dtype or n_cols differ (qtensor_owned.rs:139-141)."""
        if a._type != b._type:
            return None
        fused = fuse_vstack(a.kernel, b.kernel)
        return None if fused is None else QTensorOwned(a._type, fused)

    # ---- Kernel (qtensor_owned.rs:167-255)
    def forward_prequantized(self, input_q8, input_scales, output, n_in, n_out, ith, nth):
        self.kernel.forward_prequantized(input_q8, input_scales, output, n_in, n_out, ith, nth)

    def forward_prepared(self, input_f32, input_q8, input_scales, q8_k, output, n_in, n_out, ith, nth):
        if self._type == GGML_TYPE_Q8_0:  # Q8_0 ignores q8_k
            self.kernel.forward_prequantized(input_q8, input_scales, output, n_in, n_out, ith, nth)
        else:
            self.kernel.forward_prepared(input_f32, input_q8, input_scales, q8_k, output, n_in, n_out, ith, nth)

    # ---- Q8_K matmuls (qtensor_owned.rs:374-471)
    def matmul_into_with_q8k(self, q8k, output, row_start, row_end):
        """Rows [row_start, row_end) into `output[0 .. row_end - row_start]`."""
        if self._type == GGML_TYPE_Q8_0:
            raise ValueError("matmul_with_q8k called on non-K-quant weight type")
        n_rows = self.n_rows()
        full = np.zeros(n_rows, np.float32)
        self.kernel.forward_prepared(None, None, None, q8k, full, self.n_in(), n_rows, 0, 1)
        _out(output, row_end - row_start)[:row_end - row_start] = full[row_start:row_end]

    def matmul_with_q8k_into_buf(self, q8k, buf):
        self.matmul_into_with_q8k(q8k, buf, 0, self.n_rows())

    def matmul_with_q8k(self, q8k):
        out = np.zeros(self.n_rows(), np.float32)
        self.matmul_with_q8k_into_buf(q8k, out)
        return out

    def matmul_with_q8k_into_buf_pooled(self, q8k, buf, pool=None):
        """The reference splits rows over its pool; one launch covers them all here."""
        self.matmul_with_q8k_into_buf(q8k, buf)

    def matmul_into(self, input, output, row_start, row_end):
        """K-quants: quantize_row_q8_k, then the Q8_K dot (qtensor_owned.rs:325-371).  The Q8_0 / F32 / F16 arms of
        the reference dequantise and call dot_f32 per block, an f32-activation fallback off the quantized path."""
        if self._type == GGML_TYPE_Q8_0:
            raise NotImplementedError("QTensorOwned::matmul_into of a Q8_0 weight is the CPU dequantise-and-dot fallback")
        self.matmul_into_with_q8k(quantize_row_q8_k(as_f32(input)[:self.n_in()]), output, row_start, row_end)

    def matmul(self, input):
        out = np.zeros(self.n_rows(), np.float32)
        self.matmul_into(input, out, 0, self.n_rows())
        return out

    # ---- quantize + matmul (qtensor_owned.rs:516-589)
    def quantize_and_matmul_with_scratch(self, input, q8k_buf, q8_buf, scale_buf, buf, pool=None,
                                         rounding=hip.ROUND_TIES_EVEN):
        """K-quants: `quantize_row_q8_k_into(input, q8k_buf[..blocks])`, then the Q8_K matmul.  Q8_0:
        `quantize_q8_0_into(input, n_cols, q8_buf, scale_buf)`, then `matmul_q8_0_quantized_parallel_rows`.  The
        scratch buffers hold the quantized activation afterwards, as in the reference."""
        n_cols, n_rows = self.n_in(), self.n_rows()
        x = as_f32(input)[:n_cols]
        if self._type == GGML_TYPE_Q8_0:
            quantize_q8_0_into(x, n_cols, q8_buf, scale_buf, rounding)
            self.kernel.forward_prequantized(q8_buf[:n_cols], scale_buf[:n_cols // 32], buf, n_cols, n_rows, 0, 1)
        else:
            blocks = n_cols // 256
            q8k_buf[:blocks] = quantize_row_q8_k(x)
            self.matmul_with_q8k_into_buf_pooled(q8k_buf[:blocks], buf, pool)

    def quantize_and_matmul(self, input, q8k_buf, buf):
        n = as_f32(input).size
        self.quantize_and_matmul_with_scratch(input, q8k_buf, np.zeros(n, np.uint8), np.zeros((n + 31) // 32, np.float32),
                                              buf, None)


@dataclass
class ExecContext:
    """src/core/traits.rs:45-66.  `scratch` is accepted for signature parity; the
    GPU path dequantises in registers and never touches it."""
    scratch: np.ndarray
    kv_cache: object = None
    pos: int = 0
    layer_idx: int = 0


class Layer:
    """src/core/traits.rs:68-74"""

    def forward(self, input, output, ctx):
        raise NotImplementedError

    def input_dim(self):
        raise NotImplementedError

    def output_dim(self):
        raise NotImplementedError

    def name(self):
        raise NotImplementedError


class QuantizedLinear(Layer):
    """src/core/model.rs:12-104: always reads its weight as Q4_K, ignores bias."""

    def __init__(self, weight, bias, in_features, out_features, name, _kernel=None):
        self.kernel = _kernel if _kernel is not None else Q4_KKernel(weight, in_features, out_features)
        self.bias = bias
        self.in_features, self.out_features, self.layer_name = in_features, out_features, name

    @classmethod
    def from_weight_slice(cls, weight, bias, in_features, out_features, name):
        return cls(weight, bias, in_features, out_features, name)

    @classmethod
    def from_source(cls, source, weight_name, bias_name, in_features, out_features, name):
        """src/core/model.rs:38-55 over a `loader.GGUFLoader`: None when the weight is not in the file.  The
        bytes go from the file's mapping to HBM inside the library."""
        info = source.tensor_info(weight_name)
        if info is None:
            return None
        bias = source.tensor_data(bias_name) if bias_name else None
        if info.ggml_type == GGML_TYPE_Q4_K and info.dims == (in_features, out_features):
            return cls(None, bias, in_features, out_features, name, _kernel=source.kernel(weight_name))
        return cls(source.tensor_data(weight_name), bias, in_features, out_features, name)

    def forward_dequant(self, input, output, scratch=None):
        x = as_f32(input)
        check(lib.rmi_hip_quantized_linear_forward(self.kernel.w.handle, ptr(x, _f32p),
                                                   ptr(_out(output, self.out_features), _f32p), self.in_features,
                                                   self.out_features))

    def forward(self, input, output, ctx):
        self.forward_dequant(input, output, ctx.scratch if ctx is not None else None)

    def input_dim(self):
        return self.in_features

    def output_dim(self):
        return self.out_features

    def name(self):
        return self.layer_name


class ModelGraph:
    """src/core/model.rs:107-153: a stack of layers ping-ponging two buffers."""

    def __init__(self, config=None):
        self.config = config
        self.layers = []

    def add_layer(self, layer):
        self.layers.append(layer)

    def forward_all(self, input, output, scratch, ctx):
        if not self.layers:
            return
        dim = max(self.layers[0].output_dim(), self.layers[0].input_dim())
        buf_a = np.zeros(max(dim, max(max(l.input_dim(), l.output_dim()) for l in self.layers)), np.float32)
        buf_b = np.zeros_like(buf_a)
        x = as_f32(input)
        buf_a[:x.size] = x
        for i, layer in enumerate(self.layers):
            ctx.layer_idx = i
            if i % 2 == 0:
                layer.forward(buf_a, buf_b, ctx)
            else:
                layer.forward(buf_b, buf_a, ctx)
        src = buf_b if (len(self.layers) - 1) % 2 == 0 else buf_a
        n = min(output.size, src.size)
        output[:n] = src[:n]
