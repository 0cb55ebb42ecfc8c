"""Host-side mirror of the reference's ``GGUFLoader`` (src/core/loader.rs:187-372) over the native parser
of the C ABI, plus the uploads that go from the file's mapping to HBM without a host copy of the tensor.

Opening a file and querying it needs no GPU; ``upload*`` and ``Qwen3Session.from_gguf`` do.
"""
import ctypes as C

import numpy as np

from . import hip

# MetaValueType tags (src/core/tensor.rs:92-106)
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)


class TensorInfo:
    """TensorInfo of src/core/tensor.rs:189-230: name, dims ([columns, rows, ..]), ggml type tag, offset."""

    def __init__(self, name, dims, ggml_type, offset, nbytes):
        self.name, self.dims, self.ggml_type, self.offset, self._nbytes = name, dims, ggml_type, offset, nbytes

    def nbytes(self):
        return self._nbytes

    def n_elements(self):
        n = 1
        for d in self.dims:
            n *= d
        return n


class GGUFLoader:
    def __init__(self, handle):
        self._h = handle

    @classmethod
    def from_file(cls, path):
        """GGUFLoader::from_file; raises ValueError with the reference's message on a file it rejects."""
        h = hip.lib.rmi_hip_gguf_open(str(path).encode())
        if not h:
            raise ValueError(hip.last_error())
        return cls(h)

    def close(self):
        if self._h:
            hip.lib.rmi_hip_gguf_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    version = property(lambda self: hip.lib.rmi_hip_gguf_version(self._h))
    alignment = property(lambda self: hip.lib.rmi_hip_gguf_alignment(self._h))

    def n_tensors(self):
        return hip.lib.rmi_hip_gguf_n_tensors(self._h)

    def n_kv(self):
        return hip.lib.rmi_hip_gguf_n_kv(self._h)

    def data_offset(self):
        return hip.lib.rmi_hip_gguf_data_offset(self._h)

    def keys(self):
        return [hip.lib.rmi_hip_gguf_kv_key(self._h, i).decode() for i in range(self.n_kv())]

    # --- metadata: the MetaValue conversions, None where the reference gives None
    def meta_type(self, key):
        t = hip.lib.rmi_hip_gguf_meta_type(self._h, key.encode())
        return None if t < 0 else t

    def to_u64(self, key):
        v = C.c_uint64()
        return v.value if hip.lib.rmi_hip_gguf_meta_u64(self._h, key.encode(), C.byref(v)) else None

    def to_f64(self, key):
        v = C.c_double()
        return v.value if hip.lib.rmi_hip_gguf_meta_f64(self._h, key.encode(), C.byref(v)) else None

    def to_bool(self, key):
        v = C.c_int()
        return bool(v.value) if hip.lib.rmi_hip_gguf_meta_bool(self._h, key.encode(), C.byref(v)) else None

    def to_string_val(self, key):
        n = hip.lib.rmi_hip_gguf_meta_str(self._h, key.encode(), None, 0)
        if n < 0:
            return None
        buf = C.create_string_buffer(n + 1)
        hip.lib.rmi_hip_gguf_meta_str(self._h, key.encode(), buf, n + 1)
        return buf.raw[:n].decode()

    def array_len(self, key):
        n = hip.lib.rmi_hip_gguf_meta_array_len(self._h, key.encode(), None)
        return None if n < 0 else n

    def array_u64(self, key):
        n = self.array_len(key)
        if n is None:
            return None
        out, v = [], C.c_uint64()
        for i in range(n):
            if not hip.lib.rmi_hip_gguf_meta_array_u64(self._h, key.encode(), i, C.byref(v)):
                return None
            out.append(v.value)
        return out

    # --- tensors
    def tensor_info(self, name):
        i = name if isinstance(name, int) else hip.lib.rmi_hip_gguf_find_tensor(self._h, name.encode())
        if i < 0 or i >= self.n_tensors():
            return None
        nm, nd, dims = C.c_char_p(), C.c_uint32(), (C.c_uint64 * 8)()
        ty, off, nb = C.c_int(), C.c_uint64(), C.c_uint64()
        hip.check(hip.lib.rmi_hip_gguf_tensor_info(self._h, i, C.byref(nm), C.byref(nd), dims, 8, C.byref(ty),
                                                   C.byref(off), C.byref(nb)))
        return TensorInfo(nm.value.decode(), tuple(dims[:nd.value]), ty.value, off.value, nb.value)

    def tensors(self):
        return [self.tensor_info(i) for i in range(self.n_tensors())]

    def tensor_data(self, name):
        """uint8 view of the tensor's bytes in the mapping (valid until close()); None for an unknown name."""
        i = hip.lib.rmi_hip_gguf_find_tensor(self._h, name.encode())
        if i < 0:
            return None
        info = self.tensor_info(i)
        p = hip.lib.rmi_hip_gguf_tensor_data(self._h, i)
        return np.ctypeslib.as_array(C.cast(p, hip._u8p), shape=(info.nbytes(),)) if info.nbytes() else np.zeros(0, np.uint8)

    # --- file -> HBM
    def upload(self, *names):
        """One device weight from one matrix, or from several stacked row-wise ([q ; k ; v])."""
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        h = hip.lib.rmi_hip_gguf_upload_stack(self._h, arr, len(names))
        if not h:
            raise hip.RmiHipError(-1, hip.last_error())
        return h

    def kernel(self, *names):
        """The `Kernel` of one matrix of the file (or of several stacked row-wise), of the class its type has."""
        from . import kernel as K

        h = self.upload(*names)
        cls = {hip.DTYPE_Q8_0: K.Q8Kernel, hip.DTYPE_Q4_0: K.Q4_0Kernel, hip.DTYPE_Q4_K: K.Q4_KKernel,
               hip.DTYPE_Q6_K: K.Q6_KKernel}[hip.lib.rmi_hip_weight_dtype(h)]
        return cls(None, hip.lib.rmi_hip_weight_n_in(h), hip.lib.rmi_hip_weight_n_out(h), _handle=h)

    def qwen3_config(self, capacity, rounding=hip.ROUND_TIES_EVEN):
        c = hip.Qwen3Config()
        rc = hip.lib.rmi_hip_gguf_qwen3_config(self._h, capacity, rounding, C.byref(c))
        if rc != 0:
            raise ValueError(hip.last_error())
        return c
