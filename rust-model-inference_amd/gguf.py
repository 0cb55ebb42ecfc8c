"""Minimal GGUF v3 writer and mmap reader, enough for the synthetic all-Q8_0
Qwen3 file of the end-to-end configuration.  Layout as the reference's loader
reads it (src/core/loader.rs:217-320): magic "GGUF", u32 version, u64 tensor
count, u64 kv count, kv pairs (string = u64 length + bytes, i32 type tag,
value), tensor infos (name, u32 n_dims, u64 dims[], i32 ggml type, u64 offset),
then tensor data from the next multiple of general.alignment (default 32).
Dims are [n_in, n_out] (columns first, src/models/qwen3.rs:1297-1311).
"""
import mmap
import struct

import numpy as np

GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q8_0, GGML_Q4_K, GGML_Q6_K = 0, 1, 2, 8, 12, 14
_TYPE_TRAITS = {GGML_F32: (1, 4), GGML_F16: (1, 2), GGML_Q4_0: (32, 18), GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144),
                GGML_Q6_K: (256, 210)}
# metadata value type tags (src/core/loader.rs MetaValueType)
_U32, _I32, _F32, _BOOL, _STR, _ARR, _U64, _F64 = 4, 5, 6, 7, 8, 9, 10, 12
ALIGNMENT = 32


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _kv(key, value):
    out = _s(key)
    if isinstance(value, bool):
        return out + struct.pack("<iB", _BOOL, int(value))
    if isinstance(value, int):
        return out + struct.pack("<iI", _U32, value)
    if isinstance(value, float):
        return out + struct.pack("<if", _F32, value)
    if isinstance(value, str):
        return out + struct.pack("<i", _STR) + _s(value)
    raise TypeError(f"unsupported metadata value for {key}: {type(value)}")


def tensor_nbytes(dims, ggml_type):
    n = 1
    for d in dims:
        n *= int(d)
    block, size = _TYPE_TRAITS[ggml_type]
    return n // block * size


def write_gguf(path, metadata, tensors):
    """tensors: iterable of (name, dims, ggml_type, array-like bytes), written in order."""
    tensors = list(tensors)
    infos, offset = [], 0
    for name, dims, ggml_type, data in tensors:
        nbytes = tensor_nbytes(dims, ggml_type)
        assert np.asarray(data).nbytes == nbytes, (name, np.asarray(data).nbytes, nbytes)
        infos.append(_s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", int(d)) for d in dims)
                     + struct.pack("<iQ", ggml_type, offset))
        offset += (nbytes + ALIGNMENT - 1) // ALIGNMENT * ALIGNMENT
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(metadata))
    head += b"".join(_kv(k, v) for k, v in metadata.items()) + b"".join(infos)
    pad = (-len(head)) % ALIGNMENT
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for name, dims, ggml_type, data in tensors:
            raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
            f.write(raw.tobytes())
            f.write(b"\0" * ((-raw.size) % ALIGNMENT))


class GGUFFile:
    """mmap view of a GGUF file: `.metadata` dict, `.tensors[name] = (dims, ggml_type, uint8 view)`."""

    def __init__(self, path):
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        buf = self._mm
        if buf[:4] != b"GGUF":
            raise ValueError("Invalid GGUF magic")
        pos = 4
        (version,) = struct.unpack_from("<I", buf, pos)
        if version not in (2, 3):
            raise ValueError(f"Unsupported GGUF version: {version}")
        n_tensors, n_kv = struct.unpack_from("<QQ", buf, pos + 4)
        pos += 20

        def rd_str(p):
            (n,) = struct.unpack_from("<Q", buf, p)
            return buf[p + 8:p + 8 + n].decode(), p + 8 + n

        def rd_val(t, p):
            fmt = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q",
                   12: "<d"}
            if t in fmt:
                (v,) = struct.unpack_from(fmt[t], buf, p)
                return (bool(v) if t == 7 else v), p + struct.calcsize(fmt[t])
            if t == _STR:
                return rd_str(p)
            if t == _ARR:
                et, n = struct.unpack_from("<iQ", buf, p)
                p += 12
                vals = []
                for _ in range(n):
                    v, p = rd_val(et, p)
                    vals.append(v)
                return vals, p
            raise ValueError(f"Unknown meta value type: {t}")

        self.version = version
        self.metadata = {}
        for _ in range(n_kv):
            key, pos = rd_str(pos)
            (t,) = struct.unpack_from("<i", buf, pos)
            self.metadata[key], pos = rd_val(t, pos + 4)
        infos = []
        for _ in range(n_tensors):
            name, pos = rd_str(pos)
            (nd,) = struct.unpack_from("<I", buf, pos)
            dims = struct.unpack_from(f"<{nd}Q", buf, pos + 4)
            ggml_type, off = struct.unpack_from("<iQ", buf, pos + 4 + 8 * nd)
            pos += 4 + 8 * nd + 12
            infos.append((name, dims, ggml_type, off))
        align = int(self.metadata.get("general.alignment", ALIGNMENT))
        data_offset = (pos + align - 1) // align * align
        whole = np.frombuffer(buf, np.uint8)
        self.tensors = {}
        for name, dims, ggml_type, off in infos:
            n = tensor_nbytes(dims, ggml_type)
            if data_offset + off + n > whole.size:
                raise ValueError(f"tensor {name} exceeds GGUF data")
            self.tensors[name] = (tuple(int(d) for d in dims), ggml_type, whole[data_offset + off:data_offset + off + n])

    def tensor(self, name):
        return self.tensors[name][2]


def write_synthetic_qwen3(path, seed, n_layer=28, n_embd=1024, n_head=16, n_head_kv=8, head_dim=128, n_ff=3072,
                          vocab=151936, n_ctx=40960):
    """Random-init Qwen3 architecture, every 2-D weight Q8_0 (same distribution as
    synth.q8_0_weight), norm weights F32 = 1 + small noise, tied lm_head (no
    output.weight), no EOS id so generation cannot stop early."""
    from . import synth

    meta = {
        "general.architecture": "qwen3",
        "general.alignment": ALIGNMENT,
        "qwen3.embedding_length": n_embd,
        "qwen3.attention.head_count": n_head,
        "qwen3.attention.head_count_kv": n_head_kv,
        "qwen3.block_count": n_layer,
        "qwen3.feed_forward_length": n_ff,
        "qwen3.context_length": n_ctx,
        "qwen3.attention.layer_norm_rms_epsilon": 1e-6,
        "qwen3.rope.freq_base": 1000000.0,
        "qwen3.attention.key_length": head_dim,
        "qwen3.attention.value_length": head_dim,
        "qwen3.vocab_size": vocab,
    }
    rng = np.random.default_rng(seed)

    def norm(n):
        return (1.0 + 0.02 * rng.standard_normal(n)).astype(np.float32)

    def gen():
        tid = 0
        yield "token_embd.weight", (n_embd, vocab), GGML_Q8_0, synth.q8_0_weight(seed * 1000 + tid, vocab, n_embd)
        yield "output_norm.weight", (n_embd,), GGML_F32, norm(n_embd)
        q_dim, kv_dim = n_head * head_dim, n_head_kv * head_dim
        for layer in range(n_layer):
            p = f"blk.{layer}."
            yield p + "attn_norm.weight", (n_embd,), GGML_F32, norm(n_embd)
            yield p + "ffn_norm.weight", (n_embd,), GGML_F32, norm(n_embd)
            yield p + "attn_q_norm.weight", (head_dim,), GGML_F32, norm(head_dim)
            yield p + "attn_k_norm.weight", (head_dim,), GGML_F32, norm(head_dim)
            for name, n_in, n_out in (("attn_q", n_embd, q_dim), ("attn_k", n_embd, kv_dim), ("attn_v", n_embd, kv_dim),
                                      ("attn_output", q_dim, n_embd), ("ffn_gate", n_embd, n_ff),
                                      ("ffn_up", n_embd, n_ff), ("ffn_down", n_ff, n_embd)):
                tid += 1
                yield p + name + ".weight", (n_in, n_out), GGML_Q8_0, synth.q8_0_weight(seed * 1000 + tid, n_out, n_in)

    write_gguf(path, meta, gen())
    return meta
