"""The native GGUF parser against the reference's own loader fixtures (the byte strings its unit tests build,
src/core/loader.rs:695-1181, restated here as data) and against the Python reader on a synthetic Qwen3 file.
No GPU: open / close and the metadata and tensor queries need none."""
import struct

import numpy as np
import pytest

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
Q4K = 12


def s(text):
    b = text if isinstance(text, bytes) else text.encode()
    return struct.pack("<Q", len(b)) + b


def kv(key, tag, payload):
    return s(key) + struct.pack("<i", tag) + payload


def head(n_tensors, n_kv, version=3, magic=b"GGUF"):
    return magic + struct.pack("<IQQ", version, n_tensors, n_kv)


def pad32(b):
    return b + b"\0" * ((-len(b)) % 32)


def write(tmp_path, data, name="t.gguf", total=None):
    p = tmp_path / name
    with open(p, "wb") as f:
        f.write(data)
        if total is not None:
            f.truncate(total)  # sparse tail: tensor data nobody reads
    return p


@pytest.fixture()
def L(rmi):
    return rmi.loader


def open_err(L, path):
    with pytest.raises(ValueError) as e:
        L.GGUFLoader.from_file(path)
    return str(e.value)


def minimal_gguf():
    """build_minimal_gguf (src/core/loader.rs:695-776): 11 keys, two Q4K tensors."""
    b = head(2, 11)
    b += kv("general.architecture", STR, s("qwen2"))
    b += kv("qwen2.embedding_length", U32, struct.pack("<I", 1024))
    b += kv("qwen2.block_count", U32, struct.pack("<I", 24))
    b += kv("qwen2.attention.head_count", U32, struct.pack("<I", 16))
    b += kv("general.alignment", U64, struct.pack("<Q", 32))
    b += kv("qwen2.attention.head_count_kv", U32, struct.pack("<I", 16))
    b += kv("qwen2.feed_forward_length", U32, struct.pack("<I", 2816))
    b += kv("qwen2.context_length", U32, struct.pack("<I", 4096))
    b += kv("qwen2.vocab_size", U32, struct.pack("<I", 151936))
    b += kv("qwen2.rope.freq_base", F32, struct.pack("<f", 1_000_000.0))
    b += kv("qwen2.attention.layer_norm_rms_epsilon", F32, struct.pack("<f", 1e-6))
    embd = 1024 * 151936 // 256 * 144
    padded = (embd + 31) // 32 * 32
    b += s("token_embd.weight") + struct.pack("<IQQiQ", 2, 1024, 151936, Q4K, 0)
    b += s("blk.0.attn_q.weight") + struct.pack("<IQQiQ", 2, 1024, 1024, Q4K, padded)
    b = pad32(b)
    return b, len(b) + padded + 1024 * 1024 // 256 * 144


def test_parse_minimal(L, tmp_path):
    """test_gguf_parse_minimal (src/core/loader.rs:846-889)."""
    data, total = minimal_gguf()
    g = L.GGUFLoader.from_file(write(tmp_path, data, total=total))
    assert (g.version, g.alignment, g.n_tensors(), g.n_kv()) == (3, 32, 2, 11)
    assert g.to_string_val("general.architecture") == "qwen2"
    assert g.to_u64("qwen2.embedding_length") == 1024
    assert g.to_u64("qwen2.block_count") == 24
    t0 = g.tensor_info("token_embd.weight")
    assert (t0.dims, t0.ggml_type, t0.offset) == ((1024, 151936), Q4K, 0)
    t1 = g.tensor_info("blk.0.attn_q.weight")
    assert t1.dims == (1024, 1024)
    assert g.tensor_data("token_embd.weight").size == t0.nbytes() == 1024 * 151936 // 256 * 144
    assert g.tensor_data("blk.0.attn_q.weight").size == t1.nbytes() == 1024 * 1024 // 256 * 144
    assert g.data_offset() == len(data) and g.data_offset() % 32 == 0
    assert g.tensor_info("nope") is None and g.tensor_data("nope") is None
    assert g.keys()[0] == "general.architecture" and len(g.keys()) == 11
    # model_config_from_source over the same file (:904-907): the qwen2 prefix, no q/k norms
    c = g.qwen3_config(capacity=64)
    assert (c.n_embd, c.n_layer, c.n_head, c.n_head_kv, c.n_ff, c.vocab) == (1024, 24, 16, 16, 2816, 151936)
    assert (c.head_dim_k, c.head_dim_v, c.has_qk_norm, c.capacity) == (64, 64, 0, 64)
    assert c.freq_base == 1_000_000.0 and c.eps == np.float32(1e-6)
    with pytest.raises(ValueError, match="Session capacity 4097 exceeds model context 4096"):
        g.qwen3_config(capacity=4097)
    g.close()


def all_meta_types():
    """build_all_meta_types_gguf (src/core/loader.rs:778-833)."""
    b = head(0, 13)
    b += kv("test.uint8", U8, struct.pack("<B", 42))
    b += kv("test.int8", I8, struct.pack("<b", -1))
    b += kv("test.uint16", U16, struct.pack("<H", 1000))
    b += kv("test.int16", I16, struct.pack("<h", -100))
    b += kv("test.uint32", U32, struct.pack("<I", 1024))
    b += kv("test.int32", I32, struct.pack("<i", -24))
    b += kv("test.float32", F32, struct.pack("<f", 3.14))
    b += kv("test.bool", BOOL, b"\x01")
    b += kv("test.string", STR, s("hello"))
    b += kv("test.uint64", U64, struct.pack("<Q", 999999))
    b += kv("test.int64", I64, struct.pack("<q", -123456))
    b += kv("test.float64", F64, struct.pack("<d", 2.71828))
    b += kv("test.array", ARR, struct.pack("<iQIII", U32, 3, 10, 20, 30))
    return pad32(b)


def test_all_meta_types(L, tmp_path):
    """test_gguf_all_meta_types (src/core/loader.rs:988-1059); negative integers convert as Rust's `as u64`."""
    g = L.GGUFLoader.from_file(write(tmp_path, all_meta_types()))
    m = 1 << 64
    assert g.to_u64("test.uint8") == 42
    assert g.to_u64("test.int8") == m - 1
    assert g.to_u64("test.uint16") == 1000
    assert g.to_u64("test.int16") == m - 100
    assert g.to_u64("test.uint32") == 1024
    assert g.to_u64("test.int32") == m - 24
    assert abs(g.to_f64("test.float32") - 3.14) < 0.01
    assert g.to_f64("test.float32") == float(np.float32(3.14))
    assert g.to_bool("test.bool") is True and g.meta_type("test.bool") == BOOL
    assert g.to_string_val("test.string") == "hello"
    assert g.to_u64("test.uint64") == 999999
    assert g.to_u64("test.int64") == m - 123456
    assert g.to_f64("test.float64") == 2.71828
    assert g.meta_type("test.array") == ARR and g.array_len("test.array") == 3
    assert g.array_u64("test.array") == [10, 20, 30]
    # conversions the reference refuses (src/core/tensor.rs:147-187)
    assert g.to_u64("test.bool") is None and g.to_u64("test.string") is None and g.to_u64("test.array") is None
    assert g.to_f64("test.uint8") is None and g.to_f64("test.int16") is None and g.to_f64("test.bool") is None
    assert g.to_f64("test.int32") == -24.0 and g.to_f64("test.uint64") == 999999.0 and g.to_f64("test.int64") == -123456.0
    assert g.to_string_val("test.uint8") is None and g.array_len("test.string") is None
    assert g.to_u64("absent") is None and g.meta_type("absent") is None
    # float -> u64 saturates: 3.14 -> 3, 2.71828 -> 2
    assert g.to_u64("test.float32") == 3 and g.to_u64("test.float64") == 2


def test_float_to_u64_edges(L, tmp_path):
    b = head(0, 5)
    b += kv("neg", F32, struct.pack("<f", -1.5))
    b += kv("nan", F64, struct.pack("<d", float("nan")))
    b += kv("huge", F64, struct.pack("<d", 1e30))
    b += kv("inf", F32, struct.pack("<f", float("inf")))
    b += kv("edge", F64, struct.pack("<d", 18446744073709549568.0))  # the largest double below 2^64
    g = L.GGUFLoader.from_file(write(tmp_path, b))
    assert g.to_u64("neg") == 0 and g.to_u64("nan") == 0
    assert g.to_u64("huge") == (1 << 64) - 1 and g.to_u64("inf") == (1 << 64) - 1
    assert g.to_u64("edge") == 18446744073709549568


def test_string_and_bool_arrays(L, tmp_path):
    toks = ["<pad>", "héllo", "", "世界"]
    b = head(0, 3)
    b += kv("tokenizer.ggml.tokens", ARR, struct.pack("<iQ", STR, len(toks)) + b"".join(s(t) for t in toks))
    b += kv("flags", ARR, struct.pack("<iQ", BOOL, 3) + b"\x01\x00\x01")
    b += kv("after", U32, struct.pack("<I", 7))  # the cursor is past both arrays
    g = L.GGUFLoader.from_file(write(tmp_path, b))
    assert g.array_len("tokenizer.ggml.tokens") == 4 and g.array_u64("tokenizer.ggml.tokens") is None
    assert g.array_len("flags") == 3 and g.to_u64("after") == 7
    bad = head(0, 1) + kv("flags", ARR, struct.pack("<iQ", BOOL, 2) + b"\x01\x02")
    assert "Invalid bool value: 2" in open_err(L, write(tmp_path, bad, "bad.gguf"))


def test_malformed_files_are_rejected(L, tmp_path):
    """The rejection cases of src/core/loader.rs:1062-1181, each with the reference's message."""
    cases = {
        "bad_bool": (head(0, 1) + kv("b", BOOL, b"\x02"), "Invalid bool value: 2"),
        "bad_utf8": (head(0, 1) + struct.pack("<Q", 1) + b"\xff" + struct.pack("<iI", U32, 0), "Invalid UTF-8 string"),
        "bad_utf8_value": (head(0, 1) + kv("k", STR, struct.pack("<Q", 2) + b"\xc0\x80"), "Invalid UTF-8 string"),
        "array_count": (head(0, 1) + kv("a", ARR, struct.pack("<iQ", U8, 2)), "array count exceeds remaining bytes"),
        "nested": (pad32(head(0, 1) + kv("test.nested", ARR, struct.pack("<iQiQI", ARR, 1, U32, 1, 7))),
                   "Nested metadata arrays are not supported"),
        "kv_count": (head(0, 1), "metadata count exceeds remaining bytes"),
        "tensor_count": (head(1, 0), "tensor count exceeds remaining bytes"),
        "dim_count": (head(1, 0) + s("") + struct.pack("<I", 2) + b"\0" * 12,
                      "tensor dimension count exceeds remaining bytes"),
        "magic": (head(0, 0, magic=b"GGML"), "Invalid GGUF magic"),
        "version1": (head(0, 0, version=1), "Unsupported GGUF version: 1"),
        "version4": (head(0, 0, version=4), "Unsupported GGUF version: 4"),
        "meta_tag": (head(0, 1) + kv("k", 13, b"\0" * 16), "Unknown meta value type: 13"),
        "elem_tag": (head(0, 1) + kv("k", ARR, struct.pack("<iQ", -1, 0) + b"\0" * 16), "Unknown meta value type: -1"),
        "ggml_tag": (head(1, 0) + s("t") + struct.pack("<IQiQ", 1, 32, 4, 0) + b"\0" * 64, "Unknown GGML type: 4"),
        "alignment0": (head(0, 1) + kv("general.alignment", U32, struct.pack("<I", 0)), "GGUF alignment must be nonzero"),
        "ragged_row": (head(1, 0) + s("t") + struct.pack("<IQQiQ", 2, 48, 2, 8, 0) + b"\0" * 256,
                       "invalid tensor shape: t"),
        "no_dims": (head(1, 0) + s("t") + struct.pack("<IiQ", 0, 0, 0) + b"\0" * 64, "invalid tensor shape: t"),
        "overflow": (head(1, 0) + s("t") + struct.pack("<IQQQiQ", 3, 32, 1 << 40, 1 << 40, 8, 0) + b"\0" * 64,
                     "invalid tensor shape: t"),
        "past_end": (pad32(head(1, 0) + s("t") + struct.pack("<IQQiQ", 2, 32, 4, 8, 0)) + b"\0" * 135,
                     "tensor t exceeds GGUF data"),
        "offset_wrap": (pad32(head(1, 0) + s("t") + struct.pack("<IQQiQ", 2, 32, 4, 8, (1 << 64) - 8)) + b"\0" * 136,
                        "tensor t range overflow"),
        "empty": (b"", "EOF reading u32"),
    }
    for name, (data, want) in cases.items():
        err = open_err(L, write(tmp_path, data, name + ".gguf"))
        assert want in err, (name, err)
    assert "Failed to open GGUF file" in open_err(L, tmp_path / "absent.gguf")
    # one byte more and the tensor fits
    ok = pad32(head(1, 0) + s("t") + struct.pack("<IQQiQ", 2, 32, 4, 8, 0)) + b"\x07" * 136
    g = L.GGUFLoader.from_file(write(tmp_path, ok, "ok.gguf"))
    assert g.tensor_data("t").size == 136 and int(g.tensor_data("t")[135]) == 7


def test_every_truncation_is_an_error_not_a_crash(L, tmp_path):
    data = all_meta_types()
    end = len(data.rstrip(b"\0"))
    for n in list(range(0, 64)) + list(range(64, end, 7)):
        err = open_err(L, write(tmp_path, data[:n]))
        assert "EOF" in err or "exceeds remaining" in err, (n, err)
    mini, _ = minimal_gguf()
    for n in range(len(mini) - 200, len(mini) - 32, 5):
        assert open_err(L, write(tmp_path, mini[:n]))


def test_alignment_is_honoured(L, tmp_path):
    payload = np.arange(68, dtype=np.uint8).tobytes()
    for align, tag, fmt in ((64, U32, "<I"), (8, U64, "<Q"), (1, U8, "<B"), (32, None, None)):
        b = head(1, 0 if tag is None else 1)
        if tag is not None:
            b += kv("general.alignment", tag, struct.pack(fmt, align))
        b += s("w") + struct.pack("<IQQiQ", 2, 32, 2, 8, align)  # offset = one alignment unit into the data
        start = (len(b) + align - 1) // align * align
        b += b"\0" * (start - len(b)) + b"\xee" * align + payload
        g = L.GGUFLoader.from_file(write(tmp_path, b, f"a{align}.gguf"))
        assert g.alignment == align and g.data_offset() == start
        assert g.tensor_data("w").tobytes() == payload


def test_matches_the_python_reader_on_a_synthetic_qwen3(rmi, L, tmp_path):
    path = tmp_path / "q.gguf"
    meta = rmi.gguf.write_synthetic_qwen3(path, seed=5, n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32,
                                          n_ff=96, vocab=50, n_ctx=128)
    py = rmi.gguf.GGUFFile(path)
    g = L.GGUFLoader.from_file(path)
    assert g.n_kv() == len(py.metadata) and g.n_tensors() == len(py.tensors)
    for k, v in py.metadata.items():
        if isinstance(v, str):
            assert g.to_string_val(k) == v
        elif isinstance(v, float):
            assert g.to_f64(k) == v
        else:
            assert g.to_u64(k) == v
    for name, (dims, ty, view) in py.tensors.items():
        info = g.tensor_info(name)
        assert (info.dims, info.ggml_type, info.nbytes()) == (dims, ty, view.size)
        assert np.array_equal(g.tensor_data(name), view), name
    assert [t.name for t in g.tensors()] == list(py.tensors)
    c = g.qwen3_config(capacity=16)
    assert (c.n_embd, c.n_layer, c.n_head, c.n_head_kv, c.head_dim_k, c.head_dim_v) == (64, 2, 4, 2, 32, 32)
    assert (c.n_ff, c.vocab, c.capacity, c.has_qk_norm) == (96, 50, 16, 1)
    assert c.eps == np.float32(meta["qwen3.attention.layer_norm_rms_epsilon"]) and c.freq_base == 1e6


def test_qwen3_config_errors(L, tmp_path):
    base = {"general.architecture": ("qwen3", STR), "qwen3.embedding_length": (1024, U32),
            "qwen3.attention.head_count": (16, U32), "qwen3.block_count": (28, U32),
            "qwen3.attention.head_count_kv": (8, U32), "qwen3.feed_forward_length": (3072, U32),
            "qwen3.context_length": (40960, U32), "qwen3.attention.layer_norm_rms_epsilon": (1e-6, F32)}

    def build(d):
        b = head(0, len(d))
        for k, (v, tag) in d.items():
            b += kv(k, tag, s(v) if tag == STR else struct.pack({U32: "<I", F32: "<f", F64: "<d", BOOL: "<B"}[tag], v))
        return b

    def cfg(d, name="c.gguf", capacity=8):
        return L.GGUFLoader.from_file(write(tmp_path, build(d), name)).qwen3_config(capacity)

    c = cfg(base)  # no vocab_size, no tokens, no key_length, no freq_base: the reference's defaults
    assert (c.vocab, c.head_dim_k, c.head_dim_v, c.freq_base, c.has_qk_norm) == (0, 64, 64, 1e6, 1)
    toks = dict(base)
    toks["qwen3.attention.key_length"] = (128, U32)
    toks["qwen3.rope.freq_base"] = (10000.0, F64)
    c = cfg(toks)
    assert (c.head_dim_k, c.head_dim_v, c.freq_base) == (128, 64, 10000.0)
    for drop in ("qwen3.embedding_length", "qwen3.block_count", "qwen3.context_length",
                 "qwen3.attention.layer_norm_rms_epsilon"):
        d = {k: v for k, v in base.items() if k != drop}
        with pytest.raises(ValueError, match="Missing metadata: " + drop):
            cfg(d)
    bad = dict(base)
    bad["qwen3.attention.head_count"] = (0, U32)
    with pytest.raises(ValueError, match="Invalid qwen3 head shape: embedding_length=1024, head_count=0"):
        cfg(bad)
    bad["qwen3.attention.head_count"] = (7, U32)
    with pytest.raises(ValueError, match="Invalid qwen3 head shape"):
        cfg(bad)
    bad = dict(base)
    bad["qwen3.attention.key_length"] = (True, BOOL)
    with pytest.raises(ValueError, match="Invalid metadata: qwen3.attention.key_length"):
        cfg(bad)
    bad = dict(base)
    bad["qwen3.attention.value_length"] = (0, U32)
    with pytest.raises(ValueError, match="Invalid qwen3 attention head lengths: key=64, value=0"):
        cfg(bad)
    bad = dict(base)
    bad["general.architecture"] = ("gpt2", STR)
    with pytest.raises(ValueError, match="Unsupported Qwen3-family architecture: gpt2"):
        cfg(bad)
    with pytest.raises(ValueError, match="Missing metadata: general.architecture"):
        cfg({k: v for k, v in base.items() if k != "general.architecture"})


def test_uploads_need_init(rmi, L, tmp_path):
    if rmi.hip.lib.rmi_hip_device_info(None, 0, None, None) == 0:
        pytest.skip("library already initialised on a GPU in this process")
    ok = pad32(head(1, 0) + s("t") + struct.pack("<IQQiQ", 2, 32, 4, 8, 0)) + b"\x07" * 136
    g = L.GGUFLoader.from_file(write(tmp_path, ok))
    with pytest.raises(rmi.hip.RmiHipError, match="rmi_hip_init"):
        g.upload("t")
    with pytest.raises(rmi.hip.RmiHipError, match="Missing tensor: u"):
        g.upload("u")
