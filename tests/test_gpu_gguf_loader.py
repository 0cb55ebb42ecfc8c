"""GGUF file -> HBM: what the uploads from the file's mapping leave in device memory is byte for byte what the
host-slice uploads leave, for all four block formats, for stacked tensors and for weights of several staging
chunks; the session built from the file generates what the session built from host slices generates."""
import os
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _device_bytes(H, handle):
    n = H.lib.rmi_hip_weight_device_bytes(handle)
    out = np.empty(n, np.uint8)
    H.check(H.lib.rmi_hip_memcpy_d2h(H.ptr(out, H._u8p), H.lib.rmi_hip_weight_device_data(handle), n))
    return out


def _host_upload(H, ggml_type, data, n_in, n_out):
    fn = {2: H.lib.rmi_hip_upload_q4_0, 8: H.lib.rmi_hip_upload_q8_0, 12: H.lib.rmi_hip_upload_q4_k,
          14: H.lib.rmi_hip_upload_q6_k}[ggml_type]
    a = H.as_u8(data)
    h = fn(H.ptr(a, H._u8p), a.size, n_in, n_out)
    assert h, H.last_error()
    return h


def _weights(rmi):
    S, G = rmi.synth, rmi.gguf
    return [
        ("q8.a", G.GGML_Q8_0, 1024, 2048, S.q8_0_weight(1, 2048, 1024)),
        ("q8.b", G.GGML_Q8_0, 1024, 1024, S.q8_0_weight(2, 1024, 1024)),
        ("q8.c", G.GGML_Q8_0, 1024, 1021, S.q8_0_weight(3, 1021, 1024)),   # ends inside a tile
        ("q8.ragged", G.GGML_Q8_0, 1024, 13, S.q8_0_weight(4, 13, 1024)),  # 13 rows: the next part starts inside a tile
        ("q8.odd", G.GGML_Q8_0, 96, 50, S.q8_0_weight(5, 50, 96)),         # 3 blocks a row: a partly filled octet
        ("q8.big", G.GGML_Q8_0, 1024, 40000, S.q8_0_weight(6, 40000, 1024)),  # 43.5 MB: three staging chunks
        ("q40.a", G.GGML_Q4_0, 1024, 520, S.q4_0_weight(7, 520, 1024)),
        ("q40.b", G.GGML_Q4_0, 1024, 77, S.q4_0_weight(8, 77, 1024)),
        ("q4k.a", G.GGML_Q4_K, 1024, 256, S.q4_k_weight(9, 256, 1024)),
        ("q4k.b", G.GGML_Q4_K, 1024, 99, S.q4_k_weight(10, 99, 1024)),
        ("q6k.a", G.GGML_Q6_K, 2048, 136, S.q6_k_weight(11, 136, 2048)),
        ("q6k.b", G.GGML_Q6_K, 2048, 35, S.q6_k_weight(12, 35, 2048)),
        ("norm", G.GGML_F32, 64, None, np.arange(64, dtype=np.float32)),
    ]


@pytest.fixture(scope="module")
def model_file(hip, tmp_path_factory):
    path = os.path.join(str(tmp_path_factory.mktemp("gguf")), "weights.gguf")
    ws = _weights(hip)
    hip.gguf.write_gguf(path, {"general.architecture": "qwen3"},
                        [(n, (n_in,) if n_out is None else (n_in, n_out), ty, d) for n, ty, n_in, n_out, d in ws])
    return path, ws


def test_upload_from_file_equals_upload_from_host(hip, model_file):
    H = hip.hip
    path, ws = model_file
    with hip.loader.GGUFLoader.from_file(path) as g:
        for name, ty, n_in, n_out, data in ws:
            if n_out is None:
                continue
            a, b = g.upload(name), _host_upload(H, ty, data, n_in, n_out)
            assert (H.lib.rmi_hip_weight_n_in(a), H.lib.rmi_hip_weight_n_out(a)) == (n_in, n_out)
            assert H.lib.rmi_hip_weight_dtype(a) == ty
            assert np.array_equal(_device_bytes(H, a), _device_bytes(H, b)), name
            H.lib.rmi_hip_free_weight(a)
            H.lib.rmi_hip_free_weight(b)


def test_chunked_upload_is_the_repack_of_the_whole(hip, model_file):
    """A weight of several staging chunks against a host restatement of the Q8_0 tile stream that knows nothing
    of chunks: per 8-row tile the f16 scales [octet][row][block], then per quad of blocks q the quants as 4-byte
    pieces [row][piece][block of the quad]; rows and blocks past the end are zero."""
    H = hip.hip
    path, ws = model_file
    name, ty, n_in, n_out, data = next(w for w in ws if w[0] == "q8.big")
    with hip.loader.GGUFLoader.from_file(path) as g:
        h = g.upload(name)
    got = _device_bytes(H, h)
    H.lib.rmi_hip_free_weight(h)
    nb, n_tiles = n_in // 32, (n_out + 7) // 8
    n_oct = (nb + 7) // 8
    blocks = np.zeros((n_tiles * 8, n_oct * 8, 34), np.uint8)
    blocks[:n_out, :nb] = np.asarray(data).reshape(n_out, nb, 34)
    blocks = blocks.reshape(n_tiles, 8, n_oct * 8, 34)
    scales = blocks[..., :2].reshape(n_tiles, 8, n_oct, 8, 2).transpose(0, 2, 1, 3, 4).reshape(n_tiles, -1)
    quants = blocks[..., 2:].reshape(n_tiles, 8, n_oct * 2, 4, 8, 4).transpose(0, 2, 1, 4, 3, 5).reshape(n_tiles, -1)
    want = np.concatenate([scales, quants], axis=1).reshape(-1)
    assert got.size == want.size == n_tiles * n_oct * 2176
    assert np.array_equal(got, want)


def test_big_weight_gemv_after_chunked_upload(hip, oracle, model_file):
    path, ws = model_file
    name, ty, n_in, n_out, data = next(w for w in ws if w[0] == "q8.big")
    with hip.loader.GGUFLoader.from_file(path) as g:
        k = g.kernel(name)
    x = hip.synth.activations(21, 1, n_in).reshape(-1)
    q8, sc = oracle.quantize_q8_0(x)
    out = np.zeros(n_out, np.float32)
    k.forward_prequantized(q8, sc, out, n_in, n_out, 0, 1)
    ref = oracle.matmul_q8_0_quantized(np.asarray(data), q8, sc, n_in, n_out)
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("names", [("q8.a", "q8.b", "q8.b"), ("q8.a", "q8.c"), ("q8.ragged", "q8.b"),
                                   ("q8.c", "q8.ragged", "q8.a"), ("q40.a", "q40.b"), ("q40.b", "q40.a"),
                                   ("q4k.a", "q4k.b"), ("q4k.b", "q4k.a"), ("q6k.a", "q6k.b"), ("q6k.b", "q6k.a")])
def test_stacked_upload_equals_fuse_vstack(hip, model_file, names):
    H = hip.hip
    path, ws = model_file
    by_name = {w[0]: w for w in ws}
    with hip.loader.GGUFLoader.from_file(path) as g:
        stacked = g.upload(*names)
    acc = None
    for n in names:
        _, ty, n_in, n_out, data = by_name[n]
        w = _host_upload(H, ty, data, n_in, n_out)
        if acc is None:
            acc = w
        else:
            f = H.lib.rmi_hip_fuse_vstack(acc, w)
            assert f, H.last_error()
            H.lib.rmi_hip_free_weight(acc)
            H.lib.rmi_hip_free_weight(w)
            acc = f
    assert H.lib.rmi_hip_weight_n_out(stacked) == sum(by_name[n][3] for n in names)
    assert np.array_equal(_device_bytes(H, stacked), _device_bytes(H, acc)), names
    H.lib.rmi_hip_free_weight(stacked)
    H.lib.rmi_hip_free_weight(acc)


def test_upload_errors(hip, model_file):
    H = hip.hip
    path, _ = model_file
    with hip.loader.GGUFLoader.from_file(path) as g:
        with pytest.raises(H.RmiHipError, match="Missing tensor: nope"):
            g.upload("nope")
        with pytest.raises(H.RmiHipError, match="Invalid tensor norm"):
            g.upload("norm")
        with pytest.raises(H.RmiHipError, match="does not stack"):
            g.upload("q8.a", "q40.a")
        with pytest.raises(H.RmiHipError, match="does not stack"):
            g.upload("q8.a", "q8.odd")


def test_quantized_linear_from_source(hip, oracle, model_file):
    """QuantizedLinear::from_source (src/core/model.rs:38-55) over the loader, as the reference's
    model_config_and_linear_accept_a_tensor_source builds it (src/core/loader.rs:904-920)."""
    path, ws = model_file
    _, ty, n_in, n_out, data = next(w for w in ws if w[0] == "q4k.a")
    K = hip.kernel
    with hip.loader.GGUFLoader.from_file(path) as g:
        assert K.QuantizedLinear.from_source(g, "absent", None, n_in, n_out, "x") is None
        layer = K.QuantizedLinear.from_source(g, "q4k.a", None, n_in, n_out, "attn_q")
    direct = K.QuantizedLinear.from_weight_slice(data, None, n_in, n_out, "attn_q")
    x = hip.synth.activations(3, 1, n_in).reshape(-1)
    a, b = np.zeros(n_out, np.float32), np.zeros(n_out, np.float32)
    layer.forward(x, a, None)
    direct.forward(x, b, None)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)) and np.any(a != 0)
    assert (layer.input_dim(), layer.output_dim(), layer.name()) == (n_in, n_out, "attn_q")


def test_session_from_file_equals_session_from_host_slices(hip, tmp_path):
    path = os.path.join(str(tmp_path), "synthetic-qwen3-q8_0.gguf")
    kw = dict(n_layer=3, n_embd=512, n_head=8, n_head_kv=4, head_dim=64, n_ff=1024, vocab=5000, n_ctx=4096)
    hip.gguf.write_synthetic_qwen3(path, seed=4, **kw)
    f = hip.gguf.GGUFFile(path)
    prompt = np.random.default_rng(6).integers(0, 5000, 20, dtype=np.uint32)
    steps = list(range(31))
    host = hip.decode.Qwen3Session(f.metadata, {n: t[2] for n, t in f.tensors.items()}, capacity=32)
    want = host.generate(prompt, 12, dump_steps=steps)
    host.close()
    with hip.loader.GGUFLoader.from_file(path) as g:
        sess = hip.decode.Qwen3Session.from_gguf(g, capacity=32)
        with pytest.raises(ValueError, match="Session capacity 5000 exceeds model context 4096"):
            hip.decode.Qwen3Session.from_gguf(g, capacity=5000)
    got = sess.generate(prompt, 12, dump_steps=steps)  # the file is closed: the session owns its HBM copies
    sess.close()
    assert np.array_equal(want["tokens"], got["tokens"]) and np.array_equal(want["argmax"], got["argmax"])
    assert np.array_equal(want["dump"].view(np.uint32), got["dump"].view(np.uint32))


def test_session_from_file_rejects_what_the_reference_rejects(hip, tmp_path):
    G = hip.gguf
    kw = dict(n_layer=1, n_embd=64, n_head=2, n_head_kv=1, head_dim=32, n_ff=96, vocab=40, n_ctx=64)
    path = os.path.join(str(tmp_path), "m.gguf")
    G.write_synthetic_qwen3(path, seed=1, **kw)
    f = G.GGUFFile(path)
    meta = {k: v for k, v in f.metadata.items()}

    def rewrite(name, drop=None, retype=None, reshape=None):
        out = []
        for n, (dims, ty, view) in f.tensors.items():
            if n == drop:
                continue
            if n == retype:
                ty, view, dims = G.GGML_Q4_0, np.zeros(G.tensor_nbytes(dims, G.GGML_Q4_0), np.uint8), dims
            if n == reshape:
                dims = (dims[1], dims[0])
            out.append((n, dims, ty, view))
        p = os.path.join(str(tmp_path), name)
        G.write_gguf(p, meta, out)
        return p

    H = hip.hip
    cases = [(rewrite("a.gguf", drop="blk.0.ffn_up.weight"), "Missing tensor: blk.0.ffn_up.weight"),
             (rewrite("b.gguf", retype="blk.0.attn_k.weight"),
              r"Invalid tensor blk.0.attn_k.weight: shape \[64, 32\] type Q4_0; expected \[64, 32\] Q8_0"),
             (rewrite("c.gguf", reshape="blk.0.ffn_down.weight"),
              r"Invalid tensor blk.0.ffn_down.weight: shape \[64, 96\] type Q8_0; expected \[96, 64\] Q8_0"),
             (rewrite("d.gguf", drop="blk.0.attn_q_norm.weight"), "Missing tensor: blk.0.attn_q_norm.weight")]
    for p, msg in cases:
        with hip.loader.GGUFLoader.from_file(p) as g:
            with pytest.raises(H.RmiHipError, match=msg):
                hip.decode.Qwen3Session.from_gguf(g, capacity=8)


def test_full_size_file_to_hbm_rate(hip, tmp_path):
    """The whole Qwen3-0.6B-shaped file (0.64 GB of Q8_0) from the page cache to repacked HBM; prints the rate."""
    H = hip.hip
    path = os.path.join(str(tmp_path), "qwen3-0.6b-q8_0.gguf")
    hip.gguf.write_synthetic_qwen3(path, seed=2)
    size = os.path.getsize(path)
    with hip.loader.GGUFLoader.from_file(path) as g:
        t0 = time.perf_counter()
        sess = hip.decode.Qwen3Session.from_gguf(g, capacity=64)
        dt = time.perf_counter() - t0
        t0 = time.perf_counter()
        w = g.upload("token_embd.weight")
        dt_embd = time.perf_counter() - t0
        embd_bytes = g.tensor_info("token_embd.weight").nbytes()
    print(f"\nfile -> HBM: {size / 1e9:.2f} GB in {dt:.2f} s = {size / dt / 1e9:.2f} GB/s (session, 311 tensors); "
          f"token_embd alone {embd_bytes / dt_embd / 1e9:.2f} GB/s")
    out = sess.generate(np.arange(4, dtype=np.uint32), 4)
    assert out["tokens"].size == 4
    H.lib.rmi_hip_free_weight(w)
    sess.close()
