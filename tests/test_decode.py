"""End-to-end greedy decode of a synthetic all-Q8_0 Qwen3 GGUF.

The decode loop is the restated Qwen3Session::generate_inner of the checker;
its elementwise ops stay on the CPU ("RMSNorm / RoPE-NeoX / SiLU unchanged").
CPU test: the loop, the GGUF writer/reader and the CPU matmuls on a small model.
GPU tests: the same loop with every quantized matmul routed through the C ABI
(the function pointer of rmi_hip_q8_0_forward_prequantized is handed to the
loop, so no Python sits between the loop and the library), compared step by
step with the CPU-matmul run: logits bit-identical, argmax identical.
"""
import ctypes as C
import os

import numpy as np
import pytest


def _write_model(rmi, tmp_path, **kw):
    path = os.path.join(str(tmp_path), "synthetic-qwen3-q8_0.gguf")
    rmi.gguf.write_synthetic_qwen3(path, seed=4, **kw)
    return rmi.gguf.GGUFFile(path)


def _tensors(f):
    return {name: t[2] for name, t in f.tensors.items()}


def _hip_decoder(oracle, hip, f, pool):
    H, K = hip.hip, hip.kernel
    kernels = []

    def weight_handle(name, data, n_in, n_out):
        k = K.QuantizedTensor.from_bytes(K.GGML_TYPE_Q8_0, data, n_in, n_out).into_kernel()
        kernels.append(k)
        return k.w.handle

    fn = C.cast(H.lib.rmi_hip_q8_0_forward_prequantized, C.c_void_p).value
    dec = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool, matmul_fn=fn, weight_handle=weight_handle)
    dec._kernels = kernels
    return dec


def test_gguf_roundtrip_and_small_decode_cpu(rmi, oracle, tmp_path):
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    kw = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, vocab=1000, n_ctx=4096)
    f = _write_model(rmi, tmp_path, **kw)
    assert f.metadata["general.architecture"] == "qwen3" and f.metadata["qwen3.block_count"] == 2
    dims, ggml_type, data = f.tensors["blk.1.ffn_down.weight"]
    assert dims == (512, 256) and ggml_type == rmi.gguf.GGML_Q8_0 and data.size == 256 * (512 // 32) * 34
    assert np.array_equal(data, rmi.synth.q8_0_weight(4 * 1000 + 14, 256, 512))
    assert "output.weight" not in f.tensors  # tied lm_head
    pool = oracle.Pool(4)
    dec = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool)
    prompt = np.random.default_rng(5).integers(0, 1000, 20, dtype=np.uint32)
    a = dec.generate(prompt, 12, dump_steps=[0, 19, 30])
    b = dec.generate(prompt, 12, dump_steps=[0, 19, 30])
    assert a["tokens"].size == 12 and a["steps"] == 31
    assert np.array_equal(a["tokens"], b["tokens"]) and np.array_equal(a["hashes"], b["hashes"])  # deterministic
    assert np.all(np.isfinite(a["dump"])) and np.array_equal(a["argmax"][[0, 19, 30]], a["dump"].argmax(axis=1))
    assert np.array_equal(a["tokens"], a["argmax"][19:])  # greedy: token i is the argmax of step n_prompt-1+i
    # a longer prompt sharing the prefix must reproduce the prefix steps (causality of the KV cache)
    c = dec.generate(np.concatenate([prompt, prompt[:5]]), 3)
    assert np.array_equal(c["hashes"][:20], a["hashes"][:20])
    pool.close()


@pytest.mark.gpu
def test_small_decode_gpu_matmuls_match_cpu(hip, oracle, tmp_path):
    kw = dict(n_layer=3, n_embd=512, n_head=8, n_head_kv=4, head_dim=64, n_ff=1024, vocab=5000, n_ctx=4096)
    f = _write_model(hip, tmp_path, **kw)
    pool = oracle.Pool(8)
    prompt = np.random.default_rng(6).integers(0, 5000, 40, dtype=np.uint32)
    cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 24, dump_steps=[39, 62])
    gpu = _hip_decoder(oracle, hip, f, pool).generate(prompt, 24, dump_steps=[39, 62])
    assert np.array_equal(cpu["hashes"], gpu["hashes"])  # every step's logits, bit for bit
    assert np.array_equal(cpu["tokens"], gpu["tokens"]) and np.array_equal(cpu["argmax"], gpu["argmax"])
    assert np.array_equal(cpu["dump"].view(np.uint32), gpu["dump"].view(np.uint32))
    pool.close()


@pytest.mark.gpu
def test_full_qwen3_0_6b_decode_512_plus_128(hip, oracle, tmp_path):
    """512 prompt tokens + 128 greedy tokens = 639 forward steps of a random-init
    Qwen3-0.6B-architecture Q8_0 GGUF; logits of every step compared with the CPU run."""
    f = _write_model(hip, tmp_path)  # 28 layers, 1024 wide, vocab 151936
    pool = oracle.Pool(16)
    prompt = np.random.default_rng(7).integers(0, 151936, 512, dtype=np.uint32)
    gpu_dec = _hip_decoder(oracle, hip, f, pool)
    gpu = gpu_dec.generate(prompt, 128, dump_steps=[511, 638])
    cpu = oracle.Qwen3Decoder(f.metadata, _tensors(f), pool).generate(prompt, 128, dump_steps=[511, 638])
    assert gpu["steps"] == 639 and gpu["tokens"].size == 128
    same = cpu["hashes"] == gpu["hashes"]
    margin = (cpu["top2"][:, 0] - cpu["top2"][:, 1]).min()
    print(f"\n639 steps: logits bit-identical in {int(same.sum())}/639 steps; smallest top-1 margin {margin:.3e}; "
          f"CPU {cpu['seconds']:.1f}s ({cpu['seconds_matmul']:.1f}s in matmuls, {pool.n_threads} threads), "
          f"GPU-matmul run {gpu['seconds']:.1f}s ({gpu['seconds_matmul']:.1f}s in matmul calls incl. PCIe); "
          f"decode {128 / (gpu['seconds'] * 128 / 639):.1f} tok/s vs CPU {128 / (cpu['seconds'] * 128 / 639):.1f} tok/s")
    assert same.all()
    assert np.array_equal(cpu["argmax"], gpu["argmax"]) and np.array_equal(cpu["tokens"], gpu["tokens"])
    assert np.array_equal(cpu["dump"].view(np.uint32), gpu["dump"].view(np.uint32))
    pool.close()
