"""Host-side mirror of the reference's ``Qwen3Session`` (src/models/qwen3.rs:581-1158) over the
device-resident decode entry points of the C ABI: weights go to HBM once, then whole generations
run on the GPU with one synchronisation at the end.
"""
import ctypes as C

import numpy as np

from . import hip

_MATMULS = (("wq", "attn_q"), ("wk", "attn_k"), ("wv", "attn_v"), ("wo", "attn_output"), ("w_gate", "ffn_gate"),
            ("w_up", "ffn_up"), ("w_down", "ffn_down"))
_NORMS = (("attn_norm", "attn_norm"), ("ffn_norm", "ffn_norm"), ("q_norm", "attn_q_norm"), ("k_norm", "attn_k_norm"))


class Qwen3Session:
    """`metadata` and `tensors` as a GGUF file gives them (keys of src/core/loader.rs:379-461, tensor
    names of src/models/qwen3.rs:269-349); every 2-D weight must be Q8_0 bytes, norms f32."""

    def __init__(self, metadata, tensors, capacity, rounding=hip.ROUND_TIES_EVEN):
        g = lambda k: int(metadata[f"qwen3.{k}"])  # noqa: E731
        c = hip.Qwen3Config()
        c.n_embd, c.n_layer, c.n_head, c.n_head_kv = (g("embedding_length"), g("block_count"),
                                                      g("attention.head_count"), g("attention.head_count_kv"))
        c.head_dim_k = int(metadata.get("qwen3.attention.key_length", c.n_embd // c.n_head))
        c.head_dim_v = int(metadata.get("qwen3.attention.value_length", c.n_embd // c.n_head))
        c.n_ff, c.vocab, c.capacity = g("feed_forward_length"), int(metadata["qwen3.vocab_size"]), int(capacity)
        c.eps = float(metadata["qwen3.attention.layer_norm_rms_epsilon"])
        c.freq_base = float(metadata.get("qwen3.rope.freq_base", 1e6))
        c.has_qk_norm = 1 if "blk.0.attn_q_norm.weight" in tensors else 0
        c.rounding = rounding
        keep = []

        def raw(name):
            a = hip.as_u8(tensors[name])
            keep.append(a)
            return hip.ptr(a, hip._u8p)

        def f32(name):
            a = np.ascontiguousarray(np.asarray(tensors[name]).view(np.float32))
            keep.append(a)
            return hip.ptr(a, hip._f32p)

        w = hip.Qwen3Weights()
        w.token_embd = raw("token_embd.weight")
        w.output = raw("output.weight") if "output.weight" in tensors else None
        w.output_norm = f32("output_norm.weight")
        for field, name in _NORMS:
            if not c.has_qk_norm and field in ("q_norm", "k_norm"):
                continue
            arr = (hip._f32p * c.n_layer)(*[f32(f"blk.{layer}.{name}.weight") for layer in range(c.n_layer)])
            keep.append(arr)
            setattr(w, field, arr)
        for field, name in _MATMULS:
            arr = (hip._u8p * c.n_layer)(*[raw(f"blk.{layer}.{name}.weight") for layer in range(c.n_layer)])
            keep.append(arr)
            setattr(w, field, arr)
        self.config = c
        self._h = hip.lib.rmi_hip_qwen3_create(C.byref(c), C.byref(w))
        if not self._h:
            raise hip.RmiHipError(-1, hip.last_error())

    @classmethod
    def from_gguf(cls, loader, capacity, rounding=hip.ROUND_TIES_EVEN):
        """Qwen3Model::from_source + Qwen3Session::new over an open ``loader.GGUFLoader``: tensor bytes go from
        the file's mapping to HBM inside the library (src/models/qwen3.rs:262-349)."""
        self = cls.__new__(cls)
        self._h = None
        self.config = loader.qwen3_config(capacity, rounding)
        self._h = hip.lib.rmi_hip_qwen3_create_from_gguf(loader._h, int(capacity), rounding)
        if not self._h:
            raise hip.RmiHipError(-1, hip.last_error())
        return self

    def set_stop_ids(self, ids):
        """The tokenizer's EOS / `im_end` ids (src/models/qwen3.rs:1123-1130): generation ends before the first."""
        ids = np.ascontiguousarray(ids, np.uint32)
        hip.check(hip.lib.rmi_hip_qwen3_set_stop_ids(self._h, hip.ptr(ids, hip._u32p), ids.size))

    def set_prompt_passes(self, enabled):
        """Prompt positions 128 to a pass (True, the default), every position its own step (False), or that many to a
        pass (an int above 1, at most 128); same results either way."""
        hip.check(hip.lib.rmi_hip_qwen3_set_prompt_passes(self._h, int(enabled)))

    def generate(self, prompt, max_new, dump_steps=()):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        steps = prompt.size + max_new - 1
        gen = np.zeros(max(max_new, 1), np.uint32)
        argmax = np.zeros(steps, np.uint32)
        top2 = np.zeros((steps, 2), np.float32)
        dump_steps = np.ascontiguousarray(dump_steps, np.uint32)
        dump = np.zeros((max(dump_steps.size, 1), self.config.vocab), np.float32)
        seconds = C.c_double()
        n = hip.lib.rmi_hip_qwen3_generate(self._h, hip.ptr(prompt, hip._u32p), prompt.size, max_new,
                                           hip.ptr(gen, hip._u32p), hip.ptr(argmax, hip._u32p), hip.ptr(top2, hip._f32p),
                                           hip.ptr(dump_steps, hip._u32p), dump_steps.size, hip.ptr(dump, hip._f32p),
                                           C.byref(seconds))
        if n < 0:
            raise hip.RmiHipError(n, hip.last_error())
        return dict(tokens=gen[:n], argmax=argmax, top2=top2, dump=dump[:dump_steps.size], seconds=seconds.value,
                    steps=steps)

    def close(self):
        if self._h:
            hip.lib.rmi_hip_qwen3_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()
