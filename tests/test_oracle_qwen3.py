"""Pins of the checker's decode-step pieces (oracle/rmi_qwen3.c): the functions the GPU decode kernels are
compared against.

Where the reference holds an architecture-independent bit vector it is used as is (rms_norm, rms_norm_inplace,
rope_neox, silu_mul_inplace's scalar loop, greedy_token).  Where it holds none for the x86-64 branch (softmax,
dot_f16, the attention block, embedding_lookup_q8_0) the pin is an independent numpy statement in which every
f32 / f16 rounding point is spelled out, on inputs small enough that each can be enumerated, together with a
check that the plausible wrong statements (an f64 sum, a reciprocal multiply, an f32 dot accumulator, the other
head mapping, swapped operands) give different bits on the same inputs -- so the test set can tell them apart.
"""
import math

import numpy as np
import pytest

from conftest import bits

f32 = np.float32


def _f(bits_):
    return np.array(bits_, np.uint32).view(np.float32)


# ------------------------------------------------------------------ rms_norm

def test_rms_norm_accumulates_f32_squares_in_f64(oracle):
    """src/ops/matmul_tests.rs:127-141."""
    out = oracle.rms_norm(_f([0x3F800000, 0x39800000, 0x39800000]), np.ones(3, np.float32), 0.0)
    assert list(bits(out)) == [0x3FDDB3D6, 0x39DDB3D6, 0x39DDB3D6]


def test_rms_norm_inplace_matches_ggml_sequential_f64_accumulation(oracle):
    """src/ops/matmul_tests.rs:143-181: the q/k head norm (rms_norm_inplace -> scale_mul_avx2, src/ops/norm.rs:13-84,
    (x * scale) * weight) is the same arithmetic as rms_norm."""
    values = _f([0x3E57D77B, 0xBD828687, 0xBE102E16, 0x3D2F9FEA, 0x3DF48D0B, 0x3DED164C, 0x3BCC65AD, 0xBE18B60F])
    weight = _f([0x40910000, 0x3F9F0000, 0xBF3C0000, 0x3FDA0000, 0x40260000, 0x3FC70000, 0x3F8C0000, 0x3FBB0000])
    out = oracle.rms_norm(values, weight, float(_f([0x358637BD])[0]))
    assert list(bits(out)) == [0x40F971A9, 0xBF2568FE, 0x3F580A09, 0x3F18930B, 0x4021C6F1, 0x3FBC04BD, 0x3D641282,
                               0xBFE39AEA]


# ---------------------------------------------------------------------- rope

def test_rope_neox_matches_pinned_ggml_recurrence_and_fused_rotation(oracle):
    """src/ops/matmul_tests.rs:183-198 (position 1, head dimension 128, base 1e6)."""
    values = np.zeros(128, np.float32)
    values[[0, 1, 64, 65]] = _f([0x402A4F21, 0x3FADB711, 0xBE0E7273, 0x3EF5B8F9])
    out = oracle.rope_neox(values, 1, 1000000.0)
    assert list(bits(out[[0, 1, 64, 65]])) == [0x3FC70519, 0x3F17F682, 0x400A7FF8, 0x3FA7DC8A]
    assert not out[2:64].any() and not out[66:].any()


@pytest.mark.parametrize("pos", [0, 1, 7, 511, 12000])
def test_rope_angle_table_is_what_rope_neox_rotates_by(oracle, pos):
    """The device kernels take the host's cos/sin rows (rope_angles): rotating the unit vectors e_i gives
    (cos_i, sin_i) exactly (fma(1, c, 0 * -s) = c), and e_{i+half} gives (-sin_i, cos_i)."""
    c, s = oracle.rope_angles(pos, 128, 1000000.0)
    for i in (0, 1, 5, 63):
        e = np.zeros(128, np.float32)
        e[i] = 1.0
        out = oracle.rope_neox(e, pos, 1000000.0)
        assert bits(out[i]) == bits(c[i]) and bits(out[i + 64]) == bits(s[i])
        e = np.zeros(128, np.float32)
        e[i + 64] = 1.0
        out = oracle.rope_neox(e, pos, 1000000.0)
        assert out[i] == -s[i] and out[i + 64] == c[i]
    if pos == 0:
        assert (c == 1).all() and (s == 0).all()


# ---------------------------------------------------------------------- silu

def test_silu_mul_scalar_order_pin(oracle):
    """tests/quantized_inference.rs:21-29: up[i] *= gate[i] / (1 + exp(-gate[i])), the scalar loop every x86-64
    build runs (src/ops/activation/mod.rs:137-151)."""
    gate = np.array([0.0, 0.0, 0.0, _f([0xBF44C6B5])[0]], np.float32)
    up = np.array([0.0, 0.0, 0.0, _f([0x3DDF57E5])[0]], np.float32)
    out = oracle.silu_mul(gate, up)
    assert bits(out[3]) == 0xBCD98667 and not out[:3].any()


def test_silu_mul_operand_order_against_the_neon_fixture(oracle):
    """src/ops/matmul_tests.rs:361-372 (aarch64 fixture, vector exp): the scalar loop agrees within 2 ulp, and
    with the operands swapped it is nowhere near -- `up` is scaled by silu(`gate`), not the reverse."""
    gate = _f([0xBF46E0D2, 0xBF47EBEA, 0xBEEE8B6B, 0xBE1B692B])
    up = _f([0xBDBDAB3D, 0xBDF016EB, 0x3E08064C, 0xBF87C095])
    want = np.array([0x3CB9A7C4, 0x3CEB9536, 0xBCC37DCB, 0x3D9856F8], np.uint32)
    got = bits(oracle.silu_mul(gate, up)).astype(np.int64)
    assert np.abs(got - want.astype(np.int64)).max() <= 2
    swapped = bits(oracle.silu_mul(up, gate)).astype(np.int64)
    assert np.abs(swapped - want.astype(np.int64)).min() > 1000


def test_silu_mul_against_f64(oracle):
    rng = np.random.default_rng(11)
    gate, up = rng.standard_normal(4096).astype(np.float32) * 4, rng.standard_normal(4096).astype(np.float32)
    out = oracle.silu_mul(gate, up)
    g = gate.astype(np.float64)
    ref = up.astype(np.float64) * g / (1.0 + np.exp(-g))
    assert np.abs(out - ref).max() <= 4e-7 * np.abs(ref).max() + 1e-12


# ------------------------------------------------------------------- softmax

def _exp_f32(v):
    """exp of an f32 argument correctly rounded to f32, with a guard: the f64 value is far enough from an f32
    rounding boundary that any libm expf with < 0.51 ulp error returns the same bits."""
    v = float(f32(v))
    if v == -math.inf:
        return f32(0.0)
    e = math.exp(v)
    r = f32(e)
    for nb in (np.nextafter(r, f32(np.inf)), np.nextafter(r, f32(-np.inf))):
        mid = (float(r) + float(nb)) / 2
        assert abs(e - mid) > 2.0 ** -12 * abs(float(r) - float(nb)), "input sits on an f32 rounding boundary"
    return r


def _softmax_statement(x, sum_in_f64=False, reciprocal=False):
    """src/ops/attention.rs:28-38: max, e = exp(x - max) in f32, an f32 running sum in index order, one f32
    division per element."""
    x = np.asarray(x, np.float32)
    mx = f32(-np.inf)
    for v in x:
        mx = max(mx, v)
    e = np.array([_exp_f32(f32(v - mx)) for v in x], np.float32)
    if sum_in_f64:
        s = f32(sum(float(v) for v in e))
    else:
        s = f32(0.0)
        for v in e:
            s = f32(s + v)
    if not s > 0:
        return e
    if reciprocal:
        r = f32(f32(1.0) / s)
        return np.array([f32(v * r) for v in e], np.float32)
    return np.array([f32(v / s) for v in e], np.float32)


def _softmax_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for n_keys in (1, 2, 3, 3, 3, 5, 17, 40):
        for _ in range(6):
            x = np.full(256 if n_keys < 40 else 64, -np.inf, np.float32)  # the attention block pads with -inf
            x[:n_keys] = (rng.standard_normal(n_keys) * 3).astype(np.float32)
            cases.append(x)
    cases.append(np.array([0.25], np.float32))
    cases.append(np.array([-1.0, 0.0, 1.0, -np.inf], np.float32))
    return cases


def test_softmax_every_rounding_point(oracle):
    wrong_f64 = wrong_recip = 0
    for x in _softmax_cases():
        want = _softmax_statement(x)
        got = oracle.softmax(x)
        assert np.array_equal(bits(got), bits(want)), x[:8]
        wrong_f64 += not np.array_equal(bits(_softmax_statement(x, sum_in_f64=True)), bits(want))
        wrong_recip += not np.array_equal(bits(_softmax_statement(x, reciprocal=True)), bits(want))
    # the case set tells the reference's other two formulations (f64 sum; multiply by 1/sum) apart from this one
    assert wrong_f64 >= 1 and wrong_recip >= 3
    assert list(oracle.softmax(np.array([5.0], np.float32))) == [1.0]


def test_softmax_of_all_minus_infinity_stays_nan(oracle):
    """max = -inf, x - max = NaN, sum = NaN, `sum > 0` is false: nothing is divided (attention.rs:28-38)."""
    assert np.isnan(oracle.softmax(np.full(4, -np.inf, np.float32))).all()


# ------------------------------------------------------------------- dot_f16

def _dot_f16_statement(a16, b16, f32_accumulator=False):
    """src/ops/dot.rs:99-119: f32 products (exact: 11 x 11 significant bits) summed in f64, rounded to f32 once.
    math.fsum is the exact sum; the sizes and magnitudes here keep the sequential f64 sum exact too."""
    a, b = a16.view(np.float16).astype(np.float64), b16.view(np.float16).astype(np.float64)
    if f32_accumulator:
        s = f32(0.0)
        for p in (a * b):
            s = f32(s + f32(p))
        return s
    return f32(math.fsum(a * b))


def test_dot_f16_products_in_f32_sum_in_f64(oracle):
    rng = np.random.default_rng(7)
    differs = 0
    for n in (1, 2, 3, 4, 31, 128, 256, 1000):
        for _ in range(4):
            a = rng.standard_normal(n).astype(np.float16).view(np.uint16)
            b = rng.standard_normal(n).astype(np.float16).view(np.uint16)
            want = _dot_f16_statement(a, b)
            assert bits(oracle.dot_f16(a, b)) == bits(want), n
            differs += bits(_dot_f16_statement(a, b, f32_accumulator=True)) != bits(want)
    assert differs >= 5  # an f32 accumulator would have been caught
    one = np.array([1.0], np.float16).view(np.uint16)
    assert oracle.dot_f16(np.repeat(one, 256), np.repeat(one, 256)) == 256.0
    # subnormal and signed-zero halves go through the same conversion
    a = np.array([0x0001, 0x8000, 0x7BFF], np.uint16)
    b = np.array([0x3C00, 0x3C00, 0x0001], np.uint16)
    assert bits(oracle.dot_f16(a, b)) == bits(_dot_f16_statement(a, b))


# ----------------------------------------------------------------- attention

def _attention_statement(q, k_cache, v_cache, step, kv_stride, n_head, n_head_kv, hk, hv, head_map="div",
                         round_weights=True, round_query=True):
    """src/models/qwen3.rs:876-933 with every rounding point: q to f16; score = f32(exact q.k) * f32(1/sqrt(hk));
    the row padded to a multiple of 256 with -inf; softmax; weights to f16; out = f32(exact sum of v16 * w16)."""
    group = n_head // n_head_kv
    kq_scale = f32(f32(1.0) / np.sqrt(f32(hk)))
    n_padded = (step + 1 + 255) // 256 * 256
    k16 = k_cache.reshape(-1, kv_stride)
    v16 = v_cache.reshape(-1, kv_stride)
    out = np.zeros(n_head * hv, np.float32)
    for head in range(n_head):
        kv = head // group if head_map == "div" else head % n_head_kv
        qh = q[head * hk:(head + 1) * hk]
        qd = qh.astype(np.float16).astype(np.float64) if round_query else qh.astype(np.float64)
        scores = np.full(n_padded, -np.inf, np.float32)
        for t in range(step + 1):
            key = k16[t, kv * hk:(kv + 1) * hk].view(np.float16).astype(np.float64)
            scores[t] = f32(f32(math.fsum(qd * key)) * kq_scale)
        p = _softmax_statement(scores)
        w = p.astype(np.float16).astype(np.float64) if round_weights else p.astype(np.float64)
        for d in range(hv):
            vals = v16[:step + 1, kv * hv + d].view(np.float16).astype(np.float64)
            out[head * hv + d] = f32(math.fsum(vals * w[:step + 1]))
    return out


@pytest.mark.parametrize("shape", [(4, 2, 4, 2), (2, 2, 2, 4), (6, 2, 4, 4)])
def test_attention_block_every_rounding_point(oracle, shape):
    n_head, n_head_kv, hk, hv = shape
    kv_stride = max(n_head_kv * hk, n_head_kv * hv)
    rng = np.random.default_rng(sum(shape))
    other_map = no_w16 = no_q16 = 0
    for step in (0, 1, 2, 2, 2, 9):
        q = (rng.standard_normal(n_head * hk) * 2).astype(np.float32)
        k = rng.standard_normal((step + 1, kv_stride)).astype(np.float16).view(np.uint16)
        v = rng.standard_normal((step + 1, kv_stride)).astype(np.float16).view(np.uint16)
        args = (q, k, v, step, kv_stride, n_head, n_head_kv, hk, hv)
        want = _attention_statement(*args)
        got = oracle.attention_f16(q, k, v, step, kv_stride, n_head, n_head_kv, hk, hv)
        assert np.array_equal(bits(got), bits(want)), (shape, step)
        other_map += not np.array_equal(bits(_attention_statement(*args, head_map="mod")), bits(want))
        no_w16 += not np.array_equal(bits(_attention_statement(*args, round_weights=False)), bits(want))
        no_q16 += not np.array_equal(bits(_attention_statement(*args, round_query=False)), bits(want))
    # each of these mistakes would have been caught by the cases above
    assert no_w16 >= 3 and no_q16 >= 3
    if n_head // n_head_kv > 1 and n_head_kv > 1:
        assert other_map >= 3


def test_attention_single_key_returns_the_value_row(oracle):
    """One key: softmax = [1.0], weight f16(1) = 1, so the output is the f16 value row itself."""
    n_head, n_head_kv, hk, hv = 4, 2, 8, 8
    rng = np.random.default_rng(3)
    q = rng.standard_normal(n_head * hk).astype(np.float32)
    k = rng.standard_normal((1, 16)).astype(np.float16)
    v = rng.standard_normal((1, 16)).astype(np.float16)
    out = oracle.attention_f16(q, k.view(np.uint16), v.view(np.uint16), 0, 16, n_head, n_head_kv, hk, hv)
    want = np.concatenate([v[0, (h // 2) * hv:(h // 2 + 1) * hv] for h in range(n_head)]).astype(np.float32)
    assert np.array_equal(bits(out), bits(want))


# ----------------------------------------------------------------- embedding

def test_embedding_lookup_is_the_q8_0_dequant_of_the_row(oracle, rmi):
    """src/ops/embedding.rs:12-22: out[32 b + j] = f32(d_b) * f32(q_bj), row = token_id * (n_embd / 32) * 34."""
    n_embd, vocab = 96, 5
    table = rmi.synth.q8_0_weight(21, vocab, n_embd)
    blocks = table.reshape(vocab, n_embd // 32, 34)
    for token in (0, 3, 4):
        d = blocks[token, :, 0:2].copy().view(np.float16).astype(np.float32)  # [nb, 1]
        q = blocks[token, :, 2:].view(np.int8).astype(np.float32)
        want = (d * q).reshape(-1)
        got = oracle.embedding_lookup_q8_0(table, token, n_embd)
        assert np.array_equal(bits(got), bits(want))
    assert not np.array_equal(oracle.embedding_lookup_q8_0(table, 3, n_embd), oracle.embedding_lookup_q8_0(table, 4, n_embd))


# -------------------------------------------------------------------- greedy

def test_greedy_ties_choose_the_lowest_token_id(oracle):
    """src/models/qwen3.rs:1519-1522, and the error cases of :172-191."""
    assert oracle.greedy_token([1.0, 2.0, 2.0]) == 1
    assert oracle.greedy_token([1.0, np.nan]) is None
    assert oracle.greedy_token([np.inf, 1.0]) is None
    assert oracle.greedy_token([1.0, -np.inf]) is None
    assert oracle.greedy_token([]) is None
    assert oracle.greedy_token([-3.0]) == 0
    assert oracle.greedy_token([-3.0, -2.0, -2.5, -2.0]) == 1
    assert oracle.greedy_token([0.0, -0.0]) == 0  # -0.0 > 0.0 is false


# ------------------------------------------------- the loop that wires them

def _step_by_step(oracle, meta, t, prompt, n_steps):
    """Qwen3Session::generate_inner (src/models/qwen3.rs:581-1158) written out once more in Python over the
    pinned pieces: what goes into which matmul, which buffer the gate and up products land in, the residual
    adds, the cache rows and the positions.  Returns the logits of every step."""
    g = lambda k: int(meta[f"qwen3.{k}"])  # noqa: E731
    n_embd, n_layer, n_head, n_head_kv, n_ff = g("embedding_length"), g("block_count"), g("attention.head_count"), g(
        "attention.head_count_kv"), g("feed_forward_length")
    hk, hv, vocab = g("attention.key_length"), g("attention.value_length"), g("vocab_size")
    eps, base = f32(meta["qwen3.attention.layer_norm_rms_epsilon"]), float(meta["qwen3.rope.freq_base"])
    kv_stride = n_head_kv * max(hk, hv)
    k_cache = np.zeros((n_layer, n_steps, kv_stride), np.uint16)
    v_cache = np.zeros((n_layer, n_steps, kv_stride), np.uint16)

    def mm(name, x, n_in, n_out):
        q8, sc = oracle.quantize_q8_0(x, oracle.AVX2)
        return oracle.matmul_q8_0_quantized(t[name], q8, sc, n_in, n_out, oracle.AVX2)

    norm_w = lambda name: t[name].view(np.float32)  # noqa: E731
    logits, tokens = [], list(prompt)
    for step in range(n_steps):
        x = oracle.embedding_lookup_q8_0(t["token_embd.weight"], tokens[step], n_embd)
        for layer in range(n_layer):
            p = f"blk.{layer}."
            normed = oracle.rms_norm(x, norm_w(p + "attn_norm.weight"), eps)
            q = mm(p + "attn_q.weight", normed, n_embd, n_head * hk)
            k = mm(p + "attn_k.weight", normed, n_embd, n_head_kv * hk)
            v = mm(p + "attn_v.weight", normed, n_embd, n_head_kv * hv)
            for h in range(n_head):
                q[h * hk:(h + 1) * hk] = oracle.rope_neox(
                    oracle.rms_norm(q[h * hk:(h + 1) * hk], norm_w(p + "attn_q_norm.weight"), eps), step, base)
            for h in range(n_head_kv):
                k[h * hk:(h + 1) * hk] = oracle.rope_neox(
                    oracle.rms_norm(k[h * hk:(h + 1) * hk], norm_w(p + "attn_k_norm.weight"), eps), step, base)
            k_cache[layer, step, :n_head_kv * hk] = k.astype(np.float16).view(np.uint16)
            v_cache[layer, step, :n_head_kv * hv] = v.astype(np.float16).view(np.uint16)
            attn = oracle.attention_f16(q, k_cache[layer], v_cache[layer], step, kv_stride, n_head, n_head_kv, hk, hv)
            x = x + mm(p + "attn_output.weight", attn, n_head * hv, n_embd)
            normed = oracle.rms_norm(x, norm_w(p + "ffn_norm.weight"), eps)
            gate_product = mm(p + "ffn_gate.weight", normed, n_embd, n_ff)
            up_product = mm(p + "ffn_up.weight", normed, n_embd, n_ff)
            h_ = oracle.silu_mul(gate_product, up_product)  # up * silu(gate), qwen3.rs:996-1018
            x = x + mm(p + "ffn_down.weight", h_, n_ff, n_embd)
        normed = oracle.rms_norm(x, norm_w("output_norm.weight"), eps)
        logits.append(mm("token_embd.weight", normed, n_embd, vocab))
        if step + 1 >= len(prompt):
            tokens.append(oracle.greedy_token(logits[-1]))
    return np.stack(logits), tokens[len(prompt):]


def test_decode_loop_wiring_against_a_python_composition(oracle, rmi, tmp_path):
    if not oracle.have_avx2():
        pytest.skip("host has no AVX2")
    import os

    kw = dict(n_layer=2, n_embd=64, n_head=4, n_head_kv=2, head_dim=32, n_ff=96, vocab=200, n_ctx=64)
    path = os.path.join(str(tmp_path), "tiny.gguf")
    rmi.gguf.write_synthetic_qwen3(path, seed=9, **kw)
    f = rmi.gguf.GGUFFile(path)
    tensors = {name: t[2] for name, t in f.tensors.items()}
    prompt = [5, 199, 0, 17]
    pool = oracle.Pool(2)
    run = oracle.Qwen3Decoder(f.metadata, tensors, pool).generate(prompt, 3, dump_steps=list(range(6)))
    pool.close()
    logits, tokens = _step_by_step(oracle, f.metadata, tensors, prompt, 6)
    assert np.array_equal(bits(run["dump"]), bits(logits))
    assert list(run["tokens"]) == tokens[:3]
