// Device-resident decode step of the Qwen3 text model: everything between two
// token ids stays in HBM.  Follows Qwen3Session::generate_inner
// (src/models/qwen3.rs:581-1158) for all-Q8_0 weights, F16 KV cache, NeoX RoPE,
// per-head q/k RMS norm and greedy sampling:
//   embedding_lookup_q8_0   src/ops/embedding.rs:12-22
//   rms_norm                src/ops/norm.rs:3-19      (f64 sum of f32 squares)
//   quantize_q8_0_into      src/ops/quant/q8_0.rs     (fused into the producer)
//   rope_neox               src/ops/rope.rs:21-37     (cos/sin table from the host libm)
//   attention, F16 cache    src/models/qwen3.rs:876-933, dot_f16 src/ops/dot.rs:99-119
//   softmax                 src/ops/attention.rs:28-38
//   silu_mul_inplace        src/ops/activation/mod.rs:137-151
//   greedy_token            src/models/qwen3.rs:172-191
// The quantized matmuls are the GEMV of gemv_q8_0.hip on q/k/v and gate/up
// stacked into one weight each (src/ops/quant/fuse.rs:25-64).
//
// Every f32 rounding point of the reference is kept: products rounded to f32
// before the f64 accumulation, f16 roundings of q, k, v and of the softmax
// weights, the sequential f32 sum of softmax, one f32 division per weight, and
// exp with the bits of the platform libm (device_math.h).  Only the f64 sums of
// rms_norm run as a tree instead of in sequence; they hold f32 squares, so the
// order can matter only when the f64 sum rounds differently in its last bits
// and that flips the f32 rounding of the mean (about 2^-29 per norm).  A rounded
// int8 quant that flips would move logits by 1e-2, so the step is held to
// bit-identical logits against the CPU path, not to a tolerance.
#include <chrono>
#include <cmath>
#include <utility>
#include <vector>

#include "device_math.h"
#include "device_quant.h"
#include "rmi_internal.h"

#include "device_common.h"

namespace {

__device__ __forceinline__ uint16_t f2h(float v) { return rmi_f2h(v); }

// The step counter in HBM: the embedding kernel reads its token through it and the argmax kernel advances it,
// so the next token never visits the host.  The kernels in between get the position as a launch argument:
// reading it from HBM first would put one more memory round trip in front of their loads.  (Replaying a whole step as a HIP graph with the counter read everywhere was
// measured: 676 vs 678 token-steps/s, no gain, so the launches stay eager.)
struct StepParams {
    uint32_t step;      // position of the token being processed = row of the KV cache
    uint32_t n_prompt;  // steps below n_prompt - 1 read their token from the prompt
};

__device__ __forceinline__ double wave_sum(double v) { return wave_sum_f64(v); }

// x[e] = d * q of row `token` of a Q8_0 weight in the GEMV tile stream
__device__ __forceinline__ void embed_row(const uint8_t *__restrict__ w, uint32_t n_oct, uint32_t token, uint32_t vocab,
                                          float *__restrict__ x, uint32_t n_embd) {
    if (token >= vocab) token = vocab - 1;  // ids are validated on the host; never read outside the weight
    const uint8_t *tile = w + size_t(token >> 3) * n_oct * kOctetBytes;
    const uint32_t r = token & 7;
    for (uint32_t e = threadIdx.x; e < n_embd; e += blockDim.x) {
        const uint32_t b = e >> 5, k = e & 31;
        const uint16_t dh = *reinterpret_cast<const uint16_t *>(tile + (b >> 3) * 128 + r * 16 + (b & 7) * 2);
        const int8_t q = *reinterpret_cast<const int8_t *>(tile + size_t(n_oct) * 128 + size_t(b >> 2) * 1024 + r * 128 +
                                                           (k >> 2) * 16 + (b & 3) * 4 + (k & 3));
        x[e] = h2f(dh) * float(int(q));
    }
}
// the first step's embedding; every later one is written by the step before it (argmax_final_kernel)
__global__ __launch_bounds__(256) void embed_q8_0_kernel(const uint8_t *__restrict__ w, uint32_t n_oct,
                                                          const uint32_t *__restrict__ tok,
                                                          const StepParams *__restrict__ sp, uint32_t vocab,
                                                          float *__restrict__ x, uint32_t n_embd) {
    embed_row(w, n_oct, tok[sp->step], vocab, x, n_embd);
}

// x += r (if r), then rms_norm(x, weight) quantized to Q8_0.  One workgroup of 256; R float4 per thread stay in
// registers (n <= 1024 * R), and every load of the kernel goes out before the first wait, so the kernel sees
// one memory round trip.  Sum of squares: per thread in ascending order, f64, then lanes and waves combined.
// A launch of several workgroups does the same for as many tokens: token blockIdx.x, the arrays tok_stride.x/.y/.z
// elements apart (x, r, q8; the scales q8's stride / 32).
struct TokStride3 {
    uint32_t x, y, z;
};
template <int R>
__global__ __launch_bounds__(256) void add_rmsnorm_quant_kernel(float *__restrict__ x, const float *__restrict__ r,
                                                                 const float *__restrict__ weight, uint32_t n, float eps,
                                                                 int8_t *__restrict__ q8, float *__restrict__ scales,
                                                                 int rounding, TokStride3 tok_stride) {
    __shared__ double red[4];
    const uint32_t tid = threadIdx.x;
    x += size_t(blockIdx.x) * tok_stride.x;
    if (r) r += size_t(blockIdx.x) * tok_stride.y;
    q8 += size_t(blockIdx.x) * tok_stride.z;
    scales += size_t(blockIdx.x) * (tok_stride.z >> 5);
    float4 v[R], a[R], wv[R];
#pragma unroll
    for (int j = 0; j < R; j++) {  // unconditional loads; a vector past the end re-reads the last one and is not used
        const uint32_t i = tid * 4 + j * 1024, ic = i < n ? i : n - 4;
        v[j] = *reinterpret_cast<const float4 *>(x + ic);
        if (r) a[j] = *reinterpret_cast<const float4 *>(r + ic);
        wv[j] = *reinterpret_cast<const float4 *>(weight + ic);
    }
    double part = 0.0;
#pragma unroll
    for (int j = 0; j < R; j++) {
        const uint32_t i = tid * 4 + j * 1024;
        if (i < n) {
            if (r) {
                v[j].x += a[j].x;
                v[j].y += a[j].y;
                v[j].z += a[j].z;
                v[j].w += a[j].w;
                *reinterpret_cast<float4 *>(x + i) = v[j];
            }
            const float s0 = v[j].x * v[j].x, s1 = v[j].y * v[j].y, s2 = v[j].z * v[j].z, s3 = v[j].w * v[j].w;
            part += double(s0);
            part += double(s1);
            part += double(s2);
            part += double(s3);
        }
    }
    part = wave_sum(part);
    if ((tid & 63) == 0) red[tid >> 6] = part;
    __syncthreads();
    const double total = (red[0] + red[1]) + (red[2] + red[3]);
    const float mean_sq = float(total / double(n));
    const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
    for (int j = 0; j < R; j++) {
        const uint32_t i = tid * 4 + j * 1024;
        if (i < n) {  // n is a multiple of 32: whole 8-lane groups
            float4 o;
            o.x = (v[j].x * scale) * wv[j].x;
            o.y = (v[j].y * scale) * wv[j].y;
            o.z = (v[j].z * scale) * wv[j].z;
            o.w = (v[j].w * scale) * wv[j].w;
            float sc;
            reinterpret_cast<uint32_t *>(q8)[i >> 2] = rmi_quantize_block8(o, rounding, &sc);
            if ((tid & 7) == 0) scales[i >> 5] = sc;
        }
    }
}

constexpr uint32_t kNormMaxN = 1024 * 16;
void launch_add_rmsnorm_quant(float *x, const float *r, const float *weight, uint32_t n, float eps, int8_t *q8,
                              float *scales, int rounding, hipStream_t st, uint32_t n_tok = 1, TokStride3 ts = TokStride3{0, 0, 0}) {
    if (n <= 1024)
        hipLaunchKernelGGL(add_rmsnorm_quant_kernel<1>, dim3(n_tok), dim3(256), 0, st, x, r, weight, n, eps, q8, scales, rounding, ts);
    else if (n <= 2048)
        hipLaunchKernelGGL(add_rmsnorm_quant_kernel<2>, dim3(n_tok), dim3(256), 0, st, x, r, weight, n, eps, q8, scales, rounding, ts);
    else if (n <= 4096)
        hipLaunchKernelGGL(add_rmsnorm_quant_kernel<4>, dim3(n_tok), dim3(256), 0, st, x, r, weight, n, eps, q8, scales, rounding, ts);
    else if (n <= 8192)
        hipLaunchKernelGGL(add_rmsnorm_quant_kernel<8>, dim3(n_tok), dim3(256), 0, st, x, r, weight, n, eps, q8, scales, rounding, ts);
    else
        hipLaunchKernelGGL(add_rmsnorm_quant_kernel<16>, dim3(n_tok), dim3(256), 0, st, x, r, weight, n, eps, q8, scales, rounding, ts);
}

// Per head of the stacked q|k|v vector: q/k RMS norm, NeoX rotation, f16 rounding; k and v go to the cache row.
__global__ __launch_bounds__(64) void qk_norm_rope_store_kernel(const float *__restrict__ qkv,
                                                                const float *__restrict__ q_norm,
                                                                const float *__restrict__ k_norm,
                                                                const float *__restrict__ cos_t,
                                                                const float *__restrict__ sin_t, uint32_t pos,
                                                                uint16_t *__restrict__ q16, uint16_t *__restrict__ k_row,
                                                                uint16_t *__restrict__ v_row, uint32_t n_head,
                                                                uint32_t n_head_kv, uint32_t hk, uint32_t hv, float eps,
                                                                TokStride3 tok_stride) {
    const uint32_t head = blockIdx.x, tid = threadIdx.x;
    // token blockIdx.y of a launch over several: the next position, its qkv, q16 and cache rows tok_stride apart
    qkv += size_t(blockIdx.y) * tok_stride.x;
    q16 += size_t(blockIdx.y) * tok_stride.y;
    k_row += size_t(blockIdx.y) * tok_stride.z;
    v_row += size_t(blockIdx.y) * tok_stride.z;
    pos += blockIdx.y;
    if (head >= n_head + n_head_kv) {  // v: rounding only
        const uint32_t kvh = head - n_head - n_head_kv;
        const float *src = qkv + size_t(n_head) * hk + size_t(n_head_kv) * hk + size_t(kvh) * hv;
        if (hv == 128) {
            const float v0 = src[tid], v1 = src[tid + 64];
            v_row[kvh * 128 + tid] = f2h(v0);
            v_row[kvh * 128 + tid + 64] = f2h(v1);
            return;
        }
        for (uint32_t d = tid; d < hv; d += 64) v_row[kvh * hv + d] = f2h(src[d]);
        return;
    }
    const bool is_q = head < n_head;
    const uint32_t local = is_q ? head : head - n_head;
    const float *src = qkv + (is_q ? size_t(local) * hk : size_t(n_head) * hk + size_t(local) * hk);
    const float *nw = is_q ? q_norm : k_norm;
    if (hk == 128) {  // lane i owns the pair (i, i + 64): every load goes out before the first wait
        const float x0r = src[tid], x1r = src[tid + 64];
        const float cos_a = cos_t[size_t(pos) * 64 + tid], sin_a = sin_t[size_t(pos) * 64 + tid];
        float x0 = x0r, x1 = x1r;
        if (nw) {
            const float w0 = nw[tid], w1 = nw[tid + 64];
            const float q0 = x0r * x0r, q1 = x1r * x1r;
            double part = double(q0);
            part += double(q1);
            const double total = wave_sum(part);
            const float mean_sq = float(total / 128.0);
            const float sc = 1.0f / sqrtf(mean_sq + eps);
            x0 = (x0r * sc) * w0;
            x1 = (x1r * sc) * w1;
        }
        uint16_t *dst = is_q ? q16 + size_t(local) * 128 : k_row + size_t(local) * 128;
        const float a = x1 * -sin_a;
        const float b = x1 * cos_a;
        dst[tid] = f2h(__builtin_fmaf(x0, cos_a, a));
        dst[tid + 64] = f2h(__builtin_fmaf(x0, sin_a, b));
        return;
    }
    float scale = 1.0f;
    if (nw) {
        double part = 0.0;
        for (uint32_t d = tid; d < hk; d += 64) {
            const float sq = src[d] * src[d];
            part += double(sq);
        }
        const double total = wave_sum(part);
        const float mean_sq = float(total / double(hk));
        scale = 1.0f / sqrtf(mean_sq + eps);
    }
    const uint32_t half = hk >> 1;
    uint16_t *dst = is_q ? q16 + size_t(local) * hk : k_row + size_t(local) * hk;
    for (uint32_t i = tid; i < half; i += 64) {
        float x0 = src[i], x1 = src[i + half];
        if (nw) {
            x0 = (x0 * scale) * nw[i];
            x1 = (x1 * scale) * nw[i + half];
        }
        const float cos_a = cos_t[size_t(pos) * half + i], sin_a = sin_t[size_t(pos) * half + i];
        const float a = x1 * -sin_a;
        const float b = x1 * cos_a;
        dst[i] = f2h(__builtin_fmaf(x0, cos_a, a));
        dst[i + half] = f2h(__builtin_fmaf(x0, sin_a, b));
    }
}

// One workgroup of 1024 per query head over keys 0..step of the F16 cache; the head's output leaves quantized
// to Q8_0.  The product of two f16 values is exact in f32, so the reference's "f32 product, f64 sum" is an f64
// fma chain; those f64 sums are split over lanes and combined at the end (a different order can change a
// result only when it flips the final rounding to f32, about once in 2^26 sums).  The f32 sum of the softmax
// weights runs in sequence, as in the reference: there the order shows in the last bit.
constexpr uint32_t kAttnThreads = 1024;
constexpr uint32_t kAttnPad = 64;  // keys are padded to this in LDS
__host__ __device__ inline size_t attn_lds_bytes(uint32_t n_keys, uint32_t hk, uint32_t hv) {
    const size_t n_pad = (size_t(n_keys) + kAttnPad - 1) / kAttnPad * kAttnPad;
    const size_t slices = kAttnThreads / hv ? kAttnThreads / hv : 1;
    return n_pad * 8 + size_t(hk) * 8 + slices * hv * 8 + n_pad * 4 + size_t(hv) * 4;
}
__global__ __launch_bounds__(kAttnThreads) void attention_quant_kernel(
    const uint16_t *__restrict__ q16, const uint16_t *__restrict__ k_cache, const uint16_t *__restrict__ v_cache,
    uint32_t step, uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv, uint32_t hk, uint32_t hv,
    int8_t *__restrict__ q8, float *__restrict__ scales, int rounding) {
    extern __shared__ double lds_d[];
    __shared__ float red_f[kAttnThreads / 64];
    __shared__ uint64_t exp_tab[32];
    const uint32_t head = blockIdx.x, tid = threadIdx.x;
    const uint32_t kvh = head / (n_head / n_head_kv);
    const uint32_t n_keys = step + 1;
    const uint32_t n_pad = (n_keys + kAttnPad - 1) / kAttnPad * kAttnPad;
    const uint32_t n_slices = kAttnThreads / hv ? kAttnThreads / hv : 1;
    double *wd = lds_d;                                          // [n_pad] softmax weights (f16 values), 0 beyond n_keys
    double *qd = wd + n_pad;                                     // [hk]    the query (f16 values)
    double *part = qd + hk;                                      // [n_slices][hv]
    float *scores = reinterpret_cast<float *>(part + size_t(n_slices) * hv);  // [n_pad]
    float *outv = scores + n_pad;                                // [hv]
    for (uint32_t d = tid; d < hk; d += kAttnThreads) qd[d] = double(h2f(q16[size_t(head) * hk + d]));
    if (tid < 32) exp_tab[tid] = kRmiExp2fTab[tid];

    // values: hv columns x n_slices ranges of keys.  The first loads of this thread's range go out now and
    // arrive while the scores and the softmax are computed.
    constexpr uint32_t kPre = 16;
    const bool v_lane = tid < n_slices * hv;
    const uint32_t vd = tid % hv, slice = tid / hv;
    const uint32_t chunk = ((n_pad / 8 + n_slices - 1) / n_slices) * 8;  // keys per slice, a multiple of 8
    const uint32_t t_begin = slice * chunk, t_end = t_begin + chunk < n_pad ? t_begin + chunk : n_pad;
    const uint16_t *col = v_cache + size_t(kvh) * hv + (v_lane ? vd : 0);
    uint32_t pre[kPre];  // one register each: 16-bit destinations would chain the loads
#pragma unroll
    for (uint32_t j = 0; j < kPre; j++) {
        // unconditional loads (a guarded load would wait for itself): past the last key the row of the last key
        // is read instead; its weight is zero or the element is skipped below
        const uint32_t t = t_begin + j < n_keys ? t_begin + j : n_keys - 1;
        pre[j] = col[size_t(t) * kv_stride];
    }

    // scores: four lanes per key, a quarter of the head dimension each.  For head dimension 128 the first
    // round's keys are loaded here, with the values above, so that one memory round trip covers all of them.
    const float kq_scale = 1.0f / sqrtf(float(hk));
    const uint32_t quarter = hk >> 2, lane4 = tid & 3;
    const double *qq = qd + lane4 * quarter;
    uint4 kk0[4];
    if (quarter == 32) {
        const uint32_t t = (tid >> 2) < n_keys ? (tid >> 2) : 0;
        const uint16_t *key = k_cache + size_t(t) * kv_stride + size_t(kvh) * hk + lane4 * quarter;
#pragma unroll
        for (int c = 0; c < 4; c++) kk0[c] = *reinterpret_cast<const uint4 *>(key + 8 * c);
    }
    __syncthreads();

    float my_max = -INFINITY;
    if (quarter == 32) {  // head dimension 128: the keys of the next round are in flight while this one is summed
        uint4 kk[4], kn[4];
#pragma unroll
        for (int c = 0; c < 4; c++) kk[c] = kk0[c];
        for (uint32_t t0 = 0; t0 < n_keys; t0 += kAttnThreads / 4) {
            const uint32_t t = t0 + (tid >> 2), tn = t + kAttnThreads / 4;
            if (t0 + kAttnThreads / 4 < n_keys) {
                const uint16_t *key = k_cache + size_t(tn < n_keys ? tn : 0) * kv_stride + size_t(kvh) * hk + lane4 * 32;
#pragma unroll
                for (int c = 0; c < 4; c++) kn[c] = *reinterpret_cast<const uint4 *>(key + 8 * c);
            }
            double sum = 0.0;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t kw[4] = {kk[c].x, kk[c].y, kk[c].z, kk[c].w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    sum = __builtin_fma(double(h2f(kw[j] & 0xffffu)), qq[8 * c + 2 * j], sum);
                    sum = __builtin_fma(double(h2f(kw[j] >> 16)), qq[8 * c + 2 * j + 1], sum);
                }
            }
            sum += dpp_f64<kDppQuadXor1>(sum);
            sum += dpp_f64<kDppQuadXor2>(sum);
            if (t < n_keys) {
                const float s = float(sum) * kq_scale;
                if (lane4 == 0) scores[t] = s;
                my_max = fmaxf(my_max, s);
            }
#pragma unroll
            for (int c = 0; c < 4; c++) kk[c] = kn[c];
        }
    } else {
        for (uint32_t t0 = 0; t0 < n_keys; t0 += kAttnThreads / 4) {
            const uint32_t t = t0 + (tid >> 2);
            const bool live = t < n_keys;
            const uint16_t *key = k_cache + size_t(live ? t : 0) * kv_stride + size_t(kvh) * hk + lane4 * quarter;
            double sum = 0.0;
            for (uint32_t d = 0; d < quarter; d += 8) {
                const uint4 kk = *reinterpret_cast<const uint4 *>(key + d);
                const uint32_t kw[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    sum = __builtin_fma(double(h2f(kw[j] & 0xffffu)), qq[d + 2 * j], sum);
                    sum = __builtin_fma(double(h2f(kw[j] >> 16)), qq[d + 2 * j + 1], sum);
                }
            }
            sum += dpp_f64<kDppQuadXor1>(sum);
            sum += dpp_f64<kDppQuadXor2>(sum);
            if (live) {
                const float s = float(sum) * kq_scale;
                if (lane4 == 0) scores[t] = s;
                my_max = fmaxf(my_max, s);
            }
        }
    }
    my_max = wave_max_f32(my_max);
    if ((tid & 63) == 0) red_f[tid >> 6] = my_max;
    __syncthreads();
    float max_val = red_f[0];
#pragma unroll
    for (uint32_t i = 1; i < kAttnThreads / 64; i++) max_val = fmaxf(max_val, red_f[i]);
    for (uint32_t t = tid; t < n_pad; t += kAttnThreads) scores[t] = t < n_keys ? rmi_expf_tab(scores[t] - max_val, exp_tab) : 0.0f;
    __syncthreads();
    if (tid == 0) {  // the reference adds the weights one after the other in f32; the padding zeros change nothing
        // one lane, one dependent chain of adds: the LDS reads run a batch of 32 values ahead of it
        float acc = 0.0f;
        float4 cur[8], nxt[8];
#pragma unroll
        for (int j = 0; j < 8; j++) cur[j] = reinterpret_cast<const float4 *>(scores)[j];
        for (uint32_t t = 0; t < n_pad; t += 32) {  // n_pad is a multiple of 64
            if (t + 32 < n_pad) {
#pragma unroll
                for (int j = 0; j < 8; j++) nxt[j] = reinterpret_cast<const float4 *>(scores + t + 32)[j];
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc += cur[j].x;
                acc += cur[j].y;
                acc += cur[j].z;
                acc += cur[j].w;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) cur[j] = nxt[j];
        }
        red_f[0] = acc;
    }
    __syncthreads();
    const float sum = red_f[0];
    for (uint32_t t = tid; t < n_pad; t += kAttnThreads) {
        const float e = scores[t];
        wd[t] = t < n_keys ? double(h2f(f2h(sum > 0.0f ? e / sum : e))) : 0.0;
    }
    __syncthreads();

    if (v_lane) {
        double acc = 0.0;
#pragma unroll
        for (uint32_t j = 0; j < kPre; j++)  // keys past n_keys carry weight zero
            if (t_begin + j < t_end) acc = __builtin_fma(double(h2f(pre[j])), wd[t_begin + j], acc);
        if (t_begin + kPre < t_end) {  // longer ranges: batches of 8, the next one in flight while one is added
            uint32_t cur[8], nxt[8];
#pragma unroll
            for (uint32_t j = 0; j < 8; j++) {
                const uint32_t t = t_begin + kPre + j;
                cur[j] = col[size_t(t < n_keys ? t : n_keys - 1) * kv_stride];
            }
            for (uint32_t t0 = t_begin + kPre; t0 < t_end; t0 += 8) {
#pragma unroll
                for (uint32_t j = 0; j < 8; j++) {
                    const uint32_t t = t0 + 8 + j;
                    nxt[j] = col[size_t(t < n_keys ? t : n_keys - 1) * kv_stride];
                }
#pragma unroll
                for (uint32_t j = 0; j < 8; j++) acc = __builtin_fma(double(h2f(cur[j])), wd[t0 + j], acc);
#pragma unroll
                for (uint32_t j = 0; j < 8; j++) cur[j] = nxt[j];
            }
        }
        part[size_t(slice) * hv + vd] = acc;
    }
    __syncthreads();
    for (uint32_t d = tid; d < hv; d += kAttnThreads) {
        double acc = part[d];
        for (uint32_t sl = 1; sl < n_slices; sl++) acc += part[size_t(sl) * hv + d];
        outv[d] = float(acc);
    }
    __syncthreads();
    if (tid * 4 < hv) {  // hv is a multiple of 32: whole 8-lane groups
        const float4 o = *reinterpret_cast<const float4 *>(outv + tid * 4);
        float sc;
        reinterpret_cast<uint32_t *>(q8)[(size_t(head) * hv >> 2) + tid] = rmi_quantize_block8(o, rounding, &sc);
        if ((tid & 7) == 0) scales[(size_t(head) * hv >> 5) + (tid >> 3)] = sc;
    }
}

// ---- the same attention for head dimension 128 (keys and values), the Qwen3 shape.  Arithmetic as above;
// what differs is the schedule.  The launch has 16 workgroups on a 256-CU chip, so its time is the length of one
// thread's instruction stream plus memory round trips, not throughput: the query stays in registers as packed
// f16 (product f16 x f16 is exact in f32, then an f64 add: the same value as the f64 fma above), every load of
// the first round of keys and of the first values of each thread goes out before anything waits, values are read
// 16 bytes (8 dimensions) at a time by 32 key slices, and the four slices of a wave combine in registers.  Eight
// waves, two per SIMD: with sixteen the kernel took a third longer (the waves of a SIMD run one after another
// through such dependent code, so more of them only repeat the per-thread set-up), with four it lost on long contexts.
constexpr uint32_t kA128Threads = 512;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ half8 as_half8(const uint4 &v) { return __builtin_bit_cast(half8, v); }
__device__ __forceinline__ double quad_sum(double v) {  // (l0 + l1) + (l2 + l3) in every lane of the quad
    int lo = __double2loint(v), hi = __double2hiint(v);
    v += __hiloint2double(__builtin_amdgcn_mov_dpp(hi, 0xB1, 0xf, 0xf, true), __builtin_amdgcn_mov_dpp(lo, 0xB1, 0xf, 0xf, true));
    lo = __double2loint(v), hi = __double2hiint(v);
    v += __hiloint2double(__builtin_amdgcn_mov_dpp(hi, 0x4E, 0xf, 0xf, true), __builtin_amdgcn_mov_dpp(lo, 0x4E, 0xf, 0xf, true));
    return v;
}
template <int XOR>
__device__ __forceinline__ double swizzle_xor_f64(double v) {  // the value of lane ^ XOR (XOR < 32)
    constexpr int kPattern = 0x1f | (XOR << 10);
    return __hiloint2double(__builtin_amdgcn_ds_swizzle(__double2hiint(v), kPattern),
                            __builtin_amdgcn_ds_swizzle(__double2loint(v), kPattern));
}
__device__ __forceinline__ double swizzle_xor16_f64(double v) { return swizzle_xor_f64<16>(v); }
// Two registers exchange lanes in one vector instruction (v_permlane32_swap: lanes 32..63 of the first with lanes
// 0..31 of the second; v_permlane16_swap: the odd rows of sixteen of the first with the even rows of the second).
// a + b afterwards is, in the lower half (the even rows), a summed over both halves (both rows of a pair), and in the
// upper half (the odd rows) b summed likewise: two values to reduce become one, without the LDS crossbar.
template <bool ROWS>
__device__ __forceinline__ double swap_add_f64(double a, double b) {
    const uint64_t ab = __builtin_bit_cast(uint64_t, a), bb = __builtin_bit_cast(uint64_t, b);
    uint64_t x, y;
    if constexpr (ROWS) {
        const auto lo = __builtin_amdgcn_permlane16_swap(uint32_t(ab), uint32_t(bb), false, false);
        const auto hi = __builtin_amdgcn_permlane16_swap(uint32_t(ab >> 32), uint32_t(bb >> 32), false, false);
        x = uint64_t(lo[0]) | (uint64_t(hi[0]) << 32);
        y = uint64_t(lo[1]) | (uint64_t(hi[1]) << 32);
    } else {
        const auto lo = __builtin_amdgcn_permlane32_swap(uint32_t(ab), uint32_t(bb), false, false);
        const auto hi = __builtin_amdgcn_permlane32_swap(uint32_t(ab >> 32), uint32_t(bb >> 32), false, false);
        x = uint64_t(lo[0]) | (uint64_t(hi[0]) << 32);
        y = uint64_t(lo[1]) | (uint64_t(hi[1]) << 32);
    }
    return __builtin_bit_cast(double, x) + __builtin_bit_cast(double, y);
}
// The eight f64 sums of a lane (dimensions 8 dg .. 8 dg + 7, dg = lane % DG_LANES) added over the wave's 64 / DG_LANES
// key slices (lanes DG_LANES apart; DG_LANES = 4, 8 or 16).  Halves, then rows, halve the values as they halve the
// lanes; what is left inside a row of sixteen goes round it by DPP.  Lane l ends with two sums, those of dimensions
// 8 dg + pv_dim_base(l) and the next one.  (f64 sums of exact terms: the order of the additions is free.)
__device__ __forceinline__ uint32_t pv_dim_base(uint32_t lane) { return 2 * ((lane >> 4) & 1) + 4 * (lane >> 5); }
template <int DG_LANES>
__device__ __forceinline__ void pv_slices_sum(const double (&acc)[8], double (&u)[2]) {
    static_assert(DG_LANES == 4 || DG_LANES == 8 || DG_LANES == 16, "slices are whole parts of a row of sixteen lanes");
    double r[4];
#pragma unroll
    for (int k = 0; k < 4; k++) r[k] = swap_add_f64<false>(acc[k], acc[k + 4]);
#pragma unroll
    for (int k = 0; k < 2; k++) {
        u[k] = swap_add_f64<true>(r[k], r[k + 2]);
        if constexpr (DG_LANES <= 8) u[k] += dpp_f64<0x128>(u[k]);  // row_ror:8
        if constexpr (DG_LANES <= 4) u[k] += dpp_f64<0x124>(u[k]);  // row_ror:4
    }
}
__host__ __device__ inline size_t attn128_lds_bytes(uint32_t n_keys) {
    const size_t n_pad = (size_t(n_keys) + kAttnPad - 1) / kAttnPad * kAttnPad;
    return n_pad * 12 + (kA128Threads / 64) * 128 * 8 + 128;  // 32 floats of room behind the scores
}
// FROM_QKV: the launch also does what qk_norm_rope_store_kernel does for this step, so that the q/k/v product in
// front of it can be a plain GEMV spread over the whole chip (a head per workgroup there means 139 KB of weights
// through one compute unit).  fq points at the step's f32 [q ; k ; v] and the norm weights and angles; waves 0, 1
// and 2 turn the head's q, its key/value head's new k and new v into f16 while the first cached keys are on their
// way, the new key and value are used from LDS (and written to their cache row by the first query head of each
// key/value head), the keys 0..step-1 come from the cache as before.
// PVP > 1 (single-position launches): PVP workgroups per head.  Each computes every score, the maximum, the
// exponentials and the sequential sum of the head for itself (exchanging them would cost more than repeating them)
// and then the p.v sums of 128 / PVP of the output dimensions only, over four times as many key slices: the part of
// the launch that is vector arithmetic on one compute unit shrinks by PVP.  A part's dimensions are whole 32-value
// blocks of the quantizer.  Workgroup ids run key/value head fastest, so that on a chip of eight XCDs and a model of
// eight key/value heads every workgroup that reads a head's cache rows shares one L2.
struct AttnFromQkv {
    const float *qkv;                // [n_head * 128 q | n_head_kv * 128 k | n_head_kv * 128 v]
    const float *q_norm, *k_norm;    // [128] each, or null
    const float *cos_row, *sin_row;  // [64] each: the angles of this position
    uint16_t *k_row, *v_row;         // the cache rows of this position, [n_head_kv][128] each
    float eps;
};
// DENSE: for launches of many workgroups (a prompt pass: positions x heads).  Every phase below is a stretch of
// dependent instructions, so one workgroup leaves its compute unit idle most of the time; with the registers held
// to 128 (a short value prefetch) two workgroups share a unit and fill each other's waits.
constexpr int kDenseWaves = 6, kDenseBatch = 2;
template <bool FROM_QKV, int PVP = 1, bool DENSE = false>
__global__ __launch_bounds__(kA128Threads, DENSE ? kDenseWaves : 2) void attention128_quant_kernel(
    const uint16_t *__restrict__ q16, const uint16_t *__restrict__ k_cache, const uint16_t *__restrict__ v_cache,
    uint32_t step, uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv, int8_t *__restrict__ q8,
    float *__restrict__ scales, int rounding, AttnFromQkv fq, uint32_t tok_q16_stride, uint32_t tok_out_stride) {
    extern __shared__ double lds_d[];
    __shared__ float red_f[kA128Threads / 64];
    __shared__ uint64_t exp_tab[32];
    __shared__ __attribute__((aligned(16))) uint16_t new16[3][128];  // this step's q, k, v as f16
    // token blockIdx.z of a launch over several consecutive positions (their cache rows are filled already)
    step += blockIdx.z;
    q16 += size_t(blockIdx.z) * tok_q16_stride;
    q8 += size_t(blockIdx.z) * tok_out_stride;
    scales += size_t(blockIdx.z) * (tok_out_stride >> 5);
    // grid = (query heads per key/value head, key/value heads), or with PVP parts n_head * PVP workgroups in a row:
    // key/value head fastest, then the query head of its group, then the part
    static_assert(PVP == 1 || PVP == 2 || PVP == 4, "a part is one, two or four blocks of 32 dimensions");
    const uint32_t tid = threadIdx.x, hpk = n_head / n_head_kv;
    const uint32_t kvh = PVP == 1 ? blockIdx.y : blockIdx.x % n_head_kv;
    const uint32_t qh = PVP == 1 ? blockIdx.x : (blockIdx.x / n_head_kv) % hpk;
    const uint32_t pv_part = PVP == 1 ? 0u : blockIdx.x / n_head_kv / hpk;
    const uint32_t head = kvh * hpk + qh;
    const uint32_t n_keys = step + 1;
    // keys that come from the cache, and the last row there that may be read
    const uint32_t n_cached = FROM_QKV ? step : n_keys, last_row = n_cached ? n_cached - 1 : 0;
    const uint32_t n_pad = (n_keys + kAttnPad - 1) / kAttnPad * kAttnPad;
    double *wd = lds_d;                                        // [n_pad] softmax weights (f16 values), 0 beyond n_keys
    double *part = wd + n_pad;                                 // [waves][128]
    float *scores = reinterpret_cast<float *>(part + (kA128Threads / 64) * 128);  // [n_pad]
    const uint32_t row_u4 = kv_stride >> 3;                    // uint4 per cache row
    const uint64_t tab_entry = kRmiExp2fTab[tid & 31];         // first load out; stored to LDS after the scores

    // scores: four lanes per key; lane4 takes the 16-byte pieces lane4, 4 + lane4, 8 + lane4, 12 + lane4 of the
    // key's 256 bytes, so that the four lanes of a key read 64 consecutive bytes with each load (the memory
    // pipeline handles a quad of lanes per step, and a quad that spans several cache lines takes several)
    const uint32_t lane4 = tid & 3, key0 = tid >> 2;
    const uint4 *qp = reinterpret_cast<const uint4 *>(q16 + size_t(head) * 128) + lane4;
    const uint4 *kbase = reinterpret_cast<const uint4 *>(k_cache + size_t(kvh) * 128) + lane4;
    uint4 qv[4], kk[4];
    float raw0 = 0.0f, raw1 = 0.0f, nw0 = 1.0f, nw1 = 1.0f, cos_a = 0.0f, sin_a = 0.0f;
    if constexpr (FROM_QKV) {
        if (tid < 192) {  // wave 0: q of this head, wave 1: the new k, wave 2: the new v; lane i owns (i, i + 64)
            const uint32_t lane = tid & 63;
            const float *src = tid < 64 ? fq.qkv + size_t(head) * 128
                                        : fq.qkv + size_t(n_head) * 128 + (tid < 128 ? size_t(kvh) : size_t(n_head_kv) + kvh) * 128;
            raw0 = src[lane];
            raw1 = src[lane + 64];
            if (tid < 128) {
                cos_a = fq.cos_row[lane];
                sin_a = fq.sin_row[lane];
                const float *nw = tid < 64 ? fq.q_norm : fq.k_norm;
                if (nw) {
                    nw0 = nw[lane];
                    nw1 = nw[lane + 64];
                }
            }
        }
    } else {
#pragma unroll
        for (int c = 0; c < 4; c++) qv[c] = qp[4 * c];
    }
    {
        const uint4 *key = kbase + __umul24(key0 < n_cached ? key0 : last_row, row_u4);
#pragma unroll
        for (int c = 0; c < 4; c++) kk[c] = key[4 * c];
    }
    // values: lane = (8 dimensions dg, key slice sl): 16 consecutive lanes read the 256 bytes of one row
    // (with PVP parts: 16 / PVP lanes read the part's 256 / PVP bytes of a row, PVP times as many slices)
    constexpr uint32_t kDgLanes = 16 / PVP, kSlices = kA128Threads / kDgLanes;
    // With parts a slice is short (six keys a slice cover 768 keys with four parts; longer slices go on in the batches
    // further down) and its loads are unconditional: a load under
    // a branch makes the wait for this position's q, k, v (issued first) drain most of what was issued behind them.
    constexpr uint32_t kPre = DENSE ? 1 : (PVP == 1 ? (kA128Threads >= 1024 ? 12 : (kA128Threads >= 512 ? 20 : 40)) : 24 / PVP);
    constexpr uint32_t kBatch = DENSE ? kDenseBatch : 8;  // keys of a slice in flight beyond the first kPre
    const uint32_t dg = tid % kDgLanes, sl = tid / kDgLanes;
    const uint32_t chunk = (n_cached + kSlices - 1) / kSlices;
    const uint32_t t_begin = sl * chunk, t_end = t_begin + chunk < n_cached ? t_begin + chunk : n_cached;
    const uint4 *vbase = reinterpret_cast<const uint4 *>(v_cache + size_t(kvh) * 128 + pv_part * (128 / PVP) + dg * 8);
    uint4 vp[kPre];
#pragma unroll
    for (uint32_t j = 0; j < kPre; j++) {  // j < chunk is uniform: no lane waits on a guarded load of its own
        if (PVP > 1 || j < chunk) {
            const uint32_t t = t_begin + j < n_cached ? t_begin + j : last_row;
            vp[j] = vbase[__umul24(t, row_u4)];
        }
    }
    if constexpr (FROM_QKV) {
        // head norm (when the model has the weights), NeoX rotation, rounding to f16: src/models/qwen3.rs:776-874
        if (tid < 192) {
            const uint32_t lane = tid & 63, which = tid >> 6;
            uint16_t h0, h1;
            if (which == 2) {
                h0 = f2h(raw0);
                h1 = f2h(raw1);
            } else {
                float x0 = raw0, x1 = raw1;
                if (which == 0 ? fq.q_norm != nullptr : fq.k_norm != nullptr) {
                    const float q0 = raw0 * raw0, q1 = raw1 * raw1;
                    double part = double(q0);
                    part += double(q1);
                    part = wave_sum_f64(part);
                    const float mean_sq = float(part / 128.0);
                    const float sc = 1.0f / sqrtf(mean_sq + fq.eps);
                    x0 = (raw0 * sc) * nw0;
                    x1 = (raw1 * sc) * nw1;
                }
                const float ta = x1 * -sin_a;
                const float tb = x1 * cos_a;
                h0 = f2h(__builtin_fmaf(x0, cos_a, ta));
                h1 = f2h(__builtin_fmaf(x0, sin_a, tb));
            }
            new16[which][lane] = h0;
            new16[which][lane + 64] = h1;
            if (which && qh == 0 && pv_part == 0) {  // the first query head of the key/value head fills the cache row
                uint16_t *dst = (which == 1 ? fq.k_row : fq.v_row) + size_t(kvh) * 128;
                dst[lane] = h0;
                dst[lane + 64] = h1;
            }
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 4; c++) qv[c] = reinterpret_cast<const uint4 *>(new16[0])[lane4 + 4 * c];
    }
    const float kq_scale = 1.0f / sqrtf(128.0f);  // two f32 roundings, as the reference computes it
    float my_max = -INFINITY;
    for (uint32_t t0 = 0; t0 < n_keys; t0 += kA128Threads / 4) {
        const uint32_t t = t0 + key0, tn = t + kA128Threads / 4;
        // The next round's keys are in flight while this one is summed.  The loads are unconditional (after the
        // last round they read the last key again): behind a branch they could not be counted on, and the wait
        // for this round's keys would have to drain them, too.
        uint4 kn[4];
        {
            const uint4 *key = kbase + __umul24(tn < n_cached ? tn : last_row, row_u4);
#pragma unroll
            for (int c = 0; c < 4; c++) kn[c] = key[4 * c];
        }
        if constexpr (FROM_QKV) {
            if (t == n_cached) {  // this step's key: not in the cache yet for this launch, in LDS
#pragma unroll
                for (int c = 0; c < 4; c++) kk[c] = reinterpret_cast<const uint4 *>(new16[1])[lane4 + 4 * c];
            }
        }
        double s4[4] = {0.0, 0.0, 0.0, 0.0};  // four chains of eight adds, not one of thirty-two
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const half8 kh = as_half8(kk[c]), qh = as_half8(qv[c]);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float prod = __builtin_fmaf(float(kh[j]), float(qh[j]), 0.0f);  // exact
                s4[c] += double(prod);
            }
        }
        double sum = quad_sum((s4[0] + s4[1]) + (s4[2] + s4[3]));
        if (t < n_keys) {
            const float sc = float(sum) * kq_scale;
            if (lane4 == 0) scores[t] = sc;
            my_max = fmaxf(my_max, sc);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) kk[c] = kn[c];
    }
    my_max = wave_max_f32(my_max);
    if ((tid & 63) == 0) red_f[tid >> 6] = my_max;
    if (tid < 32) exp_tab[tid] = tab_entry;
    __syncthreads();
    float max_val = red_f[0];
#pragma unroll
    for (uint32_t i = 1; i < kA128Threads / 64; i++) max_val = fmaxf(max_val, red_f[i]);
    for (uint32_t t = tid; t < n_pad; t += kA128Threads) scores[t] = t < n_keys ? rmi_expf_tab(scores[t] - max_val, exp_tab) : 0.0f;
    __syncthreads();
    if (tid == 0) {  // the reference adds the weights one after the other in f32; the padding zeros change nothing
        // one lane, one dependent chain of adds; the LDS reads run 32 values ahead of it (two buffers, no copies)
        float acc = 0.0f;
        constexpr int kAhead = DENSE ? 4 : 8;  // float4 of each buffer
        float4 a[kAhead], b[kAhead];
#pragma unroll
        for (int j = 0; j < kAhead; j++) a[j] = reinterpret_cast<const float4 *>(scores)[j];
        for (uint32_t t = 0; t < n_pad; t += 8 * kAhead) {  // n_pad is a multiple of 64
#pragma unroll
            for (int j = 0; j < kAhead; j++) b[j] = reinterpret_cast<const float4 *>(scores + t + 4 * kAhead)[j];
#pragma unroll
            for (int j = 0; j < kAhead; j++) {
                acc += a[j].x;
                acc += a[j].y;
                acc += a[j].z;
                acc += a[j].w;
            }
            // unconditional (the array has 32 floats of room behind n_pad): under a branch the registers would be
            // copied every round, on the chain's own lane
#pragma unroll
            for (int j = 0; j < kAhead; j++) a[j] = reinterpret_cast<const float4 *>(scores + t + 8 * kAhead)[j];
#pragma unroll
            for (int j = 0; j < kAhead; j++) {
                acc += b[j].x;
                acc += b[j].y;
                acc += b[j].z;
                acc += b[j].w;
            }
        }
        red_f[0] = acc;
    }
    __syncthreads();
    const float total = red_f[0];
    for (uint32_t t = tid; t < n_pad; t += kA128Threads) {
        const float e = scores[t];
        wd[t] = t < n_keys ? double(h2f(f2h(total > 0.0f ? e / total : e))) : 0.0;
    }
    __syncthreads();

    double acc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = 0.0;
#pragma unroll
    for (uint32_t j = 0; j < kPre; j++) {
        if (t_begin + j < t_end) {
            const double w = wd[t_begin + j];
            const half8 vh = as_half8(vp[j]);
#pragma unroll
            for (int d = 0; d < 8; d++) acc[d] = __builtin_fma(double(float(vh[d])), w, acc[d]);
        }
    }
    if (t_begin + kPre < t_end) {  // longer slices: batches of kBatch keys, the next one in flight while one is added
        uint4 cur[kBatch], nxt[kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kBatch; j++) {
            const uint32_t t = t_begin + kPre + j;
            cur[j] = vbase[__umul24(t < n_cached ? t : last_row, row_u4)];
        }
        for (uint32_t t0 = t_begin + kPre; t0 < t_end; t0 += kBatch) {
#pragma unroll
            for (uint32_t j = 0; j < kBatch; j++) {
                const uint32_t t = t0 + kBatch + j;
                nxt[j] = vbase[__umul24(t < n_cached ? t : last_row, row_u4)];
            }
#pragma unroll
            for (uint32_t j = 0; j < kBatch; j++) {
                if (t0 + j < t_end) {
                    const double w = wd[t0 + j];
                    const half8 vh = as_half8(cur[j]);
#pragma unroll
                    for (int d = 0; d < 8; d++) acc[d] = __builtin_fma(double(float(vh[d])), w, acc[d]);
                }
            }
#pragma unroll
            for (uint32_t j = 0; j < kBatch; j++) cur[j] = nxt[j];
        }
    }
    if constexpr (FROM_QKV) {
        if (sl == 0) {  // this step's value, from LDS: one more exact term of the f64 sums
            const double w = wd[n_cached];
            const half8 vh = as_half8(reinterpret_cast<const uint4 *>(new16[2])[pv_part * kDgLanes + dg]);
#pragma unroll
            for (int d = 0; d < 8; d++) acc[d] = __builtin_fma(double(float(vh[d])), w, acc[d]);
        }
    }
    {  // the slices of a wave: lanes kDgLanes apart
        double u[2];
        pv_slices_sum<kDgLanes>(acc, u);
        if ((tid & 15) < kDgLanes) {  // one lane of each row for every dg
            double *dst = part + (tid >> 6) * 128 + dg * 8 + pv_dim_base(tid & 63);
            dst[0] = u[0];
            dst[1] = u[1];
        }
    }
    __syncthreads();
    if (tid < 32 / PVP) {  // four dimensions per lane: whole 8-lane groups for the quantizer
        double o[4];
#pragma unroll
        for (int d = 0; d < 4; d++) o[d] = part[tid * 4 + d];
        for (uint32_t w = 1; w < kA128Threads / 64; w++) {
#pragma unroll
            for (int d = 0; d < 4; d++) o[d] += part[w * 128 + tid * 4 + d];
        }
        const float4 of = make_float4(float(o[0]), float(o[1]), float(o[2]), float(o[3]));
        float sc;
        const size_t first = size_t(head) * 128 + pv_part * (128 / PVP);  // of this workgroup's output dimensions
        reinterpret_cast<uint32_t *>(q8)[(first >> 2) + tid] = rmi_quantize_block8(of, rounding, &sc);
        if ((tid & 7) == 0) scales[(first >> 5) + (tid >> 3)] = sc;
    }
}

// ---- head dimension 128 over long contexts: a head's keys split over several workgroups, two launches.
// One workgroup per head leaves most of the chip idle and costs about 54 clocks of one compute unit per key; of
// the head's arithmetic only the f32 sum of the softmax weights has to run in key order (about 8 clocks a key
// on one lane).  The scores and the p.v sums are f64 sums of exact terms, which are split over lanes already
// and here over workgroups as well:
//   attn128_scores_kernel    workgroup (head, part): the scores of its keys to HBM, and their maximum;
//   attn128_weights_pv_kernel workgroup (head, part): the head's maximum, exp of every score of the head into
//                            LDS, the sequential f32 sum (every part computes the same one: waiting for another
//                            workgroup's would take as long), the f16 weights of its own keys, their p.v sums;
//                            the part that finishes last adds the parts' sums in part order and quantizes.
// Every f32 / f16 rounding point is that of attention128_quant_kernel.  Workgroup ids are head + n_head * part,
// so with a multiple of 8 heads the parts of a head sit on one XCD and share its L2.
constexpr uint32_t kAttnSplitThreads = 512;
constexpr uint32_t kAttnSplitMaxParts = 16;
struct AttnSplitScratch {  // device memory of one attention launch pair; the counters start, and are left, at zero
    float *scores;      // [n_head][score_stride]
    float *part_max;    // [n_head][kAttnSplitMaxParts]
    double *part_sums;  // [n_head][kAttnSplitMaxParts][128]
    uint32_t *arrived;  // [n_head]
    uint32_t score_stride;
};
__host__ __device__ inline size_t attn128_split_lds_bytes(uint32_t n_keys, uint32_t keys_per_part) {
    const size_t n_pad = (size_t(n_keys) + kAttnPad - 1) / kAttnPad * kAttnPad;
    return n_pad * 4 + size_t(keys_per_part) * 8 + (kAttnSplitThreads / 64) * 128 * 8 + 128;  // 32 floats of room behind e
}
__global__ __launch_bounds__(kAttnSplitThreads) void attn128_scores_kernel(
    const uint16_t *__restrict__ q16, const uint16_t *__restrict__ k_cache, uint32_t n_keys, uint32_t keys_per_part,
    uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv, AttnSplitScratch ws) {
    __shared__ float red_f[kAttnSplitThreads / 64];
    const uint32_t head = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    const uint32_t kvh = head / (n_head / n_head_kv);
    const uint32_t t_first = part * keys_per_part;
    const uint32_t t_stop = t_first + keys_per_part < n_keys ? t_first + keys_per_part : n_keys;
    const uint32_t row_u4 = kv_stride >> 3;
    // four lanes per key, the 16-byte pieces interleaved as in attention128_quant_kernel
    const uint32_t lane4 = tid & 3, key0 = t_first + (tid >> 2);
    const uint4 *qp = reinterpret_cast<const uint4 *>(q16 + size_t(head) * 128) + lane4;
    const uint4 *kbase = reinterpret_cast<const uint4 *>(k_cache + size_t(kvh) * 128) + lane4;
    uint4 qv[4], kk[4];
#pragma unroll
    for (int c = 0; c < 4; c++) qv[c] = qp[4 * c];
    {
        const uint4 *key = kbase + size_t(key0 < n_keys ? key0 : n_keys - 1) * row_u4;
#pragma unroll
        for (int c = 0; c < 4; c++) kk[c] = key[4 * c];
    }
    const float kq_scale = 1.0f / sqrtf(128.0f);  // two f32 roundings, as the reference computes it
    float my_max = -INFINITY;
    float *scores = ws.scores + size_t(head) * ws.score_stride;
    for (uint32_t t = key0; t - (tid >> 2) < t_stop; t += kAttnSplitThreads / 4) {
        const uint32_t tn = t + kAttnSplitThreads / 4;
        uint4 kn[4];  // the next round's keys, unconditionally (after the last round the last key again)
        {
            const uint4 *key = kbase + size_t(tn < n_keys ? tn : n_keys - 1) * row_u4;
#pragma unroll
            for (int c = 0; c < 4; c++) kn[c] = key[4 * c];
        }
        double s4[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const half8 kh = as_half8(kk[c]), qh = as_half8(qv[c]);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float prod = __builtin_fmaf(float(kh[j]), float(qh[j]), 0.0f);  // exact
                s4[c] += double(prod);
            }
        }
        const double sum = quad_sum((s4[0] + s4[1]) + (s4[2] + s4[3]));
        if (t < t_stop) {
            const float sc = float(sum) * kq_scale;
            if (lane4 == 0) scores[t] = sc;
            my_max = fmaxf(my_max, sc);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) kk[c] = kn[c];
    }
    my_max = wave_max_f32(my_max);
    if ((tid & 63) == 0) red_f[tid >> 6] = my_max;
    __syncthreads();
    if (tid == 0) {
        float m = red_f[0];
#pragma unroll
        for (uint32_t i = 1; i < kAttnSplitThreads / 64; i++) m = fmaxf(m, red_f[i]);
        ws.part_max[head * kAttnSplitMaxParts + part] = m;
    }
}

__global__ __launch_bounds__(kAttnSplitThreads) void attn128_weights_pv_kernel(
    const uint16_t *__restrict__ v_cache, uint32_t n_keys, uint32_t keys_per_part, uint32_t n_parts, uint32_t kv_stride,
    uint32_t n_head, uint32_t n_head_kv, AttnSplitScratch ws, int8_t *__restrict__ q8, float *__restrict__ scales,
    int rounding) {
    extern __shared__ double lds_d[];
    __shared__ float red_f[2];
    __shared__ uint64_t exp_tab[32];
    const uint32_t head = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    const uint32_t kvh = head / (n_head / n_head_kv);
    const uint32_t n_pad = (n_keys + kAttnPad - 1) / kAttnPad * kAttnPad;
    const uint32_t t_first = part * keys_per_part;
    const uint32_t t_stop = t_first + keys_per_part < n_keys ? t_first + keys_per_part : n_keys;
    double *wd = lds_d;                                       // [keys_per_part] this part's weights (f16 values)
    double *wave_sums = wd + keys_per_part;                   // [waves][128]
    float *e = reinterpret_cast<float *>(wave_sums + (kAttnSplitThreads / 64) * 128);  // [n_pad] exp(score - max), 0 beyond n_keys
    const uint32_t row_u4 = kv_stride >> 3;
    if (tid < 32) exp_tab[tid] = kRmiExp2fTab[tid];

    // values: lane = (8 dimensions dg, key slice sl) of this part's keys; the first loads go out now
    constexpr uint32_t kPre = 8;
    const uint32_t dg = tid & 15, sl = tid >> 4;
    const uint32_t n_mine = t_stop - t_first;
    const uint32_t chunk = (n_mine + kAttnSplitThreads / 16 - 1) / (kAttnSplitThreads / 16);
    const uint32_t t_begin = t_first + sl * chunk, t_end = t_begin + chunk < t_stop ? t_begin + chunk : t_stop;
    const uint4 *vbase = reinterpret_cast<const uint4 *>(v_cache + size_t(kvh) * 128 + dg * 8);
    uint4 vp[kPre];
#pragma unroll
    for (uint32_t j = 0; j < kPre; j++) {
        if (j < chunk) {
            const uint32_t t = t_begin + j < n_keys ? t_begin + j : n_keys - 1;
            vp[j] = vbase[size_t(t) * row_u4];
        }
    }
    // every score of the head, four per load and all loads out before the first is used: one memory round trip
    // (n_pad, a multiple of 64 and at most 16 384: more would not fit the LDS anyway)
    constexpr uint32_t kScoreLoads = 8;
    const float *scores = ws.scores + size_t(head) * ws.score_stride;
    float4 raw[kScoreLoads];
#pragma unroll
    for (uint32_t j = 0; j < kScoreLoads; j++) {
        if (j * kAttnSplitThreads * 4 < n_pad) {  // uniform; past the end the last group of four is read again
            const uint32_t t = (j * kAttnSplitThreads + tid) * 4;
            raw[j] = *reinterpret_cast<const float4 *>(scores + (t < n_pad ? t : n_pad - 4));
        }
    }
    float max_val = ws.part_max[head * kAttnSplitMaxParts];
    for (uint32_t i = 1; i < n_parts; i++) max_val = fmaxf(max_val, ws.part_max[head * kAttnSplitMaxParts + i]);
    __syncthreads();  // exp_tab
#pragma unroll
    for (uint32_t j = 0; j < kScoreLoads; j++) {
        const uint32_t t = (j * kAttnSplitThreads + tid) * 4;
        if (j * kAttnSplitThreads * 4 < n_pad && t < n_pad) {
            float4 ev;
            ev.x = t + 0 < n_keys ? rmi_expf_tab(raw[j].x - max_val, exp_tab) : 0.0f;
            ev.y = t + 1 < n_keys ? rmi_expf_tab(raw[j].y - max_val, exp_tab) : 0.0f;
            ev.z = t + 2 < n_keys ? rmi_expf_tab(raw[j].z - max_val, exp_tab) : 0.0f;
            ev.w = t + 3 < n_keys ? rmi_expf_tab(raw[j].w - max_val, exp_tab) : 0.0f;
            *reinterpret_cast<float4 *>(e + t) = ev;
        }
    }
    __syncthreads();
    if (tid == 0) {  // the reference adds the weights one after the other in f32; the padding zeros change nothing
        float acc = 0.0f;
        float4 a[8], b[8];
#pragma unroll
        for (int j = 0; j < 8; j++) a[j] = reinterpret_cast<const float4 *>(e)[j];
        for (uint32_t t = 0; t < n_pad; t += 64) {  // n_pad is a multiple of 64
#pragma unroll
            for (int j = 0; j < 8; j++) b[j] = reinterpret_cast<const float4 *>(e + t + 32)[j];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc += a[j].x;
                acc += a[j].y;
                acc += a[j].z;
                acc += a[j].w;
            }
            // unconditional (the array has 32 floats of room behind n_pad): under a branch the registers would be
            // copied every round, on the chain's own lane
#pragma unroll
            for (int j = 0; j < 8; j++) a[j] = reinterpret_cast<const float4 *>(e + t + 64)[j];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc += b[j].x;
                acc += b[j].y;
                acc += b[j].z;
                acc += b[j].w;
            }
        }
        red_f[0] = acc;
    }
    __syncthreads();
    const float total = red_f[0];
    for (uint32_t t = t_first + tid; t < t_stop; t += kAttnSplitThreads) {
        const float ev = e[t];
        wd[t - t_first] = double(h2f(f2h(total > 0.0f ? ev / total : ev)));
    }
    __syncthreads();

    double acc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = 0.0;
#pragma unroll
    for (uint32_t j = 0; j < kPre; j++) {
        if (t_begin + j < t_end) {
            const double w = wd[t_begin + j - t_first];
            const half8 vh = as_half8(vp[j]);
#pragma unroll
            for (int d = 0; d < 8; d++) acc[d] = __builtin_fma(double(float(vh[d])), w, acc[d]);
        }
    }
    if (t_begin + kPre < t_end) {  // longer slices: batches of 8 keys, the next one in flight while one is added
        uint4 cur[8], nxt[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            const uint32_t t = t_begin + kPre + j;
            cur[j] = vbase[size_t(t < n_keys ? t : n_keys - 1) * row_u4];
        }
        for (uint32_t t0 = t_begin + kPre; t0 < t_end; t0 += 8) {
#pragma unroll
            for (uint32_t j = 0; j < 8; j++) {
                const uint32_t t = t0 + 8 + j;
                nxt[j] = vbase[size_t(t < n_keys ? t : n_keys - 1) * row_u4];
            }
#pragma unroll
            for (uint32_t j = 0; j < 8; j++) {
                if (t0 + j < t_end) {
                    const double w = wd[t0 + j - t_first];
                    const half8 vh = as_half8(cur[j]);
#pragma unroll
                    for (int d = 0; d < 8; d++) acc[d] = __builtin_fma(double(float(vh[d])), w, acc[d]);
                }
            }
#pragma unroll
            for (uint32_t j = 0; j < 8; j++) cur[j] = nxt[j];
        }
    }
    {  // the four slices of a wave: lanes 16 apart
        double u[2];
        pv_slices_sum<16>(acc, u);
        double *dst = wave_sums + (tid >> 6) * 128 + dg * 8 + pv_dim_base(tid & 63);
        dst[0] = u[0];
        dst[1] = u[1];
    }
    __syncthreads();
    // The first wave alone hands the part's sums over: its stores, one release (the other waves have nothing in
    // flight that anybody reads), its count.  The part that counts last has every part's sums in reach after one
    // acquire, adds them in part order and quantizes.  Nobody waits for anybody.  The pair is written in its fence
    // form: an agent-scope fence in front of a relaxed counter update releases, the same fence behind the update that
    // read the last count acquires; the 64 storing lanes are one wave, whose fence covers the stores of all of them.
    // (An acq_rel update would put a second write-back in front of the acquire that nothing needs.)
    if (tid >= 64) return;
    double *mine = ws.part_sums + (size_t(head) * kAttnSplitMaxParts + part) * 128;
#pragma unroll
    for (uint32_t d = tid; d < 128; d += 64) {
        double o = wave_sums[d];
        for (uint32_t w = 1; w < kAttnSplitThreads / 64; w++) o += wave_sums[w * 128 + d];
        mine[d] = o;
    }
    __builtin_amdgcn_wave_barrier();  // the hand-over stays inside this one wave: its stores, then its fence, then its count
    __threadfence();
    uint32_t before = 0;
    if (tid == 0) before = __hip_atomic_fetch_add(ws.arrived + head, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = uint32_t(__builtin_amdgcn_readfirstlane(int(before)));
    if (before + 1 != n_parts) return;
    if (tid == 0) __hip_atomic_store(ws.arrived + head, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();
    if (tid < 32) {  // four dimensions per lane: whole 8-lane groups for the quantizer
        const double *all = ws.part_sums + size_t(head) * kAttnSplitMaxParts * 128 + tid * 4;
        double v[kAttnSplitMaxParts][4];  // every part's sums on their way before the first is added
#pragma unroll
        for (uint32_t p = 0; p < kAttnSplitMaxParts; p++) {
            if (p < n_parts) {
#pragma unroll
                for (int d = 0; d < 4; d++) v[p][d] = __builtin_nontemporal_load(all + p * 128 + d);
            }
        }
        double o[4] = {v[0][0], v[0][1], v[0][2], v[0][3]};
#pragma unroll
        for (uint32_t p = 1; p < kAttnSplitMaxParts; p++) {
            if (p < n_parts) {
#pragma unroll
                for (int d = 0; d < 4; d++) o[d] += v[p][d];
            }
        }
        const float4 of = make_float4(float(o[0]), float(o[1]), float(o[2]), float(o[3]));
        float sc;
        reinterpret_cast<uint32_t *>(q8)[(size_t(head) * 128 >> 2) + tid] = rmi_quantize_block8(of, rounding, &sc);
        if ((tid & 7) == 0) scales[(size_t(head) * 128 >> 5) + (tid >> 3)] = sc;
    }
}

// One position's attention straight from its f32 q | k | v: the launch with the p.v sums of a head split over parts.
// Four parts from 64 keys on (measured over 512..638 keys, 28 layers: 0.840 ms a generated token with one part, 0.789
// with two, 0.779 with four); below, the p.v sums are a few terms and one workgroup a head is enough.
static int attn_pv_parts(uint32_t n_keys) { return n_keys >= 64 ? 4 : 1; }
static void launch_attention128_from_qkv(const uint16_t *k_cache, const uint16_t *v_cache, uint32_t step, uint32_t kv_stride,
                                         uint32_t n_head, uint32_t n_head_kv, int8_t *q8, float *scales, int rounding,
                                         const AttnFromQkv &fq, hipStream_t st) {
    const size_t lds = attn128_lds_bytes(step + 1);
    const uint16_t *no_q16 = nullptr;
    switch (attn_pv_parts(step + 1)) {
    case 4:
        hipLaunchKernelGGL((attention128_quant_kernel<true, 4>), dim3(n_head * 4), dim3(kA128Threads), lds, st, no_q16, k_cache,
                           v_cache, step, kv_stride, n_head, n_head_kv, q8, scales, rounding, fq, 0u, 0u);
        break;
    default:
        hipLaunchKernelGGL((attention128_quant_kernel<true, 1>), dim3(n_head / n_head_kv, n_head_kv), dim3(kA128Threads), lds, st,
                           no_q16, k_cache, v_cache, step, kv_stride, n_head, n_head_kv, q8, scales, rounding, fq, 0u, 0u);
    }
}

// Dynamic LDS an attention launch may use: 64 KiB unless more has been asked for, which is done once, for both
// kernels; then what a compute unit has (160 KiB) less the kernels' static arrays (under 1 KiB).  With 12 bytes
// per key that is about 13 000 keys.
size_t attn_lds_limit() {
    static const size_t limit = [] {
        constexpr size_t kWant = 159 * 1024;
        const bool ok = hipFuncSetAttribute(reinterpret_cast<const void *>(attention128_quant_kernel<false>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, int(kWant)) == hipSuccess &&
                        hipFuncSetAttribute(reinterpret_cast<const void *>(attention_quant_kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, int(kWant)) == hipSuccess &&
                        hipFuncSetAttribute(reinterpret_cast<const void *>(attn128_weights_pv_kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, int(kWant)) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        return ok ? kWant : size_t(64 * 1024);
    }();
    return limit;
}

// From this many keys on a head's keys are split over workgroups (measured: below, the second launch and the
// hand-over through HBM cost more than the other compute units save; with four workgroups a head in the single
// launch the two meet between 1024 keys, 14.3 us against 14.7, and 1536, 18.6 against 17.2).
#ifndef RMI_ATTN_SPLIT_MIN_KEYS
#define RMI_ATTN_SPLIT_MIN_KEYS 1280
#endif
constexpr uint32_t kAttnSplitMinKeys = RMI_ATTN_SPLIT_MIN_KEYS;
inline bool attn128_use_split(uint32_t n_keys, uint32_t n_head);
// bytes of the scratch of one launch pair for n_head heads and up to max_keys keys, and its layout
inline uint32_t attn_split_score_stride(uint32_t max_keys) { return (max_keys + kAttnPad - 1) / kAttnPad * kAttnPad; }
constexpr uint32_t kAttnSplitMaxHeads = 1024;  // the arrival counters sit in front, wherever the head count puts the rest
inline size_t attn_split_scratch_bytes(uint32_t n_head, uint32_t max_keys) {
    return size_t(kAttnSplitMaxHeads) * 4 +
           size_t(n_head) * (size_t(attn_split_score_stride(max_keys)) * 4 + kAttnSplitMaxParts * 4 +
                             size_t(kAttnSplitMaxParts) * 128 * 8);
}
inline AttnSplitScratch attn_split_scratch_at(void *base, uint32_t n_head, uint32_t max_keys) {
    AttnSplitScratch ws;
    ws.score_stride = attn_split_score_stride(max_keys);
    uint8_t *p = static_cast<uint8_t *>(base);
    ws.arrived = reinterpret_cast<uint32_t *>(p);
    p += size_t(kAttnSplitMaxHeads) * 4;
    ws.part_sums = reinterpret_cast<double *>(p);
    p += size_t(n_head) * kAttnSplitMaxParts * 128 * 8;
    ws.scores = reinterpret_cast<float *>(p);
    p += size_t(n_head) * ws.score_stride * 4;
    ws.part_max = reinterpret_cast<float *>(p);
    return ws;
}
inline bool attn128_use_split(uint32_t n_keys, uint32_t n_head) {
    return n_keys >= kAttnSplitMinKeys && n_head <= kAttnSplitMaxHeads;
}
// keys 0..n_keys-1 of every head, split; ws.arrived must be zero (the launch leaves it zero)
int launch_attention128_split(const uint16_t *q16, const uint16_t *k_cache, const uint16_t *v_cache, uint32_t n_keys,
                              uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv, const AttnSplitScratch &ws,
                              int8_t *q8, float *scales, int rounding, hipStream_t st) {
    // about 256 keys a part (two rounds of the score loop), at most kAttnSplitMaxParts parts of whole 64-key groups
    uint32_t parts = (n_keys + 255) / 256;
    if (parts > kAttnSplitMaxParts) parts = kAttnSplitMaxParts;
    if (parts < 2) parts = 2;
    const uint32_t keys_per_part = ((n_keys + parts - 1) / parts + kAttnPad - 1) / kAttnPad * kAttnPad;
    parts = (n_keys + keys_per_part - 1) / keys_per_part;
    const size_t lds = attn128_split_lds_bytes(n_keys, keys_per_part);
    if (lds > attn_lds_limit() || n_keys > ws.score_stride || n_keys > 8 * kAttnSplitThreads * 4)
        return rmi_fail(RMI_HIP_E_INVALID, "%u keys exceed what the attention kernels hold", n_keys);
    hipLaunchKernelGGL(attn128_scores_kernel, dim3(n_head, parts), dim3(kAttnSplitThreads), 0, st, q16, k_cache, n_keys,
                       keys_per_part, kv_stride, n_head, n_head_kv, ws);
    hipLaunchKernelGGL(attn128_weights_pv_kernel, dim3(n_head, parts), dim3(kAttnSplitThreads), lds, st, v_cache, n_keys,
                       keys_per_part, parts, kv_stride, n_head, n_head_kv, ws, q8, scales, rounding);
    return RMI_HIP_OK;
}

// gu = [W_gate x ; W_up x]: h = (W_up x) * silu(W_gate x), quantized to Q8_0
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(const float *__restrict__ gu, uint32_t n_ff,
                                                             int8_t *__restrict__ q8, float *__restrict__ scales,
                                                             int rounding, uint32_t tok_gu_stride, uint32_t tok_q_stride) {
    gu += size_t(blockIdx.y) * tok_gu_stride;  // token blockIdx.y of a launch over several
    q8 += size_t(blockIdx.y) * tok_q_stride;
    scales += size_t(blockIdx.y) * (tok_q_stride >> 5);
    const uint32_t i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n_ff) return;  // n_ff is a multiple of 32: whole 8-lane groups leave together
    const float4 g = *reinterpret_cast<const float4 *>(gu + i);
    const float4 u = *reinterpret_cast<const float4 *>(gu + n_ff + i);
    float4 h;
    h.x = u.x * (g.x / (1.0f + rmi_expf(-g.x)));
    h.y = u.y * (g.y / (1.0f + rmi_expf(-g.y)));
    h.z = u.z * (g.z / (1.0f + rmi_expf(-g.z)));
    h.w = u.w * (g.w / (1.0f + rmi_expf(-g.w)));
    float sc;
    reinterpret_cast<uint32_t *>(q8)[i >> 2] = rmi_quantize_block8(h, rounding, &sc);
    if ((threadIdx.x & 7) == 0) scales[i >> 5] = sc;
}

__global__ __launch_bounds__(256) void expf_kernel(const float *__restrict__ x, float *__restrict__ y, size_t n) {
    for (size_t i = blockIdx.x * size_t(256) + threadIdx.x; i < n; i += size_t(gridDim.x) * 256) y[i] = rmi_expf(x[i]);
}

// greedy_token: the first strict maximum, the second largest value, and whether every logit is finite
struct Top {
    float best, second;
    uint32_t id, finite;
};
__device__ __forceinline__ Top top_merge(const Top &a, const Top &b) {
    Top r;
    const bool a_first = a.best > b.best || (a.best == b.best && a.id < b.id);
    const Top &hi = a_first ? a : b, &lo = a_first ? b : a;
    r.best = hi.best;
    r.id = hi.id;
    r.second = fmaxf(fmaxf(hi.second, lo.second), lo.best);
    r.finite = a.finite & b.finite;
    return r;
}
__device__ __forceinline__ Top top_block_reduce(Top t, Top *sm) {
    sm[threadIdx.x] = t;
    __syncthreads();
    for (uint32_t s = blockDim.x >> 1; s > 0; s >>= 1) {
        if (threadIdx.x < s) sm[threadIdx.x] = top_merge(sm[threadIdx.x], sm[threadIdx.x + s]);
        __syncthreads();
    }
    return sm[0];
}
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *__restrict__ logits, uint32_t n,
                                                             Top *__restrict__ partial) {
    __shared__ Top sm[256];
    logits += size_t(blockIdx.y) * n;  // token blockIdx.y of a launch over several: its logits, its partial results
    partial += size_t(blockIdx.y) * gridDim.x;
    Top t{-INFINITY, -INFINITY, 0xffffffffu, 1u};
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float l = logits[i];
        if (!(fabsf(l) <= 3.4028234663852886e38f)) t.finite = 0;  // NaN or inf
        if (l > t.best) {
            t.second = t.best;
            t.best = l;
            t.id = i;
        } else if (l > t.second) {
            t.second = l;
        }
    }
    const Top r = top_block_reduce(t, sm);
    if (threadIdx.x == 0) partial[blockIdx.x] = r;
}
__global__ __launch_bounds__(256) void argmax_final_kernel(const Top *__restrict__ partial, uint32_t n_partial,
                                                           StepParams *__restrict__ sp,
                                                           uint32_t *__restrict__ tok, uint32_t *__restrict__ step_argmax,
                                                           float *__restrict__ step_top2,
                                                           uint32_t *__restrict__ nonfinite_steps,
                                                           const uint8_t *__restrict__ w_embd, uint32_t n_oct,
                                                           uint32_t vocab, float *__restrict__ x, uint32_t n_embd) {
    __shared__ Top sm[256];
    __shared__ uint32_t next_token;
    Top t{-INFINITY, -INFINITY, 0xffffffffu, 1u};
    for (uint32_t i = threadIdx.x; i < n_partial; i += 256) t = top_merge(t, partial[i]);
    const Top r = top_block_reduce(t, sm);
    if (threadIdx.x == 0) {
        const uint32_t step = sp->step, n_prompt = sp->n_prompt;
        step_argmax[step] = r.id;
        step_top2[2 * step] = r.best;
        step_top2[2 * step + 1] = r.second;
        if (!r.finite) atomicAdd(nonfinite_steps, 1u);
        if (step + 1 >= n_prompt) tok[step + 1] = r.id;  // the next step's token
        next_token = step + 1 >= n_prompt ? r.id : tok[step + 1];
        sp->step = step + 1;  // last kernel of the step: the next one sees the new position
    }
    __syncthreads();
    embed_row(w_embd, n_oct, next_token, vocab, x, n_embd);  // the next step starts from its token's embedding
}

// ---- several prompt positions in one pass (rmi_hip_qwen3_generate while the tokens are known in advance)
// the embeddings of the prompt tokens step0 .. step0 + gridDim.x - 1, n_embd apart
__global__ __launch_bounds__(256) void embed_batch_kernel(const uint8_t *__restrict__ w, uint32_t n_oct,
                                                          const uint32_t *__restrict__ tok, uint32_t step0, uint32_t vocab,
                                                          float *__restrict__ x, uint32_t n_embd) {
    embed_row(w, n_oct, tok[step0 + blockIdx.x], vocab, x + size_t(blockIdx.x) * n_embd, n_embd);
}
// argmax_final_kernel for position step0 + blockIdx.x of such a pass; the workgroup of the pass's last position also
// advances the step counter and leaves the next token's embedding where a single step starts from
__global__ __launch_bounds__(256) void argmax_final_batch_kernel(const Top *__restrict__ partial, uint32_t n_partial,
                                                                 StepParams *__restrict__ sp, uint32_t step0,
                                                                 uint32_t *__restrict__ tok, uint32_t *__restrict__ step_argmax,
                                                                 float *__restrict__ step_top2,
                                                                 uint32_t *__restrict__ nonfinite_steps,
                                                                 const uint8_t *__restrict__ w_embd, uint32_t n_oct,
                                                                 uint32_t vocab, float *__restrict__ x, uint32_t n_embd) {
    __shared__ Top sm[256];
    __shared__ uint32_t next_token;
    partial += size_t(blockIdx.x) * n_partial;
    Top t{-INFINITY, -INFINITY, 0xffffffffu, 1u};
    for (uint32_t i = threadIdx.x; i < n_partial; i += 256) t = top_merge(t, partial[i]);
    const Top r = top_block_reduce(t, sm);
    const uint32_t step = step0 + blockIdx.x;
    if (threadIdx.x == 0) {
        const uint32_t n_prompt = sp->n_prompt;
        step_argmax[step] = r.id;
        step_top2[2 * step] = r.best;
        step_top2[2 * step + 1] = r.second;
        if (!r.finite) atomicAdd(nonfinite_steps, 1u);
        if (step + 1 >= n_prompt) tok[step + 1] = r.id;  // the next step's token
        next_token = step + 1 >= n_prompt ? r.id : tok[step + 1];
    }
    if (blockIdx.x + 1 != gridDim.x) return;
    if (threadIdx.x == 0) sp->step = step + 1;
    __syncthreads();
    embed_row(w_embd, n_oct, next_token, vocab, x, n_embd);
}

}  // namespace

// ------------------------------------------------------------------ session

struct rmi_hip_qwen3 {
    rmi_hip_qwen3_config cfg{};
    uint32_t n_q = 0, n_k = 0, n_v = 0, n_attn = 0, kv_stride = 0, max_n_in = 0;
    rmi_hip_weight *embd = nullptr, *head = nullptr;  // head == embd when tied
    std::vector<rmi_hip_weight *> w_qkv, w_o, w_gu, w_down;
    std::vector<float *> attn_norm, ffn_norm, q_norm, k_norm;
    float *output_norm = nullptr;
    float *cos_t = nullptr, *sin_t = nullptr;
    uint16_t *k_cache = nullptr, *v_cache = nullptr, *q16 = nullptr;
    float *x = nullptr, *x2 = nullptr, *resid = nullptr, *qkv = nullptr, *gu = nullptr, *logits = nullptr, *act_scales = nullptr;
    int8_t *act_q8 = nullptr;
    uint32_t *tok = nullptr, *step_argmax = nullptr, *nonfinite = nullptr;
    float *step_top2 = nullptr;
    void *partial = nullptr;
    // the same buffers for kPromptBatch positions at once (prompt passes), token-major
    float *xb = nullptr, *residb = nullptr, *qkvb = nullptr, *gub = nullptr, *logitsb = nullptr, *act_scalesb = nullptr;
    uint16_t *q16b = nullptr;
    int8_t *act_q8b = nullptr;
    void *partialb = nullptr;
    void *attn_split = nullptr;          // scratch of the split attention launches (head dimension 128)
    void *params = nullptr;              // StepParams in HBM
    std::vector<void *> owned;  // every other device allocation, freed with the session
    std::vector<uint32_t> stop_ids;  // generation ends before the first of these (EOS, im_end)
    uint32_t prompt_pass = 128;      // prompt positions per pass, 0 = every position its own step (rmi_hip_qwen3_set_prompt_passes)
};

namespace {

constexpr uint32_t kArgmaxGroups = 256;
constexpr uint32_t kPromptBatch = 128;  // most positions a prompt pass takes (the buffers' size); kPromptPassDefault is what it takes
constexpr uint32_t kPromptPassDefault = 128;

template <typename T>
T *dev_alloc(rmi_hip_qwen3 *s, size_t count, bool zero = false) {
    void *p = nullptr;
    if (hipMalloc(&p, count * sizeof(T) ? count * sizeof(T) : sizeof(T)) != hipSuccess) {
        rmi_set_error("hipMalloc of %zu bytes failed", count * sizeof(T));
        return nullptr;
    }
    s->owned.push_back(p);
    if (zero && hipMemset(p, 0, count * sizeof(T)) != hipSuccess) return nullptr;
    return static_cast<T *>(p);
}

float *upload_f32(rmi_hip_qwen3 *s, const float *host, size_t n) {
    float *d = dev_alloc<float>(s, n);
    if (d && hipMemcpy(d, host, n * 4, hipMemcpyHostToDevice) != hipSuccess) {
        rmi_set_error("hipMemcpy of a norm weight failed");
        return nullptr;
    }
    return d;
}

rmi_hip_weight *upload_stack(const uint8_t *const *parts, const uint32_t *rows, int n_parts, uint32_t n_in) {
    // the session's constructor waits once, after the last weight
    return rmi_upload_stack(RMI_HIP_DTYPE_Q8_0, parts, rows, n_parts, n_in, false);
}

int gemv(const rmi_hip_weight *w, const int8_t *q8, const float *scales, float *y, hipStream_t st) {
    RmiGemvProblem p{};
    p.w = w->data;
    p.x_q8 = q8;
    p.x_scales = scales;
    p.y = y;
    p.n_in = w->n_in;
    p.n_oct = w->n_units;
    p.y_stride = w->n_out;
    p.row_start = 0;
    p.row_end = w->n_out;
    p.tile0 = 0;
    p.n_tiles = w->n_tiles;
    return rmi_launch_gemv_q8_0_single(p, 1, st);
}

// One decoder step at position `step` (the host's copy of the counter in HBM, which the last kernel advances).
// Leaves logits, argmax and the next token on the device.
int enqueue_step(rmi_hip_qwen3 *s, uint32_t step, hipStream_t st) {
    const rmi_hip_qwen3_config &c = s->cfg;
    const int rnd = c.rounding;
    StepParams *sp = static_cast<StepParams *>(s->params);
    const size_t attn_lds = attn_lds_bytes(step + 1, c.head_dim_k, c.head_dim_v);
    if (step == 0)
        hipLaunchKernelGGL(embed_q8_0_kernel, dim3(1), dim3(256), 0, st, s->embd->data, s->embd->n_units, s->tok, sp, c.vocab,
                           s->x, c.n_embd);
    const float *pending = nullptr;  // matmul output still to be added to the residual stream
    // the residual stream alternates between two buffers where the norm is folded into the next product
    float *x = s->x, *x_other = s->x2;
    auto norm_gemv = [&](const rmi_hip_weight *w, const float *resid, const float *norm_weight, float *y) -> int {
        if (rmi_gemv_q8_0_norm_fusable(w)) {
            int rc = rmi_launch_gemv_q8_0_norm(w, x, resid, norm_weight, x_other, c.eps, rnd, y, st);
            std::swap(x, x_other);
            return rc;
        }
        launch_add_rmsnorm_quant(x, resid, norm_weight, c.n_embd, c.eps, s->act_q8, s->act_scales, rnd, st);
        return gemv(w, s->act_q8, s->act_scales, y, st);
    };
    for (uint32_t l = 0; l < c.n_layer; l++) {
        int rc;
        const size_t layer_base = size_t(l) * c.capacity * s->kv_stride, row = layer_base + size_t(step) * s->kv_stride;
        const float *qn = c.has_qk_norm ? s->q_norm[l] : nullptr, *kn = c.has_qk_norm ? s->k_norm[l] : nullptr;
        const bool d128 = c.head_dim_k == 128 && c.head_dim_v == 128;
        const bool split = d128 && s->attn_split && attn128_use_split(step + 1, c.n_head);
        // Short contexts: the q/k/v product as a plain GEMV behind the norm, one wave a tile over the whole chip, and
        // the head norms, the rotation and the cache row inside the attention launch.
        const bool qkv_in_attention = d128 && !split && rmi_gemv_q8_0_norm_fusable(s->w_qkv[l]) &&
                                      attn128_lds_bytes(step + 1) <= 48 * 1024;
        if (qkv_in_attention) {
            rc = norm_gemv(s->w_qkv[l], pending, s->attn_norm[l], s->qkv);
            if (rc != RMI_HIP_OK) return rc;
            const size_t half = 64;
            const AttnFromQkv fq{s->qkv, qn, kn, s->cos_t + size_t(step) * half, s->sin_t + size_t(step) * half,
                                 s->k_cache + row, s->v_cache + row, c.eps};
            launch_attention128_from_qkv(s->k_cache + layer_base, s->v_cache + layer_base, step, s->kv_stride, c.n_head, c.n_head_kv,
                                         s->act_q8, s->act_scales, rnd, fq, st);
        } else if (rmi_gemv_q8_0_norm_rope_fusable(s->w_qkv[l], c.n_head, c.n_head_kv, c.head_dim_k, c.head_dim_v)) {
            // norm, q/k/v products, head norms, rotation and the cache row in one launch
            const size_t half = c.head_dim_k / 2;
            rc = rmi_launch_gemv_q8_0_norm_rope(s->w_qkv[l], x, pending, s->attn_norm[l], x_other, c.eps, rnd, qn, kn,
                                                s->cos_t + size_t(step) * half, s->sin_t + size_t(step) * half, s->q16,
                                                s->k_cache + row, s->v_cache + row, c.n_head, c.n_head_kv, st);
            std::swap(x, x_other);
            if (rc != RMI_HIP_OK) return rc;
        } else {
            rc = norm_gemv(s->w_qkv[l], pending, s->attn_norm[l], s->qkv);
            if (rc != RMI_HIP_OK) return rc;
            hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3(c.n_head + 2 * c.n_head_kv), dim3(64), 0, st, s->qkv, qn, kn,
                               s->cos_t, s->sin_t, step, s->q16, s->k_cache + row, s->v_cache + row, c.n_head,
                               c.n_head_kv, c.head_dim_k, c.head_dim_v, c.eps, TokStride3{0, 0, 0});
        }
        if (qkv_in_attention) {
            // done above
        } else if (split) {
            rc = launch_attention128_split(s->q16, s->k_cache + layer_base, s->v_cache + layer_base, step + 1, s->kv_stride,
                                           c.n_head, c.n_head_kv, attn_split_scratch_at(s->attn_split, c.n_head, c.capacity),
                                           s->act_q8, s->act_scales, rnd, st);
            if (rc != RMI_HIP_OK) return rc;
        } else if (d128)
            hipLaunchKernelGGL(attention128_quant_kernel<false>, dim3(c.n_head / c.n_head_kv, c.n_head_kv), dim3(kA128Threads), attn128_lds_bytes(step + 1),
                               st, s->q16, s->k_cache + layer_base, s->v_cache + layer_base, step, s->kv_stride,
                               c.n_head, c.n_head_kv, s->act_q8, s->act_scales, rnd, AttnFromQkv{}, 0u, 0u);
        else
            hipLaunchKernelGGL(attention_quant_kernel, dim3(c.n_head), dim3(kAttnThreads), attn_lds, st, s->q16,
                               s->k_cache + layer_base, s->v_cache + layer_base, step, s->kv_stride, c.n_head,
                               c.n_head_kv, c.head_dim_k, c.head_dim_v, s->act_q8, s->act_scales, rnd);
        rc = gemv(s->w_o[l], s->act_q8, s->act_scales, s->resid, st);
        if (rc != RMI_HIP_OK) return rc;
        if (rmi_gemv_q8_0_norm_silu_fusable(s->w_gu[l])) {  // norm, gate/up products and SiLU*up in one launch
            rc = rmi_launch_gemv_q8_0_norm_silu(s->w_gu[l], x, s->resid, s->ffn_norm[l], x_other, c.eps, rnd, s->act_q8,
                                                s->act_scales, st);
            std::swap(x, x_other);
        } else {
            rc = norm_gemv(s->w_gu[l], s->resid, s->ffn_norm[l], s->gu);
            hipLaunchKernelGGL(silu_mul_quant_kernel, dim3((c.n_ff + 1023) / 1024), dim3(256), 0, st, s->gu, c.n_ff,
                               s->act_q8, s->act_scales, rnd, 0u, 0u);
        }
        if (rc != RMI_HIP_OK) return rc;
        rc = gemv(s->w_down[l], s->act_q8, s->act_scales, s->resid, st);
        if (rc != RMI_HIP_OK) return rc;
        pending = s->resid;
    }
    int rc = norm_gemv(s->head, pending, s->output_norm, s->logits);
    if (rc != RMI_HIP_OK) return rc;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(kArgmaxGroups), dim3(256), 0, st, s->logits, c.vocab,
                       static_cast<Top *>(s->partial));
    hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, st, static_cast<const Top *>(s->partial),
                       kArgmaxGroups, sp, s->tok, s->step_argmax, s->step_top2, s->nonfinite, s->embd->data,
                       s->embd->n_units, c.vocab, s->x, c.n_embd);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// Whether the prompt positions step0 .. step0 + n - 1 can go through one pass: head dimension 128, every launch
// of the pass within what the single-workgroup attention kernel holds, and short of the split's first position.
bool prompt_pass_possible(const rmi_hip_qwen3 *s, uint32_t step0, uint32_t n) {
    const rmi_hip_qwen3_config &c = s->cfg;
    if (!s->xb || n == 0 || n > kPromptBatch) return false;
    if (c.n_embd > kNormMaxN) return false;
    if (s->attn_split && attn128_use_split(step0 + n, c.n_head)) return false;
    return attn128_lds_bytes(step0 + n) <= 64 * 1024;
}

// n consecutive prompt positions from step0 on in one pass: every product reads its weight once for all of them
// (the x86-64-order GEMV takes up to eight tokens a launch and gives each the bits it gets alone), the other
// kernels run once per position inside one launch.  Position by position the arithmetic is that of enqueue_step's
// separate-kernel path; a position's keys and values are in the cache before any attention launch of the pass
// reads them.  Leaves every position's argmax and top-2 logits, the logits in logitsb, and, behind the last
// position, the step counter and the next token's embedding as a single step expects them.
int enqueue_prompt_pass(rmi_hip_qwen3 *s, uint32_t step0, uint32_t n, hipStream_t st) {
    const rmi_hip_qwen3_config &c = s->cfg;
    const int rnd = c.rounding;
    StepParams *sp = static_cast<StepParams *>(s->params);
    const uint32_t n_qkv = s->n_q + s->n_k + s->n_v;
    hipLaunchKernelGGL(embed_batch_kernel, dim3(n), dim3(256), 0, st, s->embd->data, s->embd->n_units, s->tok, step0, c.vocab,
                       s->xb, c.n_embd);
    const float *pending = nullptr;  // matmul output still to be added to the residual stream
    uint32_t pending_stride = 0;
    int rc;
    for (uint32_t l = 0; l < c.n_layer; l++) {
        const size_t layer_base = size_t(l) * c.capacity * s->kv_stride, row = layer_base + size_t(step0) * s->kv_stride;
        const float *qn = c.has_qk_norm ? s->q_norm[l] : nullptr, *kn = c.has_qk_norm ? s->k_norm[l] : nullptr;
        launch_add_rmsnorm_quant(s->xb, pending, s->attn_norm[l], c.n_embd, c.eps, s->act_q8b, s->act_scalesb, rnd, st, n,
                                 TokStride3{c.n_embd, pending_stride, c.n_embd});
        rc = rmi_gemv_q8_0_tokens(s->w_qkv[l], s->act_q8b, s->act_scalesb, s->qkvb, n, n_qkv, 0, n_qkv, st);
        if (rc != RMI_HIP_OK) return rc;
        hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3(c.n_head + 2 * c.n_head_kv, n), dim3(64), 0, st, s->qkvb, qn, kn,
                           s->cos_t, s->sin_t, step0, s->q16b, s->k_cache + row, s->v_cache + row, c.n_head, c.n_head_kv,
                           c.head_dim_k, c.head_dim_v, c.eps, TokStride3{n_qkv, s->n_q, s->kv_stride});
        // (a pass ends short of the split's first position, far below the 64 KiB of LDS a launch may take unasked)
        hipLaunchKernelGGL((attention128_quant_kernel<false, 1, true>), dim3(c.n_head / c.n_head_kv, c.n_head_kv, n), dim3(kA128Threads),
                           attn128_lds_bytes(step0 + n), st, s->q16b, s->k_cache + layer_base, s->v_cache + layer_base, step0,
                           s->kv_stride, c.n_head, c.n_head_kv, s->act_q8b, s->act_scalesb, rnd, AttnFromQkv{}, s->n_q, s->n_attn);
        rc = rmi_gemv_q8_0_tokens(s->w_o[l], s->act_q8b, s->act_scalesb, s->residb, n, c.n_embd, 0, c.n_embd, st);
        if (rc != RMI_HIP_OK) return rc;
        launch_add_rmsnorm_quant(s->xb, s->residb, s->ffn_norm[l], c.n_embd, c.eps, s->act_q8b, s->act_scalesb, rnd, st, n,
                                 TokStride3{c.n_embd, c.n_embd, c.n_embd});
        rc = rmi_gemv_q8_0_tokens(s->w_gu[l], s->act_q8b, s->act_scalesb, s->gub, n, 2 * c.n_ff, 0, 2 * c.n_ff, st);
        if (rc != RMI_HIP_OK) return rc;
        hipLaunchKernelGGL(silu_mul_quant_kernel, dim3((c.n_ff + 1023) / 1024, n), dim3(256), 0, st, s->gub, c.n_ff, s->act_q8b,
                           s->act_scalesb, rnd, 2 * c.n_ff, c.n_ff);
        rc = rmi_gemv_q8_0_tokens(s->w_down[l], s->act_q8b, s->act_scalesb, s->residb, n, c.n_embd, 0, c.n_embd, st);
        if (rc != RMI_HIP_OK) return rc;
        pending = s->residb;
        pending_stride = c.n_embd;
    }
    launch_add_rmsnorm_quant(s->xb, pending, s->output_norm, c.n_embd, c.eps, s->act_q8b, s->act_scalesb, rnd, st, n,
                             TokStride3{c.n_embd, pending_stride, c.n_embd});
    rc = rmi_gemv_q8_0_tokens(s->head, s->act_q8b, s->act_scalesb, s->logitsb, n, c.vocab, 0, c.vocab, st);
    if (rc != RMI_HIP_OK) return rc;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(kArgmaxGroups, n), dim3(256), 0, st, s->logitsb, c.vocab,
                       static_cast<Top *>(s->partialb));
    hipLaunchKernelGGL(argmax_final_batch_kernel, dim3(n), dim3(256), 0, st, static_cast<const Top *>(s->partialb), kArgmaxGroups,
                       sp, step0, s->tok, s->step_argmax, s->step_top2, s->nonfinite, s->embd->data, s->embd->n_units, c.vocab,
                       s->x, c.n_embd);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

}  // namespace

extern "C" {

int rmi_hip_expf_dev(const float *x, float *y, size_t n, void *stream) {
    RMI_REQUIRE_INIT();
    if (n == 0) return RMI_HIP_OK;
    if (!x || !y) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    const size_t groups = (n + 255) / 256;
    hipLaunchKernelGGL(expf_kernel, dim3(uint32_t(groups < 4096 ? groups : 4096)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), x, y, n);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_hip_rms_norm_quantize_q8_0_dev(float *x, const float *residual, const float *weight, uint32_t n, float eps,
                                       int8_t *q8, float *scales, int rounding, void *stream) {
    RMI_REQUIRE_INIT();
    if (n == 0) return RMI_HIP_OK;
    if (n % 32 != 0) return rmi_fail(RMI_HIP_E_INVALID, "n=%u is not a multiple of 32", n);
    if (n > kNormMaxN) return rmi_fail(RMI_HIP_E_INVALID, "n=%u exceeds the %u elements the norm kernel holds", n, kNormMaxN);
    if (!x || !weight || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    launch_add_rmsnorm_quant(x, residual, weight, n, eps, q8, scales, rounding, static_cast<hipStream_t>(stream));
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_hip_rms_norm_gemv_q8_0_dev(const rmi_hip_weight *w, const float *x_in, const float *residual,
                                   const float *norm_weight, float eps, int rounding, float *x_out, float *y,
                                   void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (!x_in || !norm_weight || !x_out || !y || x_in == x_out) return rmi_fail(RMI_HIP_E_INVALID, "null or aliased pointer");
    return rmi_launch_gemv_q8_0_norm(w, x_in, residual, norm_weight, x_out, eps, rounding, y,
                                     static_cast<hipStream_t>(stream));
}

int rmi_hip_rms_norm_qkv_rope_q8_0_dev(const rmi_hip_weight *w_qkv, const float *x_in, const float *residual,
                                       const float *norm_weight, float eps, int rounding, float *x_out,
                                       const float *q_norm, const float *k_norm, const float *cos_row,
                                       const float *sin_row, uint16_t *q16, uint16_t *k_row, uint16_t *v_row,
                                       uint32_t n_head, uint32_t n_head_kv, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w_qkv || w_qkv->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (!x_in || !norm_weight || !x_out || !cos_row || !sin_row || !q16 || !k_row || !v_row || x_in == x_out)
        return rmi_fail(RMI_HIP_E_INVALID, "null or aliased pointer");
    if (n_head == 0 || n_head_kv == 0) return rmi_fail(RMI_HIP_E_INVALID, "bad head shape");
    return rmi_launch_gemv_q8_0_norm_rope(w_qkv, x_in, residual, norm_weight, x_out, eps, rounding, q_norm, k_norm,
                                          cos_row, sin_row, q16, k_row, v_row, n_head, n_head_kv,
                                          static_cast<hipStream_t>(stream));
}

int rmi_hip_rms_norm_ffn_gate_up_q8_0_dev(const rmi_hip_weight *w_gate_up, const float *x_in, const float *residual,
                                          const float *norm_weight, float eps, int rounding, float *x_out,
                                          int8_t *h_q8, float *h_scales, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w_gate_up || w_gate_up->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (!x_in || !norm_weight || !x_out || !h_q8 || !h_scales || x_in == x_out)
        return rmi_fail(RMI_HIP_E_INVALID, "null or aliased pointer");
    return rmi_launch_gemv_q8_0_norm_silu(w_gate_up, x_in, residual, norm_weight, x_out, eps, rounding, h_q8, h_scales,
                                          static_cast<hipStream_t>(stream));
}

int rmi_hip_silu_mul_quantize_q8_0_dev(const float *gate_up, uint32_t n_ff, int8_t *q8, float *scales, int rounding,
                                       void *stream) {
    RMI_REQUIRE_INIT();
    if (n_ff == 0) return RMI_HIP_OK;
    if (n_ff % 32 != 0) return rmi_fail(RMI_HIP_E_INVALID, "n_ff=%u is not a multiple of 32", n_ff);
    if (!gate_up || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    hipLaunchKernelGGL(silu_mul_quant_kernel, dim3((n_ff + 1023) / 1024), dim3(256), 0, static_cast<hipStream_t>(stream),
                       gate_up, n_ff, q8, scales, rounding, 0u, 0u);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_hip_qk_norm_rope_f16_dev(const float *qkv, const float *q_norm, const float *k_norm, const float *cos_row,
                                 const float *sin_row, uint16_t *q16, uint16_t *k_row, uint16_t *v_row, uint32_t n_head,
                                 uint32_t n_head_kv, uint32_t head_dim_k, uint32_t head_dim_v, float eps, void *stream) {
    RMI_REQUIRE_INIT();
    if (!qkv || !cos_row || !sin_row || !q16 || !k_row || !v_row) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    if (n_head == 0 || n_head_kv == 0 || head_dim_k % 2) return rmi_fail(RMI_HIP_E_INVALID, "bad head shape");
    hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3(n_head + 2 * n_head_kv), dim3(64), 0,
                       static_cast<hipStream_t>(stream), qkv, q_norm, k_norm, cos_row, sin_row, 0u, q16, k_row, v_row,
                       n_head, n_head_kv, head_dim_k, head_dim_v, eps, TokStride3{0, 0, 0});
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// The calling thread's scratch for the two-launch attention: sized for n_head heads and max_keys keys, counters zero.
constexpr int kAttnSplitSlot = 5;
constexpr uint32_t kAttnSplitReserveKeys = 16384;  // what the two launches hold at most: sized once for any context
static int attn_split_reserve(RmiThreadCtx *c, uint32_t n_head, uint32_t max_keys) {
    const size_t need = attn_split_scratch_bytes(n_head, max_keys);
    if (c->dev_cap[kAttnSplitSlot] >= need) return RMI_HIP_OK;
    void *fresh = rmi_dev_buf(c, kAttnSplitSlot, need);
    if (!fresh) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemset(fresh, 0, c->dev_cap[kAttnSplitSlot]));  // the arrival counters start at zero
    return RMI_HIP_OK;
}

int rmi_hip_attention_reserve(uint32_t n_head, uint32_t max_keys) {
    RMI_REQUIRE_INIT();
    if (n_head == 0 || n_head > kAttnSplitMaxHeads) return rmi_fail(RMI_HIP_E_INVALID, "1..%u heads", kAttnSplitMaxHeads);
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    (void)attn_lds_limit();  // the kernels' dynamic-LDS limit is raised here, too, not at the first launch
    RMI_HIP_CHECK(hipDeviceSynchronize());  // a launch of this thread may still use the region this call replaces
    return attn_split_reserve(c, n_head, max_keys < kAttnSplitReserveKeys ? kAttnSplitReserveKeys : max_keys);
}

int rmi_hip_attention_f16_quantize_q8_0_dev(const uint16_t *q16, const uint16_t *k_cache, const uint16_t *v_cache,
                                            uint32_t n_keys, uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv,
                                            uint32_t head_dim_k, uint32_t head_dim_v, int8_t *q8, float *scales,
                                            int rounding, void *stream) {
    RMI_REQUIRE_INIT();
    if (!q16 || !k_cache || !v_cache || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    if (n_keys == 0 || n_head == 0 || n_head_kv == 0 || n_head % n_head_kv || head_dim_k % 32 || head_dim_v % 32 ||
        head_dim_k == 0 || head_dim_v == 0 || head_dim_k > 1024 || head_dim_v > 1024 || kv_stride % 8)
        return rmi_fail(RMI_HIP_E_INVALID, "bad attention shape");
    const bool d128 = head_dim_k == 128 && head_dim_v == 128;
    if (d128 && attn128_use_split(n_keys, n_head)) {
        // The scratch of the two launches is the calling thread's (slot 5 of its staging buffers, never used by
        // the host-slice entry points): calls of one thread that overlap on different streams would share it.
        // rmi_hip_attention_reserve makes it ahead of time; without that call it is made here, once.  (What the two
        // launches hold in LDS is their own figure, checked where they are launched.)
        RmiThreadCtx *c = rmi_thread_ctx();
        if (!c) return RMI_HIP_E_RUNTIME;
        const uint32_t max_keys = n_keys < kAttnSplitReserveKeys ? kAttnSplitReserveKeys : n_keys;
        if (c->dev_cap[kAttnSplitSlot] < attn_split_scratch_bytes(n_head, max_keys)) {
            RMI_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));  // it may still read the old one
            const int rc = attn_split_reserve(c, n_head, max_keys);
            if (rc != RMI_HIP_OK) return rc;
        }
        const int rc = launch_attention128_split(q16, k_cache, v_cache, n_keys, kv_stride, n_head, n_head_kv,
                                                 attn_split_scratch_at(c->dev[kAttnSplitSlot], n_head, max_keys), q8, scales,
                                                 rounding, static_cast<hipStream_t>(stream));
        if (rc != RMI_HIP_OK) return rc;
        RMI_HIP_CHECK(hipGetLastError());
        return RMI_HIP_OK;
    }
    const size_t lds = d128 ? attn128_lds_bytes(n_keys) : attn_lds_bytes(n_keys, head_dim_k, head_dim_v);
    if (lds > attn_lds_limit()) return rmi_fail(RMI_HIP_E_INVALID, "%u keys exceed what the kernel holds in LDS", n_keys);
    if (d128 && attn_pv_parts(n_keys) == 4 && lds <= 64 * 1024)  // four workgroups a head, as in the session's own launch
        hipLaunchKernelGGL((attention128_quant_kernel<false, 4>), dim3(n_head * 4), dim3(kA128Threads), lds, static_cast<hipStream_t>(stream),
                           q16, k_cache, v_cache, n_keys - 1, kv_stride, n_head, n_head_kv, q8, scales, rounding, AttnFromQkv{}, 0u, 0u);
    else if (d128)
        hipLaunchKernelGGL(attention128_quant_kernel<false>, dim3(n_head / n_head_kv, n_head_kv), dim3(kA128Threads), lds, static_cast<hipStream_t>(stream),
                           q16, k_cache, v_cache, n_keys - 1, kv_stride, n_head, n_head_kv, q8, scales, rounding, AttnFromQkv{}, 0u, 0u);
    else
        hipLaunchKernelGGL(attention_quant_kernel, dim3(n_head), dim3(kAttnThreads), lds, static_cast<hipStream_t>(stream),
                           q16, k_cache, v_cache, n_keys - 1, kv_stride, n_head, n_head_kv, head_dim_k, head_dim_v, q8,
                           scales, rounding);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_hip_qkv_attention_f16_quantize_q8_0_dev(const float *qkv, const float *q_norm, const float *k_norm,
                                                const float *cos_row, const float *sin_row, uint16_t *k_cache,
                                                uint16_t *v_cache, uint32_t n_keys, uint32_t kv_stride, uint32_t n_head,
                                                uint32_t n_head_kv, float eps, int8_t *q8, float *scales, int rounding,
                                                void *stream) {
    RMI_REQUIRE_INIT();
    if (!qkv || !cos_row || !sin_row || !k_cache || !v_cache || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null pointer");
    if (n_keys == 0 || n_head == 0 || n_head_kv == 0 || n_head % n_head_kv || kv_stride % 8 || kv_stride < n_head_kv * 128)
        return rmi_fail(RMI_HIP_E_INVALID, "bad attention shape");
    const size_t lds = attn128_lds_bytes(n_keys);
    if (lds > 48 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "%u keys: beyond %u the rotation runs in its own launch "
                        "(rmi_hip_qk_norm_rope_f16_dev, then rmi_hip_attention_f16_quantize_q8_0_dev)", n_keys,
                        uint32_t((48 * 1024 - (kA128Threads / 64) * 128 * 8 - 128) / 12 / kAttnPad * kAttnPad));
    const size_t row = size_t(n_keys - 1) * kv_stride;
    const AttnFromQkv fq{qkv, q_norm, k_norm, cos_row, sin_row, k_cache + row, v_cache + row, eps};
    launch_attention128_from_qkv(k_cache, v_cache, n_keys - 1, kv_stride, n_head, n_head_kv, q8, scales, rounding, fq,
                                 static_cast<hipStream_t>(stream));
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

void rmi_hip_qwen3_destroy(rmi_hip_qwen3 *s) {
    if (!s) return;
    if (s->head && s->head != s->embd) rmi_hip_free_weight(s->head);
    if (s->embd) rmi_hip_free_weight(s->embd);
    for (auto *w : s->w_qkv) rmi_hip_free_weight(w);
    for (auto *w : s->w_o) rmi_hip_free_weight(w);
    for (auto *w : s->w_gu) rmi_hip_free_weight(w);
    for (auto *w : s->w_down) rmi_hip_free_weight(w);
    for (void *p : s->owned) (void)hipFree(p);
    delete s;
}

rmi_hip_qwen3 *rmi_hip_qwen3_create(const rmi_hip_qwen3_config *cfg, const rmi_hip_qwen3_weights *wt) {
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    if (!cfg || !wt || !wt->token_embd || !wt->output_norm) {
        rmi_set_error("null configuration or weights");
        return nullptr;
    }
    const rmi_hip_qwen3_config &c = *cfg;
    if (!wt->attn_norm || !wt->ffn_norm || !wt->wq || !wt->wk || !wt->wv || !wt->wo || !wt->w_gate || !wt->w_up ||
        !wt->w_down || (c.has_qk_norm && (!wt->q_norm || !wt->k_norm))) {
        rmi_set_error("null per-layer weight array");
        return nullptr;
    }
    for (uint32_t l = 0; l < c.n_layer; l++)
        if (!wt->attn_norm[l] || !wt->ffn_norm[l] || !wt->wq[l] || !wt->wk[l] || !wt->wv[l] || !wt->wo[l] ||
            !wt->w_gate[l] || !wt->w_up[l] || !wt->w_down[l] || (c.has_qk_norm && (!wt->q_norm[l] || !wt->k_norm[l]))) {
            rmi_set_error("null weights in layer %u", l);
            return nullptr;
        }
    // widths and cache rows are 32-bit in the kernels (the reference's checked_product, src/models/qwen3.rs:96-121)
    const uint64_t kMax32 = 0x7fffffffull;
    const uint64_t wide_q = uint64_t(c.n_head) * c.head_dim_k, wide_attn = uint64_t(c.n_head) * c.head_dim_v;
    const uint64_t wide_kv = uint64_t(c.n_head_kv) * (c.head_dim_k > c.head_dim_v ? c.head_dim_k : c.head_dim_v);
    if (wide_q > kMax32 || wide_attn > kMax32 || uint64_t(c.n_ff) * 2 > kMax32 || wide_q + 2 * wide_kv > kMax32 ||
        uint64_t(c.capacity) * wide_kv > 0xffffffffull ||
        uint64_t(c.n_layer) * c.capacity * wide_kv > (uint64_t(1) << 40)) {
        rmi_set_error("unsupported model shape: a width or the KV cache overflows");
        return nullptr;
    }
    if (c.n_embd == 0 || c.n_embd % 32 || c.n_ff == 0 || c.n_ff % 32 || c.n_layer == 0 || c.n_head == 0 ||
        c.n_head_kv == 0 || c.n_head % c.n_head_kv || c.head_dim_k == 0 || c.head_dim_k % 32 || c.head_dim_v == 0 ||
        c.head_dim_v % 32 || c.head_dim_k > 1024 || c.head_dim_v > 1024 || c.vocab == 0 || c.capacity == 0 ||
        c.n_embd > kNormMaxN ||
        (c.rounding != RMI_HIP_ROUND_TIES_EVEN && c.rounding != RMI_HIP_ROUND_HALF_AWAY && c.rounding != RMI_HIP_ROUND_NEON)) {
        rmi_set_error("unsupported model shape");
        return nullptr;
    }
    // attention keeps the scores of one head in LDS
    if ((c.head_dim_k == 128 && c.head_dim_v == 128 ? attn128_lds_bytes(c.capacity)
                                                    : attn_lds_bytes(c.capacity, c.head_dim_k, c.head_dim_v)) > attn_lds_limit()) {
        rmi_set_error("capacity %u exceeds what the attention kernel holds in LDS", c.capacity);
        return nullptr;
    }
    if (!rmi_thread_ctx()) return nullptr;
    rmi_hip_qwen3 *s = new rmi_hip_qwen3();
    s->cfg = c;
    s->n_q = c.n_head * c.head_dim_k;
    s->n_k = c.n_head_kv * c.head_dim_k;
    s->n_v = c.n_head_kv * c.head_dim_v;
    s->n_attn = c.n_head * c.head_dim_v;
    s->kv_stride = s->n_k > s->n_v ? s->n_k : s->n_v;
    s->max_n_in = c.n_embd;
    if (s->n_attn > s->max_n_in) s->max_n_in = s->n_attn;
    if (c.n_ff > s->max_n_in) s->max_n_in = c.n_ff;
    bool ok = true;
    {
        const uint32_t rows[1] = {c.vocab};
        const uint8_t *parts[1] = {wt->token_embd};
        ok = ok && (s->embd = upload_stack(parts, rows, 1, c.n_embd));
        if (ok && wt->output) {
            parts[0] = wt->output;
            ok = ok && (s->head = upload_stack(parts, rows, 1, c.n_embd));
        } else {
            s->head = s->embd;
        }
    }
    ok = ok && (s->output_norm = upload_f32(s, wt->output_norm, c.n_embd));
    for (uint32_t l = 0; ok && l < c.n_layer; l++) {
        const uint8_t *qkv[3] = {wt->wq[l], wt->wk[l], wt->wv[l]};
        const uint32_t qkv_rows[3] = {s->n_q, s->n_k, s->n_v};
        const uint8_t *gu[2] = {wt->w_gate[l], wt->w_up[l]};
        const uint32_t gu_rows[2] = {c.n_ff, c.n_ff};
        const uint8_t *o[1] = {wt->wo[l]}, *dn[1] = {wt->w_down[l]};
        const uint32_t o_rows[1] = {c.n_embd};
        rmi_hip_weight *w;
        ok = ok && (w = upload_stack(qkv, qkv_rows, 3, c.n_embd));
        if (ok) s->w_qkv.push_back(w);
        ok = ok && (w = upload_stack(o, o_rows, 1, s->n_attn));
        if (ok) s->w_o.push_back(w);
        ok = ok && (w = upload_stack(gu, gu_rows, 2, c.n_embd));
        if (ok) s->w_gu.push_back(w);
        ok = ok && (w = upload_stack(dn, o_rows, 1, c.n_ff));
        if (ok) s->w_down.push_back(w);
        float *f;
        ok = ok && (f = upload_f32(s, wt->attn_norm[l], c.n_embd));
        if (ok) s->attn_norm.push_back(f);
        ok = ok && (f = upload_f32(s, wt->ffn_norm[l], c.n_embd));
        if (ok) s->ffn_norm.push_back(f);
        if (ok && c.has_qk_norm) {
            ok = ok && (f = upload_f32(s, wt->q_norm[l], c.head_dim_k));
            if (ok) s->q_norm.push_back(f);
            ok = ok && (f = upload_f32(s, wt->k_norm[l], c.head_dim_k));
            if (ok) s->k_norm.push_back(f);
        }
    }
    if (ok) {  // rope_neox angles, with the host libm as the reference's CPU path uses it (src/ops/rope.rs:21-37)
        const uint32_t half = c.head_dim_k / 2;
        std::vector<float> ct(size_t(c.capacity) * half), stv(size_t(c.capacity) * half);
        const float theta_scale = powf(c.freq_base, -2.0f / float(c.head_dim_k));
        for (uint32_t pos = 0; pos < c.capacity; pos++) {
            float theta = float(pos);
            for (uint32_t i = 0; i < half; i++) {
                ct[size_t(pos) * half + i] = cosf(theta);
                stv[size_t(pos) * half + i] = sinf(theta);
                theta *= theta_scale;
            }
        }
        ok = ok && (s->cos_t = upload_f32(s, ct.data(), ct.size())) && (s->sin_t = upload_f32(s, stv.data(), stv.size()));
    }
    const size_t cache = size_t(c.n_layer) * c.capacity * s->kv_stride;
    ok = ok && (s->k_cache = dev_alloc<uint16_t>(s, cache, true)) && (s->v_cache = dev_alloc<uint16_t>(s, cache, true)) &&
         (s->q16 = dev_alloc<uint16_t>(s, s->n_q)) && (s->x = dev_alloc<float>(s, c.n_embd)) && (s->x2 = dev_alloc<float>(s, c.n_embd)) &&
         (s->resid = dev_alloc<float>(s, c.n_embd)) && (s->qkv = dev_alloc<float>(s, size_t(s->n_q) + s->n_k + s->n_v)) &&
         (s->gu = dev_alloc<float>(s, size_t(2) * c.n_ff)) && (s->logits = dev_alloc<float>(s, c.vocab)) &&
         (s->act_q8 = dev_alloc<int8_t>(s, s->max_n_in)) && (s->act_scales = dev_alloc<float>(s, s->max_n_in / 32)) &&
         (s->tok = dev_alloc<uint32_t>(s, size_t(c.capacity) + 1, true)) &&
         (s->step_argmax = dev_alloc<uint32_t>(s, c.capacity, true)) &&
         (s->step_top2 = dev_alloc<float>(s, size_t(2) * c.capacity, true)) &&
         (s->nonfinite = dev_alloc<uint32_t>(s, 1, true)) && (s->partial = dev_alloc<Top>(s, kArgmaxGroups)) &&
         (s->params = dev_alloc<StepParams>(s, 1, true));
    if (ok && c.head_dim_k == 128 && c.head_dim_v == 128)  // prompt passes of kPromptBatch positions (head dimension 128)
        ok = (s->xb = dev_alloc<float>(s, size_t(kPromptBatch) * c.n_embd)) &&
             (s->residb = dev_alloc<float>(s, size_t(kPromptBatch) * c.n_embd)) &&
             (s->qkvb = dev_alloc<float>(s, size_t(kPromptBatch) * (size_t(s->n_q) + s->n_k + s->n_v))) &&
             (s->q16b = dev_alloc<uint16_t>(s, size_t(kPromptBatch) * s->n_q)) &&
             (s->gub = dev_alloc<float>(s, size_t(kPromptBatch) * 2 * c.n_ff)) &&
             (s->logitsb = dev_alloc<float>(s, size_t(kPromptBatch) * c.vocab)) &&
             (s->act_q8b = dev_alloc<int8_t>(s, size_t(kPromptBatch) * s->max_n_in)) &&
             (s->act_scalesb = dev_alloc<float>(s, size_t(kPromptBatch) * s->max_n_in / 32)) &&
             (s->partialb = dev_alloc<Top>(s, size_t(kPromptBatch) * kArgmaxGroups));
    if (ok && c.head_dim_k == 128 && c.head_dim_v == 128 && attn128_use_split(c.capacity, c.n_head))
        ok = (s->attn_split = dev_alloc<uint8_t>(s, attn_split_scratch_bytes(c.n_head, c.capacity), true)) != nullptr;
    if (ok && hipStreamSynchronize(rmi_thread_ctx()->stream) != hipSuccess) {  // the uploads enqueued above
        rmi_set_error("weight upload failed");
        ok = false;
    }
    if (!ok) {
        rmi_hip_qwen3_destroy(s);
        return nullptr;
    }
    return s;
}

int rmi_hip_qwen3_generate(rmi_hip_qwen3 *s, const uint32_t *prompt, uint32_t n_prompt, uint32_t max_new,
                           uint32_t *generated, uint32_t *step_argmax, float *step_top2, const uint32_t *dump_steps,
                           uint32_t n_dump, float *dump_logits, double *seconds) {
    RMI_REQUIRE_INIT();
    if (!s || !prompt || n_prompt == 0 || (max_new && !generated))
        return rmi_fail(RMI_HIP_E_INVALID, "null session, prompt or output");
    const rmi_hip_qwen3_config &c = s->cfg;
    if (size_t(n_prompt) + max_new > c.capacity)
        return rmi_fail(RMI_HIP_E_INVALID, "%u prompt + %u new tokens exceed the capacity %u", n_prompt, max_new,
                        c.capacity);
    for (uint32_t i = 0; i < n_prompt; i++)
        if (prompt[i] >= c.vocab) return rmi_fail(RMI_HIP_E_INVALID, "token id %u outside the vocabulary", prompt[i]);
    RmiThreadCtx *ctx = rmi_thread_ctx();
    if (!ctx) return RMI_HIP_E_RUNTIME;
    hipStream_t st = ctx->stream;
    const uint32_t steps = n_prompt + max_new - 1;
    float *d_dump = nullptr;
    if (n_dump) {
        if (!dump_steps || !dump_logits) return rmi_fail(RMI_HIP_E_INVALID, "null dump arrays");
        RMI_HIP_CHECK(hipMalloc(reinterpret_cast<void **>(&d_dump), size_t(n_dump) * c.vocab * 4));
    }
    int rc = RMI_HIP_OK;
    const StepParams start{0u, n_prompt};
    hipError_t e = hipMemcpyAsync(s->tok, prompt, size_t(n_prompt) * 4, hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipMemcpyAsync(s->params, &start, sizeof start, hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipMemsetAsync(s->nonfinite, 0, 4, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    const auto t0 = std::chrono::steady_clock::now();
    // Without stop ids every step is enqueued at once.  With them the host looks at the tokens every
    // kStopCheck generated steps (one small copy) and ends the run at the first stop id, which is not part of
    // the result (src/models/qwen3.rs:1123-1130: the loop breaks before the token is pushed).
    constexpr uint32_t kStopCheck = 32;
    const bool stops = !s->stop_ids.empty() && max_new > 0;
    uint32_t n_valid = max_new, steps_done = 0, checked = 0;
    std::vector<uint32_t> seen(stops ? max_new : 0);
    while (e == hipSuccess && rc == RMI_HIP_OK && steps_done < steps) {
        uint32_t until = steps;
        if (stops) {
            const uint32_t base = steps_done < n_prompt - 1 ? n_prompt - 1 : steps_done;
            until = steps - base > kStopCheck ? base + kStopCheck : steps;
        }
        for (uint32_t step = steps_done; e == hipSuccess && rc == RMI_HIP_OK && step < until;) {
            // prompt positions go eight to a pass while they can (their tokens are known); the rest step by step
            uint32_t n = step < n_prompt ? n_prompt - step : 0;
            if (n > s->prompt_pass) n = s->prompt_pass;
            if (n > until - step) n = until - step;
            if (n > 1 && prompt_pass_possible(s, step, n)) {
                rc = enqueue_prompt_pass(s, step, n, st);
                for (uint32_t d = 0; rc == RMI_HIP_OK && d < n_dump; d++)
                    if (dump_steps[d] >= step && dump_steps[d] < step + n)
                        e = hipMemcpyAsync(d_dump + size_t(d) * c.vocab, s->logitsb + size_t(dump_steps[d] - step) * c.vocab,
                                           size_t(c.vocab) * 4, hipMemcpyDeviceToDevice, st);
                step += n;
                continue;
            }
            rc = enqueue_step(s, step, st);
            for (uint32_t d = 0; rc == RMI_HIP_OK && d < n_dump; d++)
                if (dump_steps[d] == step)
                    e = hipMemcpyAsync(d_dump + size_t(d) * c.vocab, s->logits, size_t(c.vocab) * 4, hipMemcpyDeviceToDevice, st);
            step++;
        }
        steps_done = until;
        if (!stops || e != hipSuccess || rc != RMI_HIP_OK) continue;
        const uint32_t have = steps_done - (n_prompt - 1);  // tokens sampled so far
        e = hipStreamSynchronize(st);
        if (e == hipSuccess && have > checked)
            e = hipMemcpy(seen.data() + checked, s->tok + n_prompt + checked, size_t(have - checked) * 4, hipMemcpyDeviceToHost);
        bool hit = false;
        for (; e == hipSuccess && checked < have && !hit; checked++)
            for (uint32_t id : s->stop_ids)
                if (seen[checked] == id) {
                    n_valid = checked;
                    hit = true;
                    break;
                }
        if (hit) break;
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (seconds) *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    uint32_t nonfinite = 0;
    if (e == hipSuccess && rc == RMI_HIP_OK) {
        if (n_valid) e = hipMemcpy(generated, s->tok + n_prompt, size_t(n_valid) * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess && step_argmax) e = hipMemcpy(step_argmax, s->step_argmax, size_t(steps_done) * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess && step_top2) e = hipMemcpy(step_top2, s->step_top2, size_t(steps_done) * 8, hipMemcpyDeviceToHost);
        if (e == hipSuccess && n_dump) e = hipMemcpy(dump_logits, d_dump, size_t(n_dump) * c.vocab * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(&nonfinite, s->nonfinite, 4, hipMemcpyDeviceToHost);
    }
    if (d_dump) (void)hipFree(d_dump);
    if (rc != RMI_HIP_OK) return rc;
    if (e != hipSuccess) return rmi_fail(RMI_HIP_E_RUNTIME, "decode failed: %s", hipGetErrorString(e));
    if (nonfinite) return rmi_fail(RMI_HIP_E_RUNTIME, "non-finite logits in %u steps", nonfinite);
    return int(n_valid);
}

int rmi_hip_qwen3_set_prompt_passes(rmi_hip_qwen3 *s, int enabled) {
    if (!s) return rmi_fail(RMI_HIP_E_INVALID, "null session");
    // 0: off; 1: the default size; more: that many positions a pass, up to the buffers' size
    s->prompt_pass = enabled <= 0 ? 0u : enabled == 1 ? kPromptPassDefault : uint32_t(enabled) < kPromptBatch ? uint32_t(enabled) : kPromptBatch;
    return RMI_HIP_OK;
}

int rmi_hip_qwen3_set_stop_ids(rmi_hip_qwen3 *s, const uint32_t *ids, uint32_t n_ids) {
    if (!s || (n_ids && !ids)) return rmi_fail(RMI_HIP_E_INVALID, "null session or ids");
    if (n_ids > 16) return rmi_fail(RMI_HIP_E_INVALID, "at most 16 stop ids");
    s->stop_ids.assign(ids, ids + n_ids);
    return RMI_HIP_OK;
}

}  // extern "C"
