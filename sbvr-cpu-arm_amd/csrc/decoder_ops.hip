// Small single-token kernels around the SBVR linears of a Llama-shaped decoder:
// residual add + RMSNorm, rotary embedding + cache append + attention of one
// query over the cache, SiLU(gate) * up.  They exist so that a decode step is a
// short chain of launches (8 per layer) instead of dozens of elementwise ops;
// the arithmetic follows models/sbvr_llama.py of the reference:
//   LlamaRMSNorm.forward            :118-123  (fp32 statistics, weight * x.to(fp16))
//   rotate_half / apply_rotary...   :193-224  (q*cos + rotate_half(q)*sin)
//   eager_attention_forward         :255-278  (softmax in fp32, weights rounded to fp16)
//   LlamaMLP.forward                :238-240  (act_fn(gate) * up in fp16)
// gfx950 only.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sbvr_hip_decoder.h"

namespace {

__device__ __forceinline__ float h2f(uint16_t h)
{
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return static_cast<float>(v);
}

__device__ __forceinline__ uint16_t f2h(float f)
{
    const _Float16 v = static_cast<_Float16>(f);
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

constexpr int kNormThreads = 1024;
constexpr int kAttnThreads = 256;

// sum (or max) over the workgroup; every thread gets the result
template <bool IsMax>
__device__ __forceinline__ float block_reduce(float v, float *scratch)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, 64);
        v = IsMax ? fmaxf(v, o) : v + o;
    }
    const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    __syncthreads();                   // scratch may still be read from an earlier call
    if ((threadIdx.x & 63) == 0)
        scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int w = 1; w < waves; ++w)
        r = IsMax ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

// x <- fp16(x + delta) (delta may be null), h <- weight * fp16(x * rsqrt(mean(x^2) + eps)).
// A thread keeps its elements (pairs, up to kNormPairs of them) in registers between the two passes.
constexpr int kNormPairs = 4;

__global__ void __launch_bounds__(kNormThreads)
add_rmsnorm_kernel(uint16_t *x, const uint16_t *delta, const uint16_t *weight, uint16_t *h, int n, float eps)
{
    __shared__ float scratch[kNormThreads / 64];
    const int pairs = n >> 1;                       // n is even (checked by the caller)
    uint32_t *x2 = reinterpret_cast<uint32_t *>(x);
    const uint32_t *d2 = reinterpret_cast<const uint32_t *>(delta);
    const uint32_t *w2 = reinterpret_cast<const uint32_t *>(weight);
    uint32_t *h2 = reinterpret_cast<uint32_t *>(h);
    float v0[kNormPairs], v1[kNormPairs];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kNormPairs; ++j) {
        const int i = threadIdx.x + j * kNormThreads;
        v0[j] = v1[j] = 0.f;
        if (i < pairs) {
            const uint32_t xv = x2[i];
            v0[j] = h2f(static_cast<uint16_t>(xv & 0xffffu));
            v1[j] = h2f(static_cast<uint16_t>(xv >> 16));
            if (delta) {
                const uint32_t dv = d2[i];
                const uint16_t r0 = f2h(v0[j] + h2f(static_cast<uint16_t>(dv & 0xffffu)));
                const uint16_t r1 = f2h(v1[j] + h2f(static_cast<uint16_t>(dv >> 16)));
                x2[i] = static_cast<uint32_t>(r0) | (static_cast<uint32_t>(r1) << 16);
                v0[j] = h2f(r0);
                v1[j] = h2f(r1);
            }
            ss = fmaf(v0[j], v0[j], fmaf(v1[j], v1[j], ss));
        }
    }
    for (int i = threadIdx.x + kNormPairs * kNormThreads; i < pairs; i += kNormThreads) {     // beyond the cached part
        const uint32_t xv = x2[i];
        float a = h2f(static_cast<uint16_t>(xv & 0xffffu)), b = h2f(static_cast<uint16_t>(xv >> 16));
        if (delta) {
            const uint32_t dv = d2[i];
            const uint16_t r0 = f2h(a + h2f(static_cast<uint16_t>(dv & 0xffffu)));
            const uint16_t r1 = f2h(b + h2f(static_cast<uint16_t>(dv >> 16)));
            x2[i] = static_cast<uint32_t>(r0) | (static_cast<uint32_t>(r1) << 16);
            a = h2f(r0);
            b = h2f(r1);
        }
        ss = fmaf(a, a, fmaf(b, b, ss));
    }
    const float var = block_reduce<false>(ss, scratch) / static_cast<float>(n);
    const float inv = rsqrtf(var + eps);
    auto emit = [&](int i, float a, float b) {
        const uint32_t wv = w2[i];
        const uint16_t r0 = f2h(h2f(static_cast<uint16_t>(wv & 0xffffu)) * h2f(f2h(a * inv)));
        const uint16_t r1 = f2h(h2f(static_cast<uint16_t>(wv >> 16)) * h2f(f2h(b * inv)));
        h2[i] = static_cast<uint32_t>(r0) | (static_cast<uint32_t>(r1) << 16);
    };
#pragma unroll
    for (int j = 0; j < kNormPairs; ++j) {
        const int i = threadIdx.x + j * kNormThreads;
        if (i < pairs)
            emit(i, v0[j], v1[j]);
    }
    for (int i = threadIdx.x + kNormPairs * kNormThreads; i < pairs; i += kNormThreads) {
        const uint32_t xv = x2[i];
        emit(i, h2f(static_cast<uint16_t>(xv & 0xffffu)), h2f(static_cast<uint16_t>(xv >> 16)));
    }
}

// One workgroup per query head.  qkv = [q heads | k heads | v heads] of the
// new token; the rotated key and the value are appended to the caches at
// position *pos by the first query head of each key/value group, and every
// head uses its own copy of them, so no workgroup waits for another.
// head_dim / 8 lanes share a cache row (16 bytes each), 256 / (head_dim / 8)
// rows are in flight per pass over the positions.
__global__ void __launch_bounds__(kAttnThreads)
attention_kernel(const uint16_t *qkv, const float *cos_t, const float *sin_t, const long long *pos_p,
                 uint16_t *kcache, uint16_t *vcache, uint16_t *ctx, int heads, int kv_heads, int head_dim, int max_seq)
{
    extern __shared__ float lds[];
    float *q = lds;                          // head_dim
    float *knew = q + head_dim;              // head_dim
    float *vnew = knew + head_dim;           // head_dim
    float *scores = vnew + head_dim;         // max_seq
    float *part = scores + max_seq;          // rows * head_dim
    __shared__ float scratch[kAttnThreads / 64];

    const int h = blockIdx.x;
    const int group = heads / kv_heads;
    const int kvh = h / group;
    const int half = head_dim / 2;
    long long p64 = *pos_p;
    const int p = p64 < 0 ? 0 : (p64 >= max_seq ? max_seq - 1 : static_cast<int>(p64));
    const uint16_t *qh = qkv + static_cast<size_t>(h) * head_dim;
    const uint16_t *kh = qkv + static_cast<size_t>(heads + kvh) * head_dim;
    const uint16_t *vh = qkv + static_cast<size_t>(heads + kv_heads + kvh) * head_dim;
    uint16_t *kc = kcache + static_cast<size_t>(kvh) * max_seq * head_dim;
    uint16_t *vc = vcache + static_cast<size_t>(kvh) * max_seq * head_dim;

    for (int d = threadIdx.x; d < half; d += blockDim.x) {
        const float c = cos_t[static_cast<size_t>(p) * half + d], s = sin_t[static_cast<size_t>(p) * half + d];
        const float qa = h2f(qh[d]), qb = h2f(qh[d + half]);
        const float ka = h2f(kh[d]), kb = h2f(kh[d + half]);
        q[d] = h2f(f2h(qa * c - qb * s));
        q[d + half] = h2f(f2h(qb * c + qa * s));
        const uint16_t k0 = f2h(ka * c - kb * s), k1 = f2h(kb * c + ka * s);
        knew[d] = h2f(k0);
        knew[d + half] = h2f(k1);
        vnew[d] = h2f(vh[d]);
        vnew[d + half] = h2f(vh[d + half]);
        if (h % group == 0) {
            kc[static_cast<size_t>(p) * head_dim + d] = k0;
            kc[static_cast<size_t>(p) * head_dim + d + half] = k1;
            vc[static_cast<size_t>(p) * head_dim + d] = vh[d];
            vc[static_cast<size_t>(p) * head_dim + d + half] = vh[d + half];
        }
    }
    __syncthreads();

    const int lpr = head_dim >> 3;                   // lanes per row: 8 or 16 (a power of two)
    const int rows = kAttnThreads / lpr;
    const int sub = threadIdx.x & (lpr - 1), row = threadIdx.x / lpr;
    float qr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        qr[i] = q[sub * 8 + i];
    const float scaling = rsqrtf(static_cast<float>(head_dim));
    float mx = -INFINITY;
    constexpr int kBatch = 8;                        // cache rows a lane has in flight
    for (int t0 = 0; t0 <= p; t0 += rows * kBatch) {
        uint4 kw[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * rows + row;
            kw[b] = uint4{0u, 0u, 0u, 0u};
            if (t < p)
                kw[b] = *reinterpret_cast<const uint4 *>(kc + static_cast<size_t>(t) * head_dim + sub * 8);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * rows + row;
            float acc = 0.f;
            if (t == p) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc = fmaf(qr[i], knew[sub * 8 + i], acc);
            } else {
                const uint32_t ws[4] = {kw[b].x, kw[b].y, kw[b].z, kw[b].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc = fmaf(qr[2 * i], h2f(static_cast<uint16_t>(ws[i] & 0xffffu)), acc);
                    acc = fmaf(qr[2 * i + 1], h2f(static_cast<uint16_t>(ws[i] >> 16)), acc);
                }
            }
            for (int off = lpr >> 1; off > 0; off >>= 1)
                acc += __shfl_xor(acc, off, 64);
            if (t <= p) {
                acc = h2f(f2h(acc)) * scaling;           // the reference's q @ k^T is an fp16 matmul
                if (sub == 0)
                    scores[t] = acc;
                mx = fmaxf(mx, acc);
            }
        }
    }
    mx = block_reduce<true>(mx, scratch);            // (its barriers also publish the scores)
    float sum = 0.f;
    for (int t = threadIdx.x; t <= p; t += blockDim.x) {
        const float e = __expf(scores[t] - mx);
        scores[t] = e;
        sum += e;
    }
    sum = block_reduce<false>(sum, scratch);
    const float inv = 1.f / sum;
    __syncthreads();

    // context: the lanes of a row slot add weight * value for their 8 dimensions
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = 0.f;
    for (int t0 = 0; t0 <= p; t0 += rows * kBatch) {
        uint4 vw[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * rows + row;
            vw[b] = uint4{0u, 0u, 0u, 0u};
            if (t < p)
                vw[b] = *reinterpret_cast<const uint4 *>(vc + static_cast<size_t>(t) * head_dim + sub * 8);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * rows + row;
            if (t > p)
                continue;
            const float w = h2f(f2h(scores[t] * inv));
            if (t < p) {
                const uint32_t vs[4] = {vw[b].x, vw[b].y, vw[b].z, vw[b].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] = fmaf(w, h2f(static_cast<uint16_t>(vs[i] & 0xffffu)), acc[2 * i]);
                    acc[2 * i + 1] = fmaf(w, h2f(static_cast<uint16_t>(vs[i] >> 16)), acc[2 * i + 1]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc[i] = fmaf(w, vnew[sub * 8 + i], acc[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
        part[row * head_dim + sub * 8 + i] = acc[i];
    __syncthreads();
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float total = 0.f;
        for (int r = 0; r < rows; ++r)
            total += part[r * head_dim + d];
        ctx[static_cast<size_t>(h) * head_dim + d] = f2h(total);
    }
}

// token <- argmax(logits) (lowest index among equals), generated[*pos] <- token, *pos <- *pos + 1
__global__ void __launch_bounds__(kNormThreads)
argmax_advance_kernel(const uint16_t *logits, int n, long long *token, long long *generated, long long *pos, int max_seq)
{
    __shared__ float best_v[kNormThreads / 64];
    __shared__ int best_i[kNormThreads / 64];
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    };
    // 16-byte pieces, four in flight per thread (logits is 16-byte aligned: checked by the caller)
    const int chunks = n >> 3;
    const uint4 *l4 = reinterpret_cast<const uint4 *>(logits);
    for (int c0 = 0; c0 < chunks; c0 += 4 * kNormThreads) {
        uint4 w[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int c = c0 + b * kNormThreads + threadIdx.x;
            w[b] = uint4{0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u};      // -inf
            if (c < chunks)
                w[b] = l4[c];
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int c = c0 + b * kNormThreads + threadIdx.x;
            if (c < chunks) {
                const uint32_t ws[4] = {w[b].x, w[b].y, w[b].z, w[b].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    take(h2f(static_cast<uint16_t>(ws[i] & 0xffffu)), c * 8 + 2 * i);
                    take(h2f(static_cast<uint16_t>(ws[i] >> 16)), c * 8 + 2 * i + 1);
                }
            }
        }
    }
    for (int i = chunks * 8 + threadIdx.x; i < n; i += blockDim.x)
        take(h2f(logits[i]), i);
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        best_v[threadIdx.x >> 6] = bv;
        best_i[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < static_cast<int>(blockDim.x >> 6); ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        if (bi == 0x7fffffff)
            bi = 0;                      // all NaN
        const long long p = *pos;
        *token = bi;
        if (p >= 0 && p < max_seq)
            generated[p] = bi;
        *pos = p + 1;
    }
}

__global__ void __launch_bounds__(256)
silu_mul_kernel(const uint16_t *gu, uint16_t *out, int ffn)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= ffn)
        return;
    const float g = h2f(gu[i]), u = h2f(gu[ffn + i]);
    const float act = h2f(f2h(g / (1.f + __expf(-g))));
    out[i] = f2h(act * u);
}

}  // namespace

extern "C" {

int sbvr_hip_dec_add_rmsnorm_f16(void *x, const void *delta, const void *weight, void *h, int n, float eps,
                                 void *stream)
{
    if (!x || !weight || !h || n <= 0 || n % 2)
        return -1;
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint16_t *>(x), static_cast<const uint16_t *>(delta),
                       static_cast<const uint16_t *>(weight), static_cast<uint16_t *>(h), n, eps);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int sbvr_hip_dec_attention_f16(const void *qkv, const float *cos_table, const float *sin_table, const long long *pos,
                               void *kcache, void *vcache, void *ctx, int heads, int kv_heads, int head_dim,
                               int max_seq, void *stream)
{
    if (!qkv || !cos_table || !sin_table || !pos || !kcache || !vcache || !ctx)
        return -1;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || (head_dim != 64 && head_dim != 128) || max_seq <= 0 ||
        max_seq > 8192)
        return -2;
    const size_t lds = (3 * static_cast<size_t>(head_dim) + max_seq + static_cast<size_t>(kAttnThreads) * 8) * sizeof(float);
    hipLaunchKernelGGL(attention_kernel, dim3(heads), dim3(kAttnThreads), lds, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(qkv), cos_table, sin_table, pos, static_cast<uint16_t *>(kcache),
                       static_cast<uint16_t *>(vcache), static_cast<uint16_t *>(ctx), heads, kv_heads, head_dim,
                       max_seq);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int sbvr_hip_dec_silu_mul_f16(const void *gate_up, void *out, int ffn, void *stream)
{
    if (!gate_up || !out || ffn <= 0)
        return -1;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((ffn + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(gate_up), static_cast<uint16_t *>(out), ffn);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int sbvr_hip_dec_argmax_advance_f16(const void *logits, int n, long long *token, long long *generated, long long *pos,
                                    int max_seq, void *stream)
{
    if (!logits || !token || !generated || !pos || n <= 0 || max_seq <= 0 || reinterpret_cast<uintptr_t>(logits) % 16)
        return -1;
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(logits), n, token, generated, pos, max_seq);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
