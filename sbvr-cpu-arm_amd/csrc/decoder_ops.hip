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

typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef v4u __attribute__((may_alias)) v4u_any;      // for 16-byte reads of memory written as fp16 elements

// Sum / max over groups of kLanes consecutive lanes (8 or 16) by DPP moves inside
// a row of 16 lanes: no LDS round trips.  Every lane of a group gets the result.
#define SBVR_DPP_F(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, true))
template <int kLanes>
__device__ __forceinline__ float group_sum(float v)
{
    v += SBVR_DPP_F(v, 0xB1);        // quad_perm 1,0,3,2
    v += SBVR_DPP_F(v, 0x4E);        // quad_perm 2,3,0,1
    v += SBVR_DPP_F(v, 0x141);       // row_half_mirror
    if constexpr (kLanes == 16)
        v += SBVR_DPP_F(v, 0x140);   // row_mirror
    return v;
}

// over the 64 lanes; wave-uniform result
template <bool IsMax>
__device__ __forceinline__ float wave_reduce(float v)
{
#define SBVR_STEP(ctrl) v = IsMax ? fmaxf(v, SBVR_DPP_F(v, ctrl)) : v + SBVR_DPP_F(v, ctrl)
    SBVR_STEP(0xB1);
    SBVR_STEP(0x4E);
    SBVR_STEP(0x141);
    SBVR_STEP(0x140);
#undef SBVR_STEP
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return IsMax ? fmaxf(fmaxf(r0, r1), fmaxf(r2, r3)) : (r0 + r1) + (r2 + r3);
}

// 8 fp16 times 8 fp16 (four packed words each), products and sum in fp32
__device__ __forceinline__ float dot8(v4u a, v4u b)
{
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // (the words go through scalars: a bit cast applied to a vector element expression
        // directly takes element 0 whatever the index, with this compiler)
        const uint32_t ai = a[i], bi = b[i];
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h, ai), __builtin_bit_cast(v2h, bi), acc, false);
    }
    return acc;
}

// acc += weight * 8 fp16
__device__ __forceinline__ void axpy8(float (&acc)[8], float w, v4u v)
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc[2 * i] = fmaf(w, h2f(static_cast<uint16_t>(v[i] & 0xffffu)), acc[2 * i]);
        acc[2 * i + 1] = fmaf(w, h2f(static_cast<uint16_t>(v[i] >> 16)), acc[2 * i + 1]);
    }
}

__device__ __forceinline__ v4u pick(bool c, v4u a, v4u b)
{
    v4u r;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        r[i] = c ? a[i] : b[i];
    return r;
}

// One workgroup per query head.  qkv = [q heads | k heads | v heads] of the
// new token; the rotated key and the value are appended to the caches at
// position *pos by the first query head of each key/value group, and every
// head uses its own copy of them, so no workgroup waits for another.
// HD / 8 lanes share a cache row (16 bytes each), kRows = 256 / (HD / 8) rows
// are covered per step over the positions.
// The kernel is a chain of memory round trips with little work between them, so
// it asks for everything before it knows the position: the first kAttnPre * kRows
// cache rows of keys and of values are requested together with the position
// itself (rows past the position are fetched for nothing and ignored; the row
// of the position itself is never taken from the cache), and so is the
// rotation of the position when the caller has it ready (rot_now).  The work on
// those rows is straight-line code without branches, so that the rows of a
// thread overlap.  Longer caches go on in loops that wait step by step.
constexpr int kAttnPre = 16;

#ifdef SBVR_TRACE
__device__ unsigned long long g_attn_trace[8];      // development builds: timestamps of workgroup 0
#define SBVR_ASTAMP(i)                                                \
    do {                                                              \
        if (blockIdx.x == 0 && threadIdx.x == 0)                      \
            g_attn_trace[i] = wall_clock64();                         \
    } while (0)
#else
#define SBVR_ASTAMP(i) do { } while (0)
#endif

template <int HD>
__global__ void __launch_bounds__(kAttnThreads)
attention_kernel(const uint16_t *qkv, const float *cos_t, const float *sin_t, const float *rot_now,
                 const long long *pos_p, uint16_t *kcache, uint16_t *vcache, uint16_t *ctx, int heads, int kv_heads,
                 int max_seq)
{
    constexpr int kLanes = HD / 8;                   // lanes per cache row
    constexpr int kRows = kAttnThreads / kLanes;
    constexpr int kHalf = HD / 2;
    extern __shared__ float lds[];
    uint16_t *qn = reinterpret_cast<uint16_t *>(lds);        // rotated query, rotated new key, new value: HD fp16 each
    uint16_t *kn = qn + HD;
    uint16_t *vn = kn + HD;
    float *scores = lds + 3 * HD;            // max_seq
    float *part = scores + max_seq;          // kRows * HD, and before that a dump for unwanted scores
    __shared__ float red_max[kAttnThreads / 64], red_sum[kAttnThreads / 64];

    const int tid = threadIdx.x;
    const int h = blockIdx.x;
    const int group = heads / kv_heads;
    const int kvh = h / group;
    const uint16_t *qh = qkv + static_cast<size_t>(h) * HD;
    const uint16_t *kh = qkv + static_cast<size_t>(heads + kvh) * HD;
    const uint16_t *vh = qkv + static_cast<size_t>(heads + kv_heads + kvh) * HD;
    uint16_t *kc = kcache + static_cast<size_t>(kvh) * max_seq * HD;
    uint16_t *vc = vcache + static_cast<size_t>(kvh) * max_seq * HD;
    const int sub = tid & (kLanes - 1), row = tid / kLanes;

    SBVR_ASTAMP(0);
    // -- requests that need no position
    const long long p64 = *pos_p;
    const int dd = min(tid, kHalf - 1);              // the threads past kHalf repeat the last pair and drop it
    const uint16_t qa_h = qh[dd], qb_h = qh[dd + kHalf], ka_h = kh[dd], kb_h = kh[dd + kHalf];
    const uint16_t va_h = vh[dd], vb_h = vh[dd + kHalf];
    float c_now = 0.f, s_now = 0.f;
    if (rot_now) {                                   // uniform
        c_now = rot_now[dd];
        s_now = rot_now[kHalf + dd];
    }
    v4u kpre[kAttnPre], vpre[kAttnPre];
#pragma unroll
    for (int b = 0; b < kAttnPre; ++b) {
        const int t = min(b * kRows + row, max_seq - 1);
        kpre[b] = *reinterpret_cast<const v4u_any *>(kc + static_cast<size_t>(t) * HD + sub * 8);
    }
#pragma unroll
    for (int b = 0; b < kAttnPre; ++b) {
        const int t = min(b * kRows + row, max_seq - 1);
        vpre[b] = *reinterpret_cast<const v4u_any *>(vc + static_cast<size_t>(t) * HD + sub * 8);
    }
    const int p = p64 < 0 ? 0 : (p64 >= max_seq ? max_seq - 1 : static_cast<int>(p64));
    if (!rot_now) {
        c_now = cos_t[static_cast<size_t>(p) * kHalf + dd];
        s_now = sin_t[static_cast<size_t>(p) * kHalf + dd];
    }
    SBVR_ASTAMP(1);

    if (tid < kHalf) {
        const float qa = h2f(qa_h), qb = h2f(qb_h), ka = h2f(ka_h), kb = h2f(kb_h);
        const uint16_t k0 = f2h(ka * c_now - kb * s_now), k1 = f2h(kb * c_now + ka * s_now);
        qn[tid] = f2h(qa * c_now - qb * s_now);
        qn[tid + kHalf] = f2h(qb * c_now + qa * s_now);
        kn[tid] = k0;
        kn[tid + kHalf] = k1;
        vn[tid] = va_h;
        vn[tid + kHalf] = vb_h;
        if (h % group == 0) {
            kc[static_cast<size_t>(p) * HD + tid] = k0;
            kc[static_cast<size_t>(p) * HD + tid + kHalf] = k1;
            vc[static_cast<size_t>(p) * HD + tid] = va_h;
            vc[static_cast<size_t>(p) * HD + tid + kHalf] = vb_h;
        }
    }
    __syncthreads();
    SBVR_ASTAMP(2);

    const v4u qp = *reinterpret_cast<const v4u_any *>(qn + sub * 8);
    const v4u knp = *reinterpret_cast<const v4u_any *>(kn + sub * 8);
    const v4u vnp = *reinterpret_cast<const v4u_any *>(vn + sub * 8);
    const float scaling = rsqrtf(static_cast<float>(HD));
    float mx = -INFINITY;
    // scores of the first part: all rows of a thread at once (the reference's q @ k^T is an fp16 matmul)
    {
        float sc[kAttnPre];
#pragma unroll
        for (int b = 0; b < kAttnPre; ++b) {
            const int t = b * kRows + row;
            sc[b] = dot8(qp, pick(t == p, knp, kpre[b]));
        }
#pragma unroll
        for (int b = 0; b < kAttnPre; ++b)
            sc[b] = group_sum<kLanes>(sc[b]);
#pragma unroll
        for (int b = 0; b < kAttnPre; ++b) {
            const int t = b * kRows + row;
            const float v = h2f(f2h(sc[b])) * scaling;
            const bool mine = t <= p && sub == 0;
            (mine ? scores + t : part + tid)[0] = v;         // the others drop theirs in the dump
            mx = t <= p ? fmaxf(mx, v) : mx;
        }
    }
    constexpr int kBatch = 8;                        // cache rows a lane has in flight beyond the first part
    for (int t0 = kAttnPre * kRows; t0 <= p; t0 += kRows * kBatch) {
        v4u kw[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = min(t0 + b * kRows + row, max_seq - 1);
            kw[b] = *reinterpret_cast<const v4u_any *>(kc + static_cast<size_t>(t) * HD + sub * 8);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * kRows + row;
            const float v = h2f(f2h(group_sum<kLanes>(dot8(qp, pick(t == p, knp, kw[b]))))) * scaling;
            if (t <= p) {
                if (sub == 0)
                    scores[t] = v;
                mx = fmaxf(mx, v);
            }
        }
    }
    SBVR_ASTAMP(3);
    // softmax over 0..p: the maximum, then the exponentials and their sum (both barriers also publish LDS data)
    mx = wave_reduce<true>(mx);
    if ((tid & 63) == 0)
        red_max[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
    float sum = 0.f;
    for (int t = tid; t <= p; t += kAttnThreads) {
        const float e = __expf(scores[t] - mx);
        scores[t] = e;
        sum += e;
    }
    sum = wave_reduce<false>(sum);
    if ((tid & 63) == 0)
        red_sum[tid >> 6] = sum;
    __syncthreads();
    const float inv = 1.f / ((red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]));
    SBVR_ASTAMP(4);

    // context: the lanes of a row slot add weight * value for their 8 dimensions
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = 0.f;
    const v4u zero4 = {0u, 0u, 0u, 0u};
    {
        float w[kAttnPre];
#pragma unroll
        for (int b = 0; b < kAttnPre; ++b)
            w[b] = scores[min(b * kRows + row, p)];
#pragma unroll
        for (int b = 0; b < kAttnPre; ++b) {
            const int t = b * kRows + row;
            const float wt = t <= p ? h2f(f2h(w[b] * inv)) : 0.f;       // weights are rounded to fp16
            axpy8(acc, wt, pick(t < p, vpre[b], pick(t == p, vnp, zero4)));      // rows past p may hold anything
        }
    }
    for (int t0 = kAttnPre * kRows; t0 <= p; t0 += kRows * kBatch) {
        v4u vw[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = min(t0 + b * kRows + row, max_seq - 1);
            vw[b] = *reinterpret_cast<const v4u_any *>(vc + static_cast<size_t>(t) * HD + sub * 8);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int t = t0 + b * kRows + row;
            const float wt = t <= p ? h2f(f2h(scores[min(t, p)] * inv)) : 0.f;
            axpy8(acc, wt, pick(t < p, vw[b], pick(t == p, vnp, zero4)));
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)                      // (the dump in `part` was last written two barriers ago)
        part[row * HD + sub * 8 + i] = acc[i];
    SBVR_ASTAMP(5);
    __syncthreads();
    for (int d = tid; d < HD; d += kAttnThreads) {
        float total = 0.f;
#pragma unroll
        for (int r = 0; r < kRows; ++r)
            total += part[r * HD + d];
        ctx[static_cast<size_t>(h) * HD + d] = f2h(total);
    }
    SBVR_ASTAMP(6);
}
#undef SBVR_DPP_F

// token <- argmax(logits) (lowest index among equals), generated[*pos] <- token, *pos <- *pos + 1
__global__ void __launch_bounds__(kNormThreads)
argmax_advance_kernel(const uint16_t *logits, int n, long long *token, long long *generated, long long *pos, int max_seq,
                      const float *cos_t, const float *sin_t, int half, float *rot_now)
{
    __shared__ float best_v[kNormThreads / 64];
    __shared__ int best_i[kNormThreads / 64];
    __shared__ long long new_pos;
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
        new_pos = p + 1;
    }
    if (rot_now) {
        // the rotation of the new position, side by side, for the attention kernels of the next step
        __syncthreads();
        const long long p1 = new_pos;
        const int row = p1 < 0 ? 0 : (p1 >= max_seq ? max_seq - 1 : static_cast<int>(p1));
        for (int d = threadIdx.x; d < half; d += blockDim.x) {
            rot_now[d] = cos_t[static_cast<size_t>(row) * half + d];
            rot_now[half + d] = sin_t[static_cast<size_t>(row) * half + d];
        }
    }
}

// The end of a decode step in one launch: r = fp16(x + delta), h = weight * fp16(r * rsqrt(mean(r^2) + eps))
// (the final norm), logits = fp16(h . head[v]) for every row v of the fp16 output head, token = argmax, and the
// bookkeeping of argmax_advance_kernel.  The head is the largest read of the step (vocab * K * 2 bytes), so the
// kernel is a plain stream: a wave takes rows two at a time, a row is K/512 loads of 16 bytes per lane, the
// loads of the next pair are in flight while the current pair is multiplied (v_dot2_f32_f16, fp32 sums) and
// summed over the lanes (DPP).  Every wave works the norm out by itself (its 64 lanes hold all of h, packed).
// The argmax crosses workgroups in one 64-bit word: (orderable fp16 value << 32) | ~index under an atomic
// maximum at memory, then a counter; the counter's addend depends on the value the maximum returned, so it is
// issued after the maximum has been applied (no fence).  The workgroup that completes the count reads the
// word, does the bookkeeping and leaves both words zero for the next launch.
constexpr int kHeadThreads = 256;
constexpr int kHeadWorkgroupsPerCu = 3;     // as many as fit at K = 4096: every wave of the launch is resident at once

template <int KI>                                   // K = 512 * KI
__global__ void __launch_bounds__(kHeadThreads)
head_argmax_kernel(const uint16_t *x, const uint16_t *delta, const uint16_t *weight, float eps, const uint16_t *head,
                   int vocab, int rows_per_wave, uint16_t *logits, long long *token, long long *generated, long long *pos,
                   int max_seq, const float *cos_t, const float *sin_t, int half, float *rot_now,
                   unsigned long long *work, const uint16_t *embed, uint16_t *x_next)
{
    constexpr int K = 512 * KI;
    __shared__ unsigned long long best[kHeadThreads / 64];
    __shared__ long long new_pos, new_token;
    __shared__ int last;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row0 = (blockIdx.x * (kHeadThreads / 64) + wave) * rows_per_wave;      // rows_per_wave: a multiple of 4

    // -- requests: the first pair of rows, then the activations (needed first, so asked for first)
    v4u xs[KI], ds[KI], ws[KI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        xs[i] = reinterpret_cast<const v4u_any *>(x)[lane + 64 * i];
        ws[i] = reinterpret_cast<const v4u_any *>(weight)[lane + 64 * i];
        ds[i] = v4u{0u, 0u, 0u, 0u};
        if (delta)                                   // uniform
            ds[i] = reinterpret_cast<const v4u_any *>(delta)[lane + 64 * i];
    }
    auto row_ptr = [&](int r) __attribute__((always_inline)) {
        return reinterpret_cast<const v4u_any *>(head + static_cast<size_t>(min(r, vocab - 1)) * K) + lane;
    };
    // (non-temporal: the head is read once per step and should not push anything out of the caches on its way;
    // measured 172 us against 185 us for the 1.05 GB head of the 8B shape)
#define SBVR_ROW_LOAD(ptr, i) __builtin_nontemporal_load(reinterpret_cast<const v4u *>(ptr) + 64 * (i))
    v4u a0[KI], a1[KI], b0[KI], b1[KI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        a0[i] = SBVR_ROW_LOAD(row_ptr(row0), i);
        a1[i] = SBVR_ROW_LOAD(row_ptr(row0 + 1), i);
    }

    // -- the norm
    v4u h[KI];
    {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < KI; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t xv = xs[i][e], dv = ds[i][e];
                const uint32_t lo = f2h(h2f(static_cast<uint16_t>(xv & 0xffffu)) + h2f(static_cast<uint16_t>(dv & 0xffffu)));
                const uint32_t hi = f2h(h2f(static_cast<uint16_t>(xv >> 16)) + h2f(static_cast<uint16_t>(dv >> 16)));
                xs[i][e] = lo | (hi << 16);
                const float fl = h2f(static_cast<uint16_t>(lo)), fh = h2f(static_cast<uint16_t>(hi));
                ss = fmaf(fl, fl, fmaf(fh, fh, ss));
            }
        const float inv = rsqrtf(wave_reduce<false>(ss) / static_cast<float>(K) + eps);
#pragma unroll
        for (int i = 0; i < KI; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t rv = xs[i][e], wv = ws[i][e];
                const uint32_t lo = f2h(h2f(static_cast<uint16_t>(wv & 0xffffu)) * h2f(f2h(h2f(static_cast<uint16_t>(rv & 0xffffu)) * inv)));
                const uint32_t hi = f2h(h2f(static_cast<uint16_t>(wv >> 16)) * h2f(f2h(h2f(static_cast<uint16_t>(rv >> 16)) * inv)));
                h[i][e] = lo | (hi << 16);
            }
    }

    // -- the rows
    unsigned long long mine = 0ull;                  // wave-uniform: best (value, ~index) so far
    auto finish = [&](int r, float sum) __attribute__((always_inline)) {
        const uint16_t v = f2h(wave_reduce<false>(sum));
        if (r < vocab && r < row0 + rows_per_wave) {     // uniform
            if (lane == 0 && logits)
                logits[r] = v;
            const bool nan = (v & 0x7fffu) > 0x7c00u;
            const uint32_t ord = nan ? 0u : ((v & 0x8000u) ? (~static_cast<uint32_t>(v)) & 0xffffu : static_cast<uint32_t>(v) | 0x8000u);
            const unsigned long long key = (static_cast<unsigned long long>(ord) << 32) | (0xffffffffu - static_cast<uint32_t>(r));
            mine = key > mine ? key : mine;
        }
    };
    auto dot_row = [&](const v4u (&a)[KI]) __attribute__((always_inline)) -> float {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < KI; ++i)
            acc += dot8(h[i], a[i]);
        return acc;
    };
    for (int p = 0; p < rows_per_wave; p += 4) {
        const int r = row0 + p;
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            b0[i] = SBVR_ROW_LOAD(row_ptr(r + 2), i);
            b1[i] = SBVR_ROW_LOAD(row_ptr(r + 3), i);
        }
        finish(r, dot_row(a0));
        finish(r + 1, dot_row(a1));
#pragma unroll
        for (int i = 0; i < KI; ++i) {               // (past the wave's rows these repeat a row and are dropped)
            a0[i] = SBVR_ROW_LOAD(row_ptr(min(r + 4, row0 + rows_per_wave - 1)), i);
            a1[i] = SBVR_ROW_LOAD(row_ptr(min(r + 5, row0 + rows_per_wave - 1)), i);
        }
        finish(r + 2, dot_row(b0));
        finish(r + 3, dot_row(b1));
    }

    // -- argmax across the waves, then across the workgroups
    if (lane == 0)
        best[wave] = mine;
    __syncthreads();
    if (tid == 0) {
        unsigned long long key = best[0];
        for (int w = 1; w < kHeadThreads / 64; ++w)
            key = best[w] > key ? best[w] : key;
        const unsigned long long before = __hip_atomic_fetch_max(work, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // The count must not be raised before this workgroup's maximum is in place: the workgroup that completes the
        // count reads the maximum and zeroes both words.  The addend is made to depend on the value the maximum
        // returned (the empty statement takes `before` in a register and gives `one` back as something the compiler
        // cannot see through), so the add is issued only once that value has come back, i.e. once the maximum has
        // been applied where all workgroups' atomics meet.  Both are returning atomics of one thread on neighbouring
        // words; no fence is involved (an agent-scope fence writes back the XCD's whole L2).
        unsigned long long one = 1ull;
        asm volatile("" : "+v"(one) : "v"(before));
        const unsigned long long count = __hip_atomic_fetch_add(work + 1, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = count + 1 == gridDim.x;
        if (last) {
            const unsigned long long win = __hip_atomic_load(work, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const long long bi = static_cast<long long>(0xffffffffu - static_cast<uint32_t>(win & 0xffffffffu));
            const long long pnow = *pos;
            *token = bi;
            if (pnow >= 0 && pnow < max_seq)
                generated[pnow] = bi;
            *pos = pnow + 1;
            new_pos = pnow + 1;
            new_token = bi;
            __hip_atomic_store(work, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(work + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __syncthreads();
    if (last && rot_now) {
        const long long p1 = new_pos;
        const int row = p1 < 0 ? 0 : (p1 >= max_seq ? max_seq - 1 : static_cast<int>(p1));
        for (int d = tid; d < half; d += kHeadThreads) {
            rot_now[d] = cos_t[static_cast<size_t>(row) * half + d];
            rot_now[half + d] = sin_t[static_cast<size_t>(row) * half + d];
        }
    }
    // the chosen token's embedding row, where the next step's residual stream starts (every other workgroup has
    // read x and added its maximum by now, so x_next may be x)
    if (last && x_next) {
        const long long t = new_token < 0 ? 0 : (new_token >= vocab ? vocab - 1 : new_token);
        const v4u_any *src = reinterpret_cast<const v4u_any *>(embed + static_cast<size_t>(t) * K);
        for (int c = tid; c < K / 8; c += kHeadThreads)
            reinterpret_cast<v4u_any *>(x_next)[c] = src[c];
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

#ifdef SBVR_TRACE
int sbvr_hip_debug_attn_trace(unsigned long long *out8)
{
    return hipMemcpyFromSymbol(out8, HIP_SYMBOL(g_attn_trace), 8 * sizeof(unsigned long long)) == hipSuccess ? 0 : -3;
}
#endif

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

int sbvr_hip_dec_attention_f16(const void *qkv, const float *cos_table, const float *sin_table, const float *rot_now,
                               const long long *pos, void *kcache, void *vcache, void *ctx, int heads, int kv_heads,
                               int head_dim, int max_seq, void *stream)
{
    if (!qkv || !cos_table || !sin_table || !pos || !kcache || !vcache || !ctx)
        return -1;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || (head_dim != 64 && head_dim != 128) || max_seq <= 0 ||
        max_seq > 8192)
        return -2;
    if ((reinterpret_cast<uintptr_t>(kcache) | reinterpret_cast<uintptr_t>(vcache)) % 16)
        return -1;
    const size_t lds = (3 * static_cast<size_t>(head_dim) + max_seq + static_cast<size_t>(kAttnThreads) * 8) * sizeof(float);
    const dim3 grid(heads), block(kAttnThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (head_dim == 128)
        hipLaunchKernelGGL(attention_kernel<128>, grid, block, lds, st, static_cast<const uint16_t *>(qkv), cos_table,
                           sin_table, rot_now, pos, static_cast<uint16_t *>(kcache), static_cast<uint16_t *>(vcache),
                           static_cast<uint16_t *>(ctx), heads, kv_heads, max_seq);
    else
        hipLaunchKernelGGL(attention_kernel<64>, grid, block, lds, st, static_cast<const uint16_t *>(qkv), cos_table,
                           sin_table, rot_now, pos, static_cast<uint16_t *>(kcache), static_cast<uint16_t *>(vcache),
                           static_cast<uint16_t *>(ctx), heads, kv_heads, max_seq);
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
                                    int max_seq, const float *cos_table, const float *sin_table, int head_dim,
                                    float *rot_now, void *stream)
{
    if (!logits || !token || !generated || !pos || n <= 0 || max_seq <= 0 || reinterpret_cast<uintptr_t>(logits) % 16)
        return -1;
    if (rot_now && (!cos_table || !sin_table || head_dim <= 0 || head_dim % 2))
        return -1;
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(logits), n, token, generated, pos, max_seq, cos_table, sin_table,
                       head_dim / 2, rot_now);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int sbvr_hip_dec_head_argmax_f16(const void *x, const void *delta, const void *norm_weight, float eps, const void *head,
                                 int vocab, int K, void *logits, long long *token, long long *generated, long long *pos,
                                 int max_seq, const float *cos_table, const float *sin_table, int head_dim,
                                 float *rot_now, void *workspace, void *stream)
{
    return sbvr_hip_dec_head_argmax_embed_f16(x, delta, norm_weight, eps, head, vocab, K, logits, token, generated, pos,
                                              max_seq, cos_table, sin_table, head_dim, rot_now, workspace, nullptr, nullptr,
                                              stream);
}

int sbvr_hip_dec_head_argmax_embed_f16(const void *x, const void *delta, const void *norm_weight, float eps,
                                       const void *head, int vocab, int K, void *logits, long long *token,
                                       long long *generated, long long *pos, int max_seq, const float *cos_table,
                                       const float *sin_table, int head_dim, float *rot_now, void *workspace,
                                       const void *embed, void *x_next, void *stream)
{
    if ((embed == nullptr) != (x_next == nullptr) ||
        (reinterpret_cast<uintptr_t>(embed) | reinterpret_cast<uintptr_t>(x_next)) % 16)
        return -1;
    if (!x || !norm_weight || !head || !token || !generated || !pos || !workspace || vocab <= 0 || max_seq <= 0)
        return -1;
    if (rot_now && (!cos_table || !sin_table || head_dim <= 0 || head_dim % 2))
        return -1;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(delta) | reinterpret_cast<uintptr_t>(norm_weight) |
         reinterpret_cast<uintptr_t>(head)) % 16 || reinterpret_cast<uintptr_t>(workspace) % 8)
        return -1;
    // one wave per wave slot of the chip, the rows dealt out evenly (in fours): no second round of workgroups
    static int cus[16];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
        return -3;
    if (cus[dev] == 0 && hipDeviceGetAttribute(&cus[dev], hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return -3;
    const int waves_per_wg = kHeadThreads / 64;
    int wgs = cus[dev] * kHeadWorkgroupsPerCu;
    int rows_per_wave = ((vocab + wgs * waves_per_wg - 1) / (wgs * waves_per_wg) + 3) / 4 * 4;
    wgs = (vocab + rows_per_wave * waves_per_wg - 1) / (rows_per_wave * waves_per_wg);
    const dim3 grid(wgs), block(kHeadThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define SBVR_HEAD(ki)                                                                                               \
    case 512 * ki:                                                                                                  \
        hipLaunchKernelGGL(head_argmax_kernel<ki>, grid, block, 0, st, static_cast<const uint16_t *>(x),            \
                           static_cast<const uint16_t *>(delta), static_cast<const uint16_t *>(norm_weight), eps,   \
                           static_cast<const uint16_t *>(head), vocab, rows_per_wave,                               \
                           static_cast<uint16_t *>(logits), token,                                                  \
                           generated, pos, max_seq, cos_table, sin_table, head_dim / 2, rot_now,                    \
                           static_cast<unsigned long long *>(workspace), static_cast<const uint16_t *>(embed),      \
                           static_cast<uint16_t *>(x_next));                                                        \
        break
    switch (K) {
        SBVR_HEAD(1); SBVR_HEAD(2); SBVR_HEAD(4); SBVR_HEAD(8); SBVR_HEAD(16);
    default:
        return -2;
    }
#undef SBVR_HEAD
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
