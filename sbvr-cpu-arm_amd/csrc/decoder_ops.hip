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

}  // extern "C"
