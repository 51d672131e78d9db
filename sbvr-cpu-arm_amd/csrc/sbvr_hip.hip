// libsbvr_hip.so -- HIP kernels for gfx950 (MI355X) behind the C ABI of
// include/sbvr_hip.h: the SBVR compressed-domain linear layer.
//
// Decode path (M <= 8 by default, M <= 16 on request and with 6 or 8 planes), sbvr_gemv_mfma_kernel (and, from
// 5 rows on, sbvr_gemv_batch_kernel, whose waves share the activation operands of a sub-group).  The work is one bit per weight
// element and plane, far too many bits for one VALU lane-op each, so the masked
// sums run on the matrix cores:
//   * a 32-bit plane word becomes four dwords of fp4 (e2m1) values with one AND
//     (or shift+AND) each: nibble q of dword t carries bit 4q+t of the word as
//     0.5, 1.0 or 2.0;
//   * the fp16 activations of one 128-element sub-group are written as three
//     fp8 (e4m3) terms h1 + h2 + h3/256 = x * 2^e * f_t, which reproduce the
//     fp16 value exactly (4 significant bits each, the third taken from the
//     residual scaled by 256), in the register image of the A operand; the
//     per-position factor f_t undoes the 0.5/1/2 of the B nibbles, 2^e is a
//     power of two per (row, sub-group);
//   * v_mfma_f32_16x16x128_f8f6f4 (A fp8, B fp4) then yields, for 16 columns
//     and one plane, the three partial plane sums per batch row; they are added,
//     rescaled and multiplied by the group's coefficient in fp32.
// The packed layout of the reference (sbvr/core.py:724-731, 782-805) is read as
// it is: a lane loads the S plane words of one (word, column) pair with one
// vector load, 16 neighbouring columns give 256 contiguous bytes.
// Work split: a workgroup owns 16*CT columns, its waves split K and add their
// partial results in LDS in a fixed order; when N alone does not give enough
// workgroups, K is also split across workgroups, whose partial sums meet in
// 64-bit fixed-point accumulators (exact, so the result does not depend on
// the order of arrival).
//
// For one batch row the kernel can take the elementwise step in front of the
// linear along (SiLU(gate) * up, or residual add + RMSNorm) while it turns the
// activations into A operands: sbvr_hip_linear_f16_swiglu / _add_rmsnorm.
//
// Prefill path (M > 32): fp16 MFMA, fp32 accumulation; sbvr_gemm_lut_kernel (2..4
// planes: weights decoded by table look-up in registers, activations shared
// through LDS) or sbvr_gemm_mfma_kernel (weights decoded to fp16 tiles in LDS by
// producer waves).  In between, 9..32 rows (17..32 with 6
// or 8 planes): the batch rows are the 32 rows of one MFMA, weights decoded in
// registers -- by table look-up for 2..4 planes (sbvr_gemm_rows32_lut_kernel),
// arithmetically otherwise (sbvr_gemm_rows32_kernel).
//
// The reference's own operator forms: both operands encoded: the decode kernel
// with the left operand's planes as batch rows (one left row of up to 4 planes),
// else sbvr_mm_T_popc_kernel (popcounts per group, lane per column);
// sbvr_row_deq_mfma_kernel (trans=True
// weight: bits transposed across lanes, then the decode path's plane sums) and
// sbvr_row_deq_lanes_kernel (the same for other plane counts, lanes along K).
//
// Portable kernels (any shape, one thread per output) back all of them.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <mutex>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/sbvr_hip.h"
#include "../../include/sbvr_hip_decoder.h"

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

thread_local char g_err[256] = "";
thread_local int g_last_kernel = 0;       // SBVR_HIP_KERNEL_* of the last linear launched from this thread
thread_local int g_last_rounding = 0;     // SBVR_HIP_ROUNDING_* of that launch

int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

struct DevInfo {
    bool ready = false;
    int cus = 256;
};
DevInfo g_dev[16];
std::mutex g_dev_lock;           // guards g_dev[] and the scratch addresses: first use may come from several threads

// ------------------------------------------------------------------ helpers

__device__ __forceinline__ float h2f(uint16_t h)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
}

__device__ __forceinline__ uint16_t f2h(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// fp16 add of two fp16 values: exact sum rounded once (what __hadd does).
__device__ __forceinline__ uint16_t hadd(uint16_t a, uint16_t b)
{
    return f2h(h2f(a) + h2f(b));
}

template <typename IdxT>
__device__ __forceinline__ int load_idx(const void *p, size_t i)
{
    return static_cast<int>(static_cast<const IdxT *>(p)[i]);
}

// ---------------------------------------------------- portable kernel (any shape)

// One thread per output element.  Slow; used for shapes the MFMA kernel does
// not take and as a second implementation to test against.
template <typename IdxT>
__global__ void __launch_bounds__(256)
sbvr_linear_portable_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ bvr,
                            const void *__restrict__ idx, const uint16_t *__restrict__ cache,
                            const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                            int M, int N, int K, int S, int G)
{
    const size_t o = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= static_cast<size_t>(M) * N)
        return;
    const int m = static_cast<int>(o / N), n = static_cast<int>(o % N);
    const int wpg = G / 32;
    float acc = 0.f;
    for (int g = 0; g < K / G; ++g) {
        const int line = load_idx<IdxT>(idx, static_cast<size_t>(g) * N + n);
        for (int j = 0; j < S; ++j) {
            float ps = 0.f;
            for (int w = 0; w < wpg; ++w) {
                const int kw = g * wpg + w;
                uint32_t bits = bvr[(static_cast<size_t>(kw) * N + n) * S + j];
                const uint16_t *xr = x + static_cast<size_t>(m) * K + kw * 32;
                while (bits) {
                    const int b = __builtin_ctz(bits);
                    bits &= bits - 1;
                    ps += h2f(xr[b]);
                }
            }
            acc = fmaf(h2f(cache[static_cast<size_t>(line) * S + j]), ps, acc);
        }
    }
    uint16_t r = f2h(acc);
    if (bias)
        r = hadd(r, bias[n]);
    out[o] = r;
}

// --------------------------------------------------------------- MFMA decode

constexpr int kSub = 128;        // K elements per MFMA (one sub-group)
constexpr int kMaxWaves = 16;    // waves of a workgroup; they split K among themselves
constexpr int kMaxM = 16;        // batch rows of the decode kernel (row tiles of 4)
constexpr int kUnitsAhead = 3;   // units of plane words a wave of the decode kernel keeps in flight
constexpr int kUnitsFirst = 2;   // of those, requested before the wave makes its A operands (the rest right behind them)
constexpr float kLastTermScale = 256.f;  // third fp8 term of an activation holds residual * 256

// Split-K accumulator: one 64-bit word per output, [count:8 | sum:56].  Every
// workgroup adds (1 << 56) + (v + 2^47) with v = rint(partial * 2^30); integer
// addition is exact and order-free, so the result does not depend on which
// workgroup comes first.  The adder that finds count == ksplit-1 owns the total.
constexpr int kAccFracBits = 30;
constexpr long long kAccBias = 1ll << 47;
constexpr float kAccClamp = 130000.f;    // |partial| beyond this becomes +-inf in fp16 anyway
constexpr int kMaxKsplit = 255;

struct GemvArgs {
    const uint16_t *x;
    const uint32_t *bvr;
    const void *idx;
    const uint16_t *cache;
    const uint16_t *bias;
    uint16_t *out;
    unsigned long long *acc;   // (M, N) split-K accumulators, all zero between calls (ksplit > 1 only)
    int M, N, K, L;
    int gshift;           // a coefficient group is 128 << gshift elements
    int idx16;            // line indices are uint16 (else uint8)
    int ksplit;           // workgroups along K
    int xstride;          // elements between batch rows of x
    int wstride;          // columns a workgroup owns: a multiple of 8, (CT - 1) * 16 < wstride <= CT * 16
    // fused activation prologues (see XM of the kernel)
    const uint16_t *delta;      // XM == 2: added to x before the norm
    const uint16_t *norm_w;     // XM == 2: RMSNorm weight
    uint16_t *x_out;            // XM == 2: receives fp16(x + delta)
    float eps;
    // XM == kXPlanes: the left operand, SBVR-encoded (one row, M planes, default layout)
    const uint32_t *xbvr;       // (K / 32, 1, M)
    const void *xidx;           // (K / G, 1)
    const uint16_t *xcache;     // (xL, M)
    int x_idx16, xL;
#ifdef SBVR_TRACE
    unsigned long long *trace;   // 8 timestamps per workgroup (development builds only)
#endif
};

#ifdef SBVR_TRACE
#define SBVR_STAMP(i)                                                         \
    do {                                                                      \
        if (a.trace && (threadIdx.x & 63) == 0)                               \
            a.trace[((blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64(); \
    } while (0)
unsigned long long *g_trace = nullptr;
#else
#define SBVR_STAMP(i) do { } while (0)
#endif

// Where element k (0..127) of row `row` (0..15) of a sub-group sits in the A
// operand of v_mfma_f32_16x16x128_f8f6f4 with fp8 A and fp4 B, given that B
// dword t, nibble q of the lane holding word c carries bit 4q+t of that word:
//   B side: reduction index kk = 32c + 8t + q           (lane block c, nibble 8t+q)
//   A side: byte p of lane 16*kb + row holds kk = 64*(p/16) + 16*kb + p%16
__device__ __forceinline__ int a_image_byte_offset(int k, int row)
{
    const int c = k >> 5, r = k & 31, q = r >> 2, t = r & 3;
    const int kk = 32 * c + 8 * t + q;
    const int p = 16 * (kk >> 6) + (kk & 15);
    const int lane = 16 * ((kk >> 4) & 3) + row;
    return lane * 32 + p;
}

template <int S>
struct Planes {
    uint32_t w[S];
};

typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v3raw __attribute__((ext_vector_type(3)));
typedef v3raw v3u __attribute__((aligned(4)));          // (as it lies in a row of 3 or 6 plane words)

// The S plane words of one (word of K, column) pair.  kStream: non-temporal loads, for kernels that
// read every plane word once per launch and are bound by that stream (measured on the decode kernel:
// 8.3 us instead of 8.8 us at the 4096 -> 14336 shape, 13.5 instead of 14.5 us at 4096 -> 28672; the
// 32-row, row-dequant and popcount kernels, bound by their arithmetic, gain nothing from it).
template <int S, bool kStream = false>
__device__ __forceinline__ Planes<S> load_planes(const uint32_t *p)
{
    auto ld4 = [](const uint32_t *q) __attribute__((always_inline)) -> v4u {
        return kStream ? __builtin_nontemporal_load(reinterpret_cast<const v4u *>(q)) : *reinterpret_cast<const v4u *>(q);
    };
    auto ld2 = [](const uint32_t *q) __attribute__((always_inline)) -> v2u {
        return kStream ? __builtin_nontemporal_load(reinterpret_cast<const v2u *>(q)) : *reinterpret_cast<const v2u *>(q);
    };
    Planes<S> r;
    if constexpr (S == 4) {
        const v4u v = ld4(p);
        r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z; r.w[3] = v.w;
    } else if constexpr (S == 2) {
        const v2u v = ld2(p);
        r.w[0] = v.x; r.w[1] = v.y;
    } else if constexpr (S == 8) {
        const v4u v0 = ld4(p), v1 = ld4(p + 4);
        r.w[0] = v0.x; r.w[1] = v0.y; r.w[2] = v0.z; r.w[3] = v0.w;
        r.w[4] = v1.x; r.w[5] = v1.y; r.w[6] = v1.z; r.w[7] = v1.w;
    } else if constexpr (S == 3) {
        // (12 bytes in one request: a global load wants dword alignment only)
        const v3raw v = kStream ? __builtin_nontemporal_load(reinterpret_cast<const v3u *>(p)) : *reinterpret_cast<const v3u *>(p);
        r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z;
    } else if constexpr (S == 6) {
        const v3raw v0 = kStream ? __builtin_nontemporal_load(reinterpret_cast<const v3u *>(p)) : *reinterpret_cast<const v3u *>(p);
        const v3raw v1 = kStream ? __builtin_nontemporal_load(reinterpret_cast<const v3u *>(p + 3)) : *reinterpret_cast<const v3u *>(p + 3);
        r.w[0] = v0.x; r.w[1] = v0.y; r.w[2] = v0.z; r.w[3] = v1.x; r.w[4] = v1.y; r.w[5] = v1.z;
    } else {
#pragma unroll
        for (int j = 0; j < S; ++j)
            r.w[j] = kStream ? __builtin_nontemporal_load(p + j) : p[j];
    }
    return r;
}

// The S fp16 coefficients of table line p as (S + 1) / 2 dwords, in as few loads as the line's alignment allows.
template <int S>
__device__ __forceinline__ void load_line_words(const uint16_t *p, uint32_t (&c)[(S + 1) / 2])
{
    constexpr int CW = (S + 1) / 2;
    if constexpr (S == 4) {
        const uint2 t = *reinterpret_cast<const uint2 *>(p);
        c[0] = t.x; c[1] = t.y;
    } else if constexpr (S == 8) {
        const uint4 t = *reinterpret_cast<const uint4 *>(p);
        c[0] = t.x; c[1] = t.y; c[2] = t.z; c[3] = t.w;
    } else if constexpr (S % 2 == 0) {
#pragma unroll
        for (int j = 0; j < CW; ++j)
            c[j] = reinterpret_cast<const uint32_t *>(p)[j];
    } else {
#pragma unroll
        for (int j = 0; j < CW; ++j)
            c[j] = static_cast<uint32_t>(p[2 * j]) | (2 * j + 1 < S ? static_cast<uint32_t>(p[2 * j + 1]) << 16 : 0u);
    }
}

// Waves per SIMD the register allocator is asked to leave room for: the A operands and the activations
// they are made from, the results, the MFMA outputs and plane sums of a unit, the plane words in flight
// and working registers.
constexpr int gemv_waves(int S, int MT, int CT, int SP)
{
    const int regs = 12 * SP * MT + CT * MT + 5 * MT * S + 3 * S + 4 * S + 48;
    const int w = 512 / regs;
    return w < 1 ? 1 : (w > 8 ? 8 : w);
}

// Waves of a workgroup at most: 16, or 8 for the instances that want more than 128 registers a lane
// (four row tiles).
constexpr int gemv_max_waves(int MT, int CT)
{
    (void)CT;
    return MT == 4 ? 8 : kMaxWaves;
}

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ v2h as_v2h(uint32_t u) { return __builtin_bit_cast(v2h, u); }
__device__ __forceinline__ int as_int(v2s b) { return __builtin_bit_cast(int, b); }

// max over the 64 lanes of a non-negative integer; the result is wave-uniform
__device__ __forceinline__ uint32_t wave_umax(uint32_t v)
{
    v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, true)));   // quad_perm 1,0,3,2
    v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, true)));   // quad_perm 2,3,0,1
    v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, true)));  // row_half_mirror
    v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, true)));  // row_mirror
    const uint32_t r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
    const uint32_t r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
    return max(max(r0, r1), max(r2, r3));
}

// sum over the 64 lanes; the result is wave-uniform
__device__ __forceinline__ float wave_fsum(float v)
{
#define SBVR_DPP_ADD(ctrl) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, true))
    SBVR_DPP_ADD(0xB1);      // quad_perm 1,0,3,2
    SBVR_DPP_ADD(0x4E);      // quad_perm 2,3,0,1
    SBVR_DPP_ADD(0x141);     // row_half_mirror
    SBVR_DPP_ADD(0x140);     // row_mirror
#undef SBVR_DPP_ADD
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// Activation prologues of the decode kernel: what the A operands are made from.
//   kXPlain   x itself;
//   kXSwiGLU  M == 1, x is (1, 2K) = gate | up: fp16(fp16(silu(gate)) * up), the MLP's
//             act_fn(gate_proj(x)) * up_proj(x) (models/sbvr_llama.py:238-239);
//   kXAddNorm M == 1: r = fp16(x + delta), weight * fp16(r * rsqrt(mean(r^2) + eps)),
//             the decoder layer's residual add followed by its RMSNorm
//             (models/sbvr_llama.py:396-400 and :118-124); every workgroup works out
//             the mean over all of K by itself: its threads share out x and delta in
//             16-byte chunks (one each, or two each with kXAddNorm2), leave r in LDS,
//             where the waves then find their own elements; workgroup (0, 0) writes r
//             to x_out.
constexpr int kXPlain = 0, kXSwiGLU = 1, kXAddNorm = 2, kXAddNorm2 = 3;   // (3: two chunks of x per thread for the norm)
constexpr int kXFloor = 4;      // measurement aid: the launch's plane-word and index requests only, no arithmetic, no output
// kXPlanes: the left operand is SBVR-encoded as well (one left row of M <= 4 planes, the reference's both-encoded
//           product, sbvr_kernel.cu:464-562): batch row r of the A operands is plane r times its coefficient, a_r
//           or 0 per element (exact in fp16, hence in the three fp8 terms), so the MFMAs give
//           sum_k a_r L_r[k] R_j[k] = a_r * popcount(L_r & R_j) per sub-group, and the rows are added up at the end.
constexpr int kXPlanes = 5;
constexpr int kNormChunksMax = 2;             // 16-byte chunks of x a thread sums for the norm, at most

__device__ __forceinline__ uint32_t swiglu_pair(uint32_t g, uint32_t u)
{
    auto one = [](uint16_t gh, uint16_t uh) __attribute__((always_inline)) -> uint32_t {
        const float gf = h2f(gh);
        const float act = h2f(f2h(gf / (1.f + __expf(-gf))));
        return f2h(act * h2f(uh));
    };
    return one(static_cast<uint16_t>(g & 0xffffu), static_cast<uint16_t>(u & 0xffffu)) |
           (one(static_cast<uint16_t>(g >> 16), static_cast<uint16_t>(u >> 16)) << 16);
}

__device__ __forceinline__ uint32_t add_pair(uint32_t x, uint32_t d)
{
    const uint32_t lo = f2h(h2f(static_cast<uint16_t>(x & 0xffffu)) + h2f(static_cast<uint16_t>(d & 0xffffu)));
    const uint32_t hi = f2h(h2f(static_cast<uint16_t>(x >> 16)) + h2f(static_cast<uint16_t>(d >> 16)));
    return lo | (hi << 16);
}

__device__ __forceinline__ uint32_t norm_pair(uint32_t r, uint32_t w, float inv)
{
    const uint32_t lo = f2h(h2f(static_cast<uint16_t>(w & 0xffffu)) * h2f(f2h(h2f(static_cast<uint16_t>(r & 0xffffu)) * inv)));
    const uint32_t hi = f2h(h2f(static_cast<uint16_t>(w >> 16)) * h2f(f2h(h2f(static_cast<uint16_t>(r >> 16)) * inv)));
    return lo | (hi << 16);
}

// float -> the split-K accumulator's fixed point (2^-kAccFracBits), |v| <= kAccClamp.
// hi = rint(y * 2^(F-24)) and lo = y * 2^F - hi * 2^24 are exact in fp32.
__device__ __forceinline__ long long to_fixed(float y)
{
    y = fminf(fmaxf(y, -kAccClamp), kAccClamp);
    const float hi = __builtin_rintf(y * static_cast<float>(1 << (kAccFracBits - 24)));
    const float lo = fmaf(hi, -16777216.f, y * static_cast<float>(1 << kAccFracBits));
    return (static_cast<long long>(static_cast<int>(hi)) << 24) + static_cast<long long>(static_cast<int>(lo));
}

// S planes, MT row tiles (4 batch rows each), CT column tiles of 16 columns,
// SP sub-groups (128 elements of K) per wave.  A workgroup owns 16*CT columns;
// its waves (blockDim.x / 64 of them) split K: wave w of workgroup (nt, kp)
// takes sub-groups [(kp * waves + w) * SP, +SP), i.e. U = CT*SP units of 1 KiB
// of plane words.  The waves share nothing until their partial results meet in
// LDS, so nothing in a wave waits for another wave before that.  Straight-line
// code; every wait is for exactly the oldest outstanding load.  In a wave:
//   1. its first requests: its activations (one dword per lane, row and
//      sub-group), the line indices of its units, the plane words of its first
//      units (the later units are requested one at a time, in step 4);
//   2. the activations arrive first: they become the fp8 A operands (through
//      a 2 KiB LDS buffer of the wave's own, which does the byte transpose);
//   3. the indices arrive: the coefficient lines are gathered (vector loads
//      queued behind the stream, they arrive right after the last plane words);
//   4. every unit: four ANDs per plane word, MFMA, plane sums kept in registers;
//   5. coefficients applied; partial results to LDS, barrier, summed in a fixed
//      order by the first waves, written out (or added to the split-K words).
template <int S, int MT, int CT, int SP, int XM>
__global__ void __launch_bounds__(64 * gemv_max_waves(MT, CT))
__attribute__((amdgpu_waves_per_eu(gemv_waves(S, MT, CT, SP), 8)))
sbvr_gemv_mfma_kernel(const GemvArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int N = a.N, K = a.K;
    const int col = lane & 15;   // column inside a tile (B and D operands)
    const int blk = lane >> 4;   // word of the sub-group (B), batch row of the tile (D)
    const int sg0 = (blockIdx.y * waves + wave) * SP;     // first sub-group of this wave
    // The workgroup owns columns [n_own, n_own + wstride), wstride <= 16*CT a multiple
    // of 8 (half a tile is 128 bytes per word of K: whole cache lines).  It computes
    // a full window of 16*CT columns; a window that would stick out of N is moved
    // left, and the columns it then shares with its neighbour are left to the
    // neighbour.
    // Workgroups go to the 8 XCDs in turn (by their linear index, x first): give each XCD a contiguous range of
    // column windows instead of every eighth one (2-3 % at the 4096 <-> 14336 shapes).
    const int bx = gridDim.x % 8 == 0 ? static_cast<int>((blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8)
                                      : static_cast<int>(blockIdx.x);
    const int n_own = bx * a.wstride;
    const int n_base = min(n_own, N - CT * 16);
    // columns of the window that are this workgroup's to load: with wstride < 16*CT the rest of the last
    // tile is the next workgroup's (those lanes repeat the last own column: same cache line, no traffic,
    // and their results are dropped); a window moved left at the edge of N loads all of its columns
    const int w_lim = n_base == n_own ? a.wstride : CT * 16;
    unsigned char *const mine = smem + wave * 2048;        // this wave's buffer

    SBVR_STAMP(0);
    // -- 1. requests.  Unit u = (sub-group u / CT, column tile u % CT).
    constexpr int U = SP * CT;
    constexpr bool kNorm = XM == kXAddNorm || XM == kXAddNorm2;
    constexpr int NV = XM == kXAddNorm2 ? 2 : 1;                        // chunks of x and of delta per thread
    uint32_t xx[SP][MT][4];
    uint32_t x2[XM == kXSwiGLU ? SP : 1][XM == kXSwiGLU ? MT : 1][4];   // up (SwiGLU)
    uint32_t xw[kNorm ? SP : 1];                                        // norm weights
    v4u sx[NV], sd[NV];                                                 // this thread's share of all of x and delta
    if constexpr (XM == kXFloor) {
        // (no activations)
    } else if constexpr (XM == kXPlanes) {
        // lane l holds elements 2l, 2l + 1 of a sub-group: bits 2 (l % 16) and + 1 of its word l / 16
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi) {
            const int sg = sg0 + sgi;
            const int g = sg >> a.gshift;
            const int lline = a.x_idx16 ? static_cast<int>(static_cast<const uint16_t *>(a.xidx)[g])
                                        : static_cast<int>(static_cast<const uint8_t *>(a.xidx)[g]);
            const uint16_t *la = a.xcache + static_cast<size_t>(min(lline, a.xL - 1)) * a.M;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    xx[sgi][mt][r] = 0u;
                    if (mt == 0 && r < a.M) {                       // wave-uniform
                        const uint32_t w = a.xbvr[(static_cast<size_t>(4 * sg) + blk) * a.M + r];
                        const uint32_t two = (w >> (2 * col)) & 3u;
                        xx[sgi][mt][r] = __umul24((two & 1u) | ((two & 2u) << 15), static_cast<uint32_t>(la[r]));
                    }
                }
        }
    } else if constexpr (!kNorm) {
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    xx[sgi][mt][r] = 0u;
                    if constexpr (XM == kXSwiGLU)
                        x2[sgi][mt][r] = 0u;
                    if (XM != kXPlain ? mt * 4 + r < 1 : mt * 4 + r < a.M) {    // wave-uniform; one row with a prologue
                        const size_t at = static_cast<size_t>(mt * 4 + r) * a.xstride + static_cast<size_t>(sg0 + sgi) * kSub;
                        xx[sgi][mt][r] = reinterpret_cast<const uint32_t *>(a.x + at)[lane];
                        if constexpr (XM == kXSwiGLU)
                            x2[sgi][mt][r] = reinterpret_cast<const uint32_t *>(a.x + at + K)[lane];
                    }
                }
    } else {
        // (never conditional: a chunk past the end repeats the last one and is left out of the sum)
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = min(tid + j * static_cast<int>(blockDim.x), (K >> 3) - 1);
            sx[j] = reinterpret_cast<const v4u *>(a.x)[c];
            sd[j] = reinterpret_cast<const v4u *>(a.delta)[c];
        }
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi)
            xw[sgi] = reinterpret_cast<const uint32_t *>(a.norm_w + static_cast<size_t>(sg0 + sgi) * kSub)[lane];
        // (the waves meet before any of them asks for plane words: every wave's share of x is then ahead of
        // all of those in the CU's queue; no fence, nothing has been written yet.  0.1-0.15 us per launch)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    // line indices: one load per sub-group and 64 columns of the window, lane l takes the index of column
    // n_base + 64*iw + l; they are handed to the (tile, column) lanes later, in LDS permutes: every
    // vector-memory instruction saved is tens of nanoseconds of issue time
    constexpr int IW = (16 * CT + 63) / 64;
    int lraw[SP][IW];
#pragma unroll
    for (int iw = 0; iw < IW; ++iw) {
        const uint32_t lane_i = static_cast<uint32_t>(n_base + min(64 * iw + lane, 16 * CT - 1));
        if (a.idx16) {
#pragma unroll
            for (int sgi = 0; sgi < SP; ++sgi)
                lraw[sgi][iw] = static_cast<const uint16_t *>(a.idx)[static_cast<size_t>((sg0 + sgi) >> a.gshift) * N + lane_i];
        } else {
#pragma unroll
            for (int sgi = 0; sgi < SP; ++sgi)
                lraw[sgi][iw] = static_cast<const uint8_t *>(a.idx)[static_cast<size_t>((sg0 + sgi) >> a.gshift) * N + lane_i];
        }
    }
    Planes<S> q[U];
    const uint32_t lane_w = (static_cast<uint32_t>(blk) * N + n_base + col) * S;   // words
    const uint32_t lane_w_last = (static_cast<uint32_t>(blk) * N + n_base + min((CT - 1) * 16 + col, w_lim - 1)) * S;
    auto request_units = [&](int u0, int u1) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u >= u0 && u < u1) {
                const uint32_t *wrow = a.bvr + static_cast<size_t>(sg0 + u / CT) * 4 * N * S;     // wave-uniform
                q[u] = load_planes<S, true>(u % CT == CT - 1 ? wrow + lane_w_last : wrow + lane_w + (u % CT) * 16 * S);
            }
    };
    if constexpr (XM == kXFloor) {
        // every request of the real launch, then nothing: how long the memory system alone takes
        request_units(0, U);
        uint32_t seen = 0;
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi)
#pragma unroll
            for (int iw = 0; iw < IW; ++iw)
                seen ^= static_cast<uint32_t>(lraw[sgi][iw]);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < S; ++j)
                seen ^= q[u].w[j];
        if (seen == 0x9e3779b9u && a.M == 0x7fffffff)       // never true: keeps the loads alive
            a.out[lane] = static_cast<uint16_t>(seen);
        return;
    }
    // A wave keeps kUnitsAhead units in flight: the first ones are requested here, before the A operands are
    // made, and each unit that is worked on asks for the one kUnitsAhead behind it.  A CU takes about 48 such
    // requests at a time and hands the free places to its oldest waves first: a wave that asked for all of its
    // units at once would sit in the issue of its loads for microseconds (the youngest waves until the launch
    // is nearly over) and make its operands only after that.
    // (workgroups of at most 8 waves keep twice as many, for the same number of requests per CU)
    constexpr int kAhead = gemv_max_waves(MT, CT) == 8 ? 2 * kUnitsAhead : kUnitsAhead;
    constexpr int kPre = U < kAhead ? U : kAhead;
    // Only kUnitsFirst of them before the operands are made, the rest right behind them: with every wave's full
    // share asked for at once the CU's queue is full when its youngest waves come to ask for their activations,
    // and those waves then start their units a microsecond and more behind the oldest (4096 -> 14336: 7.8 -> 7.5 us;
    // one unit first was slower again).
    constexpr int kPre0 = kUnitsFirst * (kAhead / kUnitsAhead) < kPre ? kUnitsFirst * (kAhead / kUnitsAhead) : kPre;
    request_units(0, kPre0);
    __builtin_amdgcn_sched_barrier(0);       // these requests are out before anything waits
    SBVR_STAMP(1);

    // -- 2. A operands.  A lane turns two elements of a batch row into 3 fp8
    //       terms each and drops the bytes where the MFMA wants them; the lane
    //       then reads its 32 bytes back.  Row tiles go from the last one, the
    //       only one that may have fewer than 4 rows, to the first, so a row of
    //       the buffer that is not rewritten holds zeros.
    float inv = 0.f;             // with the norm: rsqrt(mean((x + delta)^2) + eps)
    if constexpr (kNorm) {
        float ss = 0.f;
        float *const sums = reinterpret_cast<float *>(smem + waves * 2048);
        v4u *const rbuf = reinterpret_cast<v4u *>(smem + waves * 2048 + 64);      // r = fp16(x + delta), all of K
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = tid + j * static_cast<int>(blockDim.x);
            const bool counts = c < (K >> 3);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t r = add_pair(sx[j][e], sd[j][e]);
                sx[j][e] = r;
                const float lo = h2f(static_cast<uint16_t>(r & 0xffffu)), hi = h2f(static_cast<uint16_t>(r >> 16));
                ss += counts ? fmaf(lo, lo, hi * hi) : 0.f;
            }
            if (counts)
                rbuf[c] = sx[j];
        }
        ss = wave_fsum(ss);
        if (lane == 0)
            sums[wave] = ss;
        __syncthreads();
        float total = 0.f;
        for (int w = 0; w < waves; ++w)
            total += sums[w];
        inv = rsqrtf(total / static_cast<float>(K) + a.eps);
        // the wave's own elements of r (batch row 0)
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    xx[sgi][mt][r] = 0u;
            xx[sgi][0][0] = reinterpret_cast<const uint32_t *>(rbuf)[(sg0 + sgi) * (kSub / 2) + lane];
        }
    }
#ifdef SBVR_TRACE
    if constexpr (!kNorm) {
        asm volatile("" :: "v"(xx[SP - 1][0][0]));
        SBVR_STAMP(7);
    }
#endif
    // (raised priority: the SIMD's other waves are in their units by now, and this wave would get a turn
    // only between their MFMAs -- measured up to 2.5 us for the 0.3 us of work; its own units wait for this)
    __builtin_amdgcn_s_setprio(3);
    v8i A[SP][MT];
    float scale[SP][MT];         // of this lane's batch row (blk)
    const int m_rows = XM == kXPlain || XM == kXPlanes ? a.M : 1;
    // Lane l = 4g + t of a row's 64 takes elements 8g + t and 8g + t + 4 of the sub-group: the same bit t of two
    // neighbouring nibbles of a plane word, which are neighbouring bytes of the A image (one 16-bit store per
    // term) and share the weight of their B digits (0.5, 1, 2, 2 for t = 0..3, made up for here: 4, 2, 1, 1).
    const int off = a_image_byte_offset(8 * (lane >> 2) + (lane & 3), 0);
    const uint32_t half_sel = (lane & 1) ? 0x07060302u : 0x05040100u;      // (odd t: the high halves of the dwords)
    const int fac_log2 = (lane & 3) == 0 ? 2 : ((lane & 3) == 1 ? 1 : 0);
    // the operands of sub-groups [s0, s1) of this wave
    auto make_operands = [&](int s0, int s1) __attribute__((always_inline)) {
#pragma unroll
        for (int sgi = 0; sgi < SP; ++sgi) {
            if (sgi < s0 || sgi >= s1)
                continue;
            reinterpret_cast<uint4 *>(mine)[lane * 2] = uint4{0u, 0u, 0u, 0u};
            reinterpret_cast<uint4 *>(mine)[lane * 2 + 1] = uint4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int mt = MT - 1; mt >= 0; --mt) {
                scale[sgi][mt] = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (mt * 4 + r < m_rows) {      // wave-uniform
                        uint32_t v = xx[sgi][mt][r];
                        if constexpr (XM == kXSwiGLU)
                            v = swiglu_pair(v, x2[sgi][mt][r]);
                        if constexpr (kNorm)
                            v = norm_pair(v, xw[sgi], inv);
                        // 2^e puts the largest magnitude of the sub-group into [32, 64)
                        // (fp16 bits order like magnitudes; subnormals count as 2^-15)
                        const uint32_t amax = wave_umax(max(v & 0x7fffu, (v >> 16) & 0x7fffu));
                        const int eh = min(max(static_cast<int>(amax >> 10), 1), 30);
                        const int e = 20 - eh;
                        if (blk == r)            // products come out as 2 * x * 2^e
                            scale[sgi][mt] = __uint_as_float(static_cast<uint32_t>(126 - e) << 23);
                        // the lane's two elements, from the dwords (2l, 2l + 1) the lanes of its quad loaded
                        const int va = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x50, 0xF, 0xF, true);   // quad_perm 0,0,1,1
                        const int vb = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xFA, 0xF, 0xF, true);   // quad_perm 2,2,3,3
                        v2h z = as_v2h(__builtin_amdgcn_perm(static_cast<uint32_t>(vb), static_cast<uint32_t>(va), half_sel));
                        // h1 + h2 + h3/256 == z * 2^e * weight exactly: each fp8 takes the next 4 significant bits
                        // (the conversions divide by their scale operand), the last one of the residual scaled up
                        // out of the subnormals; the residuals are exact in fp16
                        const float sc = __uint_as_float(static_cast<uint32_t>(127 - e - fac_log2) << 23);
                        const float sc_last = __uint_as_float(static_cast<uint32_t>(127 - 8 - e - fac_log2) << 23);
                        static_assert(kLastTermScale == 256.f, "the last term's scale is 2^8 here");
                        v2s b = {0, 0};
                        b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, false);
                        z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, false);
                        b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, true);
                        z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, true);
                        const v2s b3 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(v2s{0, 0}, z, sc_last, false);
                        *reinterpret_cast<short *>(mine + off + (r * 4 + 0) * 32) = b[0];
                        *reinterpret_cast<short *>(mine + off + (r * 4 + 1) * 32) = b[1];
                        *reinterpret_cast<short *>(mine + off + (r * 4 + 2) * 32) = b3[0];
                    }
                }
                A[sgi][mt] = *reinterpret_cast<const v8i *>(mine + lane * 32);
            }
        }
    };
    make_operands(0, SP);
    request_units(kPre0, kPre);
    __builtin_amdgcn_sched_barrier(0);
    SBVR_STAMP(2);

    // -- 3. coefficient lines (S fp16 each): lane l gathers the line of column n_base + l for each
    //       sub-group, then the (tile, column) lanes pick theirs up with LDS permutes
    constexpr int CW = (S + 1) / 2;          // dwords per line
    uint32_t cl[SP][IW][CW];
#pragma unroll
    for (int sgi = 0; sgi < SP; ++sgi)
#pragma unroll
        for (int iw = 0; iw < IW; ++iw) {
            const uint32_t line = static_cast<uint32_t>(min(lraw[sgi][iw], a.L - 1));
            load_line_words<S>(a.cache + line * S, cl[sgi][iw]);
        }
    SBVR_STAMP(3);

    // -- 4. the units: plane sums of every (unit, row tile, plane), and one unit behind them
    // -- 5. coefficients and scales: the lane holds column n_base + 16*ct + col of batch row 4*mt + blk.
    //       The coefficients of unit u - 1 are applied behind the MFMAs of unit u: arithmetic that does not
    //       depend on them, for the time they take; and only one unit's plane sums are alive at a time.
    float y[CT][MT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            y[ct][mt] = 0.f;
    float ps[MT][S];                 // plane sums of the unit before the one in the matrix cores
    uint32_t cqu[CW];                // and that unit's coefficient line, on its way through the LDS permute
    // (the lane that gathered the line of column 16*ct + col of the window hands it over)
    auto fetch_coefficients = [&](int u) __attribute__((always_inline)) {
        const int sgi = u / CT, ct = u % CT;
#pragma unroll
        for (int j = 0; j < CW; ++j)
            cqu[j] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(((ct * 16 + col) & 63) * 4,
                                                                          static_cast<int>(cl[sgi][(ct * 16) / 64][j])));
    };
    auto apply_coefficients = [&](int u) __attribute__((always_inline)) {
        const int sgi = u / CT, ct = u % CT;
        float c[S];
#pragma unroll
        for (int j = 0; j < S; ++j)
            c[j] = h2f(static_cast<uint16_t>(j & 1 ? cqu[j / 2] >> 16 : cqu[j / 2] & 0xffffu));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < S; ++j)
                acc = fmaf(c[j], ps[mt][j], acc);
            y[ct][mt] = fmaf(acc, scale[sgi][mt], y[ct][mt]);
        }
    };
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int sgi = u / CT;
        // A wave's priority falls as it gets through its units (2, 2, 1, 0 over their quarters, below the 3 of a
        // wave that is making its operands): the CU gives its instruction slots and the free places of its memory
        // queue to the oldest wave among equals, so with one priority for all the youngest waves of a workgroup
        // finished their units 2 us after the oldest, which then sat at the barrier below (median wait 1.2 us, 0.6 us
        // with this; 7.5 -> 7.4 us at 4096 -> 14336).
        if (u == 0 || (u * 4) / U != ((u - 1) * 4) / U)
            switch ((0x2210 >> (4 * (3 - (u * 4) / U))) & 0xf) {               // (u is a constant once the loop is unrolled)
            case 3: __builtin_amdgcn_s_setprio(3); break;
            case 2: __builtin_amdgcn_s_setprio(2); break;
            case 1: __builtin_amdgcn_s_setprio(1); break;
            default: __builtin_amdgcn_s_setprio(0); break;
            }
        request_units(u + kPre, u + kPre + 1);      // keeps kPre units of this wave in flight
        if (u > 0)
            fetch_coefficients(u - 1);              // (on its way while this unit's operands are made)
        __builtin_amdgcn_sched_barrier(0);
        v4f D[MT][S];
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const uint32_t w = q[u].w[j];
            v8i B;
            B[0] = static_cast<int>(w & 0x11111111u);
            B[1] = static_cast<int>(w & 0x22222222u);
            B[2] = static_cast<int>(w & 0x44444444u);
            B[3] = static_cast<int>((w >> 1) & 0x44444444u);
            B[4] = 0; B[5] = 0; B[6] = 0; B[7] = 0;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4f z = {0.f, 0.f, 0.f, 0.f};
                D[mt][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[sgi][mt], B, z, 0, 4, 0, 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (u > 0)
            apply_coefficients(u - 1);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < S; ++j) {
                ps[mt][j] = fmaf(D[mt][j][2], 1.f / kLastTermScale, D[mt][j][0] + D[mt][j][1]);
                asm volatile("" : "+v"(ps[mt][j]));          // keeps the units in program order
            }
        __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
    fetch_coefficients(U - 1);
    apply_coefficients(U - 1);
    SBVR_STAMP(4);
    //       partial results meet in LDS: wave w's buffer holds [ct][mt][lane] floats
    // (up to 8 blocks per wave they fit the wave's own 2 KiB buffer; more go behind the buffers of all waves,
    // because another wave may still be building operands in its buffer)
    constexpr int kRedStride = CT * MT <= 8 ? 512 : CT * MT * 64;        // floats per wave
    float *const red = reinterpret_cast<float *>(smem + (CT * MT <= 8 ? 0 : waves * 2048));
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            red[wave * kRedStride + (ct * MT + mt) * 64 + lane] = y[ct][mt];
    __syncthreads();
    SBVR_STAMP(5);

    const bool shifted = n_base != n_own;            // window moved left at the edge of N
    for (int o = wave; o < CT * MT; o += waves) {    // wave-uniform
        const int ct = o / MT, mt = o % MT;
        float total = 0.f;
        for (int w = 0; w < waves; ++w)
            total += red[w * kRedStride + o * 64 + lane];
        if constexpr (XM == kXPlanes) {      // the rows are the left operand's planes: the output is their sum
            total += __shfl_xor(total, 16, 64);
            total += __shfl_xor(total, 32, 64);
        }
        const int n = n_base + ct * 16 + col, m = mt * 4 + blk;
        const bool valid = (XM == kXPlanes ? m == 0 : m < a.M) && (!shifted || n >= n_own) && n < n_own + a.wstride;
        const size_t at = static_cast<size_t>(m) * N + n;
        if (a.ksplit > 1) {
            // through the accumulators: the adder that completes the count converts
            unsigned long long tot = (1ull << 56) + static_cast<unsigned long long>(to_fixed(total) + kAccBias);
            unsigned long long old = 0ull;
            if (valid)
                old = __hip_atomic_fetch_add(a.acc + at, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            tot += old;
            if (!valid || static_cast<int>(tot >> 56) != a.ksplit)
                continue;
            // the sum without the count and the ksplit biases, back to float:
            // sum = hi * 2^24 + lo, both halves exact in fp32, one rounding
            const long long sum = static_cast<long long>(tot & ((1ull << 56) - 1)) - (static_cast<long long>(a.ksplit) << 47);
            const float hi = static_cast<float>(static_cast<int>(sum >> 24));
            const float lo = static_cast<float>(static_cast<int>(sum & 0xffffff));
            total = fmaf(hi, 1.f / (1 << (kAccFracBits - 24)), lo * (1.f / (1 << kAccFracBits)));
            __hip_atomic_store(a.acc + at, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (!valid) {
            continue;
        }
        uint16_t r = f2h(total);
        if (a.bias)
            r = hadd(r, a.bias[n]);
        a.out[at] = r;
    }
    if constexpr (kNorm) {
        if (blockIdx.x == 0 && blockIdx.y == 0) {
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int c = tid + j * static_cast<int>(blockDim.x);
                if (c < (K >> 3))
                    reinterpret_cast<v4u *>(a.x_out)[c] = sx[j];
            }
        }
    }
    SBVR_STAMP(6);
}

// 5..16 batch rows (MT = 2 or 4 row tiles of 4).  Per row and sub-group the A operands cost some 30 VALU
// instructions, as much as a unit's own arithmetic, so here MT waves share the operands of a sub-group: wave
// (group g, role r) of a workgroup makes row tile r of the group's SP sub-groups (into LDS, where the byte
// transpose happens anyway), and after one barrier reads all MT tiles back and takes CTW of the group's
// CTW * MT column tiles.  A workgroup owns 16 * CTW * MT columns and waves / MT sub-group sets; everything
// else (requests a few units ahead, edge windows, LDS reduction, split-K accumulators) is as in the kernel
// above.  The MFMAs of a unit go two planes at a time, so that four row tiles fit 128 registers.
template <int S, int MT, int CTW, int SP>
__global__ void __launch_bounds__(64 * kMaxWaves)
sbvr_gemv_batch_kernel(const GemvArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    static_assert(MT == 2 || MT == 4, "two or four row tiles");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int groups = waves / MT;
    const int grp = wave / MT, role = wave % MT;
    const int N = a.N;
    const int col = lane & 15;   // column inside a tile (B and D operands)
    const int blk = lane >> 4;   // word of the sub-group (B), batch row of the tile (D)
    const int sg0 = (blockIdx.y * groups + grp) * SP;     // first sub-group of this wave's group
    constexpr int W = CTW * MT * 16;                      // columns of the workgroup's window
    const int bx = gridDim.x % 8 == 0 ? static_cast<int>((blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8)
                                      : static_cast<int>(blockIdx.x);
    const int n_own = bx * a.wstride;
    const int n_base = min(n_own, N - W);
    const int w_lim = n_base == n_own ? a.wstride : W;    // (columns of the window that are this workgroup's to load)
    const int ws = role * CTW * 16;                       // this wave's columns of the window start here
    unsigned char *const images = smem;                                                    // [group][sub-group][row tile] 2 KiB
    float *const scl = reinterpret_cast<float *>(smem + waves * SP * 2048);                // [group][sub-group][row tile][row]
    float *const red = reinterpret_cast<float *>(smem + waves * SP * (2048 + 16));         // [wave][tile][row tile][lane]

    SBVR_STAMP(0);
    // -- 1. requests
    constexpr int U = SP * CTW;
    uint32_t xx[SP][4];
#pragma unroll
    for (int sgi = 0; sgi < SP; ++sgi)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            xx[sgi][r] = 0u;
            if (role * 4 + r < a.M) {        // wave-uniform
                const size_t at = static_cast<size_t>(role * 4 + r) * a.xstride + static_cast<size_t>(sg0 + sgi) * kSub;
                xx[sgi][r] = reinterpret_cast<const uint32_t *>(a.x + at)[lane];
            }
        }
    constexpr int IW = (16 * CTW + 63) / 64;
    int lraw[SP][IW];
#pragma unroll
    for (int iw = 0; iw < IW; ++iw) {
        const uint32_t lane_i = static_cast<uint32_t>(n_base + ws + min(64 * iw + lane, 16 * CTW - 1));
        if (a.idx16) {
#pragma unroll
            for (int sgi = 0; sgi < SP; ++sgi)
                lraw[sgi][iw] = static_cast<const uint16_t *>(a.idx)[static_cast<size_t>((sg0 + sgi) >> a.gshift) * N + lane_i];
        } else {
#pragma unroll
            for (int sgi = 0; sgi < SP; ++sgi)
                lraw[sgi][iw] = static_cast<const uint8_t *>(a.idx)[static_cast<size_t>((sg0 + sgi) >> a.gshift) * N + lane_i];
        }
    }
    Planes<S> q[U];
    auto request_units = [&](int u0, int u1) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u >= u0 && u < u1) {
                const uint32_t *wrow = a.bvr + static_cast<size_t>(sg0 + u / CTW) * 4 * N * S;     // wave-uniform
                // (columns past the workgroup's own repeat its last one: same cache line, results dropped)
                const int wc = min(ws + (u % CTW) * 16 + col, w_lim - 1);
                q[u] = load_planes<S, true>(wrow + (static_cast<uint32_t>(blk) * N + n_base + wc) * S);
            }
    };
    constexpr int kPre = U < kUnitsAhead ? U : kUnitsAhead;
    // (one unit before the operands are made, the others right behind them, and the priority ladder of the kernel
    // above over the units: 12.0 -> 11.4 us at 8 rows of 4096 -> 14336, 12.1 -> 11.4 at 14336 -> 4096)
    constexpr int kPre0 = 1;
    request_units(0, kPre0);
    __builtin_amdgcn_sched_barrier(0);
    SBVR_STAMP(1);

    // -- 2. this wave's row tile of the group's A operands
    const int off = a_image_byte_offset(8 * (lane >> 2) + (lane & 3), 0);
    const uint32_t half_sel = (lane & 1) ? 0x07060302u : 0x05040100u;
    const int fac_log2 = (lane & 3) == 0 ? 2 : ((lane & 3) == 1 ? 1 : 0);
    __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int sgi = 0; sgi < SP; ++sgi) {
        const int slot = (grp * SP + sgi) * MT + role;
        unsigned char *const img = images + slot * 2048;
        reinterpret_cast<uint4 *>(img)[lane * 2] = uint4{0u, 0u, 0u, 0u};
        reinterpret_cast<uint4 *>(img)[lane * 2 + 1] = uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float row_scale = 0.f;
            if (role * 4 + r < a.M) {      // wave-uniform
                const uint32_t v = xx[sgi][r];
                const uint32_t amax = wave_umax(max(v & 0x7fffu, (v >> 16) & 0x7fffu));
                const int eh = min(max(static_cast<int>(amax >> 10), 1), 30);
                const int e = 20 - eh;
                row_scale = __uint_as_float(static_cast<uint32_t>(126 - e) << 23);
                const int va = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x50, 0xF, 0xF, true);   // quad_perm 0,0,1,1
                const int vb = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xFA, 0xF, 0xF, true);   // quad_perm 2,2,3,3
                v2h z = as_v2h(__builtin_amdgcn_perm(static_cast<uint32_t>(vb), static_cast<uint32_t>(va), half_sel));
                const float sc = __uint_as_float(static_cast<uint32_t>(127 - e - fac_log2) << 23);
                const float sc_last = __uint_as_float(static_cast<uint32_t>(127 - 8 - e - fac_log2) << 23);
                v2s b = {0, 0};
                b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, false);
                z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, false);
                b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, true);
                z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, true);
                const v2s b3 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(v2s{0, 0}, z, sc_last, false);
                *reinterpret_cast<short *>(img + off + (r * 4 + 0) * 32) = b[0];
                *reinterpret_cast<short *>(img + off + (r * 4 + 1) * 32) = b[1];
                *reinterpret_cast<short *>(img + off + (r * 4 + 2) * 32) = b3[0];
            }
            if (lane == 0)
                scl[slot * 4 + r] = row_scale;
        }
    }
    request_units(kPre0, kPre);
    __builtin_amdgcn_sched_barrier(0);
    SBVR_STAMP(7);
    __syncthreads();
    SBVR_STAMP(2);

    // -- 3. coefficient lines: lane l gathers the line of this wave's column l (+ 64 iw) for each sub-group
    constexpr int CW = (S + 1) / 2;
    uint32_t cl[SP][IW][CW];
#pragma unroll
    for (int sgi = 0; sgi < SP; ++sgi)
#pragma unroll
        for (int iw = 0; iw < IW; ++iw) {
            const uint32_t line = static_cast<uint32_t>(min(lraw[sgi][iw], a.L - 1));
            load_line_words<S>(a.cache + line * S, cl[sgi][iw]);
        }

    SBVR_STAMP(3);
    // -- 4. the units
    float y[CTW][MT];
#pragma unroll
    for (int t = 0; t < CTW; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            y[t][mt] = 0.f;
#pragma unroll
    for (int sgi = 0; sgi < SP; ++sgi) {
        v8i A[MT];
        float scale[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int slot = (grp * SP + sgi) * MT + mt;
            A[mt] = *reinterpret_cast<const v8i *>(images + slot * 2048 + lane * 32);
            scale[mt] = scl[slot * 4 + blk];
        }
#pragma unroll
        for (int t = 0; t < CTW; ++t) {
            const int u = sgi * CTW + t;
            if (u == 0 || (u * 4) / U != ((u - 1) * 4) / U)
                switch ((0x2210 >> (4 * (3 - (u * 4) / U))) & 0xf) {
                case 2: __builtin_amdgcn_s_setprio(2); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                default: __builtin_amdgcn_s_setprio(0); break;
                }
            request_units(u + kPre, u + kPre + 1);
            float c[S];
            {
                uint32_t cqu[CW];
#pragma unroll
                for (int j = 0; j < CW; ++j)
                    cqu[j] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(((t * 16 + col) & 63) * 4,
                                                                                  static_cast<int>(cl[sgi][(t * 16) / 64][j])));
#pragma unroll
                for (int j = 0; j < S; ++j)
                    c[j] = h2f(static_cast<uint16_t>(j & 1 ? cqu[j / 2] >> 16 : cqu[j / 2] & 0xffffu));
            }
            float acc[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt] = 0.f;
#pragma unroll
            for (int j0 = 0; j0 < S; j0 += 2) {
                v4f D[MT][2];
#pragma unroll
                for (int j = j0; j < S && j < j0 + 2; ++j) {
                    const uint32_t w = q[u].w[j];
                    v8i B;
                    B[0] = static_cast<int>(w & 0x11111111u);
                    B[1] = static_cast<int>(w & 0x22222222u);
                    B[2] = static_cast<int>(w & 0x44444444u);
                    B[3] = static_cast<int>((w >> 1) & 0x44444444u);
                    B[4] = 0; B[5] = 0; B[6] = 0; B[7] = 0;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        const v4f z = {0.f, 0.f, 0.f, 0.f};
                        D[mt][j - j0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[mt], B, z, 0, 4, 0, 0, 0, 0);
                    }
                }
#pragma unroll
                for (int j = j0; j < S && j < j0 + 2; ++j)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt] = fmaf(c[j], fmaf(D[mt][j - j0][2], 1.f / kLastTermScale, D[mt][j - j0][0] + D[mt][j - j0][1]), acc[mt]);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                y[t][mt] = fmaf(acc[mt], scale[mt], y[t][mt]);
        }
    }

    __builtin_amdgcn_s_setprio(0);
    SBVR_STAMP(4);
    // -- 5. partial results meet in LDS; summed over the groups in a fixed order
    constexpr int kBlocks = CTW * MT;                 // (tile, row tile) blocks of a wave
#pragma unroll
    for (int t = 0; t < CTW; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            red[(wave * kBlocks + t * MT + mt) * 64 + lane] = y[t][mt];
    __syncthreads();
    SBVR_STAMP(5);

    const bool shifted = n_base != n_own;            // window moved left at the edge of N
    for (int o = wave; o < kBlocks * MT; o += waves) {    // wave-uniform
        const int role_o = o / kBlocks, rest = o % kBlocks;
        const int t = rest / MT, mt = rest % MT;
        float total = 0.f;
        for (int g = 0; g < groups; ++g)
            total += red[((g * MT + role_o) * kBlocks + rest) * 64 + lane];
        const int n = n_base + (role_o * CTW + t) * 16 + col, m = mt * 4 + blk;
        const bool valid = m < a.M && (!shifted || n >= n_own) && n < n_own + a.wstride;
        const size_t at = static_cast<size_t>(m) * N + n;
        if (a.ksplit > 1) {
            unsigned long long tot = (1ull << 56) + static_cast<unsigned long long>(to_fixed(total) + kAccBias);
            unsigned long long old = 0ull;
            if (valid)
                old = __hip_atomic_fetch_add(a.acc + at, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            tot += old;
            if (!valid || static_cast<int>(tot >> 56) != a.ksplit)
                continue;
            const long long sum = static_cast<long long>(tot & ((1ull << 56) - 1)) - (static_cast<long long>(a.ksplit) << 47);
            const float hi = static_cast<float>(static_cast<int>(sum >> 24));
            const float lo = static_cast<float>(static_cast<int>(sum & 0xffffff));
            total = fmaf(hi, 1.f / (1 << (kAccFracBits - 24)), lo * (1.f / (1 << kAccFracBits)));
            __hip_atomic_store(a.acc + at, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (!valid) {
            continue;
        }
        uint16_t r = f2h(total);
        if (a.bias)
            r = hadd(r, a.bias[n]);
        a.out[at] = r;
    }
    SBVR_STAMP(6);
}

// Launch shape for the MFMA kernel.
struct GemvPlan {
    int CT, SP, MT, waves, n_wgs, ksplit;
    size_t lds;
    int wstride;
};

// Development switches.  A library built with -DSBVR_DEV_SWITCHES reads them from the environment once per
// process (SBVR_HIP_CT, _SP, _WAVES, _WSTRIDE, _SHOW_PLAN, _POPC_Q, _ROWDEQ_LANES, _LUT_ROWS, _PF_LUT); the
// library as shipped does not look at the environment: launch shapes and the choice of kernel (and with it the
// rounding) depend on the arguments of a call alone.
struct EnvSwitches {
    int ct, sp, waves, wstride, show_plan, popc_q, rowdeq_lanes, lut_rows, pf_lut;
};

#ifndef SBVR_DEV_SWITCHES
const EnvSwitches &env_switches()
{
    static const EnvSwitches none{};
    return none;
}
#else
const EnvSwitches &env_switches()
{
    static const EnvSwitches e = [] {
        auto get = [](const char *name) {
            const char *v = getenv(name);
            return v && *v ? atoi(v) : 0;
        };
        return EnvSwitches{get("SBVR_HIP_CT"), get("SBVR_HIP_SP"), get("SBVR_HIP_WAVES"), get("SBVR_HIP_WSTRIDE"),
                           get("SBVR_HIP_SHOW_PLAN"), get("SBVR_HIP_POPC_Q"), get("SBVR_HIP_ROWDEQ_LANES"), get("SBVR_HIP_LUT_ROWS"), get("SBVR_HIP_PF_LUT")};
    }();
    return e;
}
#endif

// (CT, SP) pairs that have a kernel instance; see the dispatch below.
constexpr int kShapes[][2] = {{1, 1}, {1, 2}, {1, 4}, {1, 7}, {2, 1}, {2, 2}, {2, 4}, {2, 7}, {4, 1}, {4, 2}, {4, 4}, {7, 2}};
constexpr int kNumShapes = sizeof(kShapes) / sizeof(kShapes[0]);

constexpr bool shape_ok_for(int MT, int CT, int SP)
{
    // (the partial results of a wave, CT*MT*64 floats, fit its 2 KiB buffer up to CT*MT = 8 and get room
    // of their own beyond; two row tiles with a 16-wave launch bound, 128 registers: at most 4 sub-groups
    // of operands, and 4 only with one column tile)
    return CT * MT <= 16 && (MT == 1 || CT * SP * MT <= 16) && (MT != 2 || (SP <= 4 && CT * SP <= 8 && !(SP == 4 && CT > 1)));
}

bool has_instance(int CT, int SP)
{
    for (int i = 0; i < kNumShapes; ++i)
        if (kShapes[i][0] == CT && kShapes[i][1] == SP)
            return true;
    return false;
}

// Picks the launch shape.  Measured on MI355X (Llama-3-8B layer shapes, batch 1):
//  1. Where 16 waves can cover all of K with at most two sub-groups per column tile each, one workgroup
//     takes all of K (no accumulators, no atomics) and the columns are cut into windows of a multiple of
//     8 columns such that the workgroups are a whole multiple of the CUs: the launch is bound by what a CU
//     can have in flight, so a CU with 4 workgroups where others have 3 sets the time of the whole launch
//     (4096 -> 14336 on 256 CUs: 256 windows of 56 columns, 7.9 us against 8.6 us for 224 x 4 of 64).
//  2. Otherwise:
//  - about 4 units per wave when there is enough work for 4096 such waves, fewer otherwise, with as many
//    of them as possible along N (one sub-group per wave means one set of A operands per wave);
//  - at least two workgroups per CU, so K is split across workgroups (through
//    the accumulators) when N alone does not give that many;
//  - the largest workgroup that keeps that, but no more than 8 waves when the
//    waves do not all fit on the chip at once (finer placement).
GemvPlan plan_gemv_uncached(int M, int N, int K, int S, int cus, int min_waves)
{
    const int nsub = K / kSub;
    const int MT = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
    const int tiles16 = (N + 15) / 16;
    const EnvSwitches &env = env_switches();
    const int eCT = env.ct, eSP = env.sp, eW = env.waves;
    GemvPlan best{};
    // (the add + norm prologue, min_waves > 1, takes the same shapes: its barrier falls while the first units are in
    // flight; 4096 -> 28672 with it 12.4 us as 256 x 16 waves against 14.9 us as 512 x 8 waves of four sub-groups)
    const int wg_waves = std::min(kMaxWaves, gemv_max_waves(MT, 0));      // (never above the kernel's launch bound)
    if (best.CT == 0 && eCT <= 0 && nsub % wg_waves == 0 && wg_waves >= min_waves && N >= 16 * cus) {
        const int SP = nsub / wg_waves;
        // windows of wstride columns, r workgroups per CU; one workgroup per CU takes up to 7 tiles (4096 -> 28672:
        // 256 windows of 112 columns 11.8 us, 512 of 56 columns 13.1-13.5 us)
        const int widest = 112;
        for (int r = (N + widest * cus - 1) / (widest * cus); r <= 4; ++r) {
            const int wstride = ((N + cus * r - 1) / (cus * r) + 7) / 8 * 8;
            const int CT = (wstride + 15) / 16;
            if (wstride < 16)
                break;
            if (!has_instance(CT, SP) || !shape_ok_for(MT, CT, SP) || SP > 2 * CT || CT * 16 > N)
                continue;
            best = GemvPlan{CT, SP, MT, wg_waves, (N + wstride - 1) / wstride, 1, 0, wstride};
            break;
        }
    }
    if (best.CT == 0) {
        const long units = static_cast<long>(tiles16) * nsub;
        // (8 units per wave for the largest matrices: 14336 -> 4096 measured 8.2-8.3 us with 4 tiles x 2 sub-groups
        // against 8.6-8.7 with 4 x 1)
        int want = units >= 12L * 2048 && MT == 1 ? 8 : (units >= 8L * 2048 ? 4 : (units >= 2L * 2048 ? 2 : 1));
        while (want > 1 && want <= 4 && !shape_ok_for(MT, want, 1))
            want /= 2;
        double best_cost = 1e30;
        for (int i = 0; i < kNumShapes; ++i) {
            const int CT = kShapes[i][0], SP = kShapes[i][1];
            if (nsub % SP || !shape_ok_for(MT, CT, SP) || CT * 16 > N)
                continue;
            if (eCT > 0 && eSP > 0 && (CT != eCT || SP != eSP))
                continue;
            const int parts = nsub / SP;             // wave-sized pieces of K
            const int n_wgs = (tiles16 + CT - 1) / CT;
            const long total_waves = static_cast<long>(n_wgs) * parts;
            const int max_waves = total_waves > 32L * cus ? 8 : kMaxWaves;
            for (int waves = 1; waves <= gemv_max_waves(MT, CT); ++waves) {
                if (parts % waves || parts / waves > kMaxKsplit || (eW > 0 && waves != eW) || waves < min_waves)
                    continue;
                const int ksplit = parts / waves;
                const int U = CT * SP;
                double cost = 0.0;
                cost += U == want ? 0.0 : (U < want ? 2.0 * (want - U) : 1.0 * (U - want));
                cost += 0.5 * (SP - 1);                                          // A operands per wave
                cost += static_cast<double>(n_wgs) * CT / tiles16 - 1.0;        // columns computed twice at the edge of N
                if (static_cast<long>(n_wgs) * ksplit < 2L * cus)
                    cost += 3.0 * (1.0 - static_cast<double>(n_wgs) * ksplit / (2.0 * cus));
                if (waves > max_waves)
                    cost += 1.0;
                cost -= 0.01 * waves;                                            // larger workgroups, fewer accumulations
                if (eCT > 0 && eSP > 0 && eW > 0)
                    cost = 0.0;
                if (cost < best_cost) {
                    best_cost = cost;
                    best = GemvPlan{CT, SP, MT, waves, n_wgs, ksplit, 0, CT * 16};
                }
            }
        }
        const int ews = env.wstride;
        if (best.CT > 0 && ews > 0 && ews % 8 == 0 && ews <= best.CT * 16 && ews > (best.CT - 1) * 16) {
            best.wstride = ews;
            best.n_wgs = (N + ews - 1) / ews;
        }
    }
    best.lds = static_cast<size_t>(best.waves) * (2048 + (best.CT * best.MT <= 8 ? 0 : best.CT * best.MT * 256));
    return best;
}

// The plan is a function of the shape alone: kept per shape (a decode step asks for the same few shapes
// thousands of times a second).
GemvPlan plan_gemv(int M, int N, int K, int S, int cus, int min_waves = 1)
{
    struct Entry {
        int M, N, K, S, cus, min_waves;
        GemvPlan plan;
    };
    constexpr int kEntries = 64;
    static Entry cache[kEntries];
    static int used = 0;
    static std::mutex lock;
    std::lock_guard<std::mutex> guard(lock);
    for (int i = 0; i < used; ++i) {
        const Entry &e = cache[i];
        if (e.M == M && e.N == N && e.K == K && e.S == S && e.cus == cus && e.min_waves == min_waves)
            return e.plan;
    }
    const GemvPlan p = plan_gemv_uncached(M, N, K, S, cus, min_waves);
    if (used < kEntries)
        cache[used++] = Entry{M, N, K, S, cus, min_waves, p};
    return p;
}

bool mfma_path_ok(int M, int N, int K, int S, int G)
{
    // 32-bit element offsets into bvr
    return M >= 1 && M <= kMaxM && N >= 16 && K % kSub == 0 && G % kSub == 0 && ((G / kSub) & (G / kSub - 1)) == 0 &&
           (S == 2 || S == 3 || S == 4 || S == 6 || S == 8) &&
           static_cast<double>(K / 32) * N * S < 2147483648.0;
}

template <int S, int MT, int CT, int SP, int XM>
hipError_t launch_gemv_inst(const GemvArgs &a, const GemvPlan &p, hipStream_t st)
{
    const dim3 grid(static_cast<unsigned>(p.n_wgs), static_cast<unsigned>(p.ksplit)), block(64 * p.waves);
    if (p.lds > 65536) {        // (the wide shapes' partial results) above what a kernel gets without asking
        static bool raised_on[16] = {};
        std::lock_guard<std::mutex> guard(g_dev_lock);
        int dev_now = 0;
        if (hipGetDevice(&dev_now) != hipSuccess || dev_now < 0 || dev_now >= 16)
            dev_now = 0;
        if (!raised_on[dev_now]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sbvr_gemv_mfma_kernel<S, MT, CT, SP, XM>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess)
                return e;
            raised_on[dev_now] = true;
        }
    }
    hipLaunchKernelGGL((sbvr_gemv_mfma_kernel<S, MT, CT, SP, XM>), grid, block, p.lds, st, a);
    return hipGetLastError();
}

template <int S, int MT, int XM>
hipError_t launch_gemv_shape(const GemvArgs &a, const GemvPlan &p, hipStream_t st)
{
#define SBVR_SHAPE(ct, sp)                                  \
    if constexpr (shape_ok_for(MT, ct, sp))                 \
        if (p.CT == ct && p.SP == sp)                       \
            return launch_gemv_inst<S, MT, ct, sp, XM>(a, p, st)
    SBVR_SHAPE(1, 1); SBVR_SHAPE(1, 2); SBVR_SHAPE(1, 4); SBVR_SHAPE(1, 7);
    SBVR_SHAPE(2, 1); SBVR_SHAPE(2, 2); SBVR_SHAPE(2, 4); SBVR_SHAPE(2, 7);
    SBVR_SHAPE(4, 1); SBVR_SHAPE(4, 2); SBVR_SHAPE(4, 4); SBVR_SHAPE(7, 2);
#undef SBVR_SHAPE
    return hipErrorInvalidConfiguration;
}

// (the fused prologues exist for one batch row only)
template <int S>
hipError_t launch_gemv_mt(const GemvArgs &a, const GemvPlan &p, int xm, hipStream_t st)
{
    if (xm == kXSwiGLU)
        return p.MT == 1 ? launch_gemv_shape<S, 1, kXSwiGLU>(a, p, st) : hipErrorInvalidConfiguration;
    if (xm == kXAddNorm)
        return p.MT == 1 ? launch_gemv_shape<S, 1, kXAddNorm>(a, p, st) : hipErrorInvalidConfiguration;
    if (xm == kXAddNorm2)
        return p.MT == 1 ? launch_gemv_shape<S, 1, kXAddNorm2>(a, p, st) : hipErrorInvalidConfiguration;
    if (xm == kXFloor)
        return p.MT == 1 ? launch_gemv_shape<S, 1, kXFloor>(a, p, st) : hipErrorInvalidConfiguration;
    if (xm == kXPlanes)
        return p.MT == 1 ? launch_gemv_shape<S, 1, kXPlanes>(a, p, st) : hipErrorInvalidConfiguration;
    switch (p.MT) {
    case 1: return launch_gemv_shape<S, 1, kXPlain>(a, p, st);
    case 2: return launch_gemv_shape<S, 2, kXPlain>(a, p, st);
    default: return launch_gemv_shape<S, 4, kXPlain>(a, p, st);
    }
}

hipError_t launch_gemv(int S, const GemvArgs &a, const GemvPlan &p, int xm, hipStream_t st)
{
    switch (S) {
    case 4: return launch_gemv_mt<4>(a, p, xm, st);
#ifndef SBVR_FAST_BUILD      // development builds: one plane count only
    case 2: return launch_gemv_mt<2>(a, p, xm, st);
    case 3: return launch_gemv_mt<3>(a, p, xm, st);
    case 6: return launch_gemv_mt<6>(a, p, xm, st);
    case 8: return launch_gemv_mt<8>(a, p, xm, st);
#endif
    default: return hipErrorInvalidConfiguration;
    }
}

// ---- launch shape and dispatch of the kernel for 5..16 batch rows
struct BatchPlan {
    int MT, CTW, SP, waves, n_wgs, ksplit, wstride;
    size_t lds;
};

constexpr bool batch_shape_ok(int S, int MT, int CTW, int SP)
{
    if (SP != 1 && SP != 2 && SP != 4)
        return false;
    // (left out: the shapes that do not fit 128 registers a lane for that plane count)
    if (MT == 2)
        return CTW == 1 || CTW == 2 || CTW == 4 || ((CTW == 7 || CTW == 8) && SP < 4 && !(S == 6 && CTW == 8 && SP == 2));
    if (MT != 4)
        return false;
    if ((S == 3 || S == 8) && CTW * SP >= 8)
        return false;
    return CTW == 1 || CTW == 2 || (CTW == 4 && SP < 4);
}

bool batch_path_ok(int M, int N, int K, int S, int G)
{
    return M > 4 && mfma_path_ok(M, N, K, S, G) && N >= 16 * (M <= 8 ? 2 : 4);
}

// The shape with the smallest estimate of the launch's time: the busiest CU's workgroups one after the
// other, a workgroup's time that of its waves on one SIMD (operands, then units), plus the accumulators'
// atomic adds where K is split.
BatchPlan plan_batch_uncached(int M, int N, int K, int S, int cus)
{
    const int nsub = K / kSub;
    const int MT = M <= 8 ? 2 : 4;
    const EnvSwitches &env = env_switches();
    BatchPlan best{};
    double best_t = 1e30;
    constexpr int kCtw[] = {1, 2, 4, 7, 8}, kSp[] = {1, 2, 4}, kWaves[] = {16, 8, 4};
    for (int CTW : kCtw)
        for (int SP : kSp)
            for (int waves : kWaves) {
                if (!batch_shape_ok(S, MT, CTW, SP) || waves < MT || CTW * MT * 16 > N)
                    continue;
                if ((env.ct > 0 && CTW != env.ct) || (env.sp > 0 && SP != env.sp) || (env.waves > 0 && waves != env.waves))
                    continue;
                const int groups = waves / MT;
                if (nsub % (SP * groups) || nsub / (SP * groups) > kMaxKsplit)
                    continue;
                const int ksplit = nsub / (SP * groups);
                const int W = CTW * MT * 16;
                int windows = (N + W - 1) / W;
                const int wstride = ((N + windows - 1) / windows + 7) / 8 * 8;
                windows = (N + wstride - 1) / wstride;
                const size_t lds = static_cast<size_t>(waves) * (SP * (2048 + 16) + CTW * MT * 256);
                if (lds > 160 * 1024)
                    continue;
                const int per_cu = static_cast<int>(std::min<size_t>(16 / waves, (160 * 1024) / lds));
                const long wgs = static_cast<long>(windows) * ksplit;
                const long rounds = (wgs + static_cast<long>(cus) * per_cu - 1) / (static_cast<long>(cus) * per_cu);
                const double per_wave = SP * (4 * 160.0 + CTW * (MT * S * 32.0 + 250.0)) + CTW * MT * 30.0;
                // (below three waves per SIMD the waits of a wave are not covered by the others)
                double t = 1500.0 + static_cast<double>(rounds) * std::max(waves * per_cu / 4.0, 3.0) * per_wave;
                // (measured: 3.6 us for the 917 504 adds of 16 rows x 14336 columns x 4 parts, whatever the shape; with
                // two row tiles the sweeps are fitted better by a third of that: more of it hides behind the units)
                t += ksplit > 1 ? (MT == 4 ? 0.0082 : 0.003) * static_cast<double>(M) * N * ksplit : 0.0;
                t *= static_cast<double>(windows) * W / N;
                if (t < best_t) {
                    best_t = t;
                    best = BatchPlan{MT, CTW, SP, waves, windows, ksplit, wstride, lds};
                }
            }
    return best;
}

BatchPlan plan_batch(int M, int N, int K, int S, int cus)
{
    struct Entry {
        int M, N, K, S, cus;
        BatchPlan plan;
    };
    constexpr int kEntries = 64;
    static Entry cache[kEntries];
    static int used = 0;
    static std::mutex lock;
    std::lock_guard<std::mutex> guard(lock);
    for (int i = 0; i < used; ++i) {
        const Entry &e = cache[i];
        if (e.M == M && e.N == N && e.K == K && e.S == S && e.cus == cus)
            return e.plan;
    }
    const BatchPlan p = plan_batch_uncached(M, N, K, S, cus);
    if (used < kEntries)
        cache[used++] = Entry{M, N, K, S, cus, p};
    return p;
}

template <int S, int MT, int CTW, int SP>
hipError_t launch_batch_inst(const GemvArgs &a, const BatchPlan &p, hipStream_t st)
{
    const dim3 grid(static_cast<unsigned>(p.n_wgs), static_cast<unsigned>(p.ksplit)), block(64 * p.waves);
    if (p.lds > 65536) {        // above what a kernel gets without asking
        static bool raised_on[16] = {};
        std::lock_guard<std::mutex> guard(g_dev_lock);
        int dev_now = 0;
        if (hipGetDevice(&dev_now) != hipSuccess || dev_now < 0 || dev_now >= 16)
            dev_now = 0;
        if (!raised_on[dev_now]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sbvr_gemv_batch_kernel<S, MT, CTW, SP>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess)
                return e;
            raised_on[dev_now] = true;
        }
    }
    hipLaunchKernelGGL((sbvr_gemv_batch_kernel<S, MT, CTW, SP>), grid, block, p.lds, st, a);
    return hipGetLastError();
}

template <int S, int MT>
hipError_t launch_batch_shape(const GemvArgs &a, const BatchPlan &p, hipStream_t st)
{
#define SBVR_BSHAPE(ctw, sp)                                \
    if constexpr (batch_shape_ok(S, MT, ctw, sp))           \
        if (p.CTW == ctw && p.SP == sp)                     \
            return launch_batch_inst<S, MT, ctw, sp>(a, p, st)
    SBVR_BSHAPE(1, 1); SBVR_BSHAPE(2, 1); SBVR_BSHAPE(4, 1); SBVR_BSHAPE(7, 1); SBVR_BSHAPE(8, 1);
    SBVR_BSHAPE(1, 2); SBVR_BSHAPE(2, 2); SBVR_BSHAPE(4, 2); SBVR_BSHAPE(7, 2); SBVR_BSHAPE(8, 2);
    SBVR_BSHAPE(1, 4); SBVR_BSHAPE(2, 4); SBVR_BSHAPE(4, 4); SBVR_BSHAPE(7, 4); SBVR_BSHAPE(8, 4);
#undef SBVR_BSHAPE
    return hipErrorInvalidConfiguration;
}

template <int S>
hipError_t launch_batch_mt(const GemvArgs &a, const BatchPlan &p, hipStream_t st)
{
    return p.MT == 2 ? launch_batch_shape<S, 2>(a, p, st) : launch_batch_shape<S, 4>(a, p, st);
}

hipError_t launch_batch(int S, const GemvArgs &a, const BatchPlan &p, hipStream_t st)
{
    switch (S) {
    case 4: return launch_batch_mt<4>(a, p, st);
#ifndef SBVR_FAST_BUILD
    case 2: return launch_batch_mt<2>(a, p, st);
    case 3: return launch_batch_mt<3>(a, p, st);
    case 6: return launch_batch_mt<6>(a, p, st);
    case 8: return launch_batch_mt<8>(a, p, st);
#endif
    default: return hipErrorInvalidConfiguration;
    }
}

// ------------------------------------------------------------- MFMA prefill

// Prefill path (M > 16): a dense contraction.  A workgroup owns a 256 x 128
// tile of the output and walks K in steps of 64.  Its 12 waves have two jobs:
//   * waves 4-11 produce the weight tile of step t+1 while step t is consumed:
//     128 x 64 weights decoded to fp16: thread (column, word, half) holds the
//     S plane words of one 32-bit word of K and the coefficient line of its
//     group, and forms w = sum_j (bit_j ? c_j : 0) for 16 of the word's
//     elements, two of them (k, k+16) per packed fp16 operation:
//     (word >> k) & 0x00010001 times the 16-bit pattern of c_j is that pattern,
//     or zero, in each half.  Their global loads run three steps ahead of the
//     consumers, in three register sets used in rotation;
//   * waves 0-3 run v_mfma_f32_32x32x16_f16 over the two tiles (each wave
//     128 x 64 of the output, 8 accumulator blocks) and, before that, send for
//     the 256 x 64 activations of the step after the next: global memory to LDS directly,
//     no registers, the data lands while the MFMAs run.
// A SIMD holds one consumer and two producers, so the decode (VALU) and the
// MFMAs overlap.  The weight tile has two buffers, the activation tile three (its
// loads go out two steps ahead); one barrier per step.  Rows of the
// LDS tiles are 128 bytes; 16-byte chunk c of row r is stored at chunk
// c ^ ((r >> 1) & 7), which keeps the 16-byte operand reads of a quarter wave
// (16 rows, two of them per 256-byte line of banks) on different banks.
constexpr int kGemmBM = 256, kGemmBN = 128, kGemmBK = 64, kGemmThreads = 768;     // 4 consumer + 8 producer waves
constexpr int kGemmABufs = 3;       // activation tiles in LDS: the one in use and the next two
constexpr int kGemmATile = kGemmBM * kGemmBK * 2, kGemmBTile = kGemmBN * kGemmBK * 2;

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct GemmArgs {
    const uint16_t *x;
    const uint32_t *bvr;
    const void *idx;
    const uint16_t *cache;
    const uint16_t *bias;
    uint16_t *out;
    int M, N, K, L;
    int steps_per_group;   // G / 64
    int idx16;
    int ksplit;            // workgroups along K (blockIdx.z); 1: results go straight to out
    float *part;           // ksplit > 1: (ksplit, M, N) fp32 partial results, all zero between launches
#ifdef SBVR_TRACE
    unsigned long long *trace;
#endif
};

// The S fp16 coefficients of one table line as packed pairs, in as few load instructions as the
// line's alignment allows (a line starts at a multiple of 2*S bytes; the table is 16-byte aligned).
template <int S>
__device__ __forceinline__ void load_line_coeffs(const uint16_t *cp, uint32_t (&cr)[(S + 1) / 2])
{
    if constexpr (S == 4) {
        const v2u t = *reinterpret_cast<const v2u *>(cp);
        cr[0] = t.x; cr[1] = t.y;
    } else if constexpr (S == 8) {
        const v4u t = *reinterpret_cast<const v4u *>(cp);
        cr[0] = t.x; cr[1] = t.y; cr[2] = t.z; cr[3] = t.w;
    } else if constexpr (S % 2 == 0) {
#pragma unroll
        for (int j = 0; j < S / 2; ++j)
            cr[j] = reinterpret_cast<const uint32_t *>(cp)[j];
    } else {
#pragma unroll
        for (int j = 0; j < (S + 1) / 2; ++j)
            cr[j] = static_cast<uint32_t>(cp[2 * j]) | (2 * j + 1 < S ? static_cast<uint32_t>(cp[2 * j + 1]) << 16 : 0u);
    }
}

#ifdef SBVR_TRACE
#define SBVR_GSTAMP(step, slot)                                                                   \
    do {                                                                                          \
        if (a.trace && blockIdx.x == 7 && blockIdx.y == 1 && (threadIdx.x & 63) == 0 && (step) < 96) \
            a.trace[(step) * 8 + (slot)] = wall_clock64();                                        \
    } while (0)
#else
#define SBVR_GSTAMP(step, slot) do { } while (0)
#endif

template <int S>
__global__ void __launch_bounds__(kGemmThreads)
__attribute__((amdgpu_waves_per_eu(3, 3)))
sbvr_gemm_mfma_kernel(const GemmArgs a)
{
    extern __shared__ __align__(16) unsigned char gsm[];
    unsigned char *const As = gsm;                       // 2 tiles
    unsigned char *const Bs = gsm + kGemmABufs * kGemmATile;      // 2 tiles

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = a.N, K = a.K, M = a.M;
    const int n0 = blockIdx.x * kGemmBN, m0 = blockIdx.y * kGemmBM;
    const int steps = K / kGemmBK / a.ksplit;            // of this workgroup: tiles t_base .. t_base + steps - 1 of K
    const int t_base = blockIdx.z * steps;
    const int rounds = (steps + 2) / 3;                  // both kinds of waves run 3 * rounds steps (same barriers)

    if (wave >= 4) {
        // ------------------------------------------------------------ producers
        const int pt = tid - 256;
        // decode role: column of the tile, word of the step, and which 8 of the word's 16 pairs (k, k+16)
        const int bn = pt & (kGemmBN - 1), bw = (pt >> 7) & 1, bh = pt >> 8;
        const int n_ld = min(n0 + bn, N - 1);
        const int b_dst = bn * 128;
        const int sw = (bn >> 1) & 7, cb = bw * 4;       // chunk swizzle of row bn, see the consumers

        constexpr int CW = (S + 1) / 2;
        uint32_t wreg0[S], wreg1[S], wreg2[S];           // three register sets, used in rotation
        uint32_t creg0[CW], creg1[CW], creg2[CW];
        // The aligned 32-bit word that holds the line index of the tile a register set is filled with next:
        // loaded when the set is requested, used three steps later by the same set's next request, and
        // untouched in between (a move, or a byte load's zero extension, ends up at the top of the loop,
        // where it makes the step wait for the youngest loads in flight).
        uint32_t raw0 = 0, raw1 = 0, raw2 = 0;

        // (two byte loads whatever the index width: a branch between a 16-bit and an 8-bit load
        // inside the loop would make every later wait a wait for all loads)
        auto line_address = [&](int t) __attribute__((always_inline)) -> uintptr_t {
            const size_t at = (static_cast<size_t>((t_base + t) / a.steps_per_group) * N + n_ld) << a.idx16;
            return reinterpret_cast<uintptr_t>(static_cast<const uint8_t *>(a.idx) + at);
        };
        auto load_line = [&](int t, uint32_t &raw) __attribute__((always_inline)) {
            // (a global-memory pointer by type: from a bare integer the compiler would make a flat load,
            // whose completion order it does not know)
            raw = *reinterpret_cast<const __attribute__((address_space(1))) uint32_t *>(line_address(t) & ~static_cast<uintptr_t>(3));
        };
        auto line_of = [&](int t, uint32_t raw) __attribute__((always_inline)) -> int {
            const uint32_t v = raw >> (8 * static_cast<uint32_t>(line_address(t) & 3));
            return min(static_cast<int>(a.idx16 ? v & 0xffffu : v & 0xffu), a.L - 1);
        };
        // global loads of tile t into one register set
        auto request = [&](int t, uint32_t (&wr)[S], uint32_t (&cr)[CW], uint32_t &raw) __attribute__((always_inline)) {
            const int k0 = (t_base + t) * kGemmBK;
            const uint32_t *wp = a.bvr + (static_cast<size_t>(k0 / 32 + bw) * N + n_ld) * S;
            // (ordinary loads: every row tile of the launch reads these again; non-temporal ones measured 2-3 % slower)
            const Planes<S> pl = load_planes<S>(wp);
#pragma unroll
            for (int j = 0; j < S; ++j)
                wr[j] = pl.w[j];
            asm volatile("" : "+v"(raw));                // not to be taken apart before this step (see pin)
            const uint16_t *cp = a.cache + static_cast<size_t>(line_of(t, raw)) * S;
            load_line_coeffs<S>(cp, cr);
            load_line(min(t + 3, steps - 1), raw);
        };
        // Makes a register set opaque at the start of the step that decodes it: without this the compiler
        // moves part of the decode up into the step before (arithmetic may cross a barrier), where the
        // set's loads are the youngest in flight and the wait for them drains the whole queue.
        auto pin = [&](uint32_t (&wr)[S], uint32_t (&cr)[CW], uint32_t &) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < S; ++j)
                asm volatile("" : "+v"(wr[j]));
#pragma unroll
            for (int j = 0; j < CW; ++j)
                asm volatile("" : "+v"(cr[j]));
        };
        // one register set -> LDS buffers t % 2
        auto produce = [&](int t, const uint32_t (&wr)[S], const uint32_t (&cr)[CW], uint32_t) __attribute__((always_inline)) {
            unsigned char *Bt = Bs + (t & 1) * kGemmBTile;
            uint32_t cbits[S];
#pragma unroll
            for (int j = 0; j < S; ++j)
                cbits[j] = j & 1 ? cr[j / 2] >> 16 : cr[j / 2] & 0xffffu;
            uint32_t wsh[S];
#pragma unroll
            for (int j = 0; j < S; ++j)
                wsh[j] = wr[j] >> (8 * bh);
            uint32_t pr[8];          // pr[e] = {w[8 bh + e], w[16 + 8 bh + e]}
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v2h v = __builtin_bit_cast(v2h, __umul24((wsh[0] >> e) & 0x00010001u, cbits[0]));
#pragma unroll
                for (int j = 1; j < S; ++j)
                    v = v + __builtin_bit_cast(v2h, __umul24((wsh[j] >> e) & 0x00010001u, cbits[j]));
                pr[e] = __builtin_bit_cast(uint32_t, v);
            }
            v4u lo, hi;              // k 8 bh .. + 7 (low halves) and 16 + 8 bh .. + 7 (high halves)
            lo.x = __builtin_amdgcn_perm(pr[1], pr[0], 0x05040100u); hi.x = __builtin_amdgcn_perm(pr[1], pr[0], 0x07060302u);
            lo.y = __builtin_amdgcn_perm(pr[3], pr[2], 0x05040100u); hi.y = __builtin_amdgcn_perm(pr[3], pr[2], 0x07060302u);
            lo.z = __builtin_amdgcn_perm(pr[5], pr[4], 0x05040100u); hi.z = __builtin_amdgcn_perm(pr[5], pr[4], 0x07060302u);
            lo.w = __builtin_amdgcn_perm(pr[7], pr[6], 0x05040100u); hi.w = __builtin_amdgcn_perm(pr[7], pr[6], 0x07060302u);
            *reinterpret_cast<v4u *>(Bt + b_dst + (((cb + bh) ^ sw) << 4)) = lo;
            *reinterpret_cast<v4u *>(Bt + b_dst + (((cb + 2 + bh) ^ sw) << 4)) = hi;
        };
#define SBVR_SET(n) wreg##n, creg##n, raw##n
        // Requests are never conditional (beyond the last tile they repeat it): after a
        // branch that may or may not have issued loads, the wait for an older set would
        // have to assume it had not, and wait for everything.
        const int last = steps - 1;
        load_line(0, raw0);
        load_line(min(1, last), raw1);
        load_line(min(2, last), raw2);
        request(0, SBVR_SET(0));
        request(min(1, last), SBVR_SET(1));
        request(min(2, last), SBVR_SET(2));
        produce(0, SBVR_SET(0));
        __syncthreads();
        // step i: the consumers read tile i; tile i+1 goes to the other buffers, tile i+3 is requested
        for (int r = 0; r < rounds; ++r) {
            const int i = 3 * r;
            // (tiles beyond the last are produced too, from repeated loads, into buffers nobody reads:
            // a loop body without branches keeps the waits of the three register sets apart)
            if (wave == 4) SBVR_GSTAMP(i, 2);
            pin(SBVR_SET(1));
            request(min(i + 3, last), SBVR_SET(0));
            if (wave == 4) SBVR_GSTAMP(i, 3);
            produce(i + 1, SBVR_SET(1));
            if (wave == 4) SBVR_GSTAMP(i, 4);
            __syncthreads();
            if (wave == 4) SBVR_GSTAMP(i + 1, 2);
            pin(SBVR_SET(2));
            request(min(i + 4, last), SBVR_SET(1));
            if (wave == 4) SBVR_GSTAMP(i + 1, 3);
            produce(i + 2, SBVR_SET(2));
            if (wave == 4) SBVR_GSTAMP(i + 1, 4);
            __syncthreads();
            if (wave == 4) SBVR_GSTAMP(i + 2, 2);
            pin(SBVR_SET(0));
            request(min(i + 5, last), SBVR_SET(2));
            if (wave == 4) SBVR_GSTAMP(i + 2, 3);
            produce(i + 3, SBVR_SET(0));
            if (wave == 4) SBVR_GSTAMP(i + 2, 4);
            __syncthreads();
        }
#undef SBVR_SET
        return;
    }

    // ---------------------------------------------------------------- consumers
    v16f acc[4][2];
#pragma unroll
    for (int bi = 0; bi < 4; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[bi][bj][r] = 0.f;
    const int wm = wave >> 1, wn = wave & 1;
    const int arow = wm * 128 + (lane & 31), brow = wn * 64 + (lane & 31);      // + 32 bi / bj: same (row >> 1) & 7
    // Chunk c of tile row r sits at chunk position c ^ ((r >> 1) & 7) of the row's 128 bytes.  A 16-byte read
    // is served 16 lanes (rows) at a time by 64 banks of 4 bytes, i.e. two rows side by side: with the row pair
    // as the swizzle key the 16 rows hit 16 different bank groups (keyed by r & 7, rows r and r + 8 collided
    // and every read took two turns).
    const int rsw = (lane >> 1) & 7, chi = lane >> 5;
    // The activation tile goes from global memory straight into LDS (no registers): instruction j
    // of wave w fills the 1 KiB block 8w + j, i.e. rows 8 (8w + j) .. + 7, lane l the 16-byte slot l
    // of it; with the row swizzle, slot l of a block holds chunk (l & 7) ^ ((4j + (l >> 4)) & 7) of row l >> 3.
    uint32_t xoff[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = 8 * (8 * wave + j) + (lane >> 3);
        xoff[j] = static_cast<uint32_t>(min(m0 + row, M - 1)) * K + 8 * ((lane & 7) ^ ((row >> 1) & 7));     // M * K < 2^31 (checked)
    }
    auto fetch_a = [&](int t, int buf) __attribute__((always_inline)) {        // tile t -> buffer buf, asynchronously
        unsigned char *dst = As + buf * kGemmATile + wave * 8192;
        const uint16_t *src = a.x + static_cast<size_t>(t_base + t) * kGemmBK;
        // Written as assembly (M0 = LDS address of lane 0's slot): the compiler counts the builtin form as a
        // memory operation whose order of completion it does not know, and from then on turns every wait for
        // an LDS read into a wait for all of them.
        const uint32_t lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst));
#pragma unroll
        for (int j = 0; j < 8; ++j)
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         :: "v"(src + xoff[j]), "s"(lds + j * 1024) : "memory", "m0");
    };
    fetch_a(0, 0);
    fetch_a(min(1, steps - 1), 1);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0): the tiles are in LDS
    int cur = 0;                                 // activation buffer of tile i
    __syncthreads();
    // operand registers of two k-slices in turn: the reads of slice s+1 are issued before the MFMAs of slice s
    auto read_slice = [&](const unsigned char *At, const unsigned char *Bt, int ks, v8h (&af)[4], v8h (&bf)[2])
                          __attribute__((always_inline)) {
        const int coff = ((2 * ks + chi) ^ rsw) << 4;
#pragma unroll
        for (int bi = 0; bi < 4; ++bi)
            af[bi] = *reinterpret_cast<const v8h *>(At + (arow + 32 * bi) * 128 + coff);
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
            bf[bj] = *reinterpret_cast<const v8h *>(Bt + (brow + 32 * bj) * 128 + coff);
    };
    auto mfma_slice = [&](const v8h (&af)[4], const v8h (&bf)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int bi = 0; bi < 4; ++bi)
#pragma unroll
            for (int bj = 0; bj < 2; ++bj)
                acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[bi], bf[bj], acc[bi][bj], 0, 0, 0);
    };
    for (int i = 0; i < 3 * rounds; ++i) {
        if (i < steps) {
            const unsigned char *At = As + cur * kGemmATile, *Bt = Bs + (i & 1) * kGemmBTile;
            if (wave == 0) SBVR_GSTAMP(i, 0);
            // the tile after the next goes to the buffer that the tile before this one has left; it has two
            // steps to land
            fetch_a(min(i + 2, steps - 1), cur == 0 ? 2 : cur - 1);
            // (With 168 registers a wave the compiler keeps one activation operand at a time and moves each
            // read down to its MFMAs: fenced into the order written here the loop needs about 200.)
            v8h af0[4], bf0[2], af1[4], bf1[2];
            read_slice(At, Bt, 0, af0, bf0);
            read_slice(At, Bt, 1, af1, bf1);
            mfma_slice(af0, bf0);
            read_slice(At, Bt, 2, af0, bf0);
            mfma_slice(af1, bf1);
            read_slice(At, Bt, 3, af1, bf1);
            mfma_slice(af0, bf0);
            mfma_slice(af1, bf1);
            if (wave == 0) SBVR_GSTAMP(i, 1);
            __builtin_amdgcn_sched_barrier(0);   // (or the wait moves up in front of the MFMAs)
            __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): all but the 8 loads above, i.e. this wave's part of the next tile is in LDS
            cur = cur == 2 ? 0 : cur + 1;
        }
        __syncthreads();
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);          // no load into LDS is left in flight when the wave ends

    // ---- D[i][j] sits in lane j + 32*((i/4)%2), register (i%4) + 4*(i/8)
    if (a.ksplit > 1) {
        // K split across workgroups: every workgroup leaves its fp32 tile in `part`; sbvr_gemm_reduce_kernel,
        // launched behind this kernel, adds the tiles up in the order of blockIdx.z and rounds once.
        float *mine = a.part + blockIdx.z * (static_cast<size_t>(M) * N);
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
            const int n = n0 + wn * 64 + bj * 32 + (lane & 31);
#pragma unroll
            for (int bi = 0; bi < 4; ++bi)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * 128 + bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < M && n < N)
                        mine[static_cast<size_t>(m) * N + n] = acc[bi][bj][r];
                }
        }
        return;
    }
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
        const int n = n0 + wn * 64 + bj * 32 + (lane & 31);
        if (n >= N)
            continue;
        const uint16_t bias = a.bias ? a.bias[n] : 0;
#pragma unroll
        for (int bi = 0; bi < 4; ++bi)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 128 + bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < M) {
                    uint16_t v = f2h(acc[bi][bj][r]);
                    if (a.bias)
                        v = hadd(v, bias);
                    a.out[static_cast<size_t>(m) * N + n] = v;
                }
            }
    }
}

// Second pass of a split prefill launch: out[m, n] = fp16(sum over z, in order, of part[z][m][n]) (+ bias),
// and the partial results are set back to zero (the workspace is shared with the decode kernel's
// accumulators, which must find zeros).  Four outputs per thread.
__global__ void __launch_bounds__(256)
sbvr_gemm_reduce_kernel(float *__restrict__ part, const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                        int M, int N, int ksplit)
{
    const size_t total = static_cast<size_t>(M) * N;
    const size_t at = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
    if (at >= total)
        return;
    // (N is a multiple of 4 here, so the four outputs share a row and the 16-byte accesses are aligned)
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < ksplit; ++z) {
        v4f *cell = reinterpret_cast<v4f *>(part + z * total + at);
        sum += *cell;
        *cell = v4f{0.f, 0.f, 0.f, 0.f};
    }
    const int n = static_cast<int>(at % N);
    uint16_t r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r[i] = f2h(sum[i]);
        if (bias)
            r[i] = hadd(r[i], bias[n + i]);
    }
    *reinterpret_cast<uint2 *>(out + at) = uint2{static_cast<uint32_t>(r[0]) | (static_cast<uint32_t>(r[1]) << 16),
                                                 static_cast<uint32_t>(r[2]) | (static_cast<uint32_t>(r[3]) << 16)};
}

// ------------------------------------------------- MFMA, 5 to 32 batch rows

// Between the decode kernel (whose cost grows with the batch rows: each needs
// its own fp8 A operands) and the prefill kernel (256-row tiles) sits a kernel
// for up to 32 rows: v_mfma_f32_32x32x16_f16 with the batch rows as the 32 rows
// of A, read from global memory as they are, and 32 columns of decoded weights
// as B.  A wave walks a range of K one 32-bit word (two MFMAs) at a time; lane
// (column j, half h) decodes bits 8h..8h+7 and 16+8h..16+8h+7 of the word, two
// elements (k, k+16) per packed fp16 operation as in the prefill kernel, which
// are exactly its B elements of the two MFMAs.  No LDS on the way; the 8 waves
// of a workgroup split K and add their 32 x 32 partial results in LDS at the
// end.  Bound by the decode arithmetic (about 7.5 VALU operations per weight),
// not by the batch size.
constexpr int kRowsMax = 32, kRowsWaves = 8, kRowsBlock = 2;

struct RowsArgs {
    const uint16_t *x;
    const uint32_t *bvr;
    const void *idx;
    const uint16_t *cache;
    const uint16_t *bias;
    uint16_t *out;
    int M, N, K, L;
    int words_per_group;   // G / 32
    int words_per_wave;    // a multiple of kRowsBlock
    int idx16;
    // the table look-up form only
    unsigned long long *acc;   // (M, N) split-K accumulators as in the decode kernel (ksplit > 1)
    int ksplit;                // workgroups along K (blockIdx.y)
    int pairs_per_wg;          // word pairs (64 elements of K) of a workgroup
};

template <int S>
__global__ void __launch_bounds__(64 * kRowsWaves)
sbvr_gemm_rows32_kernel(const RowsArgs a)
{
    __shared__ float red[kRowsWaves][16][64];
    constexpr int CW = (S + 1) / 2;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = a.N, K = a.K, M = a.M;
    const int j = lane & 31, h = lane >> 5;
    const int n = blockIdx.x * 32 + j, n_ld = min(n, N - 1);
    const int words = K / 32;
    const int w_begin = wave * a.words_per_wave, w_end = min(words, w_begin + a.words_per_wave);
    const bool row_ok = j < M;                        // lane's batch row for the A operand is j as well
    const uint16_t *xrow = a.x + static_cast<size_t>(min(j, M - 1)) * K + 8 * h;

    struct Block {
        v4u planes[kRowsBlock];      // S <= 4 words used directly; more planes: see below
        uint32_t more[kRowsBlock][S > 4 ? S - 4 : 1];
        v4u xa[kRowsBlock][2];
        uint32_t c[kRowsBlock][CW];
    };
    auto load_lines = [&](int w0, int (&line)[kRowsBlock]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kRowsBlock; ++i) {
            const int w = min(w0 + i, words - 1);
            const size_t at = (static_cast<size_t>(w / a.words_per_group) * N + n_ld) << a.idx16;
            const uint8_t *ib = static_cast<const uint8_t *>(a.idx);
            const int lo = ib[at], hi = ib[at + a.idx16];      // two byte loads whatever the width: no branch
            line[i] = lo | (hi << 16);                          // raw: decoded where it is used (see the prefill kernel)
        }
    };
    auto load_block = [&](int w0, Block &b, const int (&line)[kRowsBlock]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kRowsBlock; ++i) {
            const int w = min(w0 + i, words - 1);        // beyond the range: repeats the last word, never used
            const uint32_t *wp = a.bvr + (static_cast<size_t>(w) * N + n_ld) * S;
            const Planes<S> pl = load_planes<S>(wp);
#pragma unroll
            for (int q = 0; q < S; ++q) {
                if (q < 4)
                    b.planes[i][q] = pl.w[q];
                else
                    b.more[i][q - 4] = pl.w[q];
            }
            b.xa[i][0] = v4u{0u, 0u, 0u, 0u};
            b.xa[i][1] = v4u{0u, 0u, 0u, 0u};
            if (row_ok) {
                b.xa[i][0] = *reinterpret_cast<const v4u *>(xrow + 32 * w);
                b.xa[i][1] = *reinterpret_cast<const v4u *>(xrow + 32 * w + 16);
            }
            const int ln = min(a.idx16 ? (line[i] & 0xff) | ((line[i] >> 8) & 0xff00) : line[i] & 0xff, a.L - 1);
            load_line_coeffs<S>(a.cache + static_cast<size_t>(ln) * S, b.c[i]);
        }
    };

    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        acc[r] = 0.f;

    auto compute = [&](int w0, const Block &b) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kRowsBlock; ++i) {
            if (w0 + i >= w_end)          // wave-uniform
                break;
            uint32_t wsh[S], cbits[S];
#pragma unroll
            for (int q = 0; q < S; ++q) {
                const uint32_t word = q < 4 ? b.planes[i][q < 4 ? q : 0] : b.more[i][q < 4 ? 0 : q - 4];
                wsh[q] = word >> (8 * h);
                cbits[q] = q & 1 ? b.c[i][q / 2] >> 16 : b.c[i][q / 2] & 0xffffu;
            }
            uint32_t pr[8];               // pr[e] = {w[8h+e], w[16+8h+e]}
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v2h v = __builtin_bit_cast(v2h, __umul24((wsh[0] >> e) & 0x00010001u, cbits[0]));
#pragma unroll
                for (int q = 1; q < S; ++q)
                    v = v + __builtin_bit_cast(v2h, __umul24((wsh[q] >> e) & 0x00010001u, cbits[q]));
                pr[e] = __builtin_bit_cast(uint32_t, v);
            }
            v4u b0, b1;
            b0.x = __builtin_amdgcn_perm(pr[1], pr[0], 0x05040100u); b1.x = __builtin_amdgcn_perm(pr[1], pr[0], 0x07060302u);
            b0.y = __builtin_amdgcn_perm(pr[3], pr[2], 0x05040100u); b1.y = __builtin_amdgcn_perm(pr[3], pr[2], 0x07060302u);
            b0.z = __builtin_amdgcn_perm(pr[5], pr[4], 0x05040100u); b1.z = __builtin_amdgcn_perm(pr[5], pr[4], 0x07060302u);
            b0.w = __builtin_amdgcn_perm(pr[7], pr[6], 0x05040100u); b1.w = __builtin_amdgcn_perm(pr[7], pr[6], 0x07060302u);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, b.xa[i][0]), __builtin_bit_cast(v8h, b0), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, b.xa[i][1]), __builtin_bit_cast(v8h, b1), acc, 0, 0, 0);
        }
    };

    // two register blocks in turn; the line indices run one block further ahead
    // (loads are never conditional, see the prefill kernel)
    Block b0, b1;
    int line[kRowsBlock];
    load_lines(w_begin, line);
    load_block(w_begin, b0, line);
    load_lines(w_begin + kRowsBlock, line);
    for (int w0 = w_begin; w0 < w_end; w0 += 2 * kRowsBlock) {
        load_block(w0 + kRowsBlock, b1, line);
        load_lines(w0 + 2 * kRowsBlock, line);
        compute(w0, b0);
        load_block(w0 + 2 * kRowsBlock, b0, line);
        load_lines(w0 + 3 * kRowsBlock, line);
        compute(w0 + kRowsBlock, b1);
    }

    // ---- partial results meet in LDS; D[i][jj] sits in lane jj + 32*((i/4)%2), register (i%4) + 4*(i/8)
#pragma unroll
    for (int r = 0; r < 16; ++r)
        red[wave][r][lane] = acc[r];
    __syncthreads();
    if (n >= N)
        return;
    const uint16_t bias = a.bias ? a.bias[n] : 0;
#pragma unroll
    for (int rr = 0; rr < 16 / kRowsWaves; ++rr) {
        const int r = wave * (16 / kRowsWaves) + rr;
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kRowsWaves; ++w)
            total += red[w][r][lane];
        const int m = 8 * (r >> 2) + 4 * h + (r & 3);
        if (m < M) {
            uint16_t v = f2h(total);
            if (a.bias)
                v = hadd(v, bias);
            a.out[static_cast<size_t>(m) * N + n] = v;
        }
    }
}

bool rows32_path_ok(int M, int N, int K, int S, int G)
{
    return M > 4 && M <= kRowsMax && K % 32 == 0 && G % 32 == 0 && (S == 2 || S == 3 || S == 4 || S == 6 || S == 8) &&
           static_cast<double>(K / 32) * N * S < 2147483648.0;
}

// The arithmetic form of the 32-row kernel: for 17..32 rows where the table look-up form has no instance (6 or 8
// planes, K or G not a multiple of 64), and for 5..16 rows of shapes the decode kernels do not cover.
bool rows32_preferred(int M, int N, int K, int S, int G, int cus)
{
    (void)cus;
    if (!rows32_path_ok(M, N, K, S, G))
        return false;
    // up to 16 rows the decode kernels are faster wherever they have a shape for (M, N)
    return !(M <= kMaxM && mfma_path_ok(M, N, K, S, G));
}

hipError_t launch_rows32(int S, RowsArgs a, hipStream_t st)
{
    const int words = a.K / 32;
    int wpw = (words + kRowsWaves - 1) / kRowsWaves;
    wpw = (wpw + kRowsBlock - 1) / kRowsBlock * kRowsBlock;
    a.words_per_wave = wpw;
    const dim3 grid(static_cast<unsigned>((a.N + 31) / 32)), block(64 * kRowsWaves);
    switch (S) {
    case 4: hipLaunchKernelGGL(sbvr_gemm_rows32_kernel<4>, grid, block, 0, st, a); break;
#ifndef SBVR_FAST_BUILD
    case 2: hipLaunchKernelGGL(sbvr_gemm_rows32_kernel<2>, grid, block, 0, st, a); break;
    case 3: hipLaunchKernelGGL(sbvr_gemm_rows32_kernel<3>, grid, block, 0, st, a); break;
    case 6: hipLaunchKernelGGL(sbvr_gemm_rows32_kernel<6>, grid, block, 0, st, a); break;
    case 8: hipLaunchKernelGGL(sbvr_gemm_rows32_kernel<8>, grid, block, 0, st, a); break;
#endif
    default: return hipErrorInvalidConfiguration;
    }
    return hipGetLastError();
}

// ------------------------------------- MFMA, up to 32 batch rows, weights decoded by table look-up
//
// The same contraction as sbvr_gemm_rows32_kernel (batch rows = the 32 rows of v_mfma_f32_32x32x16_f16, 32
// columns of decoded fp16 weights as B), with a cheaper decode for 2, 3 and 4 planes.  A weight of a group is
// one of the 2^S subset sums of the group's coefficient line; the lane builds those once per group
// (each the fp32 sum rounded to fp16 once, as the reference's decode() rounds a weight) and keeps
// them as byte tables: the low bytes of entries 0..3, 4..7, ... and the high bytes likewise.  A lane owns a
// whole word of K per step (half h of the wave takes word 2i + h of the word pair i).  Its plane words are
// merged into four "nibble words" Q_p, p = 0..3: nibble n of Q_p is the S-bit selector of element p + 4n, at
// the cost of a rotate and an and-or per plane and p.  Then (Q_p >> 0 or 4) & 0x07070707 is four selectors in
// four bytes, for elements p (+ 4), + 8, + 16, + 24, i.e. a ready v_perm_b32 selector into the byte tables:
// two permutes fetch the low and the high bytes of four weights (four permutes and two bit-field inserts
// with 16 entries, where selector bit 3 chooses between the table halves), two more interleave them into
// packed fp16 pairs.  About 4 VALU operations per weight against 7.5 for the arithmetic decode.
// The k order inside an MFMA follows from that: elements 2q, 2q+8, 2q+16, 2q+24, 2q+1, 2q+9, 2q+17, 2q+25 of
// the lane's word for MFMA q = 0..3 of a step; the activations (the lane's batch row, the same 32 elements:
// 64 bytes, four loads) are put into that order with four permutes per MFMA.
// K can be split across workgroups (blockIdx.y) through the decode kernel's 64-bit accumulators.
constexpr int kLutWaves = 8;
// Batch rows from which the linear takes this kernel.  Measured at 4096 -> 14336 / 14336 -> 4096, 4 planes: 15.3-16.1 us
// for any row count up to 16 (17.3-17.5 at 32; 11.4-12.5 with 2 planes, 12.6-13.7 with 3), against 11.7-12.5 us at
// 5..8 rows and 17.9-20.9 us at 9..16 rows for the decode kernels (13.6-16.0 with 2 planes, 19.6-22.5 with 3).
constexpr int kLutMinRows = 9;

// ---- decode by table look-up, shared by sbvr_gemm_rows32_lut_kernel and sbvr_gemm_lut_kernel (2, 3 or 4 planes)
template <int S>
struct LutTables {
    static constexpr int TW = S == 4 ? 4 : (S == 3 ? 2 : 1);       // dwords of a byte table
    uint32_t lo[TW], hi[TW];       // low and high bytes of the subset sums 0..3, 4..7, ...
};

// The 2^S subset sums of a coefficient line, entries (2i, 2i + 1) as packed pairs, then as byte tables.  Entry i is
// the sum of the coefficients whose bit is set in i, added up in fp32 and rounded to fp16 once: the reference's
// decode() takes a weight from bin_combs @ coeff (sbvr/core.py:345-366, 927-949), the exact sum rounded once.  The
// fp32 sums are exact, and the entries therefore decode()'s weights bit for bit, whenever the exponents of a line's
// coefficients lie within 11 of each other (every partial sum is then a multiple of the smallest coefficient's
// last place below 2^24 of them); a line that mixes coefficients 2^12 apart and more can differ from decode() in
// the last place of an entry that lands on a rounding tie.
template <int S>
__device__ __forceinline__ void lut_build_tables(const uint32_t (&c)[(S + 1) / 2], LutTables<S> &t)
{
    float cf[S];
#pragma unroll
    for (int q = 0; q < S; ++q)
        cf[q] = h2f(static_cast<uint16_t>(q & 1 ? c[q / 2] >> 16 : c[q / 2] & 0xffffu));
    float s[1 << S];
    s[0] = 0.f;
#pragma unroll
    for (int q = 0; q < S; ++q)
#pragma unroll
        for (int i = 0; i < (1 << q); ++i)
            s[(1 << q) + i] = i == 0 ? cf[q] : s[i] + cf[q];
    v2h e[1 << (S - 1)];
#pragma unroll
    for (int i = 0; i < (1 << (S - 1)); ++i) {
        e[i][0] = static_cast<_Float16>(s[2 * i]);         // (one v_cvt_pk_f16_f32 per pair, round to nearest even)
        e[i][1] = static_cast<_Float16>(s[2 * i + 1]);
    }
#pragma unroll
    for (int i = 0; i < LutTables<S>::TW; ++i) {
        const uint32_t e0 = __builtin_bit_cast(uint32_t, e[2 * i]), e1 = __builtin_bit_cast(uint32_t, e[2 * i + 1]);
        t.lo[i] = __builtin_amdgcn_perm(e1, e0, 0x06040200u);
        t.hi[i] = __builtin_amdgcn_perm(e1, e0, 0x07050301u);
    }
}

// Nibble words of one word of K: nibble n of Q[p] = selector (one bit per plane) of element p + 4n.
template <int S>
__device__ __forceinline__ void lut_nibble_words(const uint32_t (&w)[S], uint32_t (&Q)[4])
{
    auto rotr = [](uint32_t v, int r) __attribute__((always_inline)) -> uint32_t {
        return (r & 31) == 0 ? v : __builtin_amdgcn_alignbit(v, v, r & 31);
    };
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        uint32_t v = rotr(w[0], p) & 0x11111111u;
        v = (rotr(w[1], p - 1) & 0x22222222u) | v;
        if constexpr (S >= 3)
            v = (rotr(w[2], p - 2) & 0x44444444u) | v;
        if constexpr (S == 4)
            v = (rotr(w[3], p - 3) & 0x88888888u) | v;
        Q[p] = v;
    }
}

// The weights of elements p, p + 8 (w01) and p + 16, p + 24 (w23) of the word, p = 0..7, as packed fp16 pairs.
template <int S>
__device__ __forceinline__ void lut_look_up(const LutTables<S> &t, const uint32_t (&Q)[4], int p, uint32_t &w01, uint32_t &w23)
{
    const uint32_t qs = p < 4 ? Q[p & 3] : Q[p & 3] >> 4;
    const uint32_t sel = qs & (S == 2 ? 0x03030303u : 0x07070707u);
    uint32_t lo, hi;
    if constexpr (S == 2) {
        lo = __builtin_amdgcn_perm(t.lo[0], t.lo[0], sel);
        hi = __builtin_amdgcn_perm(t.hi[0], t.hi[0], sel);
    } else {
        lo = __builtin_amdgcn_perm(t.lo[1], t.lo[0], sel);
        hi = __builtin_amdgcn_perm(t.hi[1], t.hi[0], sel);
    }
    if constexpr (S == 4) {
        // bytes of ones where selector bit 3 is set: a look-up in the two-entry table {0x00, 0xff}
        const uint32_t upper = __builtin_amdgcn_perm(0x0000ff00u, 0x0000ff00u, (qs >> 3) & 0x01010101u);
        const uint32_t lo_u = __builtin_amdgcn_perm(t.lo[3], t.lo[2], sel), hi_u = __builtin_amdgcn_perm(t.hi[3], t.hi[2], sel);
        lo = (lo_u & upper) | (lo & ~upper);
        hi = (hi_u & upper) | (hi & ~upper);
    }
    w01 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
    w23 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
}

// The B operand of MFMA q = 0..3 of the word: elements 2q, 2q+8, 2q+16, 2q+24, 2q+1, 2q+9, 2q+17, 2q+25.
template <int S>
__device__ __forceinline__ v4u lut_operand(const LutTables<S> &t, const uint32_t (&Q)[4], int q)
{
    uint32_t b0, b1, b2, b3;
    lut_look_up<S>(t, Q, 2 * q, b0, b1);
    lut_look_up<S>(t, Q, 2 * q + 1, b2, b3);
    return v4u{b0, b1, b2, b3};
}

// kHalfRows: up to 16 batch rows (the activation loads of rows 16..31 are left out); kShare: groups of a multiple
// of 128 elements, so the two steps of a loop iteration (an even word pair and the next) share a coefficient line:
// one index load, one gather and one table per two steps.
template <int S, bool kHalfRows, bool kShare>
__global__ void __launch_bounds__(64 * kLutWaves)
sbvr_gemm_rows32_lut_kernel(const RowsArgs a)
{
    static_assert(S >= 2 && S <= 4, "tables of 4, 8 or 16 entries");
    __shared__ float red[kLutWaves][16][64];
    // a wave's activations of one step: 32 rows of 128 bytes (the word pair), rows 144 bytes apart so that 16 lanes
    // reading the same 16-byte chunk of 16 rows hit 16 different bank groups
    constexpr int kXRow = 144;
    __shared__ __align__(16) unsigned char xs[kLutWaves][32 * kXRow];
    constexpr int CW = (S + 1) / 2;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = a.N, K = a.K, M = a.M;
    const int j = lane & 31, h = lane >> 5;
    const int n = blockIdx.x * 32 + j, n_ld = min(n, N - 1);
    const int pairs = K / 64;
    const int wg_begin = blockIdx.y * a.pairs_per_wg, wg_end = min(pairs, wg_begin + a.pairs_per_wg);
    const int ppw = ((wg_end - wg_begin + kLutWaves - 1) / kLutWaves + 1) / 2 * 2;     // even: see the loop
    const int p_begin = wg_begin + wave * ppw, p_end = min(wg_end, p_begin + ppw);
    // The activations come in whole cache lines: load i of a step brings rows 8i .. 8i+7, eight lanes per row (128
    // bytes: the 64 elements of the word pair), and goes through LDS to the lanes that want a row each.  (A lane
    // loading its own row's 64 bytes touches 64 cache lines per load instruction; the launch was bound by that.)
    const uint16_t *xsrc = a.x + 8 * (lane & 7);
    size_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        xoff[i] = static_cast<size_t>(min(8 * i + (lane >> 3), M - 1)) * K;     // (rows past M repeat the last one; dropped at the end)
    unsigned char *const xw = xs[wave] + (lane >> 3) * kXRow + (lane & 7) * 16;  // + 8 i rows
    const unsigned char *const xr = xs[wave] + j * kXRow + 64 * h;                // this lane's row, its word's 64 bytes

    struct Step {
        uint32_t w[S];
        v4u x[4];
        uint32_t c[CW];
    };
    // (loads are never conditional: a pair past the range repeats the last one of K and is not computed)
    // The two bytes of a line index stay as they were loaded until the step that uses them: any arithmetic on them
    // here (even putting them into one word) would have to wait for them, and with them for every load issued before.
    struct Line {
        int lo, hi;
    };
    auto load_line = [&](int ip) __attribute__((always_inline)) -> Line {
        const int word = 2 * min(ip, pairs - 1);
        const size_t at = (static_cast<size_t>(word / a.words_per_group) * N + n_ld) << a.idx16;
        const uint8_t *ib = static_cast<const uint8_t *>(a.idx);
        return Line{ib[at], ib[at + a.idx16]};                 // two byte loads whatever the width: no branch
    };
    auto load_step = [&](int ip, Step &st, const Line &line, bool with_line) __attribute__((always_inline)) {
        const int word = 2 * min(ip, pairs - 1) + h;
        const Planes<S> pl = load_planes<S, true>(a.bvr + (static_cast<size_t>(word) * N + n_ld) * S);
#pragma unroll
        for (int q = 0; q < S; ++q)
            st.w[q] = pl.w[q];
#pragma unroll
        for (int i = 0; i < (kHalfRows ? 2 : 4); ++i)
            st.x[i] = *reinterpret_cast<const v4u *>(xsrc + xoff[i] + 64 * min(ip, pairs - 1));
        if (with_line) {                  // (known where the call is written: no branch)
            const int ln = min(a.idx16 ? line.lo | (line.hi << 8) : line.lo, a.L - 1);
            load_line_coeffs<S>(a.cache + static_cast<size_t>(ln) * S, st.c);
        }
    };

    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        acc[r] = 0.f;

    LutTables<S> tables;
    auto build_table = [&](const uint32_t (&c)[CW]) __attribute__((always_inline)) { lut_build_tables<S>(c, tables); };
    auto compute = [&](const Step &st) __attribute__((always_inline)) {
        // ---- activations: rows as loaded -> LDS -> a row per lane (the LDS serves a wave's accesses in order)
#pragma unroll
        for (int i = 0; i < (kHalfRows ? 2 : 4); ++i)
            *reinterpret_cast<v4u *>(xw + 8 * i * kXRow) = st.x[i];
        __builtin_amdgcn_wave_barrier();
        v4u xl[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            xl[i] = *reinterpret_cast<const v4u *>(xr + 16 * i);
        __builtin_amdgcn_wave_barrier();
        uint32_t Q[4];
        lut_nibble_words<S>(st.w, Q);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v4u bw = lut_operand<S>(tables, Q, q);
            v4u aw;
            // dword i of the lane's 64 bytes of activations holds elements 2i, 2i + 1
            const uint32_t d0 = xl[0][q], d1 = xl[1][q], d2 = xl[2][q], d3 = xl[3][q];
            aw.x = __builtin_amdgcn_perm(d1, d0, 0x05040100u);
            aw.y = __builtin_amdgcn_perm(d3, d2, 0x05040100u);
            aw.z = __builtin_amdgcn_perm(d1, d0, 0x07060302u);
            aw.w = __builtin_amdgcn_perm(d3, d2, 0x07060302u);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, aw), __builtin_bit_cast(v8h, bw), acc, 0, 0, 0);
        }
    };

    // (two register sets: with three, the loads two steps ahead, the kernel needs 115 registers and was 8-25 % slower)
    Step s0, s1;
    Line line = load_line(p_begin);
    load_step(p_begin, s0, line, true);
    line = load_line(p_begin + (kShare ? 2 : 1));
    // (the fences keep the loads of the next step in front of this step's arithmetic: left alone, the scheduler
    // moves them down to their first use, to save registers, and every step waits for loads it has just issued)
    // (a wave's priority falls with its progress, as in the decode kernels: the CU serves the oldest wave among
    // equals, and the youngest waves of a workgroup would finish last; 2-3 % at the 4096 <-> 14336 shapes)
    const int l_quarter = ((p_end - p_begin) / 4 + 1) / 2 * 2;
    __builtin_amdgcn_s_setprio(2);
    for (int ip = p_begin; ip < p_end; ip += 2) {
        if (ip == p_begin + 2 * l_quarter)
            __builtin_amdgcn_s_setprio(1);
        if (ip == p_begin + 3 * l_quarter)
            __builtin_amdgcn_s_setprio(0);
        load_step(ip + 1, s1, line, !kShare);
        if constexpr (!kShare)
            line = load_line(ip + 2);
        __builtin_amdgcn_sched_barrier(0);
        build_table(s0.c);
        compute(s0);
        __builtin_amdgcn_sched_barrier(0);
        load_step(ip + 2, s0, line, true);
        line = load_line(ip + (kShare ? 4 : 3));
        __builtin_amdgcn_sched_barrier(0);
        if (ip + 1 < p_end) {
            if constexpr (!kShare)
                build_table(s1.c);
            compute(s1);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    __builtin_amdgcn_s_setprio(0);
    // ---- partial results meet in LDS; D[i][jj] sits in lane jj + 32*((i/4)%2), register (i%4) + 4*(i/8)
#pragma unroll
    for (int r = 0; r < 16; ++r)
        red[wave][r][lane] = acc[r];
    __syncthreads();
    const uint16_t bias = a.bias && n < N ? a.bias[n] : 0;
#pragma unroll
    for (int rr = 0; rr < 16 / kLutWaves; ++rr) {
        const int r = wave * (16 / kLutWaves) + rr;
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kLutWaves; ++w)
            total += red[w][r][lane];
        const int m = 8 * (r >> 2) + 4 * h + (r & 3);
        const bool valid = m < M && n < N;
        const size_t at = static_cast<size_t>(m) * N + n;
        if (a.ksplit > 1) {
            unsigned long long tot = (1ull << 56) + static_cast<unsigned long long>(to_fixed(total) + kAccBias);
            unsigned long long old = 0ull;
            if (valid)
                old = __hip_atomic_fetch_add(a.acc + at, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            tot += old;
            if (!valid || static_cast<int>(tot >> 56) != a.ksplit)
                continue;
            const long long sum = static_cast<long long>(tot & ((1ull << 56) - 1)) - (static_cast<long long>(a.ksplit) << 47);
            const float hi = static_cast<float>(static_cast<int>(sum >> 24));
            const float lo = static_cast<float>(static_cast<int>(sum & 0xffffff));
            total = fmaf(hi, 1.f / (1 << (kAccFracBits - 24)), lo * (1.f / (1 << kAccFracBits)));
            __hip_atomic_store(a.acc + at, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (!valid) {
            continue;
        }
        uint16_t v = f2h(total);
        if (a.bias)
            v = hadd(v, bias);
        a.out[at] = v;
    }
}

bool lut_path_ok(int M, int N, int K, int S, int G)
{
    return M >= 1 && M <= kRowsMax && K % 64 == 0 && G % 64 == 0 && (S == 2 || S == 3 || S == 4) &&
           static_cast<double>(K / 32) * N * S < 2147483648.0;
}

// Workgroups along K: until the 32-column blocks times the parts fill the CUs, a wave keeping 4 word pairs and more.
int lut_ksplit(int N, int K, int cus)
{
    const int blocks = (N + 31) / 32, pairs = K / 64;
    int ks = 1;
    while (blocks * ks < cus && pairs / (ks * 2) >= 4 * kLutWaves && ks < 16)
        ks *= 2;
    return ks;
}

hipError_t launch_rows32_lut(int S, RowsArgs a, hipStream_t st)
{
    // (an even number of word pairs per workgroup and per wave: a loop iteration starts on an even pair, which the
    // shared coefficient line of the kShare instances relies on)
    const int pairs = a.K / 64;
    a.pairs_per_wg = ((pairs + a.ksplit - 1) / a.ksplit + 1) / 2 * 2;
    const dim3 grid(static_cast<unsigned>((a.N + 31) / 32), static_cast<unsigned>(a.ksplit)), block(64 * kLutWaves);
    const bool half = a.M <= 16, share = a.words_per_group % 4 == 0;
#define SBVR_LUT(SS)                                                                                          \
    if (half && share)                                                                                        \
        hipLaunchKernelGGL((sbvr_gemm_rows32_lut_kernel<SS, true, true>), grid, block, 0, st, a);             \
    else if (half)                                                                                            \
        hipLaunchKernelGGL((sbvr_gemm_rows32_lut_kernel<SS, true, false>), grid, block, 0, st, a);            \
    else if (share)                                                                                           \
        hipLaunchKernelGGL((sbvr_gemm_rows32_lut_kernel<SS, false, true>), grid, block, 0, st, a);            \
    else                                                                                                      \
        hipLaunchKernelGGL((sbvr_gemm_rows32_lut_kernel<SS, false, false>), grid, block, 0, st, a);           \
    break
    switch (S) {
    case 4: SBVR_LUT(4);
#ifndef SBVR_FAST_BUILD
    case 2: SBVR_LUT(2);
    case 3: SBVR_LUT(3);
#endif
    default: return hipErrorInvalidConfiguration;
    }
#undef SBVR_LUT
    return hipGetLastError();
}

bool gemm_path_ok(int M, int N, int K, int S, int G)
{
    return M > kMaxM && K % kGemmBK == 0 && G % kGemmBK == 0 && (S == 2 || S == 3 || S == 4 || S == 6 || S == 8) &&
           static_cast<double>(K / 32) * N * S < 2147483648.0 && static_cast<double>(M) * K < 2147483648.0;
}

// Workgroups along K for the prefill kernel: as long as the output tiles alone leave half of the
// chip's 256 CUs without a workgroup, and a part keeps at least 16 steps.  A function of the shape
// only, so that the workspace can be sized without a device.
constexpr int kGemmSplitCus = 256, kGemmMaxKsplit = 8;

int gemm_tiles(int M, int N)
{
    return ((N + kGemmBN - 1) / kGemmBN) * ((M + kGemmBM - 1) / kGemmBM);
}

int gemm_ksplit(int M, int N, int K)
{
    const int tiles = gemm_tiles(M, N), steps = K / kGemmBK;
    int ks = 1;
    if (N % 4)                  // the second pass works on four outputs of a row at a time
        return 1;
    while (ks < kGemmMaxKsplit && tiles * ks * 2 <= kGemmSplitCus && steps % (ks * 2) == 0 && steps / (ks * 2) >= 16)
        ks *= 2;
    return ks;
}

// Workspace of the split prefill launch: the partial results.
size_t gemm_workspace_bytes(int M, int N, int K)
{
    const int ks = gemm_ksplit(M, N, K);
    return ks == 1 ? 0 : static_cast<size_t>(ks) * M * N * sizeof(float);
}

hipError_t launch_gemm(int S, const GemmArgs &a, hipStream_t st)
{
    const dim3 grid(static_cast<unsigned>((a.N + kGemmBN - 1) / kGemmBN), static_cast<unsigned>((a.M + kGemmBM - 1) / kGemmBM),
                    static_cast<unsigned>(a.ksplit));
    const dim3 block(kGemmThreads);
    const size_t lds = kGemmABufs * kGemmATile + 2 * kGemmBTile;      // 128 KiB: above the 64 KiB a kernel gets without asking
#define SBVR_GEMM_LAUNCH(SS)                                                                                   \
    {                                                                                                          \
        static bool raised_on[16] = {};                                                                        \
        std::lock_guard<std::mutex> guard(g_dev_lock);                                                                        \
        int dev_now = 0;                                                                                       \
        if (hipGetDevice(&dev_now) != hipSuccess || dev_now < 0 || dev_now >= 16)                              \
            dev_now = 0;                                                                                       \
        bool &raised = raised_on[dev_now];                                                                     \
        if (!raised) {                                                                                         \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sbvr_gemm_mfma_kernel<SS>), \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
            if (e != hipSuccess)                                                                               \
                return e;                                                                                      \
            raised = true;                                                                                     \
        }                                                                                                      \
        hipLaunchKernelGGL(sbvr_gemm_mfma_kernel<SS>, grid, block, lds, st, a);                                \
    }                                                                                                          \
    break
    switch (S) {
    case 4: SBVR_GEMM_LAUNCH(4);
#ifndef SBVR_FAST_BUILD
    case 2: SBVR_GEMM_LAUNCH(2);
    case 3: SBVR_GEMM_LAUNCH(3);
    case 6: SBVR_GEMM_LAUNCH(6);
    case 8: SBVR_GEMM_LAUNCH(8);
#endif
    default: return hipErrorInvalidConfiguration;
    }
#undef SBVR_GEMM_LAUNCH
    return hipGetLastError();
}

// ------------------------------------------- MFMA prefill with the weights decoded by table look-up
//
// The prefill contraction with the decode of sbvr_gemm_rows32_lut_kernel: no producer and consumer waves and no
// weight tile in LDS.  A workgroup of 8 waves owns 256 rows x 256 columns of the output; wave w owns columns
// 32w .. 32w+31 for all 256 rows (8 row blocks of 32: 128 accumulator registers a lane).  Per step of 64 elements
// of K a lane (column j, half h) decodes its word 2i + h of column j by table look-up straight into the B operands
// of four MFMAs (16 registers), and the wave runs them against the 8 row blocks: 32 MFMAs per 32 weights decoded
// per lane, so the decode (about 170 VALU instructions a step) hides behind the matrix pipe (32 x 32 clocks).
// The activations of a step, 256 rows x 64 elements, are shared by the 8 waves through LDS, stored in the element
// order the MFMAs want (see sbvr_gemm_rows32_lut_kernel: that permutation is done once, by the thread that
// brings a (row, word) in, not once per wave): rows 144 bytes apart, two buffers, one barrier per step.  The loads
// of the step after the next one's (activations, plane words) are in flight while a step is computed.
// 2, 3 or 4 planes, K and G multiples of 128 (the two steps of a loop iteration share a coefficient line).
// K can be split across workgroups (blockIdx.z) as in sbvr_gemm_mfma_kernel: fp32 partial tiles, second pass.
constexpr int kPfWaves = 8, kPfBM = 256, kPfBN = 256, kPfRow = 144;
constexpr int kPfTile = kPfBM * kPfRow;

template <int S>
__global__ void __launch_bounds__(64 * kPfWaves)
sbvr_gemm_lut_kernel(const GemmArgs a)
{
    static_assert(S >= 2 && S <= 4, "tables of 4, 8 or 16 entries");
    extern __shared__ __align__(16) unsigned char psm[];
    constexpr int CW = (S + 1) / 2;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = a.N, K = a.K, M = a.M;
    const int j = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * kPfBN, m0 = blockIdx.y * kPfBM;
    const int n = n0 + 32 * wave + j, n_ld = min(n, N - 1);
    const int steps = K / 64 / a.ksplit;                 // of this workgroup, even
    const int p0 = blockIdx.z * steps, p_last = p0 + steps - 1;
    const int wpg = 2 * a.steps_per_group;               // words per group

    // bringing activations in: thread t takes (row t / 2, word t % 2) of a step, 64 bytes
    const uint16_t *xsrc = a.x + static_cast<size_t>(min(m0 + (tid >> 1), M - 1)) * K + 32 * (tid & 1);
    unsigned char *const xdst = psm + (tid >> 1) * kPfRow + (tid & 1) * 64;
    const unsigned char *const xrd = psm + j * kPfRow + h * 64;      // + 32 rb rows, + 16 q

    struct Line {
        int lo, hi;
    };
    auto load_line = [&](int ip) __attribute__((always_inline)) -> Line {
        const size_t at = (static_cast<size_t>((2 * min(ip, p_last)) / wpg) * N + n_ld) << a.idx16;
        const uint8_t *ib = static_cast<const uint8_t *>(a.idx);
        return Line{ib[at], ib[at + a.idx16]};
    };
    auto load_coefficients = [&](const Line &line, uint32_t (&c)[CW]) __attribute__((always_inline)) {
        const int ln = min(a.idx16 ? line.lo | (line.hi << 8) : line.lo, a.L - 1);
        load_line_coeffs<S>(a.cache + static_cast<size_t>(ln) * S, c);
    };
    auto load_words = [&](int ip, uint32_t (&w)[S]) __attribute__((always_inline)) {
        const int word = 2 * min(ip, p_last) + h;
        const Planes<S> pl = load_planes<S>(a.bvr + (static_cast<size_t>(word) * N + n_ld) * S);
#pragma unroll
        for (int q = 0; q < S; ++q)
            w[q] = pl.w[q];
    };
    auto load_x = [&](int ip, v4u (&x)[4]) __attribute__((always_inline)) {
        const v4u *xp = reinterpret_cast<const v4u *>(xsrc + 64 * min(ip, p_last));
#pragma unroll
        for (int i = 0; i < 4; ++i)
            x[i] = xp[i];
    };
    // the 32 elements of a (row, word), dword i = elements 2i, 2i + 1, into the order of the four MFMAs' A operands:
    // operand q = elements 2q, 2q+8, 2q+16, 2q+24, 2q+1, 2q+9, 2q+17, 2q+25
    auto store_x = [&](const v4u (&x)[4], int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t d0 = x[0][q], d1 = x[1][q], d2 = x[2][q], d3 = x[3][q];
            v4u aw;
            aw.x = __builtin_amdgcn_perm(d1, d0, 0x05040100u);
            aw.y = __builtin_amdgcn_perm(d3, d2, 0x05040100u);
            aw.z = __builtin_amdgcn_perm(d1, d0, 0x07060302u);
            aw.w = __builtin_amdgcn_perm(d3, d2, 0x07060302u);
            *reinterpret_cast<v4u *>(xdst + buf * kPfTile + 16 * q) = aw;
        }
    };

    LutTables<S> tables;
    auto build_table = [&](const uint32_t (&c)[CW]) __attribute__((always_inline)) { lut_build_tables<S>(c, tables); };

    v16f acc[8];
#pragma unroll
    for (int rb = 0; rb < 8; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[rb][r] = 0.f;

    auto compute = [&](const uint32_t (&w)[S], int buf) __attribute__((always_inline)) {
        uint32_t Q[4];
        lut_nibble_words<S>(w, Q);
        auto operand = [&](int q) __attribute__((always_inline)) -> v4u { return lut_operand<S>(tables, Q, q); };
        // MFMA q of all 8 row blocks in a row (8 different accumulators), its 8 activation operands read while
        // MFMA q - 1 runs, and the look-ups of operand q + 1 in the shadow of the matrix pipe
        const unsigned char *xt = xrd + buf * kPfTile;
        v4u A[2][8];
        auto read_a = [&](int q, v4u (&dst)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (int rb = 0; rb < 8; ++rb)
                dst[rb] = *reinterpret_cast<const v4u *>(xt + 32 * rb * kPfRow + 16 * q);
        };
        read_a(0, A[0]);
        v4u Bq = operand(0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v4u Bn = Bq;
            if (q < 3) {
                read_a(q + 1, A[(q + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
                Bn = operand(q + 1);
            }
#pragma unroll
            for (int rb = 0; rb < 8; ++rb)
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, A[q & 1][rb]), __builtin_bit_cast(v8h, Bq), acc[rb], 0, 0, 0);
            Bq = Bn;
        }
    };

    // -- prologue: the first step's activations into buffer 0, everything of the second in flight
    // (decoding a step's operands one step ahead, in the shadow of the step before's MFMAs, measured no faster)
    uint32_t wa[S], wb[S], c[CW], c_next[CW];
    v4u xa[4];
    Line line = load_line(p0);
    load_words(p0, wa);
    load_x(p0, xa);
    load_coefficients(line, c);
    line = load_line(p0 + 2);
    store_x(xa, 0);
    load_x(p0 + 1, xa);
    load_words(p0 + 1, wb);
    __syncthreads();
    for (int ip = p0; ip <= p_last; ip += 2) {
        // -- even step: buffer 0
        load_coefficients(line, c_next);              // of the next pair of steps
        line = load_line(ip + 4);
        __builtin_amdgcn_sched_barrier(0);
        build_table(c);
        compute(wa, 0);
        __builtin_amdgcn_sched_barrier(0);
        store_x(xa, 1);                                // step ip + 1
        load_x(ip + 2, xa);
        load_words(ip + 2, wa);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        // -- odd step: buffer 1
        compute(wb, 1);
        __builtin_amdgcn_sched_barrier(0);
        store_x(xa, 0);                                // step ip + 2
        load_x(ip + 3, xa);
        load_words(ip + 3, wb);
#pragma unroll
        for (int q = 0; q < CW; ++q)
            c[q] = c_next[q];
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    }

    // ---- D[i][jj] of a row block sits in lane jj + 32*((i/4)%2), register (i%4) + 4*(i/8)
    if (a.ksplit > 1) {
        float *mine = a.part + blockIdx.z * (static_cast<size_t>(M) * N);
#pragma unroll
        for (int rb = 0; rb < 8; ++rb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + 32 * rb + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < M && n < N)
                    mine[static_cast<size_t>(m) * N + n] = acc[rb][r];
            }
        return;
    }
    if (n >= N)
        return;
    const uint16_t bias = a.bias ? a.bias[n] : 0;
#pragma unroll
    for (int rb = 0; rb < 8; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + 32 * rb + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m < M) {
                uint16_t v = f2h(acc[rb][r]);
                if (a.bias)
                    v = hadd(v, bias);
                a.out[static_cast<size_t>(m) * N + n] = v;
            }
        }
}

bool gemm_lut_path_ok(int M, int N, int K, int S, int G)
{
    return M > kRowsMax && K % 128 == 0 && G % 128 == 0 && (S == 2 || S == 3 || S == 4) &&
           static_cast<double>(K / 32) * N * S < 2147483648.0 && static_cast<double>(M) * K < 2147483648.0;
}

// Workgroups along K for the table look-up prefill kernel: until the 256 x 256 tiles times the parts give three
// quarters of the chip's 256 CUs a workgroup, a part keeping 16 steps and more (an even number).  A function of the
// shape only.  (8192 -> 28672: 112 tiles at 256 rows take 229-236 us unsplit and 187 us in two parts; 224 tiles at
// 512 rows 293 us unsplit and 340 us in two parts.)
int gemm_lut_ksplit(int M, int N, int K)
{
    const int tiles = ((N + kPfBN - 1) / kPfBN) * ((M + kPfBM - 1) / kPfBM), steps = K / 64;
    int ks = 1;
    if (N % 4)
        return 1;
    while (ks < 16 && tiles * ks * 4 < 3 * kGemmSplitCus && steps % (ks * 4) == 0 && steps / (ks * 2) >= 16)
        ks *= 2;
    return ks;
}

hipError_t launch_gemm_lut(int S, const GemmArgs &a, hipStream_t st)
{
    const dim3 grid(static_cast<unsigned>((a.N + kPfBN - 1) / kPfBN), static_cast<unsigned>((a.M + kPfBM - 1) / kPfBM),
                    static_cast<unsigned>(a.ksplit));
    const dim3 block(64 * kPfWaves);
    const size_t lds = 2 * kPfTile;
#define SBVR_PF_LAUNCH(SS)                                                                                     \
    {                                                                                                          \
        static bool raised_on[16] = {};                                                                        \
        std::lock_guard<std::mutex> guard(g_dev_lock);                                                                        \
        int dev_now = 0;                                                                                       \
        if (hipGetDevice(&dev_now) != hipSuccess || dev_now < 0 || dev_now >= 16)                              \
            dev_now = 0;                                                                                       \
        bool &raised = raised_on[dev_now];                                                                     \
        if (!raised) {                                                                                         \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sbvr_gemm_lut_kernel<SS>), \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
            if (e != hipSuccess)                                                                               \
                return e;                                                                                      \
            raised = true;                                                                                     \
        }                                                                                                      \
        hipLaunchKernelGGL(sbvr_gemm_lut_kernel<SS>, grid, block, lds, st, a);                                 \
    }                                                                                                          \
    break
    switch (S) {
    case 4: SBVR_PF_LAUNCH(4);
#ifndef SBVR_FAST_BUILD
    case 2: SBVR_PF_LAUNCH(2);
    case 3: SBVR_PF_LAUNCH(3);
#endif
    default: return hipErrorInvalidConfiguration;
    }
#undef SBVR_PF_LAUNCH
    return hipGetLastError();
}

int current_cus()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
        return 256;
    std::lock_guard<std::mutex> guard(g_dev_lock);
    if (!g_dev[dev].ready) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            g_dev[dev].cus = prop.multiProcessorCount;
            g_dev[dev].ready = true;
        }
    }
    return g_dev[dev].cus;
}

// -------------------------------------------- trans=True and both-encoded forms

// One thread per output; the lanes of a wave share k and differ in n, so the
// plane words and indices are wave-uniform broadcasts.
template <typename IdxT>
__global__ void __launch_bounds__(256)
sbvr_row_deq_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ bvr,
                    const void *__restrict__ idx, const uint16_t *__restrict__ cache,
                    const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                    int M, int N, int K, int S, int G)
{
    const size_t o = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= static_cast<size_t>(M) * N)
        return;
    const int m = static_cast<int>(o / N), n = static_cast<int>(o % N);
    float acc = bias ? h2f(bias[n]) : 0.f;
    for (int k = 0; k < K; ++k) {
        const int line = load_idx<IdxT>(idx, static_cast<size_t>(n / G) * K + k);
        float w = 0.f;
        for (int j = 0; j < S; ++j) {
            const uint32_t bits = bvr[(static_cast<size_t>(n >> 5) * K + k) * S + j];
            if ((bits >> (n & 31)) & 1u)
                w += h2f(cache[static_cast<size_t>(line) * S + j]);
        }
        acc = fmaf(h2f(x[static_cast<size_t>(m) * K + k]), w, acc);
    }
    out[o] = f2h(acc);
}

// The same product with the lanes of a wave along K.  A word of the trans=True
// layout holds one row k of 32 columns, and rows follow each other in memory
// (bvr[nw][k][S]), so lane l of a wave takes row 64*step + l: its plane words,
// line index, coefficient line and activation are its own (coalesced loads, one
// gather), z_j = x[k] * c_j is formed once, and the 32 columns of the word
// block each get sum_j (bit_j ? z_j : 0) added to an accumulator of their own
// (32 per lane).  A workgroup owns one block of 32 columns and one batch row;
// its waves take the steps in turn.  At the end the 64 lanes are summed per
// column (DPP), the waves meet in LDS and the first wave adds up, in a fixed
// order.  The loads of a step are requested one step ahead, its line index two.
constexpr int kRowDeqWaves = 16;

template <int S>
__global__ void __launch_bounds__(64 * kRowDeqWaves)
sbvr_row_deq_lanes_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ bvr,
                          const void *__restrict__ idx, const uint16_t *__restrict__ cache,
                          const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                          int M, int N, int K, int L, int G, int idx16)
{
    __shared__ float part[kRowDeqWaves][32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int nw = blockIdx.x, m = blockIdx.y;
    const int steps = (K + 63) >> 6;
    const uint32_t *wbase = bvr + static_cast<size_t>(nw) * K * S;
    const size_t ibase = static_cast<size_t>((nw * 32) / G) * K;
    const uint16_t *xrow = x + static_cast<size_t>(m) * K;

    float acc[32];
#pragma unroll
    for (int b = 0; b < 32; ++b)
        acc[b] = 0.f;

    // (two byte loads whatever the index width, put together where the index is used:
    // no branch between loads, no early wait on the youngest load)
    auto load_line = [&](int step) __attribute__((always_inline)) -> int {
        const size_t at = (ibase + static_cast<size_t>(min(step * 64 + lane, K - 1))) << idx16;
        const uint8_t *ib = static_cast<const uint8_t *>(idx);
        return static_cast<int>(ib[at]) | (static_cast<int>(ib[at + idx16]) << 16);
    };
    auto line_of = [&](int raw) __attribute__((always_inline)) -> int {
        return min(idx16 ? (raw & 0xff) | ((raw >> 8) & 0xff00) : raw & 0xff, L - 1);
    };
    constexpr int CW = (S + 1) / 2;
    auto load_coeffs = [&](int raw, uint32_t (&c)[CW]) __attribute__((always_inline)) {
        load_line_coeffs<S>(cache + static_cast<size_t>(line_of(raw)) * S, c);
    };
    const int last = steps - 1;
    // pipeline: raw index of step i+2, and words / coefficients / activation of step i+1
    int raw_next = load_line(min(wave, last));
    int raw_after = load_line(min(wave + waves, last));
    Planes<S> w_next = load_planes<S>(wbase + static_cast<size_t>(min(min(wave, last) * 64 + lane, K - 1)) * S);
    uint16_t x_next = xrow[min(min(wave, last) * 64 + lane, K - 1)];
    uint32_t c_next[CW];
    load_coeffs(raw_next, c_next);

    for (int step = wave; step < steps; step += waves) {
        const Planes<S> w = w_next;
        uint32_t c[CW];
#pragma unroll
        for (int j = 0; j < CW; ++j)
            c[j] = c_next[j];
        const float xv = step * 64 + lane < K ? h2f(x_next) : 0.f;
        // requests of the following steps (beyond the end they repeat the last step)
        const int s1 = min(step + waves, last), s2 = min(step + 2 * waves, last);
        w_next = load_planes<S>(wbase + static_cast<size_t>(min(s1 * 64 + lane, K - 1)) * S);
        x_next = xrow[min(s1 * 64 + lane, K - 1)];
        load_coeffs(raw_after, c_next);
        raw_after = load_line(s2);

        uint32_t z[S];
#pragma unroll
        for (int j = 0; j < S; ++j)
            z[j] = __float_as_uint(xv * h2f(static_cast<uint16_t>(j & 1 ? c[j / 2] >> 16 : c[j / 2] & 0xffffu)));
#pragma unroll
        for (int b = 0; b < 32; ++b) {
#pragma unroll
            for (int j = 0; j < S; ++j) {
                // all ones where bit b of the plane word is set
                const uint32_t mask = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(w.w[j]), b, 1));
                acc[b] += __uint_as_float(z[j] & mask);
            }
        }
    }

    float mine = 0.f;
#pragma unroll
    for (int b = 0; b < 32; ++b) {
        const float v = wave_fsum(acc[b]);
        mine = lane == b ? v : mine;
    }
    if (lane < 32)
        part[wave][lane] = mine;
    __syncthreads();
    if (wave == 0 && lane < 32) {
        const int n = nw * 32 + lane;
        float total = bias ? h2f(bias[n]) : 0.f;
        for (int w = 0; w < waves; ++w)
            total += part[w][lane];
        out[static_cast<size_t>(m) * N + n] = f2h(total);
    }
}

// The trans=True product on the matrix cores (4 planes, K a multiple of 128, groups of 64 columns and more).
// A word of this layout holds one row k of 32 columns, so the bits that an MFMA wants along K lie across rows.
// The lanes of a wave, each holding one row's word, transpose the four 16 x 16 bit blocks of every 32 rows between
// them in four exchange stages (two DPP quad permutes, one DPP row rotate, one ds_swizzle; per stage a rotate and a
// bit-field insert): lane 16q + c then holds column c's bits of rows 16q .. 16q+15 in its low half and column
// 16 + c's in its high half.  Two such loads (rows 0-63 and 64-127 of a sub-group) give the B operands of the word's
// two column tiles without moving anything between lanes: the low halves of both, side by side, are tile 0's
// operand (lane group q of an MFMA operand is lanes 16q .. 16q+15: rows 16q .. 16q+15 and 64+16q .. 64+16q+15 of
// column c), the high halves tile 1's; the A image's bytes are laid out in that order of K.
// The A operand carries z_j[k] = fp16(x[k] * c_j(line of the column group at row k)) for the four planes as its
// "batch rows" (plane j: rows 4j .. 4j+2, three exact fp8 terms as in the decode kernel), and the four MFMAs of a
// unit each use a copy with the other planes' rows zeroed, so they accumulate into one result: lane group j keeps
// plane j's sum.  A workgroup owns 64 columns of one coefficient group and one batch row; its waves take the
// sub-groups of K in turn (one A image serves all the workgroup's columns).
// Numerics: z is rounded to fp16 once (2^-12 relative per product, random sign), everything after that is exact up
// to the fp32 sums; the one-lane-per-row kernel above keeps z in fp32.
__device__ __forceinline__ uint32_t transpose_16x16_blocks_across_lanes(uint32_t w, int lane)
{
    const int r = lane & 15;
#define SBVR_TSTAGE(s, Ms, EXCH)                                                             \
    {                                                                                         \
        const uint32_t p = EXCH;                                                              \
        const uint32_t rot = __builtin_amdgcn_alignbit(p, p, (r & s) ? s : 32 - s);           \
        const uint32_t keep = (r & s) ? Ms : ~Ms;                                             \
        w = (w & keep) | (rot & ~keep);                                                       \
    }
    SBVR_TSTAGE(8, 0xFF00FF00u, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w), 0x128, 0xF, 0xF, true)))   // row_ror 8
    SBVR_TSTAGE(4, 0xF0F0F0F0u, static_cast<uint32_t>(__builtin_amdgcn_ds_swizzle(static_cast<int>(w), (4 << 10) | 0x1f)))
    SBVR_TSTAGE(2, 0xCCCCCCCCu, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w), 0x4E, 0xF, 0xF, true)))    // quad_perm 2,3,0,1
    SBVR_TSTAGE(1, 0xAAAAAAAAu, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w), 0xB1, 0xF, 0xF, true)))    // quad_perm 1,0,3,2
#undef SBVR_TSTAGE
    return w;
}

template <int NWW>
__global__ void __launch_bounds__(64 * kRowDeqWaves)
sbvr_row_deq_mfma_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ bvr,
                         const void *__restrict__ idx, const uint16_t *__restrict__ cache,
                         const uint16_t *__restrict__ bias, uint16_t *__restrict__ out, unsigned long long *__restrict__ acc_words,
                         int M, int N, int K, int L, int G, int idx16, int ksplit)
{
    constexpr int S = 4;
    __shared__ __align__(16) unsigned char images[kRowDeqWaves][2048];
    __shared__ float red[kRowDeqWaves][2 * NWW][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int blk = lane >> 4;
    const int m = blockIdx.y;
    const int nwords = N / 32;
    const int nw0 = NWW * blockIdx.x;                     // the workgroup's NWW column words (the last ones may be missing)
    const int nsub = K / kSub;
    const size_t ibase = static_cast<size_t>((nw0 * 32) / G) * K;
    const uint16_t *xrow = x + static_cast<size_t>(m) * K;
    unsigned char *const img = images[wave];

    // where this lane's two elements (rows 8g + t and 8g + t + 4 of the sub-group, see the decode kernel) sit in the A
    // image: row k = 64 b + 16 q + i is bit 16 b + i of lane group q's B words
    const int el = 8 * (lane >> 2) + (lane & 3);
    const int off = a_image_byte_offset(32 * ((el >> 4) & 3) + 16 * (el >> 6) + (el & 15), 0);
    const uint32_t half_sel = (lane & 1) ? 0x07060302u : 0x05040100u;
    const int fac_log2 = (lane & 3) == 0 ? 2 : ((lane & 3) == 1 ? 1 : 0);
    const int row_plane = (lane & 15) >> 2;               // plane whose terms this lane's A row carries

    // (K split across workgroups, blockIdx.z, where the columns alone leave CUs idle: the parts meet in the 64-bit
    // fixed-point accumulators of the decode kernel)
    const int per_part = (nsub + ksplit - 1) / ksplit;
    const int sg_begin = static_cast<int>(blockIdx.z) * per_part, sg_end = min(nsub, sg_begin + per_part);
    float acc[NWW][2];
#pragma unroll
    for (int h = 0; h < NWW; ++h)
        acc[h][0] = acc[h][1] = 0.f;
    // The coefficient lines of a sub-group are two round trips away (line index, then the gather): both are sent for
    // one sub-group ahead, the indices at the top of the step before, the gathers at its end.
    auto load_x_idx = [&](int sg, uint32_t &xv, uint32_t &raw) __attribute__((always_inline)) {
        const int k0 = sg * kSub;
        xv = reinterpret_cast<const uint32_t *>(xrow + k0)[lane];
        if (idx16)
            raw = reinterpret_cast<const uint32_t *>(static_cast<const uint16_t *>(idx) + ibase + k0)[lane];
        else
            raw = reinterpret_cast<const uint16_t *>(static_cast<const uint8_t *>(idx) + ibase + k0)[lane];
    };
    auto gather_lines = [&](uint32_t raw, uint32_t (&c0)[2], uint32_t (&c1)[2]) __attribute__((always_inline)) {
        const int l0 = static_cast<int>(idx16 ? raw & 0xffffu : raw & 0xffu), l1 = static_cast<int>(idx16 ? raw >> 16 : (raw >> 8) & 0xffu);
        load_line_words<S>(cache + static_cast<size_t>(min(l0, L - 1)) * S, c0);
        load_line_words<S>(cache + static_cast<size_t>(min(l1, L - 1)) * S, c1);
    };
    uint32_t xv = 0u, x_next = 0u, raw_next = 0u;
    uint32_t c0[2] = {0u, 0u}, c1[2] = {0u, 0u}, n0[2] = {0u, 0u}, n1[2] = {0u, 0u};
    if (sg_begin + wave < sg_end) {
        uint32_t raw_first;
        load_x_idx(sg_begin + wave, x_next, raw_first);
        gather_lines(raw_first, n0, n1);
    }
    for (int sg = sg_begin + wave; sg < sg_end; sg += waves) {          // wave-uniform
        const int k0 = sg * kSub;
        // -- requests: plane words of the column words (rows k0 .. k0+63 and k0+64 .. k0+127); activations and line
        //    indices of the next sub-group
        // (asking for the next sub-group's plane words here as well measured slower: 16.9 against 15.3 us)
        v4u wa[NWW], wb[NWW];
#pragma unroll
        for (int h = 0; h < NWW; ++h) {
            const uint32_t *base = bvr + static_cast<size_t>(min(nw0 + h, nwords - 1)) * K * S;
            wa[h] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(base + static_cast<size_t>(k0 + lane) * S));
            wb[h] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(base + static_cast<size_t>(k0 + 64 + lane) * S));
        }
        xv = x_next;
        c0[0] = n0[0]; c0[1] = n0[1]; c1[0] = n1[0]; c1[1] = n1[1];
        const bool more = sg + waves < sg_end;
        if (more)
            load_x_idx(sg + waves, x_next, raw_next);

        // -- A image: plane j's row is z_j = fp16(x * c_j) of the 128 rows
        const float x0 = h2f(static_cast<uint16_t>(xv & 0xffffu)), x1 = h2f(static_cast<uint16_t>(xv >> 16));
        reinterpret_cast<uint4 *>(img)[lane * 2] = uint4{0u, 0u, 0u, 0u};
        reinterpret_cast<uint4 *>(img)[lane * 2 + 1] = uint4{0u, 0u, 0u, 0u};
        float scale_mine = 0.f;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const float cj0 = h2f(static_cast<uint16_t>(j & 1 ? c0[j / 2] >> 16 : c0[j / 2] & 0xffffu));
            const float cj1 = h2f(static_cast<uint16_t>(j & 1 ? c1[j / 2] >> 16 : c1[j / 2] & 0xffffu));
            const uint32_t v = static_cast<uint32_t>(f2h(x0 * cj0)) | (static_cast<uint32_t>(f2h(x1 * cj1)) << 16);
            const uint32_t amax = wave_umax(max(v & 0x7fffu, (v >> 16) & 0x7fffu));
            const int eh = min(max(static_cast<int>(amax >> 10), 1), 30);
            const int e = 20 - eh;
            if (blk == j)
                scale_mine = __uint_as_float(static_cast<uint32_t>(126 - e) << 23);
            const int va = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x50, 0xF, 0xF, true);   // quad_perm 0,0,1,1
            const int vb = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xFA, 0xF, 0xF, true);   // quad_perm 2,2,3,3
            v2h z = as_v2h(__builtin_amdgcn_perm(static_cast<uint32_t>(vb), static_cast<uint32_t>(va), half_sel));
            const float sc = __uint_as_float(static_cast<uint32_t>(127 - e - fac_log2) << 23);
            const float sc_last = __uint_as_float(static_cast<uint32_t>(127 - 8 - e - fac_log2) << 23);
            v2s b = {0, 0};
            b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, false);
            z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, false);
            b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, true);
            z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, true);
            const v2s b3 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(v2s{0, 0}, z, sc_last, false);
            *reinterpret_cast<short *>(img + off + (j * 4 + 0) * 32) = b[0];
            *reinterpret_cast<short *>(img + off + (j * 4 + 1) * 32) = b[1];
            *reinterpret_cast<short *>(img + off + (j * 4 + 2) * 32) = b3[0];
        }
        const v8i A = *reinterpret_cast<const v8i *>(img + lane * 32);
        v8i Aj[S];
#pragma unroll
        for (int j = 0; j < S; ++j)
#pragma unroll
            for (int q = 0; q < 8; ++q)
                Aj[j][q] = row_plane == j ? A[q] : 0;

        // -- the units: per column word, transposed words of the two row halves -> B operands of its two tiles
#pragma unroll
        for (int h = 0; h < NWW; ++h) {
            v4f D[2];
            D[0] = v4f{0.f, 0.f, 0.f, 0.f};
            D[1] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < S; ++j) {
                const uint32_t ta = transpose_16x16_blocks_across_lanes(wa[h][j], lane);
                const uint32_t tb = transpose_16x16_blocks_across_lanes(wb[h][j], lane);
                const uint32_t pr[2] = {(ta & 0xffffu) | (tb << 16), (ta >> 16) | (tb & 0xffff0000u)};
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t w = pr[t];
                    v8i B;
                    B[0] = static_cast<int>(w & 0x11111111u);
                    B[1] = static_cast<int>(w & 0x22222222u);
                    B[2] = static_cast<int>(w & 0x44444444u);
                    B[3] = static_cast<int>((w >> 1) & 0x44444444u);
                    B[4] = 0; B[5] = 0; B[6] = 0; B[7] = 0;
                    D[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(Aj[j], B, D[t], 0, 4, 0, 0, 0, 0);
                }
            }
#pragma unroll
            for (int t = 0; t < 2; ++t)
                acc[h][t] = fmaf(fmaf(D[t][2], 1.f / kLastTermScale, D[t][0] + D[t][1]), scale_mine, acc[h][t]);
        }
        if (more)
            gather_lines(raw_next, n0, n1);
    }
#pragma unroll
    for (int h = 0; h < NWW; ++h)
#pragma unroll
        for (int t = 0; t < 2; ++t)
            red[wave][h * 2 + t][lane] = acc[h][t];
    __syncthreads();
    // tile by tile (the first waves take one each): over the waves, then over the four planes (lane groups)
    for (int tile = wave; tile < 2 * NWW; tile += waves) {      // wave-uniform
        float total = 0.f;
        for (int w = 0; w < waves; ++w)
            total += red[w][tile][lane];
        red[0][tile][lane] = total;           // (the first row's slot of this tile: read above, by this lane only)
        __builtin_amdgcn_s_waitcnt(0xc07f);    // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
        if (lane < 16) {
            float sum = (red[0][tile][lane] + red[0][tile][lane + 16]) + (red[0][tile][lane + 32] + red[0][tile][lane + 48]);
            const int n = (nw0 + (tile >> 1)) * 32 + (tile & 1) * 16 + lane;
            if (n < N) {
                const size_t at = static_cast<size_t>(m) * N + n;
                bool mine_to_store = true;
                if (ksplit > 1) {
                    unsigned long long tot = (1ull << 56) + static_cast<unsigned long long>(to_fixed(sum) + kAccBias);
                    tot += __hip_atomic_fetch_add(acc_words + at, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    mine_to_store = static_cast<int>(tot >> 56) == ksplit;
                    if (mine_to_store) {
                        const long long fixed = static_cast<long long>(tot & ((1ull << 56) - 1)) - (static_cast<long long>(ksplit) << 47);
                        const float hi = static_cast<float>(static_cast<int>(fixed >> 24));
                        const float lo = static_cast<float>(static_cast<int>(fixed & 0xffffff));
                        sum = fmaf(hi, 1.f / (1 << (kAccFracBits - 24)), lo * (1.f / (1 << kAccFracBits)));
                        __hip_atomic_store(acc_words + at, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
                if (mine_to_store) {
                    uint16_t r = f2h(sum);
                    if (bias)
                        r = hadd(r, bias[n]);
                    out[at] = r;
                }
            }
        }
    }
}

template <typename LIdxT, typename RIdxT>
__global__ void __launch_bounds__(256)
sbvr_mm_T_kernel(const uint32_t *__restrict__ l_bvr, const void *__restrict__ l_idx,
                 const uint16_t *__restrict__ l_cache, const uint32_t *__restrict__ r_bvr,
                 const void *__restrict__ r_idx, const uint16_t *__restrict__ r_cache,
                 const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                 int M, int N, int K, int Sl, int Sr, int G)
{
    const size_t o = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= static_cast<size_t>(M) * N)
        return;
    const int m = static_cast<int>(o / N), n = static_cast<int>(o % N);
    const int wpg = G / 32;
    float acc = 0.f;
    for (int g = 0; g < K / G; ++g) {
        const uint16_t *ca = l_cache + static_cast<size_t>(load_idx<LIdxT>(l_idx, static_cast<size_t>(g) * M + m)) * Sl;
        const uint16_t *cb = r_cache + static_cast<size_t>(load_idx<RIdxT>(r_idx, static_cast<size_t>(g) * N + n)) * Sr;
        for (int l = 0; l < Sl; ++l) {
            const float al = h2f(ca[l]);
            for (int r = 0; r < Sr; ++r) {
                int pc = 0;
                for (int w = 0; w < wpg; ++w) {
                    const size_t kw = static_cast<size_t>(g) * wpg + w;
                    pc += __builtin_popcount(l_bvr[(kw * M + m) * Sl + l] & r_bvr[(kw * N + n) * Sr + r]);
                }
                acc = fmaf(static_cast<float>(pc), al * h2f(cb[r]), acc);
            }
        }
    }
    uint16_t res = f2h(acc);
    if (bias)
        res = hadd(res, bias[n]);
    out[o] = res;
}

// Both operands encoded (the form the reference's kernels compute, sbvr_kernel.cu:464-562
// and sbvr_kernel.cpp:251-399): out[m,n] = sum_g sum_{l,r} popcount_g(L_l & R_r) a_l b_r.
// A wave owns 64 / Q columns and Q parts of its share of K: lane = part * (64 / Q) + column,
// so it reads Q runs of (64 / Q) * SR consecutive plane words per word of K.  With Q = 1 the
// left operand's words and coefficients are wave-uniform (scalar loads); Q = 4 is for
// matrices with so few columns that 64-column workgroups would leave most CUs idle.  The
// waves of a workgroup split the groups of K and meet in LDS; blockIdx.y is the left row.
// Popcounts are exact integers per group; coefficients are applied in fp32.
constexpr int kPopcWaves = 8, kPopcChunk = 8;      // words of K whose plane words a lane holds at once

template <int SL, int SR, int Q>
__global__ void __launch_bounds__(64 * kPopcWaves)
sbvr_mm_T_popc_kernel(const uint32_t *__restrict__ l_bvr, const uint8_t *__restrict__ l_idx, int l_idx16,
                      const uint16_t *__restrict__ l_cache, const uint32_t *__restrict__ r_bvr,
                      const uint8_t *__restrict__ r_idx, int r_idx16, const uint16_t *__restrict__ r_cache,
                      const uint16_t *__restrict__ bias, uint16_t *__restrict__ out,
                      int M, int N, int K, int wpg, int Ll, int Lr)
{
    constexpr int C = 64 / Q;                       // columns of a wave
    __shared__ float red[kPopcWaves][C];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int m = blockIdx.y;
    const int col = lane & (C - 1), part = lane / C;
    const int n = blockIdx.x * C + col, n_ld = min(n, N - 1);
    const int words = K / 32;
    const int chunks = (words + kPopcChunk - 1) / kPopcChunk;
    const int cpw = (chunks + kPopcWaves * Q - 1) / (kPopcWaves * Q);     // chunks per (wave, part)
    const int c_begin = (wave * Q + part) * cpw, c_end = min(chunks, c_begin + cpw);      // per lane when Q > 1

    auto load_chunk = [&](int c, uint32_t (&rw)[kPopcChunk][SR], int (&line)[kPopcChunk]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kPopcChunk; ++i) {
            const int w = min(c * kPopcChunk + i, words - 1);       // beyond K: repeats the last word, never used
            const Planes<SR> pl = load_planes<SR>(r_bvr + (static_cast<size_t>(w) * N + n_ld) * SR);
#pragma unroll
            for (int r = 0; r < SR; ++r)
                rw[i][r] = pl.w[r];
            // one line index per group; read per word (same address within a group: cached)
            const size_t at = (static_cast<size_t>(w / wpg) * N + n_ld) << r_idx16;
            const int lo = r_idx[at], hi = r_idx[at + r_idx16];
            line[i] = lo | (hi << 16);                              // raw: decoded where it is used
        }
    };

    float acc = 0.f;
    uint32_t rw0[kPopcChunk][SR], rw1[kPopcChunk][SR];
    int ln0[kPopcChunk], ln1[kPopcChunk];
    // one chunk; `live` is false for a chunk past the lane's range (its counts are then masked out)
    auto compute = [&](int c, bool live, const uint32_t (&rw)[kPopcChunk][SR], const int (&line)[kPopcChunk]) __attribute__((always_inline)) {
        int cnt[SL][SR];
#pragma unroll
        for (int l = 0; l < SL; ++l)
#pragma unroll
            for (int r = 0; r < SR; ++r)
                cnt[l][r] = 0;
#pragma unroll
        for (int i = 0; i < kPopcChunk; ++i) {
            const int w = c * kPopcChunk + i;
            if constexpr (Q == 1) {
                if (w >= words)                                      // wave-uniform
                    break;
            }
            const bool counts = Q == 1 || (live && w < words);
            const int wl = Q == 1 ? w : min(w, words - 1);
            const uint32_t *lp = l_bvr + (static_cast<size_t>(wl) * M + m) * SL;      // wave-uniform when Q == 1
#pragma unroll
            for (int l = 0; l < SL; ++l) {
                uint32_t lw = lp[l];
                if constexpr (Q == 1)
                    lw = __builtin_amdgcn_readfirstlane(lw);
                else
                    lw = counts ? lw : 0u;
#pragma unroll
                for (int r = 0; r < SR; ++r)
                    cnt[l][r] += __builtin_popcount(lw & rw[i][r]);
            }
            if ((i + 1) % wpg == 0) {                                // wave-uniform: last word of its group
                const size_t lat = (static_cast<size_t>(wl / wpg) * M + m) << l_idx16;
                const int llo = l_idx[lat], lhi = l_idx[lat + l_idx16];
                int lline = min(l_idx16 ? llo | (lhi << 8) : llo, Ll - 1);
                if constexpr (Q == 1)
                    lline = __builtin_amdgcn_readfirstlane(lline);
                const uint16_t *ca = l_cache + static_cast<size_t>(lline) * SL;
                const int rline = min(r_idx16 ? (line[i] & 0xff) | ((line[i] >> 8) & 0xff00) : line[i] & 0xff, Lr - 1);
                const uint16_t *cb = r_cache + static_cast<size_t>(rline) * SR;
                float group = 0.f;
#pragma unroll
                for (int r = 0; r < SR; ++r) {
                    float t = 0.f;
#pragma unroll
                    for (int l = 0; l < SL; ++l) {
                        t = fmaf(static_cast<float>(cnt[l][r]), h2f(ca[l]), t);
                        cnt[l][r] = 0;
                    }
                    group = fmaf(t, h2f(cb[r]), group);
                }
                acc += group;
            }
        }
    };

    if constexpr (Q == 1) {
        if (c_begin < c_end) {
            load_chunk(c_begin, rw0, ln0);
            for (int c = c_begin; c < c_end; c += 2) {
                load_chunk(min(c + 1, chunks - 1), rw1, ln1);
                compute(c, true, rw0, ln0);
                load_chunk(min(c + 2, chunks - 1), rw0, ln0);
                if (c + 1 < c_end)
                    compute(c + 1, true, rw1, ln1);
            }
        }
    } else {
        // the parts of a wave walk their ranges in step: same trip count for every lane
        load_chunk(min(c_begin, chunks - 1), rw0, ln0);
        for (int t = 0; t < cpw; t += 2) {
            const int c = c_begin + t;
            load_chunk(min(c + 1, chunks - 1), rw1, ln1);
            compute(c, c < c_end, rw0, ln0);
            load_chunk(min(c + 2, chunks - 1), rw0, ln0);
            if (t + 1 < cpw)
                compute(c + 1, c + 1 < c_end, rw1, ln1);
        }
#pragma unroll
        for (int off = C; off < 64; off <<= 1)
            acc += __shfl_xor(acc, off, 64);
    }
    if (part == 0)
        red[wave][col] = acc;
    __syncthreads();
    if (wave == 0 && part == 0 && n < N) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kPopcWaves; ++w)
            total += red[w][col];
        uint16_t res = f2h(total);
        if (bias)
            res = hadd(res, bias[n]);
        out[static_cast<size_t>(m) * N + n] = res;
    }
}

template <int SL>
bool launch_mm_T_popc_sr(int Sr, int Q, hipStream_t st, const uint32_t *l_bvr, const uint8_t *l_idx, int l16,
                         const uint16_t *lc, const uint32_t *r_bvr, const uint8_t *r_idx, int r16, const uint16_t *rc,
                         const uint16_t *b, uint16_t *o, int M, int N, int K, int wpg, int Ll, int Lr)
{
    const dim3 block(64 * kPopcWaves);
    const int cols = 64 / Q;
    const dim3 grid(static_cast<unsigned>((N + cols - 1) / cols), static_cast<unsigned>(M));
#define SBVR_POPC(SR)                                                                                                \
    do {                                                                                                             \
        if (Q == 4)                                                                                                  \
            hipLaunchKernelGGL((sbvr_mm_T_popc_kernel<SL, SR, 4>), grid, block, 0, st, l_bvr, l_idx, l16, lc, r_bvr, \
                               r_idx, r16, rc, b, o, M, N, K, wpg, Ll, Lr);                                          \
        else                                                                                                         \
            hipLaunchKernelGGL((sbvr_mm_T_popc_kernel<SL, SR, 1>), grid, block, 0, st, l_bvr, l_idx, l16, lc, r_bvr, \
                               r_idx, r16, rc, b, o, M, N, K, wpg, Ll, Lr);                                          \
    } while (0)
    switch (Sr) {
    case 2: SBVR_POPC(2); return true;
    case 3: SBVR_POPC(3); return true;
    case 4: SBVR_POPC(4); return true;
    default: return false;
    }
#undef SBVR_POPC
}

} // namespace

// ---- measurement aid: a launch that only reads.  What the memory system of the part hands to a launch of a given
// size, whatever grid the decode kernel happens to use: every wave requests `units` units of 1 KiB (one
// global_load_dwordx4 per lane: the decode kernel's request) and keeps AHEAD of them in flight; nothing else.
//   pattern 0: unit i of wave w is KiB number i * (waves of the grid) + w of the buffer: at any time the grid
//              reads one contiguous band;
//   pattern 1: unit i of wave w is KiB number w * units + i: every wave walks its own contiguous piece;
//   pattern 2: the decode kernel's own: the buffer is rows of `row_bytes` (one word of K for all columns), a
//              workgroup owns `win_bytes` of every row and its waves split the rows; a unit is 256 bytes of four
//              consecutive rows (lanes past the window repeat its last 16 bytes, as the kernel's lanes do).
namespace {

template <int AHEAD>
__global__ void __launch_bounds__(1024)
sbvr_read_floor_kernel(const v4u *__restrict__ base, uint32_t units, int pattern, uint32_t row_bytes, uint32_t win_bytes,
                       uint32_t *__restrict__ sink)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * waves + wave, total = gridDim.x * waves;
    const uint32_t tiles = (win_bytes + 255u) / 256u;            // pattern 2: units per four rows of the window
    auto unit_ptr = [&](uint32_t i) __attribute__((always_inline)) -> const v4u * {
        if (pattern == 2) {
            const uint32_t sg = wave * (units / tiles) + i / tiles, ct = i % tiles;
            const size_t row = static_cast<size_t>(4u * sg + (lane >> 4));
            const uint32_t in_win = min(ct * 256u + (lane & 15u) * 16u, win_bytes - 16u);
            return reinterpret_cast<const v4u *>(reinterpret_cast<const unsigned char *>(base) + row * row_bytes +
                                                 static_cast<size_t>(blockIdx.x) * win_bytes + in_win);
        }
        const size_t kib = pattern == 0 ? static_cast<size_t>(i) * total + gw : static_cast<size_t>(gw) * units + i;
        return base + kib * 64u + lane;
    };
    v4u q[AHEAD], seen = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < AHEAD; ++j)
        q[j] = __builtin_nontemporal_load(unit_ptr(static_cast<uint32_t>(j)));
    for (uint32_t i = AHEAD; i < units; i += AHEAD) {             // (units is a multiple of AHEAD: checked by the host)
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            seen ^= q[j];
            q[j] = __builtin_nontemporal_load(unit_ptr(i + static_cast<uint32_t>(j)));
        }
    }
#pragma unroll
    for (int j = 0; j < AHEAD; ++j)
        seen ^= q[j];
    if ((seen.x ^ seen.y ^ seen.z ^ seen.w) == 0x9e3779b9u && units == 0x7fffffffu)      // never true: keeps the loads alive
        sink[lane] = seen.x;
}

} // namespace

namespace {

// ------------------------------------ attention and output projection of one decoded token, one launch
//
// The decoder layer's attention (rotary embedding, cache append, softmax(q k^T / sqrt(d)) v over the cached
// positions; reference models/sbvr_llama.py:193-224, 255-278, 307-354) followed by its SBVR-encoded o_proj, for
// batch 1 and query length 1, heads of 128 = one sub-group of the projection's K, four query heads per
// key/value head.  As two launches the pair costs two kernel boundaries and two chains of memory round trips
// for a few hundred KiB of traffic; here workgroup (g, e) does the attention of key/value head g's four query
// heads by itself and then multiplies their 512 context values into columns [128 e, 128 e + 128) of the
// projection, whose K is thereby split kv_heads ways across workgroups (the decode kernel's fixed-point
// accumulators).  Every workgroup of a key/value head repeats that head's attention (N / 128 times: cheap on the
// matrix cores, and the head's cache rows come out of one XCD's L2: workgroup (g, e) is number g + kv_heads * e
// of the launch and workgroups go to the 8 XCDs in turn); nothing waits for another workgroup.
//   * scores: v_mfma_f32_16x16x32_f16 with 16 cache positions as the rows of A and the four rotated queries as
//     columns 0..3 of B;
//   * context: the same instruction with 16 head dimensions as the rows of A and 32 positions as the reduction
//     index; B holds the softmax weights (fp16, as the reference's fp16 matmul sees them) of the four heads;
//   * both caches are kept in the element order in which the lanes of those A operands want them, so that
//     every request of a wave is 1 KiB of consecutive memory.  Per key/value head, element (position t,
//     dimension d) lies at
//        keys:   (t/16)*2048 + (d/32)*512 + (d%32/8)*128 + (t%16)*8 + d%8     [block of 16 positions][request j]
//        values: (t/32)*4096 + (d/16)*512 + (t%32/8)*128 + (d%16)*8 + t%8     [block of 32 positions][16 dimensions]
//     with lane (col = lane % 16, blk = lane / 16) reading the 8 elements at + blk*128 + col*8;
//   * a wave asks for things in the order it needs them and no earlier than it must: the new token's q, k, v,
//     the position and its line indices, then the first 256 positions' keys; after the first barrier the
//     values and coefficient lines; after the scores the plane words of its two units of the projection (head
//     wave / 4, columns 32 (wave % 4) .. + 31 of the window).  Rows past the position are fetched for nothing;
//   * the row of the position itself is never taken from the cache: workgroups with e == 0 append it, the
//     others (and they) use their own copy;
//   * the kernel is bound by the instructions its sixteen waves issue, four to a SIMD, not by its MFMAs: work
//     that only one block of positions needs (the new key, masking of values at and past the position) sits
//     behind wave-uniform branches, and a head's A operand for the projection is made by one wave, not four.
// Rounding points are the reference's: rotated q and k, scores, softmax weights and context in fp16; the
// projection is exact in its activations (three fp8 terms) with one rounding at the end.
constexpr int kAoWaves = 16, kAoThreads = 64 * kAoWaves;
constexpr int kAoHead = 128;         // head size
constexpr int kAoGroup = 4;          // query heads per key/value head
constexpr int kAoCols = 128;         // output columns of a workgroup: per head 4 waves x 2 column tiles
constexpr int kAoMaxSeq = 4096;      // 24 bytes of LDS per cache position
constexpr int kAoLdsFixed = 8192 + kAoWaves * 2048;

struct AttnOArgs {
    const uint16_t *qkv;          // [heads | kv_heads | kv_heads] x 128 of the new token
    const float *cos_t, *sin_t;   // (max_seq, 64)
    const float *rot_now;         // row *pos of cos | sin, or NULL
    const long long *pos_p;
    uint16_t *kcache;             // (kv_heads, max_seq * 128), blocked: see the kernel
    uint16_t *vcache;             // (kv_heads, max_seq * 128), blocked
    uint16_t *ctx;                // (heads * 128) or NULL
    int heads, kv_heads, max_seq;
    // the projection (default layout), K = heads * 128
    const uint32_t *bvr;
    const void *idx;
    const uint16_t *cache;
    const uint16_t *bias;
    uint16_t *out;                // (N)
    unsigned long long *acc;      // (N) split-K accumulators, all zero between calls (kv_heads > 1)
    int N, L, gshift, idx16;
};

typedef v4u __attribute__((may_alias)) v4u_alias;      // 16-byte reads of memory written as fp16 elements

#ifdef SBVR_TRACE
__device__ unsigned long long g_ao_trace[2 * 16 * 12];      // development builds: timestamps of the waves of two workgroups
#define SBVR_AOSTAMP(i)                                                                                         \
    do {                                                                                                        \
        if (blockIdx.x == 0 && (blockIdx.y == 0 || blockIdx.y == 12) && (threadIdx.x & 63) == 0)                \
            g_ao_trace[((blockIdx.y != 0) * 16 + (threadIdx.x >> 6)) * 12 + (i)] = wall_clock64();              \
    } while (0)
#else
#define SBVR_AOSTAMP(i) do { } while (0)
#endif

template <int S>
__global__ void __launch_bounds__(kAoThreads)
sbvr_attn_o_kernel(const AttnOArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int max_seq = a.max_seq;
    uint16_t *const qn = reinterpret_cast<uint16_t *>(smem);               // rotated queries of the group: 4 x 128
    uint16_t *const kn = qn + kAoGroup * kAoHead;                          // rotated new key
    uint16_t *const vn = kn + kAoHead;                                     // new value
    float *const red_max = reinterpret_cast<float *>(smem + 1536);         // [wave][head]
    float *const red_sum = red_max + kAoWaves * kAoGroup;                  // [wave]
    float *const a_scale = red_sum + kAoWaves;                             // [head]: 2^-(e+1) of its A operand
    float *const part = reinterpret_cast<float *>(smem + 2048);            // [position half][head][dimension]
    float *const ysum = reinterpret_cast<float *>(smem + 6144);            // [head][column of the window]
    unsigned char *const abuf = smem + 8192;                               // the heads' A operand images, 2 KiB each
    float *const scores = reinterpret_cast<float *>(smem + kAoLdsFixed);   // [head][position]
    uint16_t *const wts = reinterpret_cast<uint16_t *>(scores + kAoGroup * max_seq);   // [head][position], fp16

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, blk = lane >> 4;
    const int g = static_cast<int>(blockIdx.x);        // key/value head (workgroups go to the XCDs by x + 8 y with 8 heads)
    const int e = static_cast<int>(blockIdx.y);        // window of the projection's columns
    const int N = a.N;
    uint16_t *const kc = a.kcache + static_cast<size_t>(g) * max_seq * kAoHead;
    uint16_t *const vc = a.vcache + static_cast<size_t>(g) * max_seq * kAoHead;

    // -- 1. requests that need no position, in the order they are wanted
    const long long p64 = *a.pos_p;
    SBVR_AOSTAMP(0);
    // the new token: waves 0..3 take query head `wave` of the group, wave 4 the key, wave 5 the value; lane d
    // holds elements d and d + 64 (a rotation pair)
    uint16_t na = 0, nb = 0;
    float c_now = 0.f, s_now = 0.f;
    if (wave < 6) {                          // wave-uniform
        const int row = wave < 4 ? kAoGroup * g + wave : (wave == 4 ? a.heads + g : a.heads + a.kv_heads + g);
        const uint16_t *src = a.qkv + static_cast<size_t>(row) * kAoHead;
        na = src[lane];
        nb = src[lane + kAoHead / 2];
        if (wave < 5 && a.rot_now) {
            c_now = a.rot_now[lane];
            s_now = a.rot_now[kAoHead / 2 + lane];
        }
    }
    // the projection: head hq = wave / 4 of the group is sub-group sgk of its K; the wave's 32 columns, whose line
    // indices lane l % 32 asks for
    const int hq = wave >> 2;
    const int sgk = kAoGroup * g + hq;
    const int n0 = e * kAoCols + 32 * (wave & 3);
    const size_t irow = static_cast<size_t>(sgk >> a.gshift) * N + n0 + (lane & 31);
    const int lraw = a.idx16 ? static_cast<int>(static_cast<const uint16_t *>(a.idx)[irow])
                             : static_cast<int>(static_cast<const uint8_t *>(a.idx)[irow]);
    // keys: wave w takes the 16-position blocks w, w + 16, ...: 2048 elements each, four requests of 1 KiB
    v4u kpre[4];
    {
        const uint16_t *kb = kc + static_cast<size_t>(min(wave, max_seq / 16 - 1)) * 2048 + lane * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            kpre[j] = *reinterpret_cast<const v4u_alias *>(kb + j * 512);
    }
    // (the values and the projection's plane words are asked for further down, each as late as its use allows: a
    // CU takes about 48 requests of 1 KiB at a time, and a wave that stands in the queue with requests it needs
    // last keeps all sixteen from their first barrier)
    __builtin_amdgcn_sched_barrier(0);
    SBVR_AOSTAMP(1);

    // -- 2. the position is here: rotate, leave q, k, v of the new token in LDS, append (e == 0)
    const int p = p64 < 0 ? 0 : (p64 >= max_seq ? max_seq - 1 : static_cast<int>(p64));
    SBVR_AOSTAMP(2);
    if (wave < 5) {
        if (!a.rot_now) {
            c_now = a.cos_t[static_cast<size_t>(p) * (kAoHead / 2) + lane];
            s_now = a.sin_t[static_cast<size_t>(p) * (kAoHead / 2) + lane];
        }
        const float xa = h2f(na), xb = h2f(nb);
        const uint16_t r0 = f2h(xa * c_now - xb * s_now), r1 = f2h(xb * c_now + xa * s_now);
        uint16_t *const dst = wave < 4 ? qn + wave * kAoHead : kn;
        dst[lane] = r0;
        dst[lane + kAoHead / 2] = r1;
        if (wave == 4 && e == 0) {
            // dimension d of position p: block p / 16, request d / 32, lane (d % 32 / 8, p % 16), element d % 8
            uint16_t *const at = kc + static_cast<size_t>(p >> 4) * 2048 + (lane >> 5) * 512 + ((lane & 31) >> 3) * 128 +
                                 (p & 15) * 8 + (lane & 7);
            at[0] = r0;
            at[1024] = r1;                   // d + 64: two requests on
        }
    } else if (wave == 5) {
        vn[lane] = na;
        vn[lane + kAoHead / 2] = nb;
        if (e == 0) {
            // dimension d of position p: block p / 32, dimensions block d / 16, lane (p % 32 / 8, d % 16), element p % 8
            uint16_t *const at = vc + static_cast<size_t>(p >> 5) * 4096 + (lane >> 4) * 512 + ((p & 31) >> 3) * 128 +
                                 (lane & 15) * 8 + (p & 7);
            at[0] = na;
            at[2048] = nb;                   // d + 64: four blocks of dimensions on
        }
    }
    __syncthreads();
    SBVR_AOSTAMP(3);
    // values: wave (db = w % 8, ph = w / 8) takes dimensions 16 db .. + 15 of the 32-position blocks ph, ph + 2, ...:
    // 512 elements of each block, one request of 1 KiB
    const int db = wave & 7, ph = wave >> 3;
    const uint16_t *const vb = vc + db * 512 + lane * 8;
    v4u vpre[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        vpre[i] = *reinterpret_cast<const v4u_alias *>(vb + static_cast<size_t>(min(ph + 2 * i, max_seq / 32 - 1)) * 4096);
    // (the line indices came with the position: lane l gathers the coefficient line of column n0 + l % 32)
    constexpr int CW = (S + 1) / 2;
    uint32_t cl[CW];
    load_line_words<S>(a.cache + static_cast<size_t>(min(lraw, a.L - 1)) * S, cl);
    __builtin_amdgcn_sched_barrier(0);

    // -- 3. scores of the group's four heads: columns 0..3 of the product.  (The other twelve columns of B repeat
    //       them: a column of the product depends on its own column of B only, and theirs are never read.)
    const float scaling = rsqrtf(static_cast<float>(kAoHead));
    v8h qb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        qb[j] = __builtin_bit_cast(v8h, v4u(*reinterpret_cast<const v4u_alias *>(qn + (col & (kAoGroup - 1)) * kAoHead + 32 * j + 8 * blk)));
    float mx = -INFINITY;                     // of head `col` over the positions this lane sees
    auto score_block = [&](int tb, v4u (&kw)[4]) __attribute__((always_inline)) {
        if ((p >> 4) == tb) {                 // wave-uniform: the block of the new key, which is not taken from the cache
            if (col == (p & 15)) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    kw[j] = *reinterpret_cast<const v4u_alias *>(kn + 32 * j + 8 * blk);
            }
        }
        v4f d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, kw[j]), qb[j], d, 0, 0, 0);
        // the lane holds head `col`, positions 16 tb + 4 blk + i (the reference's q @ k^T is an fp16 matmul)
        const int t0 = 16 * tb + 4 * blk;
        if (col < kAoGroup) {
            float *const sp = scores + col * max_seq + t0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = h2f(f2h(d[i])) * scaling;
                if (t0 + i <= p) {
                    sp[i] = v;
                    mx = fmaxf(mx, v);
                }
            }
        }
    };
    if (16 * wave <= p)                       // wave-uniform
        score_block(wave, kpre);
    for (int tb = wave + kAoWaves; 16 * tb <= p; tb += kAoWaves) {
        v4u kw[4];
        const uint16_t *kb = kc + static_cast<size_t>(tb) * 2048 + lane * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            kw[j] = *reinterpret_cast<const v4u_alias *>(kb + j * 512);
        score_block(tb, kw);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    if (lane < kAoGroup)
        red_max[wave * kAoGroup + lane] = mx;
    __syncthreads();
    SBVR_AOSTAMP(4);
    // the plane words of the wave's two units of the projection
    Planes<S> q[2];
    {
        const uint32_t *wrow = a.bvr + (static_cast<size_t>(4 * sgk + blk) * N + n0 + col) * S;
#pragma unroll
        for (int u = 0; u < 2; ++u)
            q[u] = load_planes<S, true>(wrow + 16 * u * S);
    }
    __builtin_amdgcn_sched_barrier(0);

    // -- 4. softmax: thread (head hs = tid / 256, slot tid % 256) takes positions slot, slot + 256, ...
    const int hs = tid >> 8, slot = tid & 255;
    float *const srow = scores + hs * max_seq;
    float top = -INFINITY;
#pragma unroll
    for (int w = 0; w < kAoWaves; ++w)
        top = fmaxf(top, red_max[w * kAoGroup + hs]);
    float sum = 0.f;
    for (int t = slot; t <= p; t += 256) {
        const float ex = __expf(srow[t] - top);
        srow[t] = ex;
        sum += ex;
    }
    sum = wave_fsum(sum);
    if (lane == 0)
        red_sum[wave] = sum;
    __syncthreads();
    const float inv = 1.f / ((red_sum[4 * hs] + red_sum[4 * hs + 1]) + (red_sum[4 * hs + 2] + red_sum[4 * hs + 3]));
    const int t_pad = (p + 32) & ~31;         // the context products go over whole blocks of 32 positions
    for (int t = slot; t < t_pad; t += 256)   // (weights are rounded to fp16; positions past p weigh nothing)
        wts[hs * max_seq + t] = t <= p ? f2h(srow[t] * inv) : static_cast<uint16_t>(0);
    __syncthreads();
    SBVR_AOSTAMP(5);

    // -- 5. context: dimensions 16 db .. + 15 over the wave's blocks of 32 positions
    v4f o = {0.f, 0.f, 0.f, 0.f};
    const uint16_t *const wrow_l = wts + (col & (kAoGroup - 1)) * max_seq + 8 * blk;
    auto context_block = [&](int pb, v4u vw) __attribute__((always_inline)) {
        if (32 * pb + 31 >= p) {              // wave-uniform: the block of p (later blocks are not visited)
            // positions before p come from the cache, p itself from the new token, later ones may hold anything
            const int ts = 32 * pb + 8 * blk;     // the lane's positions ts .. ts + 7 of dimension 16 db + col
            const uint32_t vfresh = vn[16 * db + col];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int t_lo = ts + 2 * c, t_hi = t_lo + 1;
                const uint32_t lo = t_lo < p ? (vw[c] & 0xffffu) : (t_lo == p ? vfresh : 0u);
                const uint32_t hi = t_hi < p ? (vw[c] >> 16) : (t_hi == p ? vfresh : 0u);
                vw[c] = lo | (hi << 16);
            }
        }
        const v4u wb = *reinterpret_cast<const v4u_alias *>(wrow_l + 32 * pb);
        o = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, vw), __builtin_bit_cast(v8h, wb), o, 0, 0, 0);
    };
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (32 * (ph + 2 * i) <= p)           // wave-uniform
            context_block(ph + 2 * i, vpre[i]);
    for (int pb = ph + 8; 32 * pb <= p; pb += 2)
        context_block(pb, *reinterpret_cast<const v4u_alias *>(vb + static_cast<size_t>(pb) * 4096));
    // the lane holds head `col`, dimensions 16 db + 4 blk + i
    if (col < kAoGroup)
        *reinterpret_cast<v4f *>(part + (ph * kAoGroup + col) * kAoHead + 16 * db + 4 * blk) = o;
    __syncthreads();
    SBVR_AOSTAMP(6);

    // -- 6. a head's context row as the one batch row of the projection's A operand (the decode kernel's step 2:
    //       three fp8 terms per element, written where the MFMA wants them through 2 KiB of LDS); made once per
    //       head, by waves 0, 5, 10 and 15 (one on each SIMD)
    if (wave == 5 * hq) {                     // wave-uniform
        const float2 c0 = reinterpret_cast<const float2 *>(part + hq * kAoHead)[lane];
        const float2 c1 = reinterpret_cast<const float2 *>(part + (kAoGroup + hq) * kAoHead)[lane];
        const uint32_t v = static_cast<uint32_t>(f2h(c0.x + c1.x)) | (static_cast<uint32_t>(f2h(c0.y + c1.y)) << 16);
        if (a.ctx && e == 0)
            reinterpret_cast<uint32_t *>(a.ctx + static_cast<size_t>(sgk) * kAoHead)[lane] = v;
        unsigned char *const mine = abuf + hq * 2048;
        reinterpret_cast<uint4 *>(mine)[lane * 2] = uint4{0u, 0u, 0u, 0u};
        reinterpret_cast<uint4 *>(mine)[lane * 2 + 1] = uint4{0u, 0u, 0u, 0u};
        const uint32_t amax = wave_umax(max(v & 0x7fffu, (v >> 16) & 0x7fffu));
        const int eh = min(max(static_cast<int>(amax >> 10), 1), 30);
        const int ex2 = 20 - eh;              // 2^ex2 puts the head's largest magnitude into [32, 64)
        if (lane == 0)
            a_scale[hq] = __uint_as_float(static_cast<uint32_t>(126 - ex2) << 23);
        const int off = a_image_byte_offset(8 * (lane >> 2) + (lane & 3), 0);
        const uint32_t half_sel = (lane & 1) ? 0x07060302u : 0x05040100u;
        const int fac_log2 = (lane & 3) == 0 ? 2 : ((lane & 3) == 1 ? 1 : 0);
        const int va = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x50, 0xF, 0xF, true);   // quad_perm 0,0,1,1
        const int vb2 = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xFA, 0xF, 0xF, true);  // quad_perm 2,2,3,3
        v2h z = as_v2h(__builtin_amdgcn_perm(static_cast<uint32_t>(vb2), static_cast<uint32_t>(va), half_sel));
        const float sc = __uint_as_float(static_cast<uint32_t>(127 - ex2 - fac_log2) << 23);
        const float sc_last = __uint_as_float(static_cast<uint32_t>(127 - 8 - ex2 - fac_log2) << 23);
        v2s b = {0, 0};
        b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, false);
        z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, false);
        b = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(b, z, sc, true);
        z -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(as_int(b), sc, true);
        const v2s b3 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(v2s{0, 0}, z, sc_last, false);
        *reinterpret_cast<short *>(mine + off + 0 * 32) = b[0];
        *reinterpret_cast<short *>(mine + off + 1 * 32) = b[1];
        *reinterpret_cast<short *>(mine + off + 2 * 32) = b3[0];
    }
    __syncthreads();
    const v8i A = *reinterpret_cast<const v8i *>(abuf + hq * 2048 + lane * 32);
    const float scale = a_scale[hq];
    SBVR_AOSTAMP(7);

    // -- 7. the wave's two units: plane sums, coefficients (lane 16 u + col gathered the line of this lane's column)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        float ps[S];
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const uint32_t w = q[u].w[j];
            v8i B;
            B[0] = static_cast<int>(w & 0x11111111u);
            B[1] = static_cast<int>(w & 0x22222222u);
            B[2] = static_cast<int>(w & 0x44444444u);
            B[3] = static_cast<int>((w >> 1) & 0x44444444u);
            B[4] = 0; B[5] = 0; B[6] = 0; B[7] = 0;
            const v4f zf = {0.f, 0.f, 0.f, 0.f};
            const v4f d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, zf, 0, 4, 0, 0, 0, 0);
            ps[j] = fmaf(d[2], 1.f / kLastTermScale, d[0] + d[1]);
        }
        uint32_t cw[CW];
#pragma unroll
        for (int j = 0; j < CW; ++j)
            cw[j] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((16 * u + col) * 4, static_cast<int>(cl[j])));
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < S; ++j)
            acc = fmaf(h2f(static_cast<uint16_t>(j & 1 ? cw[j / 2] >> 16 : cw[j / 2] & 0xffffu)), ps[j], acc);
        if (blk == 0)                         // (rows 0..2 of the product are the three terms of the one batch row)
            ysum[hq * kAoCols + 32 * (wave & 3) + 16 * u + col] = acc * scale;
    }
    __syncthreads();
    SBVR_AOSTAMP(8);

    // -- 8. the four heads' partial results added in a fixed order; K is split kv_heads ways across workgroups
    if (tid < kAoCols) {
        float total = (ysum[tid] + ysum[kAoCols + tid]) + (ysum[2 * kAoCols + tid] + ysum[3 * kAoCols + tid]);
        const int n = e * kAoCols + tid;
        bool last = true;
        if (a.kv_heads > 1) {
            unsigned long long tot = (1ull << 56) + static_cast<unsigned long long>(to_fixed(total) + kAccBias);
            tot += __hip_atomic_fetch_add(a.acc + n, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = static_cast<int>(tot >> 56) == a.kv_heads;
            if (last) {
                const long long sum56 = static_cast<long long>(tot & ((1ull << 56) - 1)) - (static_cast<long long>(a.kv_heads) << 47);
                const float hi = static_cast<float>(static_cast<int>(sum56 >> 24));
                const float lo = static_cast<float>(static_cast<int>(sum56 & 0xffffff));
                total = fmaf(hi, 1.f / (1 << (kAccFracBits - 24)), lo * (1.f / (1 << kAccFracBits)));
                __hip_atomic_store(a.acc + n, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (last) {
            uint16_t r = f2h(total);
            if (a.bias)
                r = hadd(r, a.bias[n]);
            a.out[n] = r;
        }
    }
    SBVR_AOSTAMP(9);
}

template <int S>
hipError_t launch_attn_o_inst(const AttnOArgs &a, hipStream_t st)
{
    const dim3 grid(static_cast<unsigned>(a.kv_heads), static_cast<unsigned>(a.N / kAoCols)), block(kAoThreads);
    const size_t lds = kAoLdsFixed + 24 * static_cast<size_t>(a.max_seq);
    if (lds > 65536) {          // above what a kernel gets without asking
        static bool raised_on[16] = {};
        std::lock_guard<std::mutex> guard(g_dev_lock);
        int dev_now = 0;
        if (hipGetDevice(&dev_now) != hipSuccess || dev_now < 0 || dev_now >= 16)
            dev_now = 0;
        if (!raised_on[dev_now]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sbvr_attn_o_kernel<S>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess)
                return e;
            raised_on[dev_now] = true;
        }
    }
    hipLaunchKernelGGL((sbvr_attn_o_kernel<S>), grid, block, lds, st, a);
    return hipGetLastError();
}

hipError_t launch_attn_o(int S, const AttnOArgs &a, hipStream_t st)
{
    switch (S) {
    case 4: return launch_attn_o_inst<4>(a, st);
#ifndef SBVR_FAST_BUILD
    case 2: return launch_attn_o_inst<2>(a, st);
    case 3: return launch_attn_o_inst<3>(a, st);
    case 6: return launch_attn_o_inst<6>(a, st);
    case 8: return launch_attn_o_inst<8>(a, st);
#endif
    default: return hipErrorInvalidConfiguration;
    }
}

bool attn_o_shape_ok(int heads, int kv_heads, int head_dim, int max_seq, int N, int S, int G)
{
    return kv_heads >= 1 && kv_heads <= kMaxKsplit && heads == kAoGroup * kv_heads && head_dim == kAoHead &&
           max_seq >= 32 && max_seq <= kAoMaxSeq && max_seq % 32 == 0 && N >= kAoCols && N % kAoCols == 0 &&
           mfma_path_ok(1, N, heads * kAoHead, S, G);
}

} // namespace

// Scratch memory of sbvr_hip_linear_f16_noalloc: the split-K accumulators of the decode kernel, for callers
// that cannot bring a workspace.  One copy per GPU the library runs on, held until the process ends; zero when
// the module is loaded, and every launch leaves it zero (the adder that completes an accumulator resets it).
// In host code the array's name is only a handle: its device address is asked for once per device
// (scratch_on_current_device) and that pointer is what launches get.
constexpr size_t kScratchBytes = 4u << 20;       // 524288 accumulators: M * N of the largest decode launch it takes
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

void *g_scratch_ptr[16] = {};

// Device address of `scratch` on the current device (looked up on first use, with that device current).
int scratch_on_current_device(void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 16)
        return fail(SBVR_HIP_EUNSUPPORTED, "device %d: this library keeps scratch memory for devices 0..15", dev);
    std::lock_guard<std::mutex> guard(g_dev_lock);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(SBVR_HIP_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SBVR_HIP_OK;
}

} // namespace

// ------------------------------------------------------------------- C ABI

extern "C" {

#ifdef SBVR_TRACE
void sbvr_hip_debug_set_trace(unsigned long long *p) { g_trace = p; }
int sbvr_hip_debug_attn_o_trace(unsigned long long *out384)
{
    return hipMemcpyFromSymbol(out384, HIP_SYMBOL(g_ao_trace), sizeof(g_ao_trace)) == hipSuccess ? 0 : -3;
}
#endif

int sbvr_hip_version(void) { return 104; }      // 101: the one-row linears with a fused prologue; 102: _noalloc, _stream_floor; 103: _read_floor; 104: _dec_attention_o

const char *sbvr_hip_last_error(void) { return g_err; }

int sbvr_hip_last_kernel(void) { return g_last_kernel; }

int sbvr_hip_last_rounding(void) { return g_last_rounding; }

int sbvr_hip_init(int device)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(SBVR_HIP_ELAUNCH, "no HIP device: %s", hipGetErrorString(e));
    if (device < 0 || device >= count || device >= 16)
        return fail(SBVR_HIP_EINVAL, "device %d out of range (%d devices)", device, count);
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(SBVR_HIP_EUNSUPPORTED, "device %d is %s; this library is built for gfx950 only",
                    device, prop.gcnArchName);
    {
        std::lock_guard<std::mutex> guard(g_dev_lock);
        g_dev[device].cus = prop.multiProcessorCount;
        g_dev[device].ready = true;
    }
    // the scratch array's address on this device (each GPU holds its own copy at its own address)
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess)
        before = device;
    if (before != device && hipSetDevice(device) != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "hipSetDevice(%d) failed", device);
    void *ptr = nullptr;
    const int rc = scratch_on_current_device(&ptr);
    if (before != device)
        (void)hipSetDevice(before);
    return rc;
}

size_t sbvr_hip_linear_f16_workspace(int M, int N, int K, int S, int G)
{
    if (mfma_path_ok(M, N, K, S, G) || lut_path_ok(M, N, K, S, G))
        return static_cast<size_t>(M) * N * sizeof(unsigned long long);
    if (gemm_lut_path_ok(M, N, K, S, G)) {
        const int ks = gemm_lut_ksplit(M, N, K);
        return ks == 1 ? 0 : static_cast<size_t>(ks) * M * N * sizeof(float);
    }
    if (gemm_path_ok(M, N, K, S, G) && !rows32_path_ok(M, N, K, S, G))
        return gemm_workspace_bytes(M, N, K);
    return 0;
}

}  // extern "C"

namespace {

// What the decode kernel makes its A operands from (kXPlain: x as it is).
struct Prologue {
    int mode;
    const void *delta, *norm_weight;
    void *x_out;
    float eps;
};

int linear_core(const void *x, const uint32_t *bvr, const void *coeff_idx,
                int idx_bytes, const void *coeff_cache, const void *bias,
                void *out, int M, int N, int K, int S, int G, int L,
                void *workspace, size_t workspace_bytes, int flags,
                void *stream, const Prologue &pro)
{
    if (!x || !bvr || !coeff_idx || !coeff_cache || !out)
        return fail(SBVR_HIP_EINVAL, "null pointer argument");
    if (M <= 0 || N <= 0 || K <= 0 || S <= 0 || G <= 0 || L <= 0)
        return fail(SBVR_HIP_EINVAL, "non-positive size (M=%d N=%d K=%d S=%d G=%d L=%d)", M, N, K, S, G, L);
    if (G % 32 != 0 || K % G != 0)
        return fail(SBVR_HIP_EINVAL, "K=%d must be a multiple of G=%d, and G of 32", K, G);
    if (idx_bytes != 1 && idx_bytes != 2)
        return fail(SBVR_HIP_EINVAL, "idx_bytes must be 1 or 2, got %d", idx_bytes);
    if (idx_bytes == 1 && L > 256)
        return fail(SBVR_HIP_EINVAL, "uint8 indices cannot address L=%d lines", L);
    if (static_cast<size_t>(M) * N > 0x7fffffffu)
        return fail(SBVR_HIP_EUNSUPPORTED, "M*N too large");
    hipStream_t st = static_cast<hipStream_t>(stream);

    const bool aligned = reinterpret_cast<uintptr_t>(bvr) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(coeff_cache) % 16 == 0;
    if (pro.mode != kXPlain) {
        // the fused prologues live in the decode kernel only
        if (!aligned || !mfma_path_ok(M, N, K, S, G) || M != 1)
            return fail(SBVR_HIP_EUNSUPPORTED, "fused prologue needs M = 1 and the decode kernel's shapes (M=%d N=%d K=%d S=%d G=%d)", M, N, K, S, G);
        if (pro.mode == kXAddNorm) {
            if (!pro.delta || !pro.norm_weight || !pro.x_out)
                return fail(SBVR_HIP_EINVAL, "null pointer argument");
            if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(pro.delta) | reinterpret_cast<uintptr_t>(pro.x_out)) % 16 ||
                reinterpret_cast<uintptr_t>(pro.norm_weight) % 4)
                return fail(SBVR_HIP_EINVAL, "x, delta and x_out must be 16-byte aligned, norm_weight 4-byte");
            if (pro.x_out == x || pro.x_out == pro.delta)
                return fail(SBVR_HIP_EINVAL, "x_out must not alias x or delta (other workgroups still read them)");
        }
    }
    // from kLutMinRows batch rows on, with 2 to 4 planes: the 32-row kernel that decodes by table look-up
    // (SBVR_HIP_LUT_ROWS moves the threshold: a development switch)
    const int lut_rows = env_switches().lut_rows > 0 ? env_switches().lut_rows : kLutMinRows;
    if (pro.mode == kXPlain && !(flags & 3) && aligned && M >= lut_rows && lut_path_ok(M, N, K, S, G) &&
        reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        RowsArgs r{};
        r.x = static_cast<const uint16_t *>(x);
        r.bvr = bvr;
        r.idx = coeff_idx;
        r.cache = static_cast<const uint16_t *>(coeff_cache);
        r.bias = static_cast<const uint16_t *>(bias);
        r.out = static_cast<uint16_t *>(out);
        r.M = M; r.N = N; r.K = K; r.L = L;
        r.words_per_group = G / 32;
        r.idx16 = idx_bytes == 2;
        r.ksplit = lut_ksplit(N, K, current_cus());
        // (without the accumulators the launch is simply not split)
        if (r.ksplit > 1 && (!workspace || workspace_bytes < static_cast<size_t>(M) * N * sizeof(unsigned long long) ||
                             reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
            r.ksplit = 1;
        r.acc = static_cast<unsigned long long *>(workspace);
        if (env_switches().show_plan)
            fprintf(stderr, "sbvr_hip table look-up rows kernel M=%d N=%d K=%d S=%d: blocks=%d ksplit=%d\n", M, N, K, S, (N + 31) / 32, r.ksplit);
        const hipError_t e = launch_rows32_lut(S, r, st);
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "rows32 (table look-up) launch: %s", hipGetErrorString(e));
        g_last_kernel = SBVR_HIP_KERNEL_ROWS32;
        g_last_rounding = SBVR_HIP_ROUNDING_DECODE;
        return SBVR_HIP_OK;
    }
    if (pro.mode == kXPlain && !(flags & 3) && aligned && rows32_preferred(M, N, K, S, G, current_cus()) && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        RowsArgs r{};
        r.x = static_cast<const uint16_t *>(x);
        r.bvr = bvr;
        r.idx = coeff_idx;
        r.cache = static_cast<const uint16_t *>(coeff_cache);
        r.bias = static_cast<const uint16_t *>(bias);
        r.out = static_cast<uint16_t *>(out);
        r.M = M; r.N = N; r.K = K; r.L = L;
        r.words_per_group = G / 32;
        r.idx16 = idx_bytes == 2;
        const hipError_t e = launch_rows32(S, r, st);
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "rows32 launch: %s", hipGetErrorString(e));
        g_last_kernel = SBVR_HIP_KERNEL_ROWS32;
        g_last_rounding = SBVR_HIP_ROUNDING_PLANEWISE;
        return SBVR_HIP_OK;
    }
    if (pro.mode == kXPlain && !(flags & 1) && aligned && batch_path_ok(M, N, K, S, G)) {
        const BatchPlan p = plan_batch(M, N, K, S, current_cus());
        if (p.CTW > 0) {
            if (env_switches().show_plan)
                fprintf(stderr, "sbvr_hip batch plan M=%d N=%d K=%d S=%d: MT=%d CTW=%d SP=%d waves=%d wgs=%d ksplit=%d wstride=%d lds=%zu\n", M, N, K, S,
                        p.MT, p.CTW, p.SP, p.waves, p.n_wgs, p.ksplit, p.wstride, p.lds);
            GemvArgs a{};
            a.x = static_cast<const uint16_t *>(x);
            a.bvr = bvr;
            a.idx = coeff_idx;
            a.cache = static_cast<const uint16_t *>(coeff_cache);
            a.bias = static_cast<const uint16_t *>(bias);
            a.out = static_cast<uint16_t *>(out);
            a.M = M; a.N = N; a.K = K; a.L = L;
            a.gshift = __builtin_ctz(static_cast<unsigned>(G / kSub));
            a.idx16 = idx_bytes == 2;
            a.ksplit = p.ksplit;
            a.xstride = K;
            a.wstride = p.wstride;
#ifdef SBVR_TRACE
            a.trace = g_trace;
#endif
            if (p.ksplit > 1) {
                const size_t need = static_cast<size_t>(M) * N * sizeof(unsigned long long);
                if (!workspace || workspace_bytes < need)
                    return fail(SBVR_HIP_EWORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
                if (reinterpret_cast<uintptr_t>(workspace) % 8 != 0)
                    return fail(SBVR_HIP_EINVAL, "workspace must be 8-byte aligned");
                a.acc = static_cast<unsigned long long *>(workspace);
            }
            const hipError_t e = launch_batch(S, a, p, st);
            if (e != hipSuccess)
                return fail(SBVR_HIP_ELAUNCH, "batch launch (MT=%d CTW=%d SP=%d waves=%d ksplit=%d): %s", p.MT, p.CTW, p.SP, p.waves, p.ksplit, hipGetErrorString(e));
            g_last_kernel = SBVR_HIP_KERNEL_DECODE;
            g_last_rounding = SBVR_HIP_ROUNDING_EXACT;
            return SBVR_HIP_OK;
        }
    }
    if ((!(flags & 1) || pro.mode != kXPlain) && aligned && mfma_path_ok(M, N, K, S, G)) {
        // add + norm: the threads of a workgroup share out all of K, at most kNormChunksMax chunks of 8 each
        const int min_waves = pro.mode == kXAddNorm ? (K / 8 + 64 * kNormChunksMax - 1) / (64 * kNormChunksMax) : 1;
        GemvPlan p = plan_gemv(M, N, K, S, current_cus(), min_waves);
        if (p.CT == 0 && pro.mode != kXPlain)
            return fail(SBVR_HIP_EUNSUPPORTED, "no launch shape for the fused prologue (K=%d)", K);
        int xm = pro.mode;
        if (pro.mode == kXAddNorm) {
            p.lds += 64 + static_cast<size_t>(K) * 2;          // one partial sum of squares per wave, and fp16(x + delta)
            if (K / 8 > 64 * p.waves)
                xm = kXAddNorm2;                                 // two chunks of x per thread
        }
        if (p.CT > 0) {
        if (env_switches().show_plan)
            fprintf(stderr, "sbvr_hip plan M=%d N=%d K=%d S=%d: CT=%d SP=%d MT=%d waves=%d wgs=%d ksplit=%d wstride=%d\n", M, N, K, S, p.CT, p.SP, p.MT, p.waves, p.n_wgs, p.ksplit, p.wstride);
        GemvArgs a{};
        a.x = static_cast<const uint16_t *>(x);
        a.bvr = bvr;
        a.idx = coeff_idx;
        a.cache = static_cast<const uint16_t *>(coeff_cache);
        a.bias = static_cast<const uint16_t *>(bias);
        a.out = static_cast<uint16_t *>(out);
        a.M = M; a.N = N; a.K = K; a.L = L;
        a.gshift = __builtin_ctz(static_cast<unsigned>(G / kSub));
        a.idx16 = idx_bytes == 2;
        a.ksplit = p.ksplit;
        a.xstride = pro.mode == kXSwiGLU ? 2 * K : K;
        a.wstride = p.wstride;
        a.delta = static_cast<const uint16_t *>(pro.delta);
        a.norm_w = static_cast<const uint16_t *>(pro.norm_weight);
        a.x_out = static_cast<uint16_t *>(pro.x_out);
        a.eps = pro.eps;
#ifdef SBVR_TRACE
        a.trace = g_trace;
#endif
        if (p.ksplit > 1) {
            const size_t need = static_cast<size_t>(M) * N * sizeof(unsigned long long);
            if (!workspace || workspace_bytes < need)
                return fail(SBVR_HIP_EWORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
            if (reinterpret_cast<uintptr_t>(workspace) % 8 != 0)
                return fail(SBVR_HIP_EINVAL, "workspace must be 8-byte aligned");
            a.acc = static_cast<unsigned long long *>(workspace);
        }
        const hipError_t e = launch_gemv(S, a, p, xm, st);
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "gemv launch (CT=%d SP=%d MT=%d waves=%d ksplit=%d): %s", p.CT, p.SP, p.MT, p.waves, p.ksplit, hipGetErrorString(e));
        g_last_kernel = SBVR_HIP_KERNEL_DECODE;
        g_last_rounding = SBVR_HIP_ROUNDING_EXACT;
        return SBVR_HIP_OK;
        }
    }

    // More than 32 rows, 2 to 4 planes, K and G multiples of 128: the prefill kernel that decodes by table look-up
    // (SBVR_HIP_PF_LUT=2 keeps the tile kernel: a development switch)
    if (!(flags & 1) && aligned && env_switches().pf_lut != 2 && gemm_lut_path_ok(M, N, K, S, G) && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        GemmArgs g{};
        g.x = static_cast<const uint16_t *>(x);
        g.bvr = bvr;
        g.idx = coeff_idx;
        g.cache = static_cast<const uint16_t *>(coeff_cache);
        g.bias = static_cast<const uint16_t *>(bias);
        g.out = static_cast<uint16_t *>(out);
        g.M = M; g.N = N; g.K = K; g.L = L;
        g.steps_per_group = G / kGemmBK;
        g.idx16 = idx_bytes == 2;
        g.ksplit = 1;
        const int ks = gemm_lut_ksplit(M, N, K);
        const size_t need = ks > 1 ? static_cast<size_t>(ks) * M * N * sizeof(float) : 0;
        if (need && workspace && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
            g.ksplit = ks;
            g.part = static_cast<float *>(workspace);
        }
        if (env_switches().show_plan)
            fprintf(stderr, "sbvr_hip table look-up prefill M=%d N=%d K=%d S=%d: ksplit=%d\n", M, N, K, S, g.ksplit);
        hipError_t e = launch_gemm_lut(S, g, st);
        if (e == hipSuccess && g.ksplit > 1) {
            const size_t quads = (static_cast<size_t>(M) * N + 3) / 4;
            hipLaunchKernelGGL(sbvr_gemm_reduce_kernel, dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256), 0, st,
                               g.part, g.bias, g.out, M, N, g.ksplit);
            e = hipGetLastError();
        }
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "prefill (table look-up) launch: %s", hipGetErrorString(e));
        g_last_kernel = g.ksplit > 1 ? SBVR_HIP_KERNEL_PREFILL_SPLIT : SBVR_HIP_KERNEL_PREFILL;
        g_last_rounding = SBVR_HIP_ROUNDING_DECODE;
        return SBVR_HIP_OK;
    }
    if (!(flags & 1) && aligned && gemm_path_ok(M, N, K, S, G) && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        GemmArgs g{};
        g.x = static_cast<const uint16_t *>(x);
        g.bvr = bvr;
        g.idx = coeff_idx;
        g.cache = static_cast<const uint16_t *>(coeff_cache);
        g.bias = static_cast<const uint16_t *>(bias);
        g.out = static_cast<uint16_t *>(out);
        g.M = M; g.N = N; g.K = K; g.L = L;
        g.steps_per_group = G / kGemmBK;
        g.idx16 = idx_bytes == 2;
        g.ksplit = 1;
        // K split across workgroups where the output tiles alone would leave CUs idle, if the caller brought the
        // workspace for it (without one the launch is simply not split)
        const size_t need = gemm_workspace_bytes(M, N, K);
        if (need && workspace && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
            g.ksplit = gemm_ksplit(M, N, K);
            g.part = static_cast<float *>(workspace);
        }
#ifdef SBVR_TRACE
        g.trace = g_trace;
#endif
        hipError_t e = launch_gemm(S, g, st);
        if (e == hipSuccess && g.ksplit > 1) {
            const size_t quads = (static_cast<size_t>(M) * N + 3) / 4;
            hipLaunchKernelGGL(sbvr_gemm_reduce_kernel, dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256), 0, st,
                               g.part, g.bias, g.out, M, N, g.ksplit);
            e = hipGetLastError();
        }
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "gemm launch: %s", hipGetErrorString(e));
        g_last_kernel = g.ksplit > 1 ? SBVR_HIP_KERNEL_PREFILL_SPLIT : SBVR_HIP_KERNEL_PREFILL;
        g_last_rounding = SBVR_HIP_ROUNDING_PLANEWISE;
        return SBVR_HIP_OK;
    }

    const size_t total = static_cast<size_t>(M) * N;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
    if (idx_bytes == 1)
        hipLaunchKernelGGL(sbvr_linear_portable_kernel<uint8_t>, grid, block, 0, st,
                           static_cast<const uint16_t *>(x), bvr, coeff_idx, static_cast<const uint16_t *>(coeff_cache),
                           static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), M, N, K, S, G);
    else
        hipLaunchKernelGGL(sbvr_linear_portable_kernel<uint16_t>, grid, block, 0, st,
                           static_cast<const uint16_t *>(x), bvr, coeff_idx, static_cast<const uint16_t *>(coeff_cache),
                           static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), M, N, K, S, G);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "portable launch: %s", hipGetErrorString(e));
    g_last_kernel = SBVR_HIP_KERNEL_PORTABLE;
    g_last_rounding = SBVR_HIP_ROUNDING_EXACT;
    return SBVR_HIP_OK;
}

}  // namespace

extern "C" {

int sbvr_hip_linear_f16(const void *x, const uint32_t *bvr, const void *coeff_idx,
                        int idx_bytes, const void *coeff_cache, const void *bias,
                        void *out, int M, int N, int K, int S, int G, int L,
                        void *workspace, size_t workspace_bytes, int flags,
                        void *stream)
{
    return linear_core(x, bvr, coeff_idx, idx_bytes, coeff_cache, bias, out, M, N, K, S, G, L, workspace,
                       workspace_bytes, flags, stream, Prologue{kXPlain, nullptr, nullptr, nullptr, 0.f});
}

int sbvr_hip_linear_f16_noalloc(const void *x, const uint32_t *bvr, const void *coeff_idx,
                                int idx_bytes, const void *coeff_cache, const void *bias,
                                void *out, int M, int N, int K, int S, int G, int L,
                                int flags, void *stream)
{
    // The accumulators of the decode and 32-row kernels come from the library's own scratch array; the prefill
    // kernel runs without its optional workspace (not split along K).  Nothing is allocated or freed on the way.
    // A launch of up to 32 rows that splits K across workgroups takes its M * N accumulators from the scratch
    // array; one whose accumulators would not fit gets no workspace at all: the table look-up kernel (9 to 32
    // rows) then runs unsplit, and only a decode launch (up to 8 rows) whose shape cannot do without the split
    // is refused.
    void *ws = nullptr;
    size_t ws_bytes = 0;
    if (M >= 1 && N >= 1 && (mfma_path_ok(M, N, K, S, G) || lut_path_ok(M, N, K, S, G)) && !(flags & 1) &&
        static_cast<size_t>(M) * N * sizeof(unsigned long long) <= kScratchBytes) {
        const int rc = scratch_on_current_device(&ws);
        if (rc != SBVR_HIP_OK)
            return rc;
        ws_bytes = kScratchBytes;
    }
    const int rc = linear_core(x, bvr, coeff_idx, idx_bytes, coeff_cache, bias, out, M, N, K, S, G, L, ws, ws_bytes, flags,
                               stream, Prologue{kXPlain, nullptr, nullptr, nullptr, 0.f});
    if (rc == SBVR_HIP_EWORKSPACE)
        return fail(SBVR_HIP_EWORKSPACE, "sbvr_hip_linear_f16_noalloc: this launch splits K across workgroups and its M * N = %zu "
                    "accumulators exceed the %zu of the library's scratch array; use sbvr_hip_linear_f16 with a workspace",
                    static_cast<size_t>(M) * N, kScratchBytes / sizeof(unsigned long long));
    return rc;
}

int sbvr_hip_linear_f16_swiglu(const void *gate_up, const uint32_t *bvr, const void *coeff_idx,
                               int idx_bytes, const void *coeff_cache, const void *bias,
                               void *out, int M, int N, int K, int S, int G, int L,
                               void *workspace, size_t workspace_bytes, void *stream)
{
    return linear_core(gate_up, bvr, coeff_idx, idx_bytes, coeff_cache, bias, out, M, N, K, S, G, L, workspace,
                       workspace_bytes, 0, stream, Prologue{kXSwiGLU, nullptr, nullptr, nullptr, 0.f});
}

int sbvr_hip_linear_f16_add_rmsnorm(const void *x, const void *delta, const void *norm_weight, float eps,
                                    void *x_out, const uint32_t *bvr, const void *coeff_idx,
                                    int idx_bytes, const void *coeff_cache, const void *bias,
                                    void *out, int N, int K, int S, int G, int L,
                                    void *workspace, size_t workspace_bytes, void *stream)
{
    return linear_core(x, bvr, coeff_idx, idx_bytes, coeff_cache, bias, out, 1, N, K, S, G, L, workspace,
                       workspace_bytes, 0, stream, Prologue{kXAddNorm, delta, norm_weight, x_out, eps});
}

int sbvr_hip_linear_f16_stream_floor(const uint32_t *bvr, const void *coeff_idx, int idx_bytes,
                                     const void *coeff_cache, void *out, int N, int K, int S, int G, int L,
                                     void *workspace, size_t workspace_bytes, void *stream)
{
    // (out stands in for the activations, which this launch never reads)
    return linear_core(out, bvr, coeff_idx, idx_bytes, coeff_cache, nullptr, out, 1, N, K, S, G, L, workspace,
                       workspace_bytes, 0, stream, Prologue{kXFloor, nullptr, nullptr, nullptr, 0.f});
}

int sbvr_hip_row_deq_mm_T_ws(const void *x, const uint32_t *r_bvr, const void *r_coeff_idx,
                             int idx_bytes, const void *r_coeff_cache, const void *bias,
                             void *out, int M, int N, int K, int S, int G, int L,
                             void *workspace, size_t workspace_bytes, void *stream)
{
    if (!x || !r_bvr || !r_coeff_idx || !r_coeff_cache || !out)
        return fail(SBVR_HIP_EINVAL, "null pointer argument");
    if (M <= 0 || N <= 0 || K <= 0 || S <= 0 || G <= 0 || L <= 0)
        return fail(SBVR_HIP_EINVAL, "non-positive size");
    if (N % 32 != 0 || G % 32 != 0 || N % G != 0)
        return fail(SBVR_HIP_EINVAL, "N=%d must be a multiple of G=%d, and G of 32", N, G);
    if (idx_bytes != 1 && idx_bytes != 2)
        return fail(SBVR_HIP_EINVAL, "idx_bytes must be 1 or 2, got %d", idx_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (idx_bytes == 1 && L > 256)
        return fail(SBVR_HIP_EINVAL, "uint8 indices cannot address L=%d lines", L);
    const bool tables_aligned = reinterpret_cast<uintptr_t>(r_bvr) % 16 == 0 && reinterpret_cast<uintptr_t>(r_coeff_cache) % 16 == 0;
    if (M <= 65535 && S == 4 && K % kSub == 0 && G % 64 == 0 && tables_aligned && reinterpret_cast<uintptr_t>(x) % 4 == 0 &&
        reinterpret_cast<uintptr_t>(r_coeff_idx) % 4 == 0 && !env_switches().rowdeq_lanes) {
        // plane sums on the matrix cores over bits transposed across lanes
        const int nsub = K / kSub;
        // (128 columns per workgroup, one A image for twice the columns, measured slower: 17.3 against 15.6 us at
        // 4096 -> 14336: it wants more than 128 registers)
        const int nww = 2;
        const long col_wgs = static_cast<long>((N / 32 + nww - 1) / nww) * M;
        // K in as many parts as give the CUs a workgroup each, if the caller brought the accumulators
        int ksplit = 1;
        if (workspace && reinterpret_cast<uintptr_t>(workspace) % 8 == 0 &&
            workspace_bytes >= static_cast<size_t>(M) * N * sizeof(unsigned long long)) {
            // (measured at 4096 -> 4096 / 14336 -> 4096, 64 column workgroups: 13.2 / 39.0 us unsplit, 7.1 / 14.1 in 4
            // parts, 7.2 / 18.5 in 8; at 4096 -> 14336, 224 of them: 15.3 unsplit, 18.4 in 2)
            while (ksplit < 32 && col_wgs * ksplit < 3L * current_cus() / 4 && nsub / (ksplit * 2) >= 4)
                ksplit *= 2;
        }
        const int per_part = (nsub + ksplit - 1) / ksplit;
        ksplit = (nsub + per_part - 1) / per_part;              // (no empty parts)
        const int waves = per_part < kRowDeqWaves ? per_part : kRowDeqWaves;
        const dim3 grid(static_cast<unsigned>((N / 32 + nww - 1) / nww), static_cast<unsigned>(M), static_cast<unsigned>(ksplit)), block(64 * waves);
        if (nww == 4)
            hipLaunchKernelGGL(sbvr_row_deq_mfma_kernel<4>, grid, block, 0, st, static_cast<const uint16_t *>(x), r_bvr, r_coeff_idx,
                               static_cast<const uint16_t *>(r_coeff_cache), static_cast<const uint16_t *>(bias),
                               static_cast<uint16_t *>(out), static_cast<unsigned long long *>(workspace), M, N, K, L, G,
                               idx_bytes == 2 ? 1 : 0, ksplit);
        else
            hipLaunchKernelGGL(sbvr_row_deq_mfma_kernel<2>, grid, block, 0, st, static_cast<const uint16_t *>(x), r_bvr, r_coeff_idx,
                               static_cast<const uint16_t *>(r_coeff_cache), static_cast<const uint16_t *>(bias),
                               static_cast<uint16_t *>(out), static_cast<unsigned long long *>(workspace), M, N, K, L, G,
                               idx_bytes == 2 ? 1 : 0, ksplit);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "row_deq launch: %s", hipGetErrorString(e));
        return SBVR_HIP_OK;
    }
    if (M <= 65535 && (S == 2 || S == 3 || S == 4 || S == 6 || S == 8) && tables_aligned) {
        // lanes along K; as many waves as there are steps of 64 rows, up to kRowDeqWaves
        const int steps = (K + 63) / 64;
        const int waves = steps < kRowDeqWaves ? steps : kRowDeqWaves;
        const dim3 grid(static_cast<unsigned>(N / 32), static_cast<unsigned>(M)), block(64 * waves);
#define SBVR_ROWDEQ(s)                                                                                            \
    case s:                                                                                                       \
        hipLaunchKernelGGL(sbvr_row_deq_lanes_kernel<s>, grid, block, 0, st, static_cast<const uint16_t *>(x), r_bvr, \
                           r_coeff_idx, static_cast<const uint16_t *>(r_coeff_cache),                            \
                           static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), M, N, K, L, G,     \
                           idx_bytes == 2 ? 1 : 0);                                                               \
        break
        switch (S) {
            SBVR_ROWDEQ(2); SBVR_ROWDEQ(3); SBVR_ROWDEQ(4); SBVR_ROWDEQ(6); SBVR_ROWDEQ(8);
        }
#undef SBVR_ROWDEQ
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return fail(SBVR_HIP_ELAUNCH, "row_deq launch: %s", hipGetErrorString(e));
        return SBVR_HIP_OK;
    }
    const size_t total = static_cast<size_t>(M) * N;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
    if (idx_bytes == 1)
        hipLaunchKernelGGL(sbvr_row_deq_kernel<uint8_t>, grid, block, 0, st,
                           static_cast<const uint16_t *>(x), r_bvr, r_coeff_idx, static_cast<const uint16_t *>(r_coeff_cache),
                           static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), M, N, K, S, G);
    else
        hipLaunchKernelGGL(sbvr_row_deq_kernel<uint16_t>, grid, block, 0, st,
                           static_cast<const uint16_t *>(x), r_bvr, r_coeff_idx, static_cast<const uint16_t *>(r_coeff_cache),
                           static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), M, N, K, S, G);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "row_deq launch: %s", hipGetErrorString(e));
    return SBVR_HIP_OK;
}

int sbvr_hip_row_deq_mm_T(const void *x, const uint32_t *r_bvr, const void *r_coeff_idx,
                          int idx_bytes, const void *r_coeff_cache, const void *bias,
                          void *out, int M, int N, int K, int S, int G, int L,
                          void *stream)
{
    return sbvr_hip_row_deq_mm_T_ws(x, r_bvr, r_coeff_idx, idx_bytes, r_coeff_cache, bias, out, M, N, K, S, G, L, nullptr, 0, stream);
}

// (the launch splits K only while its column workgroups cover less than three quarters of the CUs: the predicate
// of sbvr_hip_row_deq_mm_T_ws; a prefill-sized call needs nothing)
size_t sbvr_hip_row_deq_mm_T_workspace(int M, int N)
{
    if (M <= 0 || N <= 0)
        return 0;
    const long col_wgs = static_cast<long>((N / 32 + 1) / 2) * M;
    return col_wgs * 2 < 3L * current_cus() / 4 ? static_cast<size_t>(M) * N * sizeof(unsigned long long) : 0;
}

// (only one left row runs on the decode kernel, the one form that may split K across workgroups)
size_t sbvr_hip_mm_T_workspace(int M, int N)
{
    return M == 1 && N > 0 ? static_cast<size_t>(N) * sizeof(unsigned long long) : 0;
}

int sbvr_hip_mm_T(const uint32_t *l_bvr, const void *l_coeff_idx, int l_idx_bytes,
                  const void *l_coeff_cache, const uint32_t *r_bvr,
                  const void *r_coeff_idx, int r_idx_bytes, const void *r_coeff_cache,
                  const void *bias, void *out, int M, int N, int K, int Sl, int Sr,
                  int G, int Ll, int Lr, void *stream)
{
    return sbvr_hip_mm_T_ws(l_bvr, l_coeff_idx, l_idx_bytes, l_coeff_cache, r_bvr, r_coeff_idx, r_idx_bytes, r_coeff_cache,
                            bias, out, M, N, K, Sl, Sr, G, Ll, Lr, nullptr, 0, stream);
}

int sbvr_hip_mm_T_ws(const uint32_t *l_bvr, const void *l_coeff_idx, int l_idx_bytes,
                     const void *l_coeff_cache, const uint32_t *r_bvr,
                     const void *r_coeff_idx, int r_idx_bytes, const void *r_coeff_cache,
                     const void *bias, void *out, int M, int N, int K, int Sl, int Sr,
                     int G, int Ll, int Lr, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!l_bvr || !l_coeff_idx || !l_coeff_cache || !r_bvr || !r_coeff_idx || !r_coeff_cache || !out)
        return fail(SBVR_HIP_EINVAL, "null pointer argument");
    if (M <= 0 || N <= 0 || K <= 0 || Sl <= 0 || Sr <= 0 || G <= 0 || Ll <= 0 || Lr <= 0)
        return fail(SBVR_HIP_EINVAL, "non-positive size");
    if (G % 32 != 0 || K % G != 0)
        return fail(SBVR_HIP_EINVAL, "K=%d must be a multiple of G=%d, and G of 32", K, G);
    if ((l_idx_bytes != 1 && l_idx_bytes != 2) || (r_idx_bytes != 1 && r_idx_bytes != 2))
        return fail(SBVR_HIP_EINVAL, "idx_bytes must be 1 or 2");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t total = static_cast<size_t>(M) * N;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
    const uint16_t *lc = static_cast<const uint16_t *>(l_coeff_cache), *rc = static_cast<const uint16_t *>(r_coeff_cache);
    const uint16_t *b = static_cast<const uint16_t *>(bias);
    uint16_t *o = static_cast<uint16_t *>(out);
    // One left row of up to four planes (what the reference's kernels are written for), at the decode kernel's
    // shapes: the decode kernel with the left operand's planes as its batch rows; the popcounts come out of the
    // matrix cores.  4096 -> 14336, 4 x 4 planes: about 9 us against 11.5 us for the popcount kernel below.
    if (M == 1 && Sl <= 4 && !env_switches().popc_q && mfma_path_ok(Sl, N, K, Sr, G) &&
        (l_idx_bytes == 2 || Ll <= 256) && (r_idx_bytes == 2 || Lr <= 256) &&
        reinterpret_cast<uintptr_t>(r_bvr) % 16 == 0 && reinterpret_cast<uintptr_t>(r_coeff_cache) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(l_bvr) % 4 == 0 && reinterpret_cast<uintptr_t>(l_coeff_cache) % 2 == 0) {
        const GemvPlan p = plan_gemv(Sl, N, K, Sr, current_cus());
        const size_t need = static_cast<size_t>(N) * sizeof(unsigned long long);
        const bool room = p.ksplit <= 1 || (workspace && workspace_bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 8 == 0);
        if (p.CT > 0 && p.MT == 1 && room) {
            GemvArgs a{};
            a.bvr = r_bvr;
            a.idx = r_coeff_idx;
            a.cache = rc;
            a.bias = b;
            a.out = o;
            a.M = Sl; a.N = N; a.K = K; a.L = Lr;
            a.gshift = __builtin_ctz(static_cast<unsigned>(G / kSub));
            a.idx16 = r_idx_bytes == 2;
            a.ksplit = p.ksplit;
            a.xstride = K;
            a.wstride = p.wstride;
            a.xbvr = l_bvr;
            a.xidx = l_coeff_idx;
            a.xcache = lc;
            a.x_idx16 = l_idx_bytes == 2;
            a.xL = Ll;
            a.acc = p.ksplit > 1 ? static_cast<unsigned long long *>(workspace) : nullptr;
#ifdef SBVR_TRACE
            a.trace = g_trace;
#endif
            const hipError_t e = launch_gemv(Sr, a, p, kXPlanes, st);
            if (e != hipSuccess)
                return fail(SBVR_HIP_ELAUNCH, "mm_T launch through the decode kernel (CT=%d SP=%d waves=%d ksplit=%d): %s", p.CT, p.SP, p.waves,
                            p.ksplit, hipGetErrorString(e));
            g_last_kernel = SBVR_HIP_KERNEL_DECODE;
            return SBVR_HIP_OK;
        }
    }
    // few left rows: lane-per-column popcount kernel
    const int wpg = G / 32;
    if (M <= 64 && (wpg == 1 || wpg == 2 || wpg == 4 || wpg == 8) && Sl >= 2 && Sl <= 4 &&
        reinterpret_cast<uintptr_t>(r_bvr) % 16 == 0 && static_cast<double>(K / 32) * N * Sr < 2147483648.0) {
        // 16-column windows (four parts of K inside a wave) when 64-column ones would leave half the CUs without a
        // workgroup: measured 13 us against 27 us at N=4096, K=14336, but 26 us against 11.5 us at N=14336, K=4096
        const int eq = env_switches().popc_q;
        const int pgrid = eq ? eq : (static_cast<long>((N + 63) / 64) * M * 2 <= current_cus() ? 4 : 1);
        const uint8_t *li = static_cast<const uint8_t *>(l_coeff_idx), *ri = static_cast<const uint8_t *>(r_coeff_idx);
        const int l16 = l_idx_bytes == 2, r16 = r_idx_bytes == 2;
        bool done = false;
        if (Sl == 2)
            done = launch_mm_T_popc_sr<2>(Sr, pgrid, st, l_bvr, li, l16, lc, r_bvr, ri, r16, rc, b, o, M, N, K, wpg, Ll, Lr);
        else if (Sl == 3)
            done = launch_mm_T_popc_sr<3>(Sr, pgrid, st, l_bvr, li, l16, lc, r_bvr, ri, r16, rc, b, o, M, N, K, wpg, Ll, Lr);
        else
            done = launch_mm_T_popc_sr<4>(Sr, pgrid, st, l_bvr, li, l16, lc, r_bvr, ri, r16, rc, b, o, M, N, K, wpg, Ll, Lr);
        if (done) {
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess)
                return fail(SBVR_HIP_ELAUNCH, "mm_T launch: %s", hipGetErrorString(e));
            return SBVR_HIP_OK;
        }
    }
#define SBVR_MM_LAUNCH(LT, RT)                                                                   \
    hipLaunchKernelGGL((sbvr_mm_T_kernel<LT, RT>), grid, block, 0, st, l_bvr, l_coeff_idx, lc,   \
                       r_bvr, r_coeff_idx, rc, b, o, M, N, K, Sl, Sr, G)
    if (l_idx_bytes == 1 && r_idx_bytes == 1)
        SBVR_MM_LAUNCH(uint8_t, uint8_t);
    else if (l_idx_bytes == 1)
        SBVR_MM_LAUNCH(uint8_t, uint16_t);
    else if (r_idx_bytes == 1)
        SBVR_MM_LAUNCH(uint16_t, uint8_t);
    else
        SBVR_MM_LAUNCH(uint16_t, uint16_t);
#undef SBVR_MM_LAUNCH
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "mm_T launch: %s", hipGetErrorString(e));
    return SBVR_HIP_OK;
}


int sbvr_hip_dec_attention_o_supported(int heads, int kv_heads, int head_dim, int max_seq, int N, int S, int G)
{
    if (S != 2 && S != 3 && S != 4 && S != 6 && S != 8)
        return 0;
#ifdef SBVR_FAST_BUILD
    if (S != 4)
        return 0;
#endif
    return attn_o_shape_ok(heads, kv_heads, head_dim, max_seq, N, S, G) ? 1 : 0;
}

size_t sbvr_hip_dec_attention_o_workspace(int kv_heads, int N)
{
    return kv_heads > 1 && N > 0 ? static_cast<size_t>(N) * sizeof(unsigned long long) : 0;
}

int sbvr_hip_dec_attention_o_f16(const void *qkv, const float *cos_table, const float *sin_table, const float *rot_now,
                                 const long long *pos, void *kcache, void *vcache, void *ctx, int heads, int kv_heads,
                                 int head_dim, int max_seq, const uint32_t *o_bvr, const void *o_coeff_idx, int idx_bytes,
                                 const void *o_coeff_cache, const void *o_bias, void *out, int N, int S, int G, int L,
                                 void *workspace, size_t workspace_bytes, void *stream)
{
    if (!qkv || !cos_table || !sin_table || !pos || !kcache || !vcache || !o_bvr || !o_coeff_idx || !o_coeff_cache || !out)
        return fail(SBVR_HIP_EINVAL, "null pointer argument");
    if (heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || N <= 0 || S <= 0 || G <= 0 || L <= 0)
        return fail(SBVR_HIP_EINVAL, "non-positive size");
    if (idx_bytes != 1 && idx_bytes != 2)
        return fail(SBVR_HIP_EINVAL, "idx_bytes must be 1 or 2, got %d", idx_bytes);
    if (idx_bytes == 1 && L > 256)
        return fail(SBVR_HIP_EINVAL, "uint8 indices cannot address L=%d lines", L);
    if (!sbvr_hip_dec_attention_o_supported(heads, kv_heads, head_dim, max_seq, N, S, G))
        return fail(SBVR_HIP_EUNSUPPORTED, "attention + projection in one launch: heads=%d kv_heads=%d head_dim=%d max_seq=%d N=%d S=%d G=%d",
                    heads, kv_heads, head_dim, max_seq, N, S, G);
    if ((reinterpret_cast<uintptr_t>(kcache) | reinterpret_cast<uintptr_t>(vcache) | reinterpret_cast<uintptr_t>(o_bvr) |
         reinterpret_cast<uintptr_t>(o_coeff_cache)) % 16 ||
        (reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(o_coeff_idx)) % 2 ||
        (ctx && reinterpret_cast<uintptr_t>(ctx) % 4))
        return fail(SBVR_HIP_EINVAL, "caches, bvr and coeff_cache must be 16-byte aligned, ctx 4-byte, qkv, out and uint16 indices 2-byte");
    if (kv_heads > 1 && (!workspace || workspace_bytes < sbvr_hip_dec_attention_o_workspace(kv_heads, N) ||
                         reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
        return fail(SBVR_HIP_EWORKSPACE, "attention + projection needs %zu bytes of zeroed workspace (8-byte aligned), got %zu",
                    sbvr_hip_dec_attention_o_workspace(kv_heads, N), workspace_bytes);
    AttnOArgs a{};
    a.qkv = static_cast<const uint16_t *>(qkv);
    a.cos_t = cos_table;
    a.sin_t = sin_table;
    a.rot_now = rot_now;
    a.pos_p = pos;
    a.kcache = static_cast<uint16_t *>(kcache);
    a.vcache = static_cast<uint16_t *>(vcache);
    a.ctx = static_cast<uint16_t *>(ctx);
    a.heads = heads; a.kv_heads = kv_heads; a.max_seq = max_seq;
    a.bvr = o_bvr;
    a.idx = o_coeff_idx;
    a.cache = static_cast<const uint16_t *>(o_coeff_cache);
    a.bias = static_cast<const uint16_t *>(o_bias);
    a.out = static_cast<uint16_t *>(out);
    a.acc = static_cast<unsigned long long *>(workspace);
    a.N = N; a.L = L;
    a.gshift = __builtin_ctz(static_cast<unsigned>(G / kSub));
    a.idx16 = idx_bytes == 2;
    const hipError_t e = launch_attn_o(S, a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "attention + projection launch: %s", hipGetErrorString(e));
    g_last_kernel = SBVR_HIP_KERNEL_DECODE;
    g_last_rounding = SBVR_HIP_ROUNDING_EXACT;
    return SBVR_HIP_OK;
}

int sbvr_hip_read_floor(const void *buf, size_t buf_bytes, size_t bytes, int workgroups, int waves, int ahead, int pattern,
                        int row_bytes, int win_bytes, void *sink, void *stream)
{
    if (!buf || !sink || reinterpret_cast<uintptr_t>(buf) % 16 != 0)
        return fail(SBVR_HIP_EINVAL, "read floor: buffer and sink must be given, the buffer 16-byte aligned");
    if (workgroups <= 0 || waves <= 0 || waves > 16 || ahead <= 0 || pattern < 0 || pattern > 2)
        return fail(SBVR_HIP_EINVAL, "read floor: workgroups=%d waves=%d ahead=%d pattern=%d", workgroups, waves, ahead, pattern);
    const size_t per_wave = bytes / 1024 / (static_cast<size_t>(workgroups) * waves);
    if (per_wave == 0 || per_wave > 0x7ffffffeu || per_wave * workgroups * waves * 1024 != bytes || per_wave % ahead != 0)
        return fail(SBVR_HIP_EINVAL, "read floor: %zu bytes are not a whole number of %d-KiB rounds for %d x %d waves",
                    bytes, ahead, workgroups, waves);
    if (pattern != 2) {
        if (bytes > buf_bytes)
            return fail(SBVR_HIP_EINVAL, "read floor: %zu bytes asked of a buffer of %zu", bytes, buf_bytes);
    } else {
        // rows of row_bytes, windows of win_bytes (whole 16 bytes), four rows per unit, the rows split over the waves
        if (row_bytes <= 0 || row_bytes % 16 || win_bytes < 16 || win_bytes % 16 || static_cast<size_t>(workgroups) * win_bytes > static_cast<size_t>(row_bytes))
            return fail(SBVR_HIP_EINVAL, "read floor: windows of %d bytes x %d workgroups do not fit rows of %d", win_bytes, workgroups, row_bytes);
        const size_t tiles = (static_cast<size_t>(win_bytes) + 255) / 256;
        if (per_wave % tiles)
            return fail(SBVR_HIP_EINVAL, "read floor: %zu units per wave are not whole windows of %zu tiles", per_wave, tiles);
        const size_t rows = per_wave / tiles * 4 * waves;
        if (rows * static_cast<size_t>(row_bytes) > buf_bytes)
            return fail(SBVR_HIP_EINVAL, "read floor: %zu rows of %d bytes reach beyond the buffer of %zu", rows, row_bytes, buf_bytes);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(workgroups)), block(static_cast<unsigned>(64 * waves));
    const v4u *b = static_cast<const v4u *>(buf);
    uint32_t *sk = static_cast<uint32_t *>(sink);
    const uint32_t u = static_cast<uint32_t>(per_wave);
#define SBVR_RF(A) case A: hipLaunchKernelGGL(sbvr_read_floor_kernel<A>, grid, block, 0, st, b, u, pattern, \
                                              static_cast<uint32_t>(row_bytes), static_cast<uint32_t>(win_bytes), sk); break
    switch (ahead) {
        SBVR_RF(1); SBVR_RF(2); SBVR_RF(3); SBVR_RF(4); SBVR_RF(7); SBVR_RF(8); SBVR_RF(14); SBVR_RF(16);
    default: return fail(SBVR_HIP_EINVAL, "read floor: ahead must be one of 1, 2, 3, 4, 7, 8, 14, 16");
    }
#undef SBVR_RF
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(SBVR_HIP_ELAUNCH, "read floor launch: %s", hipGetErrorString(e));
    return SBVR_HIP_OK;
}


int sbvr_hip_decode_plan(int M, int N, int K, int S, int G, int cus, int *plan)
{
    if (!plan || cus <= 0)
        return fail(SBVR_HIP_EINVAL, "decode plan: plan must be given and cus positive");
    for (int i = 0; i < 8; ++i)
        plan[i] = 0;
    if (!mfma_path_ok(M, N, K, S, G))
        return SBVR_HIP_OK;
    if (batch_path_ok(M, N, K, S, G)) {
        const BatchPlan p = plan_batch_uncached(M, N, K, S, cus);
        if (p.CTW > 0) {
            const int v[8] = {2, p.CTW, p.SP, p.MT, p.waves, p.n_wgs, p.ksplit, kMaxWaves};
            for (int i = 0; i < 8; ++i)
                plan[i] = v[i];
            return SBVR_HIP_OK;
        }
    }
    const GemvPlan p = plan_gemv_uncached(M, N, K, S, cus, 1);
    if (p.CT > 0) {
        const int v[8] = {1, p.CT, p.SP, p.MT, p.waves, p.n_wgs, p.ksplit, gemv_max_waves(p.MT, p.CT)};
        for (int i = 0; i < 8; ++i)
            plan[i] = v[i];
    }
    return SBVR_HIP_OK;
}

} // extern "C"
