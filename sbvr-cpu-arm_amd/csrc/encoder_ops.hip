// Encoder search on the GPU (libsbvr_hip.so, gfx950): the error of every (group, candidate line) pair of
// the SBVR encoder's search, for many groups at once.
//
// The search (reference sbvr/core.py:485-501, _data_diff_min_mse) takes a group of G values and n candidate
// lines, each line given by its 2^S subset sums ("points"), and wants, per line, the mean over the group of
// the squared distance from each value to its nearest point.  The reference forms the (n, G, 2^S) tensor of
// squared differences in the compute type and reduces it; at 4096 x 4096 that tensor is written and read
// 131072 times.  Here a thread owns one (group, line) pair, keeps the line's points in registers and walks
// the group's values (in LDS, read as broadcasts): nothing but the (groups, lines) matrix of errors goes to
// memory.  The arithmetic per element is the reference's: fp16 subtraction, fp16 square, minimum (packed,
// two points per instruction), then an fp32 sum over the group in element order and one division.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sbvr_hip_encoder.h"

namespace {

typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr int kEncThreads = 256;
constexpr int kEncMaxG = 4096;        // values of a group the LDS copy holds at a time (8 KiB)

// P points per line (a power of two, 2 <= P <= 256).  Grid: (ceil(n / 256), groups).  Groups longer than the
// LDS copy go through it in pieces.
template <int P>
__global__ void __launch_bounds__(kEncThreads)
sbvr_encoder_group_mse_kernel(const uint16_t *__restrict__ data, const uint16_t *__restrict__ points,
                              float *__restrict__ mse, int G, int n)
{
    __shared__ __align__(16) uint16_t group[kEncMaxG];
    const int b = blockIdx.y;
    const uint16_t *mine = data + static_cast<size_t>(b) * G;
    const int line = blockIdx.x * kEncThreads + threadIdx.x;
    const int line_c = min(line, n - 1);          // (threads past the end repeat the last line and store nothing)
    v2h p[P / 2];
    const uint32_t *src = reinterpret_cast<const uint32_t *>(points + static_cast<size_t>(line_c) * P);
#pragma unroll
    for (int j = 0; j < P / 2; ++j)
        p[j] = __builtin_bit_cast(v2h, src[j]);

    float sum = 0.f;
    for (int g0 = 0; g0 < G; g0 += kEncMaxG) {
        const int len = min(G - g0, kEncMaxG);
        __syncthreads();
        for (int i = threadIdx.x; i < len; i += kEncThreads)
            group[i] = mine[g0 + i];
        __syncthreads();
        for (int g = 0; g < len; ++g) {
            const uint16_t raw = group[g];
            const _Float16 d = __builtin_bit_cast(_Float16, raw);
            const v2h dd = {d, d};
            v2h best;
#pragma unroll
            for (int j = 0; j < P / 2; ++j) {
                const v2h diff = dd - p[j];
                const v2h sq = diff * diff;
                best = j == 0 ? sq : __builtin_elementwise_min(best, sq);
            }
            const _Float16 m = best[0] < best[1] ? best[0] : best[1];
            sum += static_cast<float>(m);
        }
    }
    if (line < n)
        mse[static_cast<size_t>(b) * n + line] = sum / static_cast<float>(G);
}

// Activations to bit planes on the fly: lane = one element x[m, k]; its selector is the first of the P
// subset sums of its group's line that is nearest to it (fp16 difference and square, as the encoder chooses
// selectors: sbvr/core.py:492-494), and the 64 lanes' selector bits become two words per plane by ballot
// (a selector counts the subset sums most significant coefficient first: plane j is its bit S - 1 - j,
// core.py:345-351 and :842-876).
// Grid: (ceil(K / 64), M), one wave per workgroup.
__global__ void __launch_bounds__(64)
sbvr_online_encode_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ points, uint32_t *__restrict__ bvr,
                          int M, int K, int G, int S)
{
    const int lane = threadIdx.x;
    const int m = blockIdx.y;
    const int k = blockIdx.x * 64 + lane;
    const int P = 1 << S;
    int sel = 0;
    if (k < K) {
        const _Float16 d = __builtin_bit_cast(_Float16, x[static_cast<size_t>(m) * K + k]);
        const uint16_t *pts = points + static_cast<size_t>(k / G) * P;
        _Float16 best = static_cast<_Float16>(0.f);
        for (int p = 0; p < P; ++p) {
            const _Float16 diff = d - __builtin_bit_cast(_Float16, pts[p]);
            const _Float16 sq = diff * diff;
            if (p == 0 || sq < best) {
                best = sq;
                sel = p;
            }
        }
    }
    const int words = K / 32;
    for (int j = 0; j < S; ++j) {
        const unsigned long long bits = __builtin_amdgcn_ballot_w64(((sel >> (S - 1 - j)) & 1) != 0);   // plane 0: the top bit
        const int kw = blockIdx.x * 2 + (lane >> 5);
        if ((lane & 31) == 0 && kw < words)
            bvr[(static_cast<size_t>(kw) * M + m) * S + j] = static_cast<uint32_t>(lane == 0 ? bits : bits >> 32);
    }
}

}  // namespace

extern "C" {

int sbvr_hip_encoder_group_mse_f16(const void *data, const void *points, float *mse, int groups, int G, int n, int P,
                                   void *stream)
{
    if (!data || !points || !mse || groups <= 0 || G <= 0 || n <= 0)
        return -1;
    if (groups > 65535 || P < 2 || P > 256 || (P & (P - 1)) != 0)
        return -2;
    if (reinterpret_cast<uintptr_t>(points) % 4 != 0)
        return -1;
    const dim3 grid(static_cast<unsigned>((n + kEncThreads - 1) / kEncThreads), static_cast<unsigned>(groups)), block(kEncThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t *d = static_cast<const uint16_t *>(data), *p = static_cast<const uint16_t *>(points);
    switch (P) {
    case 2: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<2>, grid, block, 0, st, d, p, mse, G, n); break;
    case 4: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<4>, grid, block, 0, st, d, p, mse, G, n); break;
    case 8: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<8>, grid, block, 0, st, d, p, mse, G, n); break;
    case 16: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<16>, grid, block, 0, st, d, p, mse, G, n); break;
    case 32: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<32>, grid, block, 0, st, d, p, mse, G, n); break;
    case 64: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<64>, grid, block, 0, st, d, p, mse, G, n); break;
    case 128: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<128>, grid, block, 0, st, d, p, mse, G, n); break;
    default: hipLaunchKernelGGL(sbvr_encoder_group_mse_kernel<256>, grid, block, 0, st, d, p, mse, G, n); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

int sbvr_hip_online_encode_f16(const void *x, const void *points, uint32_t *bvr, int M, int K, int G, int S, void *stream)
{
    if (!x || !points || !bvr || M <= 0 || K <= 0 || G <= 0 || S <= 0)
        return -1;
    if (S > 8 || G % 32 != 0 || K % G != 0 || M > 65535)
        return -2;
    const dim3 grid(static_cast<unsigned>((K + 63) / 64), static_cast<unsigned>(M)), block(64);
    hipLaunchKernelGGL(sbvr_online_encode_kernel, grid, block, 0, static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(x),
                       static_cast<const uint16_t *>(points), bvr, M, K, G, S);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // extern "C"
