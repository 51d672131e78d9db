// sbvr_cpu_port.cpp -- TEST / BASELINE INFRASTRUCTURE, not product code.
//
// An x86-64 port of the reference's timed CPU kernel, so that a CPU figure can
// stand beside the GPU one (the reference's own kernels are ARM-NEON only and
// do not compile on the GPU box's host).  Same algorithm and data layout as
// sbvr/kernels/sbvr_kernel.cpp:251-399 (simd_kernel_1xN_popc_first) and
// :471-539 (sbvr_mm_cpu_1xN):
//   * both operands SBVR-encoded; one activation row l_bvr (K/8, 1, Sl) uint8,
//     weight r_bvr (N/16, K/8, Sr, 16) uint8, r_coeff_idx (K/G, N);
//   * per tile of 16 columns and per group: gather the 16 coefficient lines,
//     then for every byte of the group AND the broadcast activation byte with
//     16 weight bytes, popcount per byte, accumulate in 8-bit lanes
//     (:299-329, wrapping like the reference's uint8 accumulators :273);
//   * coefficient products a_l*b_r rounded to fp16, multiplied with the counts
//     and accumulated in fp32 (:332-374); fp16 result, bias added in fp16
//     (:377-396);
//   * N split in equal chunks over a pool of pinned threads, one task each,
//     caller blocks (:480-538, sbvr/include/thread_pool.hpp:132-214).
// The 16-lane vectors map to 128-bit registers (the fp32 accumulators to two
// 256-bit ones); byte popcount is VPOPCNTB where the CPU has AVX512-BITALG+VL,
// a nibble-table PSHUFB otherwise; AVX2, FMA and F16C are required.  Only
// bench.py's cpu_baseline leg and tests/ load this library.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#include <immintrin.h>
#include <pthread.h>
#include <sched.h>

namespace {

constexpr int kLane = 16;

// ------------------------------------------------------------------ fp16
inline float h2f(uint16_t h)
{
    const uint32_t s = (h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u;
    uint32_t bits;
    if (e == 0) {
        if (m == 0) {
            bits = s;
        } else {
            int sh = 0;
            uint32_t mm = m;
            while (!(mm & 1024u)) { mm <<= 1; ++sh; }
            bits = s | ((113u - sh) << 23) | ((mm & 1023u) << 13);
        }
    } else if (e == 31) {
        bits = s | 0x7f800000u | (m << 13);
    } else {
        bits = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline uint16_t f2h(float f)   // round to nearest even
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t s = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u)
        return s | (x > 0x7f800000u ? 0x7e00u : 0x7c00u);
    if (x >= 0x477ff000u)
        return s | 0x7c00u;                       // overflows to infinity
    if (x < 0x33000001u)
        return s;                                 // below half of the smallest subnormal
    const int e = static_cast<int>(x >> 23);
    uint32_t m = (x & 0x7fffffu) | 0x800000u;
    int shift;
    int he;
    if (e < 113) { shift = 126 - e; he = 0; }     // subnormal result
    else { shift = 13; he = e - 112; }
    const uint32_t half = 1u << (shift - 1), rest = m & ((1u << shift) - 1);
    uint32_t r = m >> shift;
    if (rest > half || (rest == half && (r & 1u)))
        ++r;
    if (he == 0)
        return s | static_cast<uint16_t>(r);      // r may reach 1024 == smallest normal
    r += static_cast<uint32_t>(he - 1) << 10;     // r still carries the implicit bit (1024)
    return s | static_cast<uint16_t>(r);
}

// ------------------------------------------------------------- thread pool
// Workers pinned to core id, one shared job, the caller blocks until all tasks
// are done (thread_pool.hpp:132-214).  Workers spin briefly before sleeping so
// that a 10-microsecond job is not dominated by wake-up latency.
class Pool {
public:
    int init(int n)
    {
        if (!workers_.empty())
            return static_cast<int>(workers_.size());
        if (n <= 0) {
            const unsigned hw = std::thread::hardware_concurrency();
            n = hw ? static_cast<int>(hw) : 4;
        }
        quit_ = false;
        for (int id = 0; id < n; ++id) {
            workers_.emplace_back([this, id] { loop(id); });
            cpu_set_t set;
            CPU_ZERO(&set);
            CPU_SET(id, &set);
            pthread_setaffinity_np(workers_.back().native_handle(), sizeof(set), &set);   // best effort
        }
        return n;
    }
    int size() const { return static_cast<int>(workers_.size()); }
    void run(int tasks, const std::function<void(int)> &fn)
    {
        if (workers_.empty() || tasks <= 0) {
            for (int i = 0; i < tasks; ++i)
                fn(i);
            return;
        }
        {
            std::lock_guard<std::mutex> lk(m_);
            fn_ = &fn;
            tasks_ = tasks;
            next_.store(0);
            pending_.store(tasks);
            ++generation_;
        }
        cv_.notify_all();
        while (pending_.load(std::memory_order_acquire) != 0)
            _mm_pause();
    }
    void finalize()
    {
        {
            std::lock_guard<std::mutex> lk(m_);
            quit_ = true;
            ++generation_;
        }
        cv_.notify_all();
        for (auto &t : workers_)
            t.join();
        workers_.clear();
    }
    ~Pool() { if (!workers_.empty()) finalize(); }

private:
    void loop(int)
    {
        uint64_t seen = 0;
        for (;;) {
            int spins = 0;
            while (generation_.load(std::memory_order_acquire) == seen) {
                if (++spins < 20000) {
                    _mm_pause();
                } else {
                    std::unique_lock<std::mutex> lk(m_);
                    cv_.wait(lk, [&] { return generation_.load() != seen; });
                }
            }
            seen = generation_.load();
            if (quit_)
                return;
            for (;;) {
                const int t = next_.fetch_add(1);
                if (t >= tasks_)
                    break;
                (*fn_)(t);
                pending_.fetch_sub(1, std::memory_order_release);
            }
        }
    }
    std::vector<std::thread> workers_;
    std::mutex m_;
    std::condition_variable cv_;
    const std::function<void(int)> *fn_ = nullptr;
    int tasks_ = 0;
    std::atomic<int> next_{0}, pending_{0};
    std::atomic<uint64_t> generation_{0};
    bool quit_ = false;
};

Pool g_pool;

// ---------------------------------------------------------------- kernels
struct Job {
    const uint8_t *l_bvr; const void *l_idx; int l_idx_bytes; const uint16_t *l_cache;
    const uint8_t *r_bvr; const void *r_idx; int r_idx_bytes; const uint16_t *r_cache;
    const uint16_t *bias; uint16_t *out;
    int N, K, Sl, Sr, G;
};

inline int idx_at(const void *p, int bytes, size_t i)
{
    return bytes == 1 ? static_cast<const uint8_t *>(p)[i] : static_cast<const uint16_t *>(p)[i];
}

// One chunk of columns [n0, n1), n1-n0 a multiple of 16.  SL/SR > 0 fix the
// plane counts at compile time (the reference's 25-entry table,
// sbvr_kernel.cpp:541-590); 0 means "use the runtime values".  The body is
// stamped out once per instruction set; POPCNT8 is the per-byte popcount.
#define SBVR_CHUNK_KERNEL(NAME, TARGET, POPCNT8)                                                        \
    template <int SL, int SR>                                                                           \
    __attribute__((target(TARGET))) void NAME(const Job &j, int n0, int n1)                             \
    {                                                                                                   \
        const int Sl = SL ? SL : j.Sl, Sr = SR ? SR : j.Sr;                                             \
        const int bytes_per_group = j.G / 8, groups = j.K / j.G, Kb = j.K / 8;                          \
        constexpr int kMaxS = 10;                                                                       \
        for (int n = n0; n < n1; n += kLane) {                                                          \
            __m256 acc_lo = _mm256_setzero_ps(), acc_hi = _mm256_setzero_ps();                          \
            const uint8_t *tile = j.r_bvr + static_cast<size_t>(n / kLane) * Kb * Sr * kLane;           \
            for (int g = 0; g < groups; ++g) {                                                          \
                alignas(32) uint16_t lane_tile[kMaxS][kLane];      /* :276, 287-292 */                  \
                for (int nn = 0; nn < kLane; ++nn) {                                                    \
                    const uint16_t *src = j.r_cache +                                                   \
                        static_cast<size_t>(idx_at(j.r_idx, j.r_idx_bytes, static_cast<size_t>(g) * j.N + n + nn)) * Sr; \
                    for (int r = 0; r < Sr; ++r)                                                        \
                        lane_tile[r][nn] = src[r];                                                      \
                }                                                                                       \
                __m128i pc[kMaxS][kMaxS];                              /* :273, 294-296 */              \
                for (int l = 0; l < Sl; ++l)                                                            \
                    for (int r = 0; r < Sr; ++r)                                                        \
                        pc[l][r] = _mm_setzero_si128();                                                 \
                for (int kb = g * bytes_per_group; kb < (g + 1) * bytes_per_group; ++kb) { /* :299-329 */ \
                    const uint8_t *rrow = tile + static_cast<size_t>(kb) * Sr * kLane;                  \
                    for (int l = 0; l < Sl; ++l) {                                                      \
                        const __m128i lv = _mm_set1_epi8(static_cast<char>(j.l_bvr[static_cast<size_t>(kb) * Sl + l])); \
                        for (int r = 0; r < Sr; ++r) {                                                  \
                            const __m128i rv = _mm_loadu_si128(reinterpret_cast<const __m128i *>(rrow + r * kLane)); \
                            const __m128i a = _mm_and_si128(lv, rv);                                    \
                            pc[l][r] = _mm_add_epi8(pc[l][r], POPCNT8);                                 \
                        }                                                                               \
                    }                                                                                   \
                }                                                                                       \
                const uint16_t *la = j.l_cache + static_cast<size_t>(idx_at(j.l_idx, j.l_idx_bytes, g)) * Sl; \
                for (int l = 0; l < Sl; ++l) {                              /* :332-374 */              \
                    const __m256 av = _mm256_set1_ps(h2f(la[l]));                                       \
                    for (int r = 0; r < Sr; ++r) {                                                      \
                        const __m256 b_lo = _mm256_cvtph_ps(_mm_load_si128(reinterpret_cast<const __m128i *>(&lane_tile[r][0]))); \
                        const __m256 b_hi = _mm256_cvtph_ps(_mm_load_si128(reinterpret_cast<const __m128i *>(&lane_tile[r][8]))); \
                        /* coefficient product rounded to fp16 (vmulq_f16, :350) */                      \
                        const __m256 ab_lo = _mm256_cvtph_ps(_mm256_cvtps_ph(_mm256_mul_ps(av, b_lo), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC)); \
                        const __m256 ab_hi = _mm256_cvtph_ps(_mm256_cvtps_ph(_mm256_mul_ps(av, b_hi), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC)); \
                        const __m256 c_lo = _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(pc[l][r]));         \
                        const __m256 c_hi = _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(_mm_srli_si128(pc[l][r], 8))); \
                        acc_lo = _mm256_fmadd_ps(ab_lo, c_lo, acc_lo);       /* widening fma, :351-356 */ \
                        acc_hi = _mm256_fmadd_ps(ab_hi, c_hi, acc_hi);                                  \
                    }                                                                                   \
                }                                                                                       \
            }                                                                                           \
            alignas(32) float acc[kLane];                                                               \
            _mm256_store_ps(acc, acc_lo);                                                               \
            _mm256_store_ps(acc + 8, acc_hi);                                                           \
            for (int nn = 0; nn < kLane; ++nn) {                            /* :377-396 */              \
                uint16_t r = f2h(acc[nn]);                                                              \
                if (j.bias)                                                                             \
                    r = f2h(h2f(r) + h2f(j.bias[n + nn]));                                              \
                j.out[n + nn] = r;                                                                      \
            }                                                                                           \
        }                                                                                               \
    }

#define SBVR_POPCNT_PSHUFB                                                                              \
    _mm_add_epi8(_mm_shuffle_epi8(_mm_setr_epi8(0, 1, 1, 2, 1, 2, 2, 3, 1, 2, 2, 3, 2, 3, 3, 4),        \
                                  _mm_and_si128(a, _mm_set1_epi8(0x0f))),                               \
                 _mm_shuffle_epi8(_mm_setr_epi8(0, 1, 1, 2, 1, 2, 2, 3, 1, 2, 2, 3, 2, 3, 3, 4),        \
                                  _mm_and_si128(_mm_srli_epi16(a, 4), _mm_set1_epi8(0x0f))))

SBVR_CHUNK_KERNEL(chunk_kernel_bitalg, "avx2,fma,f16c,avx512f,avx512bw,avx512vl,avx512bitalg", _mm_popcnt_epi8(a))
SBVR_CHUNK_KERNEL(chunk_kernel_avx2, "avx2,fma,f16c,ssse3", SBVR_POPCNT_PSHUFB)

typedef void (*ChunkFn)(const Job &, int, int);

bool have_avx2()
{
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c");
}

bool have_bitalg()
{
    return have_avx2() && __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
           __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512bitalg");
}

template <int SL, int SR>
ChunkFn pick_impl(bool bitalg)
{
    return bitalg ? &chunk_kernel_bitalg<SL, SR> : &chunk_kernel_avx2<SL, SR>;
}

ChunkFn pick(int Sl, int Sr, bool bitalg)
{
#define SBVR_PICK(a, b) if (Sl == a && Sr == b) return pick_impl<a, b>(bitalg)
    SBVR_PICK(2, 2); SBVR_PICK(2, 4); SBVR_PICK(4, 2); SBVR_PICK(4, 4);
    SBVR_PICK(8, 4); SBVR_PICK(8, 6); SBVR_PICK(8, 8); SBVR_PICK(4, 8); SBVR_PICK(6, 6); SBVR_PICK(6, 4);
#undef SBVR_PICK
    return pick_impl<0, 0>(bitalg);
}

int run_job(const Job &j)
{
    if (j.N <= 0 || j.K <= 0 || j.N % kLane || j.G % 8 || j.K % j.G || j.Sl < 1 || j.Sr < 1 || j.Sl > 10 || j.Sr > 10)
        return -1;
    if (!have_avx2())
        return -2;     // no AVX2/FMA/F16C: no baseline on this host
    const ChunkFn fn = pick(j.Sl, j.Sr, have_bitalg());
    const int threads = g_pool.size() > 0 ? g_pool.size() : 1;
    int chunk = (j.N + threads - 1) / threads;
    chunk = (chunk + kLane - 1) / kLane * kLane;     // the reference refuses chunks that are not whole tiles (:503-506)
    const int tasks = (j.N + chunk - 1) / chunk;
    g_pool.run(tasks, [&](int t) {
        const int n0 = t * chunk, n1 = n0 + chunk < j.N ? n0 + chunk : j.N;
        fn(j, n0, n1);
    });
    return 0;
}

} // namespace

extern "C" {

// -1: all hardware threads (sbvr/__init__.py:12 of the reference does the same)
int sbvr_port_init_pool(int threads) { return g_pool.init(threads); }
int sbvr_port_num_threads(void) { return g_pool.size(); }
void sbvr_port_finalize_pool(void) { g_pool.finalize(); }
const char *sbvr_port_isa(void) { return have_bitalg() ? "avx512-bitalg vpopcntb" : (have_avx2() ? "avx2 pshufb" : "unsupported"); }

int sbvr_port_mm_T_v1(const uint8_t *l_bvr, const void *l_idx, int l_idx_bytes, const uint16_t *l_cache,
                      const uint8_t *r_bvr, const void *r_idx, int r_idx_bytes, const uint16_t *r_cache,
                      const uint16_t *bias, uint16_t *out, int N, int K, int Sl, int Sr, int G)
{
    const Job j{l_bvr, l_idx, l_idx_bytes, l_cache, r_bvr, r_idx, r_idx_bytes, r_cache, bias, out, N, K, Sl, Sr, G};
    return run_job(j);
}

// Mean seconds per call over `iters` calls after `warmup` calls, timed here so
// that no interpreter overhead is in the figure (protocol of
// test_sbvr.py:683-693: warm-ups, then a timed loop, mean per call).
double sbvr_port_time_mm_T_v1(const uint8_t *l_bvr, const void *l_idx, int l_idx_bytes, const uint16_t *l_cache,
                              const uint8_t *r_bvr, const void *r_idx, int r_idx_bytes, const uint16_t *r_cache,
                              const uint16_t *bias, uint16_t *out, int N, int K, int Sl, int Sr, int G,
                              int warmup, int iters)
{
    const Job j{l_bvr, l_idx, l_idx_bytes, l_cache, r_bvr, r_idx, r_idx_bytes, r_cache, bias, out, N, K, Sl, Sr, G};
    for (int i = 0; i < warmup; ++i)
        if (run_job(j) != 0)
            return -1.0;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i)
        run_job(j);
    const auto t1 = std::chrono::steady_clock::now();
    return std::chrono::duration<double>(t1 - t0).count() / (iters > 0 ? iters : 1);
}

} // extern "C"
