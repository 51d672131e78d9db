/*
 * sbvr_oracle.c -- TEST INFRASTRUCTURE, not product code.
 *
 * A plain-C, single-threaded restatement of what the reference computes on the
 * SBVR linear path: the bit packing of sbvr/core.py, its decode(), the matrix
 * products its kernels implement, and the re-layouts between its three array
 * formats.  Every function is written from the definition, with loops over
 * single elements and double accumulation, so that it is slow and obviously
 * right.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load this library; the shipped path never does.
 *
 * Conventions restated here (reference file:line in each function):
 *   sel      selector of one element, 0 .. 2^S-1, an index into
 *            itertools.product([0,1], repeat=S); plane j of an element is bit
 *            (S-1-j) of its selector, and plane j pairs with coefficient j.
 *   planes   (S, R*Kp/Wb) words of Wb bits, element w*Wb+i in bit i (LSB first).
 *   default  bvr (Kp/Wb, R, S), coeff_idx (Kp/G, R), coeff_cache (L, S) fp16.
 *   v1       bvr (R/16, Kp/8, S, 16) uint8, coeff_idx (Kp/G, R).
 *
 * How each function is pinned is listed in tests/test_oracle_*.py: the golden
 * vectors written by the reference itself (tests/golden/), brute force from the
 * definition, closed forms and round trips.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

/* ------------------------------------------------------------------ fp16 */

static double h2d(uint16_t h)
{
    int s = (h >> 15) & 1, e = (h >> 10) & 31, m = h & 1023;
    double v;
    if (e == 0)
        v = ldexp((double)m, -24);
    else if (e == 31)
        v = m ? NAN : INFINITY;
    else
        v = ldexp((double)(m + 1024), e - 25);
    return s ? -v : v;
}

/* round-to-nearest-even double -> binary16, done in one step (no float detour) */
static uint16_t d2h(double d)
{
    uint16_t sign = 0;
    if (isnan(d))
        return 0x7e00;
    if (signbit(d)) {
        sign = 0x8000;
        d = -d;
    }
    if (isinf(d))
        return sign | 0x7c00;
    if (d == 0.0)
        return sign;
    int e;
    double f = frexp(d, &e);        /* d = f * 2^e, f in [0.5, 1) */
    int E = e - 1;                  /* d = (2f) * 2^E, 2f in [1, 2) */
    double q;                       /* value in units of the target ulp */
    int biased;
    if (E < -14) {                  /* subnormal: ulp is 2^-24 */
        q = ldexp(d, 24);
        biased = 0;
    } else {
        q = ldexp(f, 11);           /* in [1024, 2048) */
        biased = E + 15;
    }
    double r = nearbyint(q);        /* default rounding mode: ties to even */
    uint32_t m = (uint32_t)r;
    if (biased == 0)                /* m == 1024 is the smallest normal: same bits */
        return sign | (uint16_t)m;
    if (m >= 2048) {
        m >>= 1;
        biased += 1;
    }
    if (biased >= 31)
        return sign | 0x7c00;
    return sign | (uint16_t)((biased << 10) | (m - 1024));
}

double sbvr_oracle_h2d(uint16_t h) { return h2d(h); }
uint16_t sbvr_oracle_d2h(double d) { return d2h(d); }

/* ------------------------------------------------------ bit plane access */

static inline int word_bit(const void *words, int word_bits, int64_t word, int bit)
{
    if (word_bits == 32)
        return (((const uint32_t *)words)[word] >> bit) & 1u;
    return (((const uint8_t *)words)[word] >> bit) & 1u;
}

static inline void word_set(void *words, int word_bits, int64_t word, int bit)
{
    if (word_bits == 32)
        ((uint32_t *)words)[word] |= (1u << bit);
    else
        ((uint8_t *)words)[word] |= (uint8_t)(1u << bit);
}

/* plane bit of element (r, k) in the default layout bvr (Kp/Wb, R, S)
 * -- core.py:726-731 (view S, R, Kp/Wb) and :783 (permute 2,1,0). */
static inline int dflt_bit(const void *bvr, int word_bits, int64_t R, int S,
                           int64_t r, int64_t k, int j)
{
    int64_t w = k / word_bits;
    return word_bit(bvr, word_bits, (w * R + r) * S + j, (int)(k % word_bits));
}

/* selectors -> planes, core.py:815-818 (_dec2bin, MSB first) and :842-876
 * (_change_coeff_sel_to_bvr, LSB first inside a word).  planes is (S, numel/Wb),
 * zeroed here. */
void sbvr_oracle_sel_to_planes(const int32_t *sel, int64_t numel, int S,
                               int word_bits, void *planes)
{
    int64_t nwords = numel / word_bits;
    memset(planes, 0, (size_t)(S * nwords * (word_bits / 8)));
    for (int64_t e = 0; e < numel; ++e)
        for (int j = 0; j < S; ++j)
            if ((sel[e] >> (S - 1 - j)) & 1)
                word_set(planes, word_bits, j * nwords + e / word_bits,
                         (int)(e % word_bits));
}

/* planes (S, R, Kp/Wb) -> default bvr (Kp/Wb, R, S), core.py:726-731, 783 */
void sbvr_oracle_planes_to_default(const void *planes, int64_t R, int64_t Kp,
                                   int S, int word_bits, void *bvr)
{
    int64_t Kw = Kp / word_bits;
    int bytes = word_bits / 8;
    for (int j = 0; j < S; ++j)
        for (int64_t r = 0; r < R; ++r)
            for (int64_t w = 0; w < Kw; ++w)
                memcpy((char *)bvr + ((w * R + r) * S + j) * bytes,
                       (const char *)planes + ((j * R + r) * Kw + w) * bytes,
                       (size_t)bytes);
}

/* planes (S, R, Kp/8) uint8 -> v1 bvr (R/16, Kp/8, S, 16), core.py:754-768 */
void sbvr_oracle_planes_to_v1(const uint8_t *planes, int64_t R, int64_t Kp,
                              int S, uint8_t *bvr)
{
    int64_t Kw = Kp / 8;
    for (int j = 0; j < S; ++j)
        for (int64_t r = 0; r < R; ++r)
            for (int64_t w = 0; w < Kw; ++w)
                bvr[(((r / 16) * Kw + w) * S + j) * 16 + (r % 16)] =
                    planes[(j * R + r) * Kw + w];
}

/* group index as the encoder emits it, (R*Kp/G) in row-major group order
 * -> coeff_idx (Kp/G, R), core.py:794-800 (and :774 for v1).  elem = 1 or 2 bytes. */
void sbvr_oracle_idx_to_default(const void *flat, int64_t R, int64_t Kg,
                                int elem, void *coeff_idx)
{
    for (int64_t r = 0; r < R; ++r)
        for (int64_t g = 0; g < Kg; ++g)
            memcpy((char *)coeff_idx + (g * R + r) * elem,
                   (const char *)flat + (r * Kg + g) * elem, (size_t)elem);
}

/* default bvr -> selectors (R*Kp), core.py:879-901 and :820-822 (_bin2dec) */
void sbvr_oracle_default_to_sel(const void *bvr, int64_t R, int64_t Kp, int S,
                                int word_bits, int32_t *sel)
{
    for (int64_t r = 0; r < R; ++r)
        for (int64_t k = 0; k < Kp; ++k) {
            int32_t v = 0;
            for (int j = 0; j < S; ++j)
                v |= dflt_bit(bvr, word_bits, R, S, r, k, j) << (S - 1 - j);
            sel[r * Kp + k] = v;
        }
}

static inline int idx_at(const void *coeff_idx, int idx_bytes, int64_t i)
{
    return idx_bytes == 1 ? ((const uint8_t *)coeff_idx)[i]
                          : ((const uint16_t *)coeff_idx)[i];
}

/* decode(), core.py:927-949: every element becomes entry `sel` of its group's
 * 2^S points, the points being bin_combs @ coeff rounded to fp16 (core.py:345-366).
 * out is (R, Kout) fp16 with Kout <= Kp (the reference truncates the padding). */
void sbvr_oracle_decode(const void *bvr, int word_bits, const void *coeff_idx,
                        int idx_bytes, const uint16_t *coeff_cache, int64_t R,
                        int64_t Kp, int64_t Kout, int S, int G, uint16_t *out)
{
    for (int64_t r = 0; r < R; ++r)
        for (int64_t k = 0; k < Kout; ++k) {
            int line = idx_at(coeff_idx, idx_bytes, (k / G) * R + r);
            double v = 0.0;
            for (int j = 0; j < S; ++j)
                if (dflt_bit(bvr, word_bits, R, S, r, k, j))
                    v += h2d(coeff_cache[(int64_t)line * S + j]);
            out[r * Kout + k] = d2h(v);
        }
}

/* The product the GPU path implements: fp16 activations x (M,K) against an
 * encoded weight (N rows, K columns, default layout):
 *   y[m,n] = f16( sum_g sum_j c[idx[g,n]][j] * sum_{k in g, bit_j(n,k)=1} x[m,k] )
 * which in real arithmetic is x @ decode(W)^T (core.py:927-949 for decode, the
 * accumulate-then-round-once and bias-after-rounding order of
 * sbvr_kernel.cu:479, 555-559).  mode 0: coefficients applied to plane sums
 * (no per-element rounding); mode 1: every element first rounded to fp16 as
 * decode() does.  yd, when not NULL, receives the unrounded double sums. */
void sbvr_oracle_linear_f16(const uint16_t *x, const void *bvr, int word_bits,
                            const void *coeff_idx, int idx_bytes,
                            const uint16_t *coeff_cache, const uint16_t *bias,
                            int64_t M, int64_t N, int64_t K, int S, int G,
                            int mode, uint16_t *y, double *yd)
{
    int64_t Kg = K / G;
    /* (every output is one thread's own sequential sum: the threads change nothing in the results) */
#pragma omp parallel for collapse(2) schedule(static) if (M * N * K > (1 << 22))
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t g = 0; g < Kg; ++g) {
                int line = idx_at(coeff_idx, idx_bytes, g * N + n);
                const uint16_t *c = coeff_cache + (int64_t)line * S;
                if (mode == 0) {
                    for (int j = 0; j < S; ++j) {
                        double ps = 0.0;
                        for (int64_t k = g * G; k < (g + 1) * G; ++k)
                            if (dflt_bit(bvr, word_bits, N, S, n, k, j))
                                ps += h2d(x[m * K + k]);
                        acc += h2d(c[j]) * ps;
                    }
                } else {
                    for (int64_t k = g * G; k < (g + 1) * G; ++k) {
                        double w = 0.0;
                        for (int j = 0; j < S; ++j)
                            if (dflt_bit(bvr, word_bits, N, S, n, k, j))
                                w += h2d(c[j]);
                        acc += h2d(x[m * K + k]) * h2d(d2h(w));
                    }
                }
            }
            if (yd)
                yd[m * N + n] = acc;
            uint16_t r = d2h(acc);
            if (bias)
                r = d2h(h2d(r) + h2d(bias[n]));
            y[m * N + n] = r;
        }
}

/* Both operands encoded (default layout, either word width):
 *   y[m,n] = f16( sum_g sum_l sum_r popcount_g(L_l & R_r) * a_l * b_r ) (+ bias)
 * sbvr_kernel_v2.cpp:135-194 (exact coefficient products, sum over groups),
 * sbvr_kernel.cu:367-417 and :464-562 (bias added after rounding). */
void sbvr_oracle_mm_T(const void *l_bvr, const void *l_idx, int l_idx_bytes,
                      const uint16_t *l_cache, const void *r_bvr,
                      const void *r_idx, int r_idx_bytes,
                      const uint16_t *r_cache, const uint16_t *bias,
                      int word_bits, int64_t M, int64_t N, int64_t K, int Sl,
                      int Sr, int G, uint16_t *y, double *yd)
{
    int64_t Kg = K / G;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t g = 0; g < Kg; ++g) {
                const uint16_t *a = l_cache + (int64_t)idx_at(l_idx, l_idx_bytes, g * M + m) * Sl;
                const uint16_t *b = r_cache + (int64_t)idx_at(r_idx, r_idx_bytes, g * N + n) * Sr;
                for (int l = 0; l < Sl; ++l)
                    for (int r = 0; r < Sr; ++r) {
                        int pc = 0;
                        for (int64_t k = g * G; k < (g + 1) * G; ++k)
                            pc += dflt_bit(l_bvr, word_bits, M, Sl, m, k, l) &
                                  dflt_bit(r_bvr, word_bits, N, Sr, n, k, r);
                        acc += (double)pc * h2d(a[l]) * h2d(b[r]);
                    }
            }
            if (yd)
                yd[m * N + n] = acc;
            uint16_t out = d2h(acc);
            if (bias)
                out = d2h(h2d(out) + h2d(bias[n]));
            y[m * N + n] = out;
        }
}

/* The same product with the weight in the v1 CPU layout and a single encoded
 * activation row in the default uint8 layout (K/8, 1, Sl):
 * sbvr_kernel.cpp:255-399 (r_bvr (N/16, K/8, Sr, 16) :259,314; coeff_idx
 * (K/G, N) :288).  wrap8 != 0 reproduces the 8-bit popcount accumulator of
 * :273,323-326, which wraps when a whole 256-bit group matches. */
void sbvr_oracle_mm_T_v1(const uint8_t *l_bvr, const void *l_idx, int l_idx_bytes,
                         const uint16_t *l_cache, const uint8_t *r_bvr,
                         const void *r_idx, int r_idx_bytes,
                         const uint16_t *r_cache, const uint16_t *bias,
                         int64_t N, int64_t K, int Sl, int Sr, int G, int wrap8,
                         uint16_t *y)
{
    int64_t Kb = K / 8, Kg = K / G;
    for (int64_t n = 0; n < N; ++n) {
        double acc = 0.0;
        for (int64_t g = 0; g < Kg; ++g) {
            const uint16_t *a = l_cache + (int64_t)idx_at(l_idx, l_idx_bytes, g) * Sl;
            const uint16_t *b = r_cache + (int64_t)idx_at(r_idx, r_idx_bytes, g * N + n) * Sr;
            for (int l = 0; l < Sl; ++l)
                for (int r = 0; r < Sr; ++r) {
                    int pc = 0;
                    for (int64_t kb = g * (G / 8); kb < (g + 1) * (G / 8); ++kb) {
                        uint8_t lv = l_bvr[kb * Sl + l];
                        uint8_t rv = r_bvr[(((n / 16) * Kb + kb) * Sr + r) * 16 + (n % 16)];
                        pc += __builtin_popcount((unsigned)(lv & rv));
                    }
                    if (wrap8)
                        pc &= 255;
                    acc += (double)pc * h2d(a[l]) * h2d(b[r]);
                }
        }
        uint16_t out = d2h(acc);
        if (bias)
            out = d2h(h2d(out) + h2d(bias[n]));
        y[n] = out;
    }
}

/* fp16 activations against a weight encoded with trans=True (core.py:244-245):
 * the encoded tensor is W^T (K rows, N columns), groups run along N, default
 * uint32 layout r_bvr (N/32, K, S), r_coeff_idx (N/G, K).
 *   y[m,n] = f16( bias[n] + sum_k x[m,k] * sum_j c[idx[n/G,k]][j] * bit_j(k,n) )
 * sbvr_kernel.cu:121-191 (bias seeds the fp32 sum there, :145). */
void sbvr_oracle_row_deq_mm_T(const uint16_t *x, const uint32_t *r_bvr,
                              const void *r_idx, int r_idx_bytes,
                              const uint16_t *r_cache, const uint16_t *bias,
                              int64_t M, int64_t N, int64_t K, int S, int G,
                              uint16_t *y)
{
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = bias ? h2d(bias[n]) : 0.0;
            for (int64_t k = 0; k < K; ++k) {
                int line = idx_at(r_idx, r_idx_bytes, (n / G) * K + k);
                double w = 0.0;
                for (int j = 0; j < S; ++j)
                    if ((r_bvr[((n / 32) * K + k) * S + j] >> (n % 32)) & 1u)
                        w += h2d(r_cache[(int64_t)line * S + j]);
                acc += h2d(x[m * K + k]) * w;
            }
            y[m * N + n] = d2h(acc);
        }
}
