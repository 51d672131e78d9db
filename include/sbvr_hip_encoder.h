/* Encoder search on the GPU (libsbvr_hip.so, gfx950).  Device pointers; the
 * launch goes to `stream` (a hipStream_t, NULL = default stream).  Return
 * values: 0 ok, -1 invalid argument, -2 unsupported shape, -3 launch error.
 */
#ifndef SBVR_HIP_ENCODER_H
#define SBVR_HIP_ENCODER_H

#ifdef __cplusplus
extern "C" {
#endif

/* mse[b, l] = mean over the G values of group b of min_p (data[b, g] - points[l, p])^2, for `groups`
 * groups and n candidate lines at once: data (groups, G) fp16, points (n, P) fp16 (the P = 2^S subset
 * sums of each line, 4-byte aligned), mse (groups, n) fp32.  Difference and square are rounded to fp16
 * and the minimum is taken there, as the reference's search does in its fp16 compute type
 * (sbvr/core.py:485-495, _data_diff_min_mse: `(data - candidate_matrix)**2`, `.min(dim=-1)`); the sum
 * over the group is fp32 in element order, divided by G (the reference: `.to(torch.float32).mean(dim=-1)`,
 * whose order of summation is torch's).  groups <= 65535, P a power of two up to 256 (S <= 8).
 * Replaces the error evaluation inside _search_coeff_bias_space (core.py:530-553), which
 * the reference runs for one group at a time (core.py:711-722). */
int sbvr_hip_encoder_group_mse_f16(const void *data, const void *points, float *mse, int groups, int G, int n, int P,
                                   void *stream);

/* Activations to bit planes on the fly: x (M, K) fp16 -> bvr (K/32, M, S) uint32, bit k%32 of
 * bvr[k/32, m, j] = bit S-1-j of the selector of x[m, k] (point p of a line is the sum of the
 * coefficients j with bit S-1-j of p set, sbvr/core.py:345-351): the index of the first of the 2^S points of group
 * k/G (points (K/G, 2^S) fp16, the subset sums of that group's input coefficients) nearest to x[m, k],
 * difference and square in fp16 (the encoder's selector rule, sbvr/core.py:492-494).  The result, with
 * coeff_idx[g, m] = g and the input coefficients as coeff_cache, is the left operand of sbvr_hip_mm_T.
 * This is what the reference's _online_tranfrom / online_mm_T (sbvr/core.py:1021-1027, both return
 * None there) are placeholders for.  G a multiple of 32, K of G, S <= 8, M <= 65535. */
int sbvr_hip_online_encode_f16(const void *x, const void *points, uint32_t *bvr, int M, int K, int G, int S, void *stream);

#ifdef __cplusplus
}
#endif

#endif
