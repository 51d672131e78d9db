/* Single-token helper kernels of the Llama-shaped decoder that measures the
 * "8B decode tokens/s" figure (libsbvr_hip.so, gfx950).  They sit between the
 * SBVR linears of a layer; the linears themselves are in sbvr_hip.h.
 *
 * All tensors are device pointers, fp16 unless stated (n even, head_dim 64 or 128), and the
 * launches go to `stream` (a hipStream_t, NULL = default stream).  Return
 * values: 0 ok, -1 invalid argument, -2 unsupported shape, -3 launch error,
 * -4 workspace missing or too small.
 */
#ifndef SBVR_HIP_DECODER_H
#define SBVR_HIP_DECODER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* x[n] <- fp16(x + delta) when delta is not NULL, then
 * h[n] <- weight * fp16(x * rsqrt(mean(x^2) + eps)), statistics in fp32.
 * Replaces the residual add of LlamaDecoderLayer.forward followed by
 * LlamaRMSNorm.forward (reference models/sbvr_llama.py:118-123, 368-420). */
int sbvr_hip_dec_add_rmsnorm_f16(void *x, const void *delta, const void *weight, void *h, int n, float eps,
                                 void *stream);

/* One new token of one sequence.  qkv = [heads*head_dim | kv_heads*head_dim |
 * kv_heads*head_dim] fp16.  Rotary embedding with row *pos of the fp32 tables
 * cos/sin (max_seq, head_dim/2) in the rotate-half convention, append of the
 * rotated key and the value to the caches (kv_heads, max_seq, head_dim) at
 * *pos, softmax(q k^T / sqrt(head_dim)) over positions 0..*pos in fp32 with
 * the weights rounded to fp16, context (heads*head_dim) fp16.
 * Replaces apply_rotary_pos_emb + the cache update + eager_attention_forward
 * (reference models/sbvr_llama.py:193-224, 255-278, 307-354) for batch 1,
 * query length 1.  *pos is read on the device, so a recorded launch can be
 * replayed for successive positions.  rot_now, when not NULL, holds row *pos
 * of the two tables side by side (cos | sin, head_dim floats), as
 * sbvr_hip_dec_argmax_advance_f16 leaves it: the kernel then need not wait
 * for *pos before it asks for the rotation.  The caches must be 16-byte
 * aligned. */
int sbvr_hip_dec_attention_f16(const void *qkv, const float *cos_table, const float *sin_table, const float *rot_now,
                               const long long *pos, void *kcache, void *vcache, void *ctx, int heads, int kv_heads,
                               int head_dim, int max_seq, void *stream);

/* sbvr_hip_dec_attention_f16 followed by the SBVR-encoded output projection
 * (sbvr_hip_linear_f16 of the context row, sbvr_hip.h) in one launch:
 * out[N] <- o_proj(attention(qkv)), i.e. `attn_output = self.o_proj(attn_output)`
 * after the attention of LlamaAttention.forward (reference
 * models/sbvr_llama.py:307-354, the projection at :352) for batch 1, query
 * length 1.  Same arguments and arithmetic as the attention call, with two
 * differences.  ctx may be NULL (when given it receives the heads*head_dim
 * context values the projection consumes).  Both caches are private to this
 * call and hold their (kv_heads, max_seq, 128) elements in a blocked order, so
 * that every request of a wave is 1 KiB of consecutive memory: per key/value
 * head, element (position t, dimension d) lies at
 *   keys:   (t/16)*2048 + (d/32)*512 + (d%32/8)*128 + (t%16)*8 + d%8
 *   values: (t/32)*4096 + (d/16)*512 + (t%32/8)*128 + (d%16)*8 + t%8.
 * Caches that start zero-filled (or whose rows past *pos do not matter) need
 * no conversion; a cache filled by sbvr_hip_dec_attention_f16 does.
 * The projection's weight is in the default layout of sbvr_hip_linear_f16 with
 * K = heads*head_dim: o_bvr (K/32, N, S) uint32, o_coeff_idx (K/G, N) uint8 or
 * uint16 (idx_bytes), o_coeff_cache (L, S) fp16, o_bias (N) fp16 or NULL (added
 * after the rounding).
 * Shapes: head_dim 128, heads = 4 * kv_heads, max_seq a multiple of 32 up to
 * 4096, N a multiple of 128, S in {2,3,4,6,8}, G a power-of-two multiple of 128;
 * sbvr_hip_dec_attention_o_supported returns 1 for a shape this call takes, and
 * anything else gets -2 (run the two calls separately).  Caches, o_bvr and
 * o_coeff_cache 16-byte aligned.
 * workspace: sbvr_hip_dec_attention_o_workspace(kv_heads, N) bytes (8 per output
 * when kv_heads > 1), zero-filled once; every launch leaves it zero-filled, and
 * launches that share it must not overlap in time (-4 when missing or small).
 * The result does not depend on the order in which workgroups finish. */
int sbvr_hip_dec_attention_o_supported(int heads, int kv_heads, int head_dim, int max_seq, int N, int S, int G);
size_t sbvr_hip_dec_attention_o_workspace(int kv_heads, int N);
int sbvr_hip_dec_attention_o_f16(const void *qkv, const float *cos_table, const float *sin_table, const float *rot_now,
                                 const long long *pos, void *kcache, void *vcache, void *ctx, int heads, int kv_heads,
                                 int head_dim, int max_seq, const uint32_t *o_bvr, const void *o_coeff_idx, int idx_bytes,
                                 const void *o_coeff_cache, const void *o_bias, void *out, int N, int S, int G, int L,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* out[ffn] <- fp16(silu(gate)) * up with gate_up = [gate | up] (2*ffn) fp16.
 * Replaces act_fn(gate_proj(x)) * up_proj(x) of LlamaMLP.forward
 * (reference models/sbvr_llama.py:238-240). */
int sbvr_hip_dec_silu_mul_f16(const void *gate_up, void *out, int ffn, void *stream);

/* Greedy choice and bookkeeping of a decode step: *token <- argmax(logits[0..n)) (the
 * lowest index among equal maxima, as torch.argmax), generated[*pos] <- *token when
 * *pos < max_seq, *pos <- *pos + 1.  Replaces `next_tokens = argmax(logits)` and the
 * cache-position update of the generation loop the reference inherits from
 * GenerationMixin (reference models/sbvr_llama.py:801).  When rot_now is not NULL
 * it receives row min(*pos, max_seq - 1) (the new position) of the rotary tables
 * cos | sin (max_seq, head_dim/2 floats each), for the attention launches of the
 * next step. */
int sbvr_hip_dec_argmax_advance_f16(const void *logits, int n, long long *token, long long *generated, long long *pos,
                                    int max_seq, const float *cos_table, const float *sin_table, int head_dim,
                                    float *rot_now, void *stream);

/* The end of a decode step in one launch: the final residual add and RMSNorm (as
 * sbvr_hip_dec_add_rmsnorm_f16, delta may be NULL, x is not written), the fp16
 * output head logits[v] = fp16(h . head[v]) for head (vocab, K) row-major
 * (reference models/sbvr_llama.py:851-853, lm_head over the last hidden state;
 * fp32 sums, one rounding), and the greedy choice and bookkeeping of
 * sbvr_hip_dec_argmax_advance_f16 on those fp16 logits.  logits may be NULL
 * (not stored).  K must be 512, 1024, 2048, 4096 or 8192 (-2 otherwise: run the
 * three steps separately); x, delta, norm_weight and head 16-byte aligned.
 * workspace: 16 bytes of device memory, zero-filled once; every launch leaves it
 * zero-filled.  Launches that share a workspace must not overlap in time. */
int sbvr_hip_dec_head_argmax_f16(const void *x, const void *delta, const void *norm_weight, float eps, const void *head,
                                 int vocab, int K, void *logits, long long *token, long long *generated, long long *pos,
                                 int max_seq, const float *cos_table, const float *sin_table, int head_dim,
                                 float *rot_now, void *workspace, void *stream);

/* sbvr_hip_dec_head_argmax_f16 that also starts the next step: x_next[K] <-
 * embed[*token] for the token it has chosen (embed: (vocab, K) fp16 row-major,
 * the model's embed_tokens, reference models/sbvr_llama.py:599), so that a
 * decode step whose input is the previous step's choice needs no launch of
 * its own for the embedding row.  embed and x_next both NULL: the call above.
 * Both 16-byte aligned; x_next may be x. */
int sbvr_hip_dec_head_argmax_embed_f16(const void *x, const void *delta, const void *norm_weight, float eps,
                                       const void *head, int vocab, int K, void *logits, long long *token,
                                       long long *generated, long long *pos, int max_seq, const float *cos_table,
                                       const float *sin_table, int head_dim, float *rot_now, void *workspace,
                                       const void *embed, void *x_next, void *stream);

#ifdef __cplusplus
}
#endif
#endif
