/* Single-token helper kernels of the Llama-shaped decoder that measures the
 * "8B decode tokens/s" figure (libsbvr_hip.so, gfx950).  They sit between the
 * SBVR linears of a layer; the linears themselves are in sbvr_hip.h.
 *
 * All tensors are device pointers, fp16 unless stated (n even, head_dim 64 or 128), and the
 * launches go to `stream` (a hipStream_t, NULL = default stream).  Return
 * values: 0 ok, -1 invalid argument, -2 unsupported shape, -3 launch error.
 */
#ifndef SBVR_HIP_DECODER_H
#define SBVR_HIP_DECODER_H

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

#ifdef __cplusplus
}
#endif
#endif
