/*
 * hydra_mix.h — C ABI of libhydra_mix.so: kernels of the sequence-mixing mechanisms that the Llama path does not have —
 * multi-stream residuals (hyper-connections) with grouped RMS norm, token shift and gated sublayer results, the tanh
 * GELU gate, and attention over a paged cache of low-rank latents (one latent row per token, shared by all heads) with a
 * sliding window.
 *
 * Same conventions as hydra_hip.h: raw device pointers, sizes and strides in ELEMENTS, a hipStream_t passed as void*,
 * asynchronous launches, no allocation, 0 or a negative hx_status (hydra_hip.h) as the result.  `dtype` is the hx_dtype
 * of the ACTIVATIONS (what the matrix products read and write): HX_F32 or HX_BF16.  The residual streams, the per-sequence
 * state, norm / shift / mixing weights and biases are always float.
 *
 * The library is separate from libhydra_hip.so so that a model that needs only these kernels builds only these.
 */
#ifndef HYDRA_MIX_H
#define HYDRA_MIX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HXM_ABI_VERSION 1
#define HXM_MAX_STREAMS 16
#define HXM_MAX_LATENT 1024     /* widest latent row the attention kernels hold in registers (the MFMA tile form: 512) */

int hxm_abi_version(void);
int hxm_last_hip_error(void);
/* A/B measurements in one process: "attn_tile_form" = 0 keeps bfloat16 attention on the row form (one wave per token
 * and head) instead of the MFMA forms, 2 keeps portions of prompts on the tile form (one wave per 16 rows) instead of
 * the group form (four waves sharing every chunk of keys), 1 = the default.  Results agree within bfloat16 rounding. */
int hxm_set_option(const char* name, int value);

/* x[t, s, :] = table[ids[t], :] * scale for every stream s.  x: float [n_tokens, n_streams, width]; table: dtype
 * [vocab, width]; ids: int32 or int64.  An id outside [0, vocab) writes zeros. */
int hxm_stream_embed(float* x, const void* table, const void* ids, int ids_are_int64, float scale, int64_t n_tokens,
                     int32_t n_streams, int64_t width, int64_t vocab, int dtype, void* stream);

/* The input of a sublayer: u = sum_s in_w[s] * x[row, s, :], h = u / sqrt(mean_group(u^2) + eps) * norm_w over `groups`
 * equal consecutive groups.  rows (optional): int32 [n_out] rows of x to take (output row i <- x row rows[i]); else
 * output row i <- x row i.  h_out: dtype [n_out, width] (may be NULL when only the shifted form is wanted).
 *
 * Token shift (shift_w != NULL; rows must be NULL): hs = h + (h_prev - h) * shift_w, h_prev = the h of the token before
 * in the same sequence: the previous row of the batch, or — for the first token of a sequence's portion — the row that
 * the sequence's state slot holds (zeros at position 0).  The slot then receives the h of the portion's last token.
 * state: float, slot s at state + s * state_slot_stride (width floats).  tok_seq: int32 [n_tokens] sequence of each
 * token; q_cu: int32 [n_seq + 1]; positions: int32 [n_tokens]; slots: int32 [n_seq]. */
int hxm_stream_norm(const float* x, const float* in_w, const float* norm_w, int32_t groups, float eps,
                    const int32_t* rows, int64_t n_out, int32_t n_streams, int64_t width, void* h_out,
                    const float* shift_w, void* hs_out, float* state, int64_t state_slot_stride,
                    const int32_t* tok_seq, const int32_t* q_cu, const int32_t* positions, const int32_t* slots,
                    int dtype, void* stream);

/* A sublayer's result enters the streams: g = y * sigmoid(gate_pre + gate_b) (gate_pre == NULL: g = y), then for every
 * target stream t: x[., t, :] <- sum_s mix[s * n_streams + t] * x[., s, :] + out_w[t] * g, all targets from the old
 * values.  y: dtype [n_tokens, >= width] with row stride y_stride; gate_pre likewise; gate_b: float [width] or NULL. */
int hxm_stream_update(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                      const float* gate_b, const float* mix, const float* out_w, int64_t n_tokens, int32_t n_streams,
                      int64_t width, int dtype, void* stream);

/* hxm_stream_update followed by the read side of the NEXT sublayer (one without a token shift) in one launch: the streams
 * are updated in place and h_out [n_tokens, width] = grouped_rms_norm(sum_s in_next[s] * x_new[., s, :]) * norm_next. */
int hxm_stream_update_norm(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                           const float* gate_b, const float* mix, const float* out_w, const float* in_next,
                           const float* norm_next, int32_t groups, float eps, void* h_out, int64_t n_tokens,
                           int32_t n_streams, int64_t width, int dtype, void* stream);

/* out[., i] = gelu_tanh(gate[., i]) * up[., i], gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))). */
int hxm_gelu_tanh_and_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t n, int64_t gate_stride,
                          int64_t up_stride, int dtype, void* stream);

/* The two latents of a token from one projection row: cq = rms_norm(proj[., q_off : q_off + q_rank]) * q_w -> cq_out
 * [n_tokens, q_rank]; c = rms_norm(proj[., kv_off : kv_off + kv_rank]) * kv_w -> the paged cache at slot_ids[token]
 * (slot = block * block_size + row; slots < 0 are skipped).  cache: dtype, block b at cache + b * cache_block_stride, row r
 * of it cache_row_stride further.  Plain (one group) RMS norms with eps inside the root. */
int hxm_latent_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_rank, int64_t kv_off,
                          int64_t kv_rank, const float* q_w, const float* kv_w, float eps, void* cq_out,
                          const int32_t* slot_ids, void* cache, int64_t cache_block_stride, int64_t cache_row_stride,
                          int32_t block_size, int64_t n_tokens, int dtype, void* stream);

typedef struct hxm_latent_attn_args {
  void* out;                 /* dtype [n_tokens, n_heads, kv_rank] (strides below): sum_j p_j c_j, times the head gate */
  const void* q;             /* dtype [n_tokens, n_heads, kv_rank]: the queries already carried into the latent space */
  const void* cache;         /* dtype paged latents */
  const void* gate_pre;      /* dtype, optional: out is multiplied by sigmoid(gate_pre[t * gate_stride + head]) */
  const int32_t* tok_seq;    /* [n_tokens] */
  const int32_t* positions;  /* [n_tokens] position of each query in its sequence (= its own key's index) */
  const int32_t* q_cu;       /* [n_seq + 1] */
  const int32_t* block_table;/* flat */
  const int32_t* cu_block_lens; /* [n_seq + 1] */
  int64_t q_token_stride, q_head_stride, out_token_stride, out_head_stride, gate_stride;
  int64_t cache_block_stride, cache_row_stride;
  int32_t n_tokens, n_seq, n_heads, kv_rank, block_size;
  int32_t window;            /* a query at position i sees keys j with 0 <= i - j < window; <= 0: every j <= i */
  int32_t max_q_len;         /* the longest portion of the batch (1: every sequence decodes) */
  float scale;
  int32_t dtype;
  int32_t max_kv_len;        /* the most keys a sequence of the batch holds (sizes the key splits) */
  int32_t n_splits;          /* from hxm_latent_attention_plan; > 1: the key range of a row tile is dealt to n_splits waves */
  float* ws_o;               /* n_splits > 1: the plan's workspace, ws_floats floats; ws_ml = where its (max, sum) pairs go */
  float* ws_ml;
} hxm_latent_attn_args;

/* How a launch with these arguments would be laid out: n_splits (1: no workspace) and the floats of workspace it needs
 * (ws_o = the first n_items * n_splits * 16 * ceil16(kv_rank) of them, ws_ml = the rest).  Pointers need not be set yet,
 * except q and cache (their alignment decides the form). */
int hxm_latent_attention_plan(const hxm_latent_attn_args* args, int32_t* n_splits, int64_t* ws_floats);

/* Softmax attention of every query over the latents of its own sequence in the paged cache (scores and weights in
 * float).  Queries of portions and single decoded tokens may share a batch. */
int hxm_latent_attention(const hxm_latent_attn_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif
