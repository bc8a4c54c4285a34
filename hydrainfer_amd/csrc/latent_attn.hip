// latent_attn.hip — attention over a paged cache of low-rank latents.  A token leaves ONE row c (kv_rank numbers) in the
// cache; every head's key and value are linear maps of it, so with the key map folded into the query (q~ = W_uk^T q) and
// the value map applied afterwards (o = W_uv sum_j p_j c_j) the kernel is multi-query attention whose keys and values
// are the same rows: score = q~ . c_j * scale, out = sum_j softmax(score)_j c_j.  Scores, weights and sums are float.
// Sliding window: a query at position i sees keys j with 0 <= i - j < window.
#include "hx_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int check_launch();
}

namespace {

using namespace hx;

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// one workgroup per token: both latents of the token from its projection row
template <typename A>
__global__ __launch_bounds__(256) void latent_norm_cache_kernel(const typename A::storage* __restrict__ proj, int64_t proj_stride,
                                                                int64_t q_off, int64_t q_rank, int64_t kv_off, int64_t kv_rank,
                                                                const float* __restrict__ q_w, const float* __restrict__ kv_w, float eps,
                                                                typename A::storage* __restrict__ cq_out,
                                                                const int32_t* __restrict__ slot_ids,
                                                                typename A::storage* __restrict__ cache, int64_t cache_block_stride,
                                                                int64_t cache_row_stride, int32_t block_size) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const typename A::storage* p = proj + t * proj_stride;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < q_rank; i += 256) {
    const float v = A::to_float(p[q_off + i]);
    ss += v * v;
  }
  float inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)q_rank + eps);
  for (int64_t i = threadIdx.x; i < q_rank; i += 256)
    cq_out[t * q_rank + i] = A::from_float(A::to_float(p[q_off + i]) * inv * q_w[i]);
  const int32_t slot = slot_ids[t];
  if (slot < 0) return;
  ss = 0.f;
  for (int64_t i = threadIdx.x; i < kv_rank; i += 256) {
    const float v = A::to_float(p[kv_off + i]);
    ss += v * v;
  }
  inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)kv_rank + eps);
  typename A::storage* dst = cache + (int64_t)(slot / block_size) * cache_block_stride + (int64_t)(slot % block_size) * cache_row_stride;
  for (int64_t i = threadIdx.x; i < kv_rank; i += 256) dst[i] = A::from_float(A::to_float(p[kv_off + i]) * inv * kv_w[i]);
}

// ---------------------------------------------------------------------------------------------------------------
// Row form: one wave per (token, head).  Keys go by in groups of 64: lane l scores key lo + l (its own row of the
// cache against the query in LDS), the group's maximum and sum are wave reductions, then the lanes turn to the latent's
// columns (lane l owns columns l, l + 64, ...) and add the 64 rows, each weighted by its lane's p.  Serves decode steps
// and short portions; long portions take the tiled form below.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxCols = HXM_MAX_LATENT / 64;

template <typename A>
__global__ __launch_bounds__(256) void latent_attn_rows_kernel(hxm_latent_attn_args a) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t total = (int64_t)a.n_tokens * a.n_heads;
  const bool live = (int64_t)blockIdx.x * 4 + wave < total;
  const int64_t item = live ? (int64_t)blockIdx.x * 4 + wave : total - 1;      // (a spare wave repeats the last row and stores nothing)
  const int32_t t = (int32_t)(item / a.n_heads), h = (int32_t)(item % a.n_heads);
  const int32_t R = a.kv_rank;
  float* q = lds + wave * R;
  const typename A::storage* qg = (const typename A::storage*)a.q + (int64_t)t * a.q_token_stride + (int64_t)h * a.q_head_stride;
  for (int i = lane; i < R; i += 64) q[i] = A::to_float(qg[i]) * a.scale;
  __syncthreads();
  const int32_t b = a.tok_seq[t];
  const int32_t pos = a.positions[t];
  const int32_t lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int32_t* table = a.block_table + a.cu_block_lens[b];
  const typename A::storage* cache = (const typename A::storage*)a.cache;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxCols];
#pragma unroll
  for (int k = 0; k < kMaxCols; ++k) acc[k] = 0.f;
  for (int32_t j0 = lo; j0 <= pos; j0 += 64) {
    const int32_t j = j0 + lane;
    const bool valid = j <= pos;
    int64_t off = 0;
    float s = -INFINITY;
    if (valid) {
      off = (int64_t)table[j / a.block_size] * a.cache_block_stride + (int64_t)(j % a.block_size) * a.cache_row_stride;
      const typename A::storage* c = cache + off;
      float d = 0.f;
      for (int i = 0; i < R; ++i) d += q[i] * A::to_float(c[i]);
      s = d;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);      // (m = -inf on the first group: 0)
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int k = 0; k < kMaxCols; ++k) acc[k] *= corr;
    const int n = min(64, pos - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int64_t oj = __shfl(off, jj, 64);
      const typename A::storage* c = cache + oj;
#pragma unroll
      for (int k = 0; k < kMaxCols; ++k) {
        const int i = lane + 64 * k;
        if (i < R) acc[k] += pj * A::to_float(c[i]);
      }
    }
  }
  float g = 1.0f / l;
  if (a.gate_pre) {
    const float z = A::to_float(((const typename A::storage*)a.gate_pre)[(int64_t)t * a.gate_stride + h]);
    g = g / (1.0f + expf(-z));
  }
  typename A::storage* og = (typename A::storage*)a.out + (int64_t)t * a.out_token_stride + (int64_t)h * a.out_head_stride;
#pragma unroll
  for (int k = 0; k < kMaxCols; ++k) {
    const int i = lane + 64 * k;
    if (i < R && live) og[i] = A::from_float(acc[k] * g);
  }
}

}  // namespace

extern "C" int hxm_latent_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_rank, int64_t kv_off,
                                     int64_t kv_rank, const float* q_w, const float* kv_w, float eps, void* cq_out,
                                     const int32_t* slot_ids, void* cache, int64_t cache_block_stride,
                                     int64_t cache_row_stride, int32_t block_size, int64_t n_tokens, int dtype, void* stream) {
  if (n_tokens < 0 || q_rank < 1 || kv_rank < 1 || block_size < 1 || q_off < 0 || kv_off < 0) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!proj || !q_w || !kv_w || !cq_out || !slot_ids || !cache) return HX_ERR_NULL;
  if (proj_stride < q_off + q_rank || proj_stride < kv_off + kv_rank || cache_row_stride < kv_rank) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case HX_F32:
      latent_norm_cache_kernel<F32><<<dim3((unsigned)n_tokens), dim3(256), 0, s>>>(
          (const float*)proj, proj_stride, q_off, q_rank, kv_off, kv_rank, q_w, kv_w, eps, (float*)cq_out, slot_ids,
          (float*)cache, cache_block_stride, cache_row_stride, block_size);
      break;
    case HX_BF16:
      latent_norm_cache_kernel<BF16><<<dim3((unsigned)n_tokens), dim3(256), 0, s>>>(
          (const u16*)proj, proj_stride, q_off, q_rank, kv_off, kv_rank, q_w, kv_w, eps, (u16*)cq_out, slot_ids,
          (u16*)cache, cache_block_stride, cache_row_stride, block_size);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_latent_attention(const hxm_latent_attn_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_latent_attn_args& a = *args;
  if (a.n_tokens < 0 || a.n_seq < 1 || a.n_heads < 1 || a.kv_rank < 1 || a.kv_rank > HXM_MAX_LATENT || a.block_size < 1)
    return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.out || !a.q || !a.cache || !a.tok_seq || !a.positions || !a.q_cu || !a.block_table || !a.cu_block_lens) return HX_ERR_NULL;
  if (a.cache_row_stride < a.kv_rank) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t items = (int64_t)a.n_tokens * a.n_heads;
  const dim3 grid((unsigned)((items + 3) / 4));
  const size_t lds = (size_t)4 * a.kv_rank * sizeof(float);
  switch (a.dtype) {
    case HX_F32: latent_attn_rows_kernel<F32><<<grid, dim3(256), lds, s>>>(a); break;
    case HX_BF16: latent_attn_rows_kernel<BF16><<<grid, dim3(256), lds, s>>>(a); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
