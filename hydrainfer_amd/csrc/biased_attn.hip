// biased_attn.hip — grouped-query attention over a paged key/value cache whose scores carry a linear distance bias,
// score(i, j) = q_i . k_j * scale - slope_h (i - j), under a causal, sliding-window or chunked mask (chunks counted from
// position 0 of the sequence).  Key and value rows may differ in size.  Scores, weights and sums are float.  Also the
// kernel in front of it: one RMS norm over a token's whole query projection and one over its whole key projection
// (all heads at once), keys and values straight into the cache.
#include <cfloat>
#include "hx_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

__device__ __forceinline__ float block_sum4(float v, float* part) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  return part[0] + part[1] + part[2] + part[3];
}

// one workgroup per token
template <typename A>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(const typename A::storage* __restrict__ proj, int64_t proj_stride,
                                                            int64_t q_off, int64_t q_size, int64_t k_off, int64_t k_size,
                                                            int64_t v_off, int64_t v_size, const float* __restrict__ q_w,
                                                            const float* __restrict__ k_w, float eps,
                                                            typename A::storage* __restrict__ q_out,
                                                            const int32_t* __restrict__ slot_ids,
                                                            typename A::storage* __restrict__ key_cache,
                                                            typename A::storage* __restrict__ value_cache,
                                                            int64_t cache_row_stride, int64_t head_stride, int kv_heads) {
  __shared__ float part[4];
  const int64_t t = blockIdx.x;
  const typename A::storage* row = proj + t * proj_stride;
  {
    float inv = 1.f;
    if (q_w) {
      float ss = 0.f;
      for (int64_t i = threadIdx.x; i < q_size; i += 256) {
        const float v = A::to_float(row[q_off + i]);
        ss += v * v;
      }
      inv = 1.0f / sqrtf(block_sum4(ss, part) / (float)q_size + eps);
    }
    for (int64_t i = threadIdx.x; i < q_size; i += 256) {
      const float v = A::to_float(row[q_off + i]);
      q_out[t * q_size + i] = q_w ? A::from_float(v * inv * q_w[i]) : row[q_off + i];
    }
  }
  if (k_size <= 0) return;
  const int64_t slot = slot_ids[t];
  float inv = 1.f;
  if (k_w) {
    float ss = 0.f;
    for (int64_t i = threadIdx.x; i < k_size; i += 256) {
      const float v = A::to_float(row[k_off + i]);
      ss += v * v;
    }
    inv = 1.0f / sqrtf(block_sum4(ss, part) / (float)k_size + eps);
  }
  if (slot < 0) return;
  const int64_t kd = k_size / kv_heads, vd = v_size / kv_heads;
  for (int64_t i = threadIdx.x; i < k_size; i += 256) {
    const float v = A::to_float(row[k_off + i]);
    key_cache[slot * cache_row_stride + (i / kd) * head_stride + i % kd] = k_w ? A::from_float(v * inv * k_w[i]) : row[k_off + i];
  }
  for (int64_t i = threadIdx.x; i < v_size; i += 256)
    value_cache[slot * cache_row_stride + (i / vd) * head_stride + i % vd] = row[v_off + i];
}

// the wave's LDS writes so far are visible to all its lanes
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// the first key a query at position i sees
__device__ __forceinline__ int first_visible(int i, int kind, int size) {
  if (kind == HXM_MASK_WINDOW) return i - size + 1 > 0 ? i - size + 1 : 0;
  if (kind == HXM_MASK_CHUNK) return i / size * size;
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Row form: one wave per (token, head), four a workgroup, no barriers.  Keys go by in groups of 64: lane l scores key
// lo + l (its row of the cache against the query in LDS), the group's maximum and sum are wave reductions, then the lanes
// turn to the value's columns (lane l owns columns l, l + 64, ...) and add the 64 rows, each weighted by its lane's p.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxVCols = 8;      // value columns per lane: vdim <= 512
template <typename A>
__global__ __launch_bounds__(256) void biased_attn_rows_kernel(hxm_biased_attn_args a) {
  extern __shared__ float lds[];
  typedef typename A::storage T;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= (int64_t)a.n_tokens * a.n_heads) return;
  const int t = (int)(item / a.n_heads), h = (int)(item - (int64_t)t * a.n_heads);
  const int D = a.dim, V = a.vdim, BS = a.block_size;
  float* qs = lds + wave * (D + 64);       // the query, then the group's weights
  float* ps = qs + D;
  const T* q = (const T*)a.q + ((int64_t)t * a.n_heads + h) * D;
  for (int d = lane; d < D; d += 64) qs[d] = A::to_float(q[d]) * a.scale;
  wave_lds_sync();
  const int seq = a.tok_seq[t], i = a.positions[t];
  const int32_t* table = a.block_table + a.cu_block_lens[seq];
  const int g = h / (a.n_heads / a.kv_heads);
  const T* kc = (const T*)a.key_cache + (int64_t)g * a.head_stride;
  const T* vc = (const T*)a.value_cache + (int64_t)g * a.head_stride;
  const float slope = a.slopes ? a.slopes[h] : 0.f;
  const int lo = first_visible(i, a.mask_kind, a.mask_size);
  float m = -FLT_MAX, l = 0.f;
  float acc[kMaxVCols];
#pragma unroll
  for (int c = 0; c < kMaxVCols; ++c) acc[c] = 0.f;
  for (int j0 = lo; j0 <= i; j0 += 64) {
    const int j = j0 + lane;
    float s = -FLT_MAX;
    if (j <= i) {
      const T* kr = kc + (int64_t)table[j / BS] * a.cache_block_stride + (int64_t)(j % BS) * a.cache_row_stride;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * A::to_float(kr[d]);
      s = dot - slope * (float)(i - j);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = j <= i ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    wave_lds_sync();
    ps[lane] = p;
    wave_lds_sync();
#pragma unroll
    for (int c = 0; c < kMaxVCols; ++c) acc[c] *= corr;
    const int n = i - j0 + 1 < 64 ? i - j0 + 1 : 64;
    for (int jj = 0; jj < n; ++jj) {
      const int jk = j0 + jj;
      const T* vr = vc + (int64_t)table[jk / BS] * a.cache_block_stride + (int64_t)(jk % BS) * a.cache_row_stride;
      const float pj = ps[jj];
#pragma unroll
      for (int c = 0; c < kMaxVCols; ++c) {
        const int col = lane + 64 * c;
        if (col < V) acc[c] += pj * A::to_float(vr[col]);
      }
    }
  }
  T* o = (T*)a.out + ((int64_t)t * a.n_heads + h) * V;
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < kMaxVCols; ++c) {
    const int col = lane + 64 * c;
    if (col < V) o[col] = A::from_float(acc[c] * inv);
  }
}

}  // namespace

extern "C" int hxm_qk_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_size, int64_t k_off,
                                 int64_t k_size, int64_t v_off, int64_t v_size, const float* q_w, const float* k_w, float eps,
                                 void* q_out, const int32_t* slot_ids, void* key_cache, void* value_cache,
                                 int64_t cache_row_stride, int64_t head_stride, int32_t kv_heads, int64_t n_tokens, int dtype,
                                 void* stream) {
  if (n_tokens < 0 || q_size < 1 || k_size < 0 || v_size < 0 || kv_heads < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!proj || !q_out) return HX_ERR_NULL;
  if (k_size > 0) {
    if (!slot_ids || !key_cache || !value_cache) return HX_ERR_NULL;
    if (k_size % kv_heads || v_size % kv_heads || v_size < 1) return HX_ERR_SHAPE;
    if (k_size / kv_heads > head_stride || v_size / kv_heads > head_stride || cache_row_stride < head_stride * kv_heads) return HX_ERR_STRIDE;
  }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), block(256);
  switch (dtype) {
    case HX_F32:
      qk_norm_cache_kernel<F32><<<grid, block, 0, s>>>((const float*)proj, proj_stride, q_off, q_size, k_off, k_size, v_off, v_size,
                                                       q_w, k_w, eps, (float*)q_out, slot_ids, (float*)key_cache, (float*)value_cache,
                                                       cache_row_stride, head_stride, kv_heads);
      break;
    case HX_BF16:
      qk_norm_cache_kernel<BF16><<<grid, block, 0, s>>>((const u16*)proj, proj_stride, q_off, q_size, k_off, k_size, v_off, v_size,
                                                        q_w, k_w, eps, (u16*)q_out, slot_ids, (u16*)key_cache, (u16*)value_cache,
                                                        cache_row_stride, head_stride, kv_heads);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_biased_attention(const hxm_biased_attn_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_biased_attn_args& a = *args;
  if (a.n_tokens < 0 || a.n_heads < 1 || a.kv_heads < 1 || a.n_heads % a.kv_heads || a.dim < 1 || a.vdim < 1 ||
      a.vdim > 64 * kMaxVCols || a.block_size < 1)
    return HX_ERR_SHAPE;
  if (a.mask_kind < HXM_MASK_CAUSAL || a.mask_kind > HXM_MASK_CHUNK || (a.mask_kind != HXM_MASK_CAUSAL && a.mask_size < 1)) return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.out || !a.q || !a.key_cache || !a.value_cache || !a.tok_seq || !a.positions || !a.block_table || !a.cu_block_lens) return HX_ERR_NULL;
  if (a.dim > a.head_stride || a.vdim > a.head_stride) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t items = (int64_t)a.n_tokens * a.n_heads;
  const size_t lds = 4 * ((size_t)a.dim + 64) * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  const dim3 grid((unsigned)((items + 3) / 4)), block(256);
  switch (a.dtype) {
    case HX_F32: biased_attn_rows_kernel<F32><<<grid, block, lds, s>>>(a); break;
    case HX_BF16: biased_attn_rows_kernel<BF16><<<grid, block, lds, s>>>(a); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
