// stream_ops.hip — multi-stream residuals (hyper-connections): embedding into the streams, the read side (weighted sum
// of the streams + grouped RMS norm + token shift with its per-sequence state) and the write side (gated sublayer
// result mixed back into every stream), and the tanh-GELU gate of the feed-forward.  Row kernels: one 256-thread
// workgroup per token, the row staged in LDS, everything in float; only what a matrix product reads or writes has the
// activation dtype.
#include "hx_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error() {
  static thread_local int e = 0;
  return e;
}
int check_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_hip_error() = (int)e;
    return HX_ERR_HIP;
  }
  return HX_OK;
}
int& tile_form() {
  static int v = 1;
  return v;
}
}  // namespace hxm

namespace {

using namespace hx;

template <typename A>
__global__ __launch_bounds__(256) void stream_embed_kernel(float* __restrict__ x, const typename A::storage* __restrict__ table,
                                                           const void* __restrict__ ids, int ids64, float scale, int32_t S,
                                                           int64_t W, int64_t vocab) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids64 ? ((const int64_t*)ids)[t] : (int64_t)((const int32_t*)ids)[t];
  const bool ok = id >= 0 && id < vocab;
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    const float v = ok ? A::to_float(table[id * W + i]) * scale : 0.f;
    for (int s = 0; s < S; ++s) x[(t * S + s) * W + i] = v;
  }
}

// buf[0 .. W) <- grouped RMS norm of sum_s in_w[s] * x[row, s, :], times norm_w.  Every thread of the workgroup calls it;
// it ends with a barrier.  A group is normalised by one wave (groups are dealt to the four waves in turn).
__device__ __forceinline__ void norm_row(float* buf, const float* __restrict__ x, int64_t row, const float* __restrict__ in_w,
                                         const float* __restrict__ norm_w, int32_t S, int64_t W, int32_t groups, float eps) {
  const float* xr = x + row * S * W;
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += in_w[s] * xr[s * W + i];
    buf[i] = u;
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t gs = W / groups;
  for (int g = wave; g < groups; g += 4) {
    float ss = 0.f;
    for (int64_t i = lane; i < gs; i += 64) {
      const float v = buf[g * gs + i];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int64_t i = lane; i < gs; i += 64) buf[g * gs + i] = buf[g * gs + i] * inv * norm_w[g * gs + i];
  }
  __syncthreads();
}

template <typename A>
__global__ __launch_bounds__(256) void stream_norm_kernel(const float* __restrict__ x, const float* __restrict__ in_w,
                                                          const float* __restrict__ norm_w, int32_t groups, float eps,
                                                          const int32_t* __restrict__ rows, int32_t S, int64_t W,
                                                          typename A::storage* __restrict__ h_out,
                                                          const float* __restrict__ shift_w,
                                                          typename A::storage* __restrict__ hs_out, float* __restrict__ state,
                                                          int64_t state_slot_stride, const int32_t* __restrict__ tok_seq,
                                                          const int32_t* __restrict__ q_cu, const int32_t* __restrict__ positions,
                                                          const int32_t* __restrict__ slots) {
  extern __shared__ float lds[];
  float* cur = lds;
  float* other = lds + W;
  const int64_t o = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[o] : o;
  norm_row(cur, x, t, in_w, norm_w, S, W, groups, eps);
  if (h_out)
    for (int64_t i = threadIdx.x; i < W; i += 256) h_out[o * W + i] = A::from_float(cur[i]);
  if (!shift_w) return;
  const int32_t b = tok_seq[t];
  const int32_t first = q_cu[b], last = q_cu[b + 1] - 1;
  if (t == first) {
    // the row before this one is the sequence's state; this workgroup alone touches the slot in this launch: it reads
    // the old row and then leaves the h of the portion's last token there
    float* st = state + (int64_t)slots[b] * state_slot_stride;
    const bool has_prev = positions[t] > 0;
    const float* nxt = cur;
    if (last != first) {
      norm_row(other, x, last, in_w, norm_w, S, W, groups, eps);
      nxt = other;
    }
    for (int64_t i = threadIdx.x; i < W; i += 256) {
      const float prev = has_prev ? st[i] : 0.f;
      const float h = cur[i];
      hs_out[t * W + i] = A::from_float(h + (prev - h) * shift_w[i]);
      st[i] = nxt[i];
    }
  } else {
    norm_row(other, x, t - 1, in_w, norm_w, S, W, groups, eps);
    for (int64_t i = threadIdx.x; i < W; i += 256) {
      const float h = cur[i];
      hs_out[t * W + i] = A::from_float(h + (other[i] - h) * shift_w[i]);
    }
  }
}

template <typename A, int MS>      // MS: 4 / 8 / 16 >= the number of streams (the loops are unrolled)
__global__ __launch_bounds__(256) void stream_update_kernel(float* __restrict__ x, const typename A::storage* __restrict__ y,
                                                            int64_t y_stride, const typename A::storage* __restrict__ gate_pre,
                                                            int64_t gate_stride, const float* __restrict__ gate_b,
                                                            const float* __restrict__ mix, const float* __restrict__ out_w,
                                                            int32_t S, int64_t W) {
  __shared__ float m[MS * MS + MS];
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) m[MS * MS + threadIdx.x] = out_w[threadIdx.x];
  __syncthreads();
  const float* ow = m + MS * MS;
  const int64_t t = blockIdx.x;
  float* xr = x + t * S * W;
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    float g = A::to_float(y[t * y_stride + i]);
    if (gate_pre) {
      const float z = A::to_float(gate_pre[t * gate_stride + i]) + (gate_b ? gate_b[i] : 0.f);
      g = g / (1.0f + expf(-z));
    }
    float old[MS];
#pragma unroll
    for (int s = 0; s < MS; ++s) old[s] = s < S ? xr[s * W + i] : 0.f;
#pragma unroll
    for (int d = 0; d < MS; ++d) {
      if (d < S) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < MS; ++s)
          if (s < S) acc += m[s * S + d] * old[s];
        xr[d * W + i] = acc + ow[d] * g;
      }
    }
  }
}

template <typename A>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_kernel(typename A::storage* __restrict__ out,
                                                                const typename A::storage* __restrict__ gate,
                                                                const typename A::storage* __restrict__ up, int64_t n,
                                                                int64_t gate_stride, int64_t up_stride) {
  const int64_t r = blockIdx.x;
  const int64_t i = (int64_t)blockIdx.y * 256 + threadIdx.x;
  if (i >= n) return;
  const float z = A::to_float(gate[r * gate_stride + i]);
  const float u = A::to_float(up[r * up_stride + i]);
  const float a = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  out[r * n + i] = A::from_float(round_to<A>(a) * u);
}

template <typename A>
int launch_embed(float* x, const void* table, const void* ids, int ids64, float scale, int64_t n, int32_t S, int64_t W,
                 int64_t vocab, hipStream_t s) {
  stream_embed_kernel<A><<<dim3((unsigned)n), dim3(256), 0, s>>>(x, (const typename A::storage*)table, ids, ids64, scale, S, W, vocab);
  return hxm::check_launch();
}

}  // namespace

extern "C" int hxm_abi_version(void) { return HXM_ABI_VERSION; }
extern "C" int hxm_last_hip_error(void) { return hxm::last_hip_error(); }
extern "C" int hxm_set_option(const char* name, int value) {
  if (name && __builtin_strcmp(name, "attn_tile_form") == 0) {
    hxm::tile_form() = value ? 1 : 0;
    return HX_OK;
  }
  return HX_ERR_UNSUPPORTED;
}

extern "C" int hxm_stream_embed(float* x, const void* table, const void* ids, int ids_are_int64, float scale,
                                int64_t n_tokens, int32_t n_streams, int64_t width, int64_t vocab, int dtype, void* stream) {
  if (n_tokens < 0 || n_streams < 1 || width < 1 || vocab < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!x || !table || !ids) return HX_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case HX_F32: return launch_embed<F32>(x, table, ids, ids_are_int64, scale, n_tokens, n_streams, width, vocab, s);
    case HX_BF16: return launch_embed<BF16>(x, table, ids, ids_are_int64, scale, n_tokens, n_streams, width, vocab, s);
    default: return HX_ERR_DTYPE;
  }
}

extern "C" int hxm_stream_norm(const float* x, const float* in_w, const float* norm_w, int32_t groups, float eps,
                               const int32_t* rows, int64_t n_out, int32_t n_streams, int64_t width, void* h_out,
                               const float* shift_w, void* hs_out, float* state, int64_t state_slot_stride,
                               const int32_t* tok_seq, const int32_t* q_cu, const int32_t* positions, const int32_t* slots,
                               int dtype, void* stream) {
  if (n_out < 0 || n_streams < 1 || n_streams > HXM_MAX_STREAMS || width < 1 || groups < 1 || width % groups) return HX_ERR_SHAPE;
  if (n_out == 0) return HX_OK;
  if (!x || !in_w || !norm_w) return HX_ERR_NULL;
  if (shift_w && (!hs_out || !state || !tok_seq || !q_cu || !positions || !slots)) return HX_ERR_NULL;
  if (shift_w && rows) return HX_ERR_UNSUPPORTED;
  if (!shift_w && !h_out) return HX_ERR_NULL;
  const size_t lds = (size_t)width * 2 * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case HX_F32:
      stream_norm_kernel<F32><<<dim3((unsigned)n_out), dim3(256), lds, s>>>(
          x, in_w, norm_w, groups, eps, rows, n_streams, width, (float*)h_out, shift_w, (float*)hs_out, state,
          state_slot_stride, tok_seq, q_cu, positions, slots);
      break;
    case HX_BF16:
      stream_norm_kernel<BF16><<<dim3((unsigned)n_out), dim3(256), lds, s>>>(
          x, in_w, norm_w, groups, eps, rows, n_streams, width, (u16*)h_out, shift_w, (u16*)hs_out, state,
          state_slot_stride, tok_seq, q_cu, positions, slots);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_stream_update(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                                 const float* gate_b, const float* mix, const float* out_w, int64_t n_tokens,
                                 int32_t n_streams, int64_t width, int dtype, void* stream) {
  if (n_tokens < 0 || n_streams < 1 || n_streams > HXM_MAX_STREAMS || width < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!x || !y || !mix || !out_w) return HX_ERR_NULL;
  if (y_stride < width || (gate_pre && gate_stride < width)) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), block(256);
#define HXM_UPDATE(A_, T_, MS_) stream_update_kernel<A_, MS_><<<grid, block, 0, s>>>( \
      x, (const T_*)y, y_stride, (const T_*)gate_pre, gate_stride, gate_b, mix, out_w, n_streams, width)
#define HXM_UPDATE_MS(A_, T_) do { if (n_streams <= 4) HXM_UPDATE(A_, T_, 4); else if (n_streams <= 8) HXM_UPDATE(A_, T_, 8); \
      else HXM_UPDATE(A_, T_, 16); } while (0)
  switch (dtype) {
    case HX_F32: HXM_UPDATE_MS(F32, float); break;
    case HX_BF16: HXM_UPDATE_MS(BF16, u16); break;
    default: return HX_ERR_DTYPE;
  }
#undef HXM_UPDATE_MS
#undef HXM_UPDATE
  return hxm::check_launch();
}

extern "C" int hxm_gelu_tanh_and_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t n,
                                     int64_t gate_stride, int64_t up_stride, int dtype, void* stream) {
  if (rows < 0 || n < 0) return HX_ERR_SHAPE;
  if (rows == 0 || n == 0) return HX_OK;
  if (!out || !gate || !up) return HX_ERR_NULL;
  if (gate_stride < n || up_stride < n) return HX_ERR_STRIDE;
  if ((n + 255) / 256 > 65535) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)rows, (unsigned)((n + 255) / 256));
  switch (dtype) {
    case HX_F32:
      gelu_tanh_and_mul_kernel<F32><<<grid, dim3(256), 0, s>>>((float*)out, (const float*)gate, (const float*)up, n, gate_stride, up_stride);
      break;
    case HX_BF16:
      gelu_tanh_and_mul_kernel<BF16><<<grid, dim3(256), 0, s>>>((u16*)out, (const u16*)gate, (const u16*)up, n, gate_stride, up_stride);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
