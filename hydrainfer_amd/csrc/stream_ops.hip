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

// four consecutive elements of an activation row <-> four floats
template <typename A> struct Vec4;
template <> struct Vec4<F32> {
  static __device__ __forceinline__ f32x4 load(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
  static __device__ __forceinline__ void store(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
};
template <> struct Vec4<BF16> {
  static __device__ __forceinline__ f32x4 load(const u16* p) {
    const u16x4 b = *reinterpret_cast<const u16x4*>(p);
    return f32x4{BF16::to_float(b[0]), BF16::to_float(b[1]), BF16::to_float(b[2]), BF16::to_float(b[3])};
  }
  static __device__ __forceinline__ void store(u16* p, f32x4 v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{BF16::from_float(v[0]), BF16::from_float(v[1]), BF16::from_float(v[2]), BF16::from_float(v[3])};
  }
};

constexpr int kMaxFastGroups = 64;

// buf[0 .. W) (complete, visible to the workgroup) <- its grouped RMS norm times norm_w; ends with a barrier.
// Fast form (rows of float4s, groups of a multiple of 256 elements): every thread squares and scales the elements it owns
// (float4 i4 = tid + 256 k), a wave's 256 consecutive elements lie in one group, so one shuffle reduction per round and
// a per-wave partial sum per group in `part` [4][64] (summed in a fixed order: no atomics).  General form: a group is
// normalised by one wave, groups dealt to the four waves in turn.
__device__ __forceinline__ void group_normalize(float* buf, float* part, const float* __restrict__ norm_w, int64_t W, int32_t groups,
                                                float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t gs = W / groups;
  if ((W & 3) == 0 && gs % 256 == 0 && groups <= kMaxFastGroups) {
    if (lane < groups) part[wave * kMaxFastGroups + lane] = 0.f;
    __syncthreads();
    const int64_t n4 = W >> 2;
    f32x4* b4 = reinterpret_cast<f32x4*>(buf);
    for (int64_t base = 0; base < n4; base += 256) {
      const int64_t i4 = base + threadIdx.x;
      float ss = 0.f;
      if (i4 < n4) {
        const f32x4 v = b4[i4];
        ss = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
      }
      ss = wave_sum(ss);
      const int64_t first = (base + 64 * wave) * 4;      // the wave's first element of this round
      if (lane == 0 && first < W) part[wave * kMaxFastGroups + first / gs] += ss;
    }
    __syncthreads();
    const f32x4* w4 = reinterpret_cast<const f32x4*>(norm_w);
    for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) {
      const int g = (int)(i4 * 4 / gs);
      const float tot = part[g] + part[kMaxFastGroups + g] + part[2 * kMaxFastGroups + g] + part[3 * kMaxFastGroups + g];
      const float inv = 1.0f / sqrtf(tot / (float)gs + eps);
      const f32x4 v = b4[i4], w = w4[i4];
      b4[i4] = f32x4{v[0] * inv * w[0], v[1] * inv * w[1], v[2] * inv * w[2], v[3] * inv * w[3]};
    }
    __syncthreads();
    return;
  }
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

// buf[0 .. W) <- grouped RMS norm of sum_s in_w[s] * x[row, s, :], times norm_w.  Every thread of the workgroup calls it;
// it ends with a barrier.
__device__ __forceinline__ void norm_row(float* buf, float* part, const float* __restrict__ x, int64_t row,
                                         const float* __restrict__ in_w, const float* __restrict__ norm_w, int32_t S, int64_t W,
                                         int32_t groups, float eps) {
  const float* xr = x + row * S * W;
  if ((W & 3) == 0) {
    const f32x4* x4 = reinterpret_cast<const f32x4*>(xr);
    const int64_t n4 = W >> 2;
    for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) {
      f32x4 u = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int s = 0; s < S; ++s) {
        const f32x4 v = x4[s * n4 + i4];
        const float w = in_w[s];
        u[0] += w * v[0]; u[1] += w * v[1]; u[2] += w * v[2]; u[3] += w * v[3];
      }
      reinterpret_cast<f32x4*>(buf)[i4] = u;
    }
  } else {
    for (int64_t i = threadIdx.x; i < W; i += 256) {
      float u = 0.f;
      for (int s = 0; s < S; ++s) u += in_w[s] * xr[s * W + i];
      buf[i] = u;
    }
  }
  __syncthreads();
  group_normalize(buf, part, norm_w, W, groups, eps);
}

// A workgroup takes `run` consecutive rows: the h of a row stays in LDS as the next row's h_prev, so only the first row
// of a run (when it is not the first of its sequence's portion) has to work out the row before it a second time.
template <typename A>
__global__ __launch_bounds__(256) void stream_norm_kernel(const float* __restrict__ x, const float* __restrict__ in_w,
                                                          const float* __restrict__ norm_w, int32_t groups, float eps,
                                                          const int32_t* __restrict__ rows, int32_t S, int64_t W,
                                                          typename A::storage* __restrict__ h_out,
                                                          const float* __restrict__ shift_w,
                                                          typename A::storage* __restrict__ hs_out, float* __restrict__ state,
                                                          int64_t state_slot_stride, const int32_t* __restrict__ tok_seq,
                                                          const int32_t* __restrict__ q_cu, const int32_t* __restrict__ positions,
                                                          const int32_t* __restrict__ slots, int64_t n_out, int32_t run) {
  extern __shared__ float lds[];
  __shared__ float part[4 * kMaxFastGroups];
  const bool vec = (W & 3) == 0;
  const int64_t n4 = W >> 2;
  const int64_t o0 = (int64_t)blockIdx.x * run;
  for (int j = 0; j < run && o0 + j < n_out; ++j) {
    const int64_t o = o0 + j;
    const int64_t t = rows ? (int64_t)rows[o] : o;
    float* cur = lds + (j & 1) * W;
    float* other = lds + ((j & 1) ^ 1) * W;      // holds the h of row t - 1 when j > 0
    norm_row(cur, part, x, t, in_w, norm_w, S, W, groups, eps);
    if (h_out) {
      if (vec)
        for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) Vec4<A>::store(h_out + o * W + 4 * i4, reinterpret_cast<f32x4*>(cur)[i4]);
      else
        for (int64_t i = threadIdx.x; i < W; i += 256) h_out[o * W + i] = A::from_float(cur[i]);
    }
    if (!shift_w) continue;
    const int32_t b = tok_seq[t];
    const int32_t first = q_cu[b], last = q_cu[b + 1] - 1;
    // the row before this one: the previous row of the batch, or — for the first token of the sequence's portion — the
    // sequence's state row (zeros at position 0).  The first token's workgroup alone touches the slot in this launch:
    // it reads the old row and then leaves the h of the portion's last token there.
    const bool is_first = t == first;
    float* st = is_first ? state + (int64_t)slots[b] * state_slot_stride : nullptr;
    const bool has_prev = !is_first || positions[t] > 0;
    const float* nxt = cur;
    if (is_first && last != first) {
      norm_row(other, part, x, last, in_w, norm_w, S, W, groups, eps);
      nxt = other;
    } else if (!is_first && j == 0) {
      norm_row(other, part, x, t - 1, in_w, norm_w, S, W, groups, eps);
    }
    const float* prev_row = is_first ? st : other;
    if (vec) {
      for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) {
        const f32x4 h = reinterpret_cast<const f32x4*>(cur)[i4], sw = reinterpret_cast<const f32x4*>(shift_w)[i4];
        const f32x4 pv = has_prev ? reinterpret_cast<const f32x4*>(prev_row)[i4] : f32x4{0.f, 0.f, 0.f, 0.f};
        Vec4<A>::store(hs_out + t * W + 4 * i4, f32x4{h[0] + (pv[0] - h[0]) * sw[0], h[1] + (pv[1] - h[1]) * sw[1],
                                                      h[2] + (pv[2] - h[2]) * sw[2], h[3] + (pv[3] - h[3]) * sw[3]});
        if (is_first) reinterpret_cast<f32x4*>(st)[i4] = reinterpret_cast<const f32x4*>(nxt)[i4];
      }
    } else {
      for (int64_t i = threadIdx.x; i < W; i += 256) {
        const float pv = has_prev ? prev_row[i] : 0.f;
        const float h = cur[i];
        hs_out[t * W + i] = A::from_float(h + (pv - h) * shift_w[i]);
        if (is_first) st[i] = nxt[i];
      }
    }
    __syncthreads();      // the rows in LDS are read to the end before the next row overwrites one of them
  }
}

// one element (or four) of the update: g = y * sigmoid(gate + bias); new_d = sum_s mix[s, d] old_s + out[d] g
template <int MS, int N>
__device__ __forceinline__ void mix_streams(float (&nw)[MS][N], const float (&old)[MS][N], const float (&g)[N], const float* m,
                                            const float* ow, int32_t S) {
#pragma unroll
  for (int d = 0; d < MS; ++d) {
    if (d < S) {
#pragma unroll
      for (int e = 0; e < N; ++e) nw[d][e] = ow[d] * g[e];
#pragma unroll
      for (int s = 0; s < MS; ++s)
        if (s < S) {
          const float w = m[s * S + d];
#pragma unroll
          for (int e = 0; e < N; ++e) nw[d][e] += w * old[s][e];
        }
    }
  }
}

__device__ __forceinline__ float sigmoid_gate(float y, float z) { return y / (1.0f + expf(-z)); }

template <typename A, int MS>      // MS: 4 / 8 / 16 >= the number of streams (the loops are unrolled)
__global__ __launch_bounds__(256) void stream_update_kernel(float* __restrict__ x, const typename A::storage* __restrict__ y,
                                                            int64_t y_stride, const typename A::storage* __restrict__ gate_pre,
                                                            int64_t gate_stride, const float* __restrict__ gate_b,
                                                            const float* __restrict__ mix, const float* __restrict__ out_w,
                                                            int32_t S, int64_t W, int vec) {
  __shared__ float m[MS * MS + MS];
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) m[MS * MS + threadIdx.x] = out_w[threadIdx.x];
  __syncthreads();
  const float* ow = m + MS * MS;
  const int64_t t = blockIdx.x;
  float* xr = x + t * S * W;
  if (vec) {
    const int64_t n4 = W >> 2;
    for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) {
      const f32x4 yv = Vec4<A>::load(y + t * y_stride + 4 * i4);
      float g[4] = {yv[0], yv[1], yv[2], yv[3]};
      if (gate_pre) {
        const f32x4 z = Vec4<A>::load(gate_pre + t * gate_stride + 4 * i4);
        const f32x4 bz = gate_b ? reinterpret_cast<const f32x4*>(gate_b)[i4] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) g[e] = sigmoid_gate(g[e], z[e] + bz[e]);
      }
      float old[MS][4], nw[MS][4];
#pragma unroll
      for (int s = 0; s < MS; ++s)
        if (s < S) {
          const f32x4 v = reinterpret_cast<const f32x4*>(xr + s * W)[i4];
          old[s][0] = v[0]; old[s][1] = v[1]; old[s][2] = v[2]; old[s][3] = v[3];
        }
      mix_streams<MS, 4>(nw, old, g, m, ow, S);
#pragma unroll
      for (int d = 0; d < MS; ++d)
        if (d < S) reinterpret_cast<f32x4*>(xr + d * W)[i4] = f32x4{nw[d][0], nw[d][1], nw[d][2], nw[d][3]};
    }
    return;
  }
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    float g[1] = {A::to_float(y[t * y_stride + i])};
    if (gate_pre) g[0] = sigmoid_gate(g[0], A::to_float(gate_pre[t * gate_stride + i]) + (gate_b ? gate_b[i] : 0.f));
    float old[MS][1], nw[MS][1];
#pragma unroll
    for (int s = 0; s < MS; ++s)
      if (s < S) old[s][0] = xr[s * W + i];
    mix_streams<MS, 1>(nw, old, g, m, ow, S);
#pragma unroll
    for (int d = 0; d < MS; ++d)
      if (d < S) xr[d * W + i] = nw[d][0];
  }
}

// stream_update followed by the NEXT sublayer's read side (no token shift) in one pass over the token's streams:
// the new streams are written back, u = sum_s in_next[s] * new_s is normalised in LDS and leaves as h_out.
template <typename A, int MS>
__global__ __launch_bounds__(256) void stream_update_norm_kernel(float* __restrict__ x, const typename A::storage* __restrict__ y,
                                                                 int64_t y_stride, const typename A::storage* __restrict__ gate_pre,
                                                                 int64_t gate_stride, const float* __restrict__ gate_b,
                                                                 const float* __restrict__ mix, const float* __restrict__ out_w,
                                                                 const float* __restrict__ in_next, const float* __restrict__ norm_next,
                                                                 int32_t groups, float eps, typename A::storage* __restrict__ h_out,
                                                                 int32_t S, int64_t W, int vec) {
  extern __shared__ float lds[];
  __shared__ float part[4 * kMaxFastGroups];
  __shared__ float m[MS * MS + 2 * MS];
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    m[MS * MS + threadIdx.x] = out_w[threadIdx.x];
    m[MS * MS + MS + threadIdx.x] = in_next[threadIdx.x];
  }
  __syncthreads();
  const float* ow = m + MS * MS;
  const float* iw = ow + MS;
  const int64_t t = blockIdx.x;
  float* xr = x + t * S * W;
  if (vec) {
    const int64_t n4 = W >> 2;
    for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) {
      const f32x4 yv = Vec4<A>::load(y + t * y_stride + 4 * i4);
      float g[4] = {yv[0], yv[1], yv[2], yv[3]};
      if (gate_pre) {
        const f32x4 z = Vec4<A>::load(gate_pre + t * gate_stride + 4 * i4);
        const f32x4 bz = gate_b ? reinterpret_cast<const f32x4*>(gate_b)[i4] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) g[e] = sigmoid_gate(g[e], z[e] + bz[e]);
      }
      float old[MS][4], nw[MS][4];
#pragma unroll
      for (int s = 0; s < MS; ++s)
        if (s < S) {
          const f32x4 v = reinterpret_cast<const f32x4*>(xr + s * W)[i4];
          old[s][0] = v[0]; old[s][1] = v[1]; old[s][2] = v[2]; old[s][3] = v[3];
        }
      mix_streams<MS, 4>(nw, old, g, m, ow, S);
      f32x4 u = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int d = 0; d < MS; ++d)
        if (d < S) {
          reinterpret_cast<f32x4*>(xr + d * W)[i4] = f32x4{nw[d][0], nw[d][1], nw[d][2], nw[d][3]};
#pragma unroll
          for (int e = 0; e < 4; ++e) u[e] += iw[d] * nw[d][e];
        }
      reinterpret_cast<f32x4*>(lds)[i4] = u;
    }
  } else {
    for (int64_t i = threadIdx.x; i < W; i += 256) {
      float g[1] = {A::to_float(y[t * y_stride + i])};
      if (gate_pre) g[0] = sigmoid_gate(g[0], A::to_float(gate_pre[t * gate_stride + i]) + (gate_b ? gate_b[i] : 0.f));
      float old[MS][1], nw[MS][1];
#pragma unroll
      for (int s = 0; s < MS; ++s)
        if (s < S) old[s][0] = xr[s * W + i];
      mix_streams<MS, 1>(nw, old, g, m, ow, S);
      float u = 0.f;
#pragma unroll
      for (int d = 0; d < MS; ++d)
        if (d < S) {
          xr[d * W + i] = nw[d][0];
          u += iw[d] * nw[d][0];
        }
      lds[i] = u;
    }
  }
  __syncthreads();
  group_normalize(lds, part, norm_next, W, groups, eps);
  if ((W & 3) == 0)
    for (int64_t i4 = threadIdx.x; i4 < (W >> 2); i4 += 256) Vec4<A>::store(h_out + t * W + 4 * i4, reinterpret_cast<f32x4*>(lds)[i4]);
  else
    for (int64_t i = threadIdx.x; i < W; i += 256) h_out[t * W + i] = A::from_float(lds[i]);
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename A>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_kernel(typename A::storage* __restrict__ out,
                                                                const typename A::storage* __restrict__ gate,
                                                                const typename A::storage* __restrict__ up, int64_t n,
                                                                int64_t gate_stride, int64_t up_stride, int vec) {
  const int64_t r = blockIdx.x;
  if (vec) {      // four elements a thread
    const int64_t i = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    const f32x4 z = Vec4<A>::load(gate + r * gate_stride + i), u = Vec4<A>::load(up + r * up_stride + i);
    Vec4<A>::store(out + r * n + i, f32x4{round_to<A>(gelu_tanh_f(z[0])) * u[0], round_to<A>(gelu_tanh_f(z[1])) * u[1],
                                          round_to<A>(gelu_tanh_f(z[2])) * u[2], round_to<A>(gelu_tanh_f(z[3])) * u[3]});
    return;
  }
  const int64_t i = (int64_t)blockIdx.y * 256 + threadIdx.x;
  if (i >= n) return;
  const float z = A::to_float(gate[r * gate_stride + i]);
  const float u = A::to_float(up[r * up_stride + i]);
  out[r * n + i] = A::from_float(round_to<A>(gelu_tanh_f(z)) * u);
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
    hxm::tile_form() = value < 0 ? 0 : value > 2 ? 2 : value;
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
  // rows a workgroup takes in a row: more than one only where that still leaves several workgroups per CU
  const int32_t run = (shift_w && n_out >= 4096) ? 4 : (shift_w && n_out >= 2048) ? 2 : 1;
  const unsigned n_wg = (unsigned)((n_out + run - 1) / run);
  switch (dtype) {
    case HX_F32:
      stream_norm_kernel<F32><<<dim3(n_wg), dim3(256), lds, s>>>(
          x, in_w, norm_w, groups, eps, rows, n_streams, width, (float*)h_out, shift_w, (float*)hs_out, state,
          state_slot_stride, tok_seq, q_cu, positions, slots, n_out, run);
      break;
    case HX_BF16:
      stream_norm_kernel<BF16><<<dim3(n_wg), dim3(256), lds, s>>>(
          x, in_w, norm_w, groups, eps, rows, n_streams, width, (u16*)h_out, shift_w, (u16*)hs_out, state,
          state_slot_stride, tok_seq, q_cu, positions, slots, n_out, run);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}


// rows of y / gate_pre can be read four elements at a time (and x, gate_b as float4s)
static int rows_vectorise(const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride, const void* gate_b,
                          int64_t width) {
  auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return (width % 4 == 0 && y_stride % 8 == 0 && al(y) && (!gate_pre || (gate_stride % 8 == 0 && al(gate_pre))) &&
          (!gate_b || al(gate_b))) ? 1 : 0;
}

extern "C" int hxm_stream_update(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                                 const float* gate_b, const float* mix, const float* out_w, int64_t n_tokens,
                                 int32_t n_streams, int64_t width, int dtype, void* stream) {
  if (n_tokens < 0 || n_streams < 1 || n_streams > HXM_MAX_STREAMS || width < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!x || !y || !mix || !out_w) return HX_ERR_NULL;
  if (y_stride < width || (gate_pre && gate_stride < width)) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int vec = rows_vectorise(y, y_stride, gate_pre, gate_stride, gate_b, width);
  const dim3 grid((unsigned)n_tokens), block(256);
#define HXM_UPDATE(A_, T_, MS_) stream_update_kernel<A_, MS_><<<grid, block, 0, s>>>( \
      x, (const T_*)y, y_stride, (const T_*)gate_pre, gate_stride, gate_b, mix, out_w, n_streams, width, vec)
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

extern "C" int hxm_stream_update_norm(float* x, const void* y, int64_t y_stride, const void* gate_pre, int64_t gate_stride,
                                      const float* gate_b, const float* mix, const float* out_w, const float* in_next,
                                      const float* norm_next, int32_t groups, float eps, void* h_out, int64_t n_tokens,
                                      int32_t n_streams, int64_t width, int dtype, void* stream) {
  if (n_tokens < 0 || n_streams < 1 || n_streams > HXM_MAX_STREAMS || width < 1 || groups < 1 || width % groups) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!x || !y || !mix || !out_w || !in_next || !norm_next || !h_out) return HX_ERR_NULL;
  if (y_stride < width || (gate_pre && gate_stride < width)) return HX_ERR_STRIDE;
  const size_t lds = (size_t)width * sizeof(float);
  if (lds > 60 * 1024) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int vec = rows_vectorise(y, y_stride, gate_pre, gate_stride, gate_b, width);
  const dim3 grid((unsigned)n_tokens), block(256);
#define HXM_UPN(A_, T_, MS_) stream_update_norm_kernel<A_, MS_><<<grid, block, lds, s>>>( \
      x, (const T_*)y, y_stride, (const T_*)gate_pre, gate_stride, gate_b, mix, out_w, in_next, norm_next, groups, eps, (T_*)h_out, n_streams, width, vec)
#define HXM_UPN_MS(A_, T_) do { if (n_streams <= 4) HXM_UPN(A_, T_, 4); else if (n_streams <= 8) HXM_UPN(A_, T_, 8); \
      else HXM_UPN(A_, T_, 16); } while (0)
  switch (dtype) {
    case HX_F32: HXM_UPN_MS(F32, float); break;
    case HX_BF16: HXM_UPN_MS(BF16, u16); break;
    default: return HX_ERR_DTYPE;
  }
#undef HXM_UPN_MS
#undef HXM_UPN
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
  auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  const int vec = (n % 4 == 0 && gate_stride % 8 == 0 && up_stride % 8 == 0 && al(out) && al(gate) && al(up)) ? 1 : 0;
  const int64_t per_block = vec ? 1024 : 256;
  const dim3 grid((unsigned)rows, (unsigned)((n + per_block - 1) / per_block));
  switch (dtype) {
    case HX_F32:
      gelu_tanh_and_mul_kernel<F32><<<grid, dim3(256), 0, s>>>((float*)out, (const float*)gate, (const float*)up, n, gate_stride, up_stride, vec);
      break;
    case HX_BF16:
      gelu_tanh_and_mul_kernel<BF16><<<grid, dim3(256), 0, s>>>((u16*)out, (const u16*)gate, (const u16*)up, n, gate_stride, up_stride, vec);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
