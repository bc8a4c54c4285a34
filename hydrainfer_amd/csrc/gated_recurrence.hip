// gated_recurrence.hip — HGRN2: a linear recurrence with a matrix state S [dim, vdim] per head whose forget gate also
// decides what is written:  f = low + (1 - low) sigmoid(f_pre + b),  S <- diag(f) S + (1 - f) v^T,  o = S^T silu(q_pre),
// then o is RMS-normed over the head's value channels.  Gates, state and sums are float.
//
// The scan: a workgroup takes (sequence, head, 64 value channels, a part of the key channels).  A lane owns one value
// channel (column of S); the part's key channels (rows of S) are dealt to the workgroup's waves, DR rows each, held in
// registers.  Rows of S evolve independently, so nothing is exchanged during the scan: per chunk of 16 tokens the gates of
// the part's rows are worked out once into LDS (f and silu(q) side by side, read back 16 bytes at a time), a lane's values
// of the chunk are loaded into registers before the scan starts (the serial chain holds no global load), the waves'
// partial o's are summed through LDS and leave for a float workspace [parts][tokens][heads * vdim].  A second kernel — one
// wave per (token, head) — sums the parts and norms over the head's value channels.
#include "hx_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

constexpr int kTC = 16;          // tokens a chunk
constexpr int kMaxWaves = 8;     // waves a workgroup

struct RecArgs {
  void* out;
  const void* q_pre;
  const void* f_pre;
  const void* v;
  int64_t q_stride, f_stride, v_stride;
  const float* f_bias;
  const float* low;
  const float* norm_w;
  float* state;
  int64_t slot_stride;
  const int32_t* q_cu;
  const int32_t* positions;
  const int32_t* slots;
  float* ws;                     // [n_parts][n_tokens][heads * vdim]
  int64_t n_tokens;
  int32_t heads, dim, vdim, n_cw, n_parts, n_waves, max_q_len;
  float eps;
};

template <typename A, int DR>
__global__ __launch_bounds__(64 * kMaxWaves) void gated_recurrence_scan_kernel(RecArgs a) {
  __shared__ __attribute__((aligned(16))) float gates[kTC * kMaxWaves * DR * 2];      // [token][row of the part][f, silu(q)]
  __shared__ __attribute__((aligned(16))) float po[kTC * kMaxWaves * 64];              // [token][wave][lane]
  __shared__ float vs[kTC * 64];                                                       // [token][lane]: the chunk's values
  typedef typename A::storage T;
  const int seq = blockIdx.x, head = blockIdx.y;
  const int cw = blockIdx.z % a.n_cw, part = blockIdx.z / a.n_cw;
  const int D = a.dim, V = a.vdim, NW = a.n_waves;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = cw * 64 + lane;
  const bool col_ok = col < V;
  const int rows_part = NW * DR;                 // key channels of this part (the last part may reach past D: f = 1, q = 0)
  const int part_d0 = part * rows_part;
  const int d0 = part_d0 + wave * DR;
  const int t_begin = a.q_cu[seq], t_end = a.q_cu[seq + 1];
  if (t_end <= t_begin) return;
  float* slot = a.state + (int64_t)a.slots[seq] * a.slot_stride + (int64_t)head * D * V;
  float S[DR];
  const bool fresh = a.positions[t_begin] == 0;
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = d0 + r;
    S[r] = (!fresh && col_ok && d < D) ? slot[(int64_t)d * V + col] : 0.f;
  }
  const T* qp = (const T*)a.q_pre + head * D;
  const T* fp = (const T*)a.f_pre + head * D;
  const T* vp = (const T*)a.v + head * V;
  const float* fb = a.f_bias + head * D;
  const float* lw = a.low + head * D;
  float* wo = a.ws + (int64_t)part * a.n_tokens * (a.heads * V) + head * V;
  const int n_threads = NW * 64;
  const bool pair_ok = (V & 1) == 0 && (((uintptr_t)a.ws) & 7) == 0;      // two floats of the workspace at a time
  // the pre-activations a thread turns into gates (element e of a chunk: token e / rows_part, row e % rows_part) and the
  // lane's values, asked for one chunk ahead
  constexpr int EPT = kTC * DR / 64;
  float qn[EPT], fn[EPT];
  auto fetch = [&](int t0) __attribute__((always_inline)) {
    const int nt = t_end - t0 < kTC ? t_end - t0 : kTC;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + e * n_threads;
      const int tt = i / rows_part, d = part_d0 + i - tt * rows_part;
      const bool ok = tt < nt && d < D;
      qn[e] = ok ? A::to_float(qp[(int64_t)(t0 + tt) * a.q_stride + d]) : 0.f;
      fn[e] = ok ? A::to_float(fp[(int64_t)(t0 + tt) * a.f_stride + d]) : 0.f;
    }
  };
  // The chunk's values [token][column of this group]: every wave of the workgroup needs the same 16 x 64, so the workgroup
  // brings them once (a few loads a thread, one chunk ahead) and hands them round through LDS — one load a lane and
  // token in every wave was the largest single cost of this kernel (vector memory instructions, not bytes).
  float vn[kTC];      // (kTC values a thread when the workgroup is a single wave, two when it has eight)
  auto fetch_v = [&](int t0) __attribute__((always_inline)) {
    const int nt = t_end - t0 < kTC ? t_end - t0 : kTC;
#pragma unroll
    for (int k = 0; k < kTC; ++k) {
      const int i = threadIdx.x + k * n_threads;      // token i / 64, column i % 64
      if (i < kTC * 64) {
        const int tt = i >> 6, c = cw * 64 + (i & 63);
        vn[k] = (tt < nt && c < V) ? A::to_float(vp[(int64_t)(t0 + tt) * a.v_stride + c]) : 0.f;
      }
    }
  };
  fetch(t_begin);
  fetch_v(t_begin);
  for (int t0 = t_begin; t0 < t_end; t0 += kTC) {
    const int nt = t_end - t0 < kTC ? t_end - t0 : kTC;
#pragma unroll
    for (int k = 0; k < kTC; ++k) {
      const int i = threadIdx.x + k * n_threads;
      if (i < kTC * 64) vs[i] = vn[k];
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + e * n_threads;
      const int tt = i / rows_part, d = part_d0 + i - tt * rows_part;
      float q = 0.f, f = 1.f;
      if (tt < nt && d < D) {
        const float qv = qn[e], fv = fn[e] + fb[d], l = lw[d];
        q = qv / (1.0f + expf(-qv));
        f = l + (1.0f - l) / (1.0f + expf(-fv));
      }
      gates[2 * i] = f;
      gates[2 * i + 1] = q;
    }
    if (t0 + kTC < t_end) {
      fetch(t0 + kTC);
      fetch_v(t0 + kTC);
    }
    __syncthreads();
    float vv[kTC];
#pragma unroll
    for (int tt = 0; tt < kTC; ++tt) vv[tt] = vs[tt * 64 + lane];
#pragma unroll
    for (int tt = 0; tt < kTC; ++tt) {
      if (tt < nt) {
        const f32x4* g4 = reinterpret_cast<const f32x4*>(gates + 2 * (tt * rows_part + wave * DR));
        const float v = vv[tt];
        float o = 0.f;
#pragma unroll
        for (int r2 = 0; r2 < DR / 2; ++r2) {
          const f32x4 g = g4[r2];                   // f, silu(q) of two rows
          S[2 * r2] = v + g[0] * (S[2 * r2] - v);   // = f S + (1 - f) v
          o += g[1] * S[2 * r2];
          S[2 * r2 + 1] = v + g[2] * (S[2 * r2 + 1] - v);
          o += g[3] * S[2 * r2 + 1];
        }
        po[(tt * kMaxWaves + wave) * 64 + lane] = o;
      }
    }
    __syncthreads();
    // the waves' partial o's of the chunk, summed: (token, pair of columns) dealt over the workgroup
    for (int i = threadIdx.x; i < nt * 32; i += n_threads) {
      const int tt = i >> 5, ln = (i & 31) * 2, c = cw * 64 + ln;
      float o0 = 0.f, o1 = 0.f;
      for (int w = 0; w < NW; ++w) {
        const float2 p2 = *reinterpret_cast<const float2*>(po + (tt * kMaxWaves + w) * 64 + ln);
        o0 += p2.x;
        o1 += p2.y;
      }
      float* dst = wo + (int64_t)(t0 + tt) * (a.heads * V) + c;
      if (c + 1 < V && pair_ok) *reinterpret_cast<float2*>(dst) = float2{o0, o1};
      else {
        if (c < V) dst[0] = o0;
        if (c + 1 < V) dst[1] = o1;
      }
    }
    // (the next chunk's gates are written while slow waves may still sum: they read po only; po is written again after
    //  the next barrier)
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = d0 + r;
    if (col_ok && d < D) slot[(int64_t)d * V + col] = S[r];
  }
}

// The same for batches in which every sequence brings ONE token (decode steps): no chunks, no staging — a wave reads its
// rows of the state, lanes 0 .. DR - 1 work out the rows' gates and hand them round with v_readlane, the state goes back.
template <typename A, int DR>
__global__ __launch_bounds__(64 * kMaxWaves) void gated_recurrence_step_kernel(RecArgs a) {
  __shared__ float po[kMaxWaves * 64];
  typedef typename A::storage T;
  const int seq = blockIdx.x, head = blockIdx.y;
  const int cw = blockIdx.z % a.n_cw, part = blockIdx.z / a.n_cw;
  const int D = a.dim, V = a.vdim, NW = a.n_waves;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = cw * 64 + lane;
  const bool col_ok = col < V;
  const int d0 = (part * NW + wave) * DR;
  const int t = a.q_cu[seq];
  if (a.q_cu[seq + 1] <= t) return;
  float* slot = a.state + (int64_t)a.slots[seq] * a.slot_stride + (int64_t)head * D * V;
  const bool fresh = a.positions[t] == 0;
  float S[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = d0 + r;
    S[r] = (!fresh && col_ok && d < D) ? slot[(int64_t)d * V + col] : 0.f;
  }
  float f = 1.f, q = 0.f;      // lane r < DR: row d0 + r (past D: the state stays, nothing is read out)
  if (lane < DR && d0 + lane < D) {
    const int hd = head * D + d0 + lane;
    const float qv = A::to_float(((const T*)a.q_pre)[(int64_t)t * a.q_stride + hd]);
    const float fv = A::to_float(((const T*)a.f_pre)[(int64_t)t * a.f_stride + hd]) + a.f_bias[hd];
    const float l = a.low[hd];
    q = qv / (1.0f + expf(-qv));
    f = l + (1.0f - l) / (1.0f + expf(-fv));
  }
  const float v = col_ok ? A::to_float(((const T*)a.v)[(int64_t)t * a.v_stride + head * V + col]) : 0.f;
  float o = 0.f;
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const float fr = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), r));
    const float qr = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(q), r));
    S[r] = v + fr * (S[r] - v);
    o += qr * S[r];
    if (col_ok && d0 + r < D) slot[(int64_t)(d0 + r) * V + col] = S[r];
  }
  po[wave * 64 + lane] = o;
  __syncthreads();
  if (wave == 0 && col_ok) {
    float sum = 0.f;
    for (int w = 0; w < NW; ++w) sum += po[w * 64 + lane];
    a.ws[(int64_t)part * a.n_tokens * (a.heads * V) + (int64_t)t * (a.heads * V) + head * V + col] = sum;
  }
}

// one wave per (token, head): the parts summed, normed over the head's value channels, times norm_w
template <typename A>
__global__ __launch_bounds__(256) void gated_recurrence_norm_kernel(RecArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= a.n_tokens * a.heads) return;
  const int V = a.vdim;
  const int64_t HV = (int64_t)a.heads * V, at = (item / a.heads) * HV + (item % a.heads) * V;
  float o[16];       // vdim <= 1024
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int c = lane + 64 * k;
    o[k] = 0.f;
    if (c < V) {
      for (int p = 0; p < a.n_parts; ++p) o[k] += a.ws[(int64_t)p * a.n_tokens * HV + at + c];
      ss += o[k] * o[k];
    }
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + a.eps);
  typename A::storage* out = (typename A::storage*)a.out + at;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int c = lane + 64 * k;
    if (c < V) out[c] = A::from_float(o[k] * inv * a.norm_w[c]);
  }
}

// rows a wave holds, waves a workgroup, parts of the key channels
void recurrence_layout(int dim, int& dr, int& n_waves, int& n_parts) {
  dr = dim > 16 ? 8 : 4;      // (16 rows a wave: the unrolled scan of a chunk holds every gate it reads in registers — too many)
  const int groups = (dim + dr - 1) / dr;
  n_waves = groups < kMaxWaves ? groups : kMaxWaves;
  n_parts = (groups + n_waves - 1) / n_waves;
}

template <typename A>
int launch_recurrence(const RecArgs& a, int n_seq, int dr, hipStream_t s) {
  const dim3 grid((unsigned)n_seq, (unsigned)a.heads, (unsigned)(a.n_cw * a.n_parts)), block((unsigned)(a.n_waves * 64));
  if (a.max_q_len == 1) {
    if (dr == 4) gated_recurrence_step_kernel<A, 4><<<grid, block, 0, s>>>(a);
    else gated_recurrence_step_kernel<A, 8><<<grid, block, 0, s>>>(a);
  } else {
    if (dr == 4) gated_recurrence_scan_kernel<A, 4><<<grid, block, 0, s>>>(a);
    else gated_recurrence_scan_kernel<A, 8><<<grid, block, 0, s>>>(a);
  }
  gated_recurrence_norm_kernel<A><<<dim3((unsigned)((a.n_tokens * a.heads + 3) / 4)), dim3(256), 0, s>>>(a);
  return hxm::check_launch();
}

}  // namespace

extern "C" int64_t hxm_gated_recurrence_workspace(int64_t n_tokens, int32_t heads, int32_t dim, int32_t vdim) {
  if (n_tokens < 0 || heads < 1 || dim < 1 || vdim < 1) return 0;
  int dr, n_waves, n_parts;
  recurrence_layout(dim, dr, n_waves, n_parts);
  return (int64_t)n_parts * n_tokens * heads * vdim;
}

extern "C" int hxm_gated_recurrence(void* out, const void* q_pre, int64_t q_stride, const void* f_pre, int64_t f_stride,
                                    const void* v, int64_t v_stride, const float* f_bias, const float* low,
                                    const float* norm_w, float eps, float* state, int64_t slot_stride, const int32_t* q_cu,
                                    const int32_t* positions, const int32_t* slots, int32_t n_seq, int64_t n_tokens,
                                    int32_t heads, int32_t dim, int32_t vdim, int32_t max_q_len, float* ws,
                                    int64_t ws_floats, int dtype, void* stream) {
  if (n_seq < 0 || n_tokens < 0 || heads < 1 || dim < 1 || vdim < 1 || vdim > 1024 || heads > 65535) return HX_ERR_SHAPE;
  if (n_seq == 0 || n_tokens == 0) return HX_OK;
  if (!out || !q_pre || !f_pre || !v || !f_bias || !low || !norm_w || !state || !q_cu || !positions || !slots || !ws) return HX_ERR_NULL;
  if (slot_stride < (int64_t)heads * dim * vdim) return HX_ERR_STRIDE;
  RecArgs a;
  a.out = out; a.q_pre = q_pre; a.f_pre = f_pre; a.v = v;
  a.q_stride = q_stride; a.f_stride = f_stride; a.v_stride = v_stride;
  a.f_bias = f_bias; a.low = low; a.norm_w = norm_w; a.state = state; a.slot_stride = slot_stride;
  a.q_cu = q_cu; a.positions = positions; a.slots = slots; a.ws = ws; a.n_tokens = n_tokens;
  a.heads = heads; a.dim = dim; a.vdim = vdim; a.eps = eps; a.max_q_len = max_q_len;
  a.n_cw = (vdim + 63) / 64;
  int dr;
  recurrence_layout(dim, dr, a.n_waves, a.n_parts);
  if ((int64_t)a.n_cw * a.n_parts > 65535) return HX_ERR_SHAPE;
  if (ws_floats < (int64_t)a.n_parts * n_tokens * heads * vdim) return HX_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case HX_F32: return launch_recurrence<F32>(a, n_seq, dr, s);
    case HX_BF16: return launch_recurrence<BF16>(a, n_seq, dr, s);
    default: return HX_ERR_DTYPE;
  }
}
