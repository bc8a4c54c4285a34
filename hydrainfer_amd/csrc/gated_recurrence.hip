// gated_recurrence.hip — HGRN2: a linear recurrence with a matrix state S [dim, vdim] per head whose forget gate also
// decides what is written:  f = low + (1 - low) sigmoid(f_pre + b),  S <- diag(f) S + (1 - f) v^T,  o = S^T silu(q_pre),
// then o is RMS-normed over the head's value channels.  Gates, state and sums are float.
//
// One workgroup per (sequence, head).  A lane owns one value channel (column of S); the key channels (rows of S) are
// dealt to `n_dg` groups of waves, DR rows each, held in registers.  Rows of S evolve independently, so the groups never
// talk during the scan: they leave partial o's in LDS, a chunk of tokens at a time, which are then summed and normed.
// The gates of a chunk are worked out once, by all threads, into LDS.  Two barriers per chunk of tokens.
#include "hx_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

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
  int32_t heads, dim, vdim, n_cw, n_dg, chunk;
  float eps;
};

template <typename A, int DR>
__global__ __launch_bounds__(1024) void gated_recurrence_kernel(RecArgs a) {
  extern __shared__ float lds[];
  typedef typename A::storage T;
  const int seq = blockIdx.x, head = blockIdx.y;
  const int D = a.dim, V = a.vdim, TC = a.chunk;
  const int n_waves = a.n_cw * a.n_dg, n_threads = n_waves * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int cw = wave % a.n_cw, dg = wave / a.n_cw;
  const int col = cw * 64 + lane;
  const bool col_ok = col < V;
  const int d0 = dg * DR;
  const int Vp = a.n_cw * 64;
  float* gq = lds;                         // [TC][D]   silu(q_pre)
  float* gf = gq + TC * D;                 // [TC][D]   f
  float* po = gf + TC * D;                 // [TC][n_dg][Vp]   partial o's
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
  T* op = (T*)a.out + head * V;
  const float* fb = a.f_bias + head * D;
  const float* lw = a.low + head * D;
  for (int t0 = t_begin; t0 < t_end; t0 += TC) {
    const int nt = t_end - t0 < TC ? t_end - t0 : TC;
    for (int i = threadIdx.x; i < nt * D; i += n_threads) {
      const int tt = i / D, d = i - tt * D;
      const float qv = A::to_float(qp[(int64_t)(t0 + tt) * a.q_stride + d]);
      const float fv = A::to_float(fp[(int64_t)(t0 + tt) * a.f_stride + d]) + fb[d];
      const float l = lw[d];
      gq[tt * D + d] = qv / (1.0f + expf(-qv));
      gf[tt * D + d] = l + (1.0f - l) / (1.0f + expf(-fv));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = col_ok ? A::to_float(vp[(int64_t)(t0 + tt) * a.v_stride + col]) : 0.f;
      const float* q_t = gq + tt * D + d0;
      const float* f_t = gf + tt * D + d0;
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < DR; ++r) {
        if (d0 + r < D) {
          const float f = f_t[r];
          S[r] = f * S[r] + (1.0f - f) * vv;
          o += q_t[r] * S[r];
        }
      }
      po[(tt * a.n_dg + dg) * Vp + col] = o;
    }
    __syncthreads();
    // sum the groups' partial o's, norm over the head's value channels: a wave takes a token at a time
    for (int tt = wave; tt < nt; tt += n_waves) {
      float ss = 0.f;
      for (int c = lane; c < V; c += 64) {
        float o = 0.f;
        for (int g = 0; g < a.n_dg; ++g) o += po[(tt * a.n_dg + g) * Vp + c];
        po[(tt * a.n_dg) * Vp + c] = o;      // (this lane alone reads and writes column c of token tt)
        ss += o * o;
      }
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)V + a.eps);
      for (int c = lane; c < V; c += 64)
        op[(int64_t)(t0 + tt) * (a.heads * V) + c] = A::from_float(po[(tt * a.n_dg) * Vp + c] * inv * a.norm_w[c]);
    }
    // (the next chunk's gates go to gq / gf, which nobody reads any more; po is written again only after the next barrier)
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = d0 + r;
    if (col_ok && d < D) slot[(int64_t)d * V + col] = S[r];
  }
}

template <typename A>
int launch_recurrence(const RecArgs& a, int n_seq, int dr, size_t lds, hipStream_t s) {
  const dim3 grid((unsigned)n_seq, (unsigned)a.heads), block((unsigned)(a.n_cw * a.n_dg * 64));
#define HXM_REC(DR_)                                                                                                      \
  do {                                                                                                                    \
    if (lds > 48 * 1024) {                                                                                                \
      hipError_t e = hipFuncSetAttribute((const void*)gated_recurrence_kernel<A, DR_>,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                           \
      if (e != hipSuccess) {                                                                                              \
        hxm::last_hip_error() = (int)e;                                                                                   \
        return HX_ERR_HIP;                                                                                                \
      }                                                                                                                   \
    }                                                                                                                     \
    gated_recurrence_kernel<A, DR_><<<grid, block, lds, s>>>(a);                                                          \
  } while (0)
  switch (dr) {
    case 8: HXM_REC(8); break;
    case 16: HXM_REC(16); break;
    case 32: HXM_REC(32); break;
    case 64: HXM_REC(64); break;
    default: return HX_ERR_SHAPE;
  }
#undef HXM_REC
  return hxm::check_launch();
}

}  // namespace

extern "C" int hxm_gated_recurrence(void* out, const void* q_pre, int64_t q_stride, const void* f_pre, int64_t f_stride,
                                    const void* v, int64_t v_stride, const float* f_bias, const float* low,
                                    const float* norm_w, float eps, float* state, int64_t slot_stride, const int32_t* q_cu,
                                    const int32_t* positions, const int32_t* slots, int32_t n_seq, int32_t heads, int32_t dim,
                                    int32_t vdim, int dtype, void* stream) {
  if (n_seq < 0 || heads < 1 || dim < 1 || vdim < 1 || dim > 1024 || vdim > 1024) return HX_ERR_SHAPE;
  if (n_seq == 0) return HX_OK;
  if (!out || !q_pre || !f_pre || !v || !f_bias || !low || !norm_w || !state || !q_cu || !positions || !slots) return HX_ERR_NULL;
  if (slot_stride < (int64_t)heads * dim * vdim) return HX_ERR_STRIDE;
  RecArgs a;
  a.out = out; a.q_pre = q_pre; a.f_pre = f_pre; a.v = v;
  a.q_stride = q_stride; a.f_stride = f_stride; a.v_stride = v_stride;
  a.f_bias = f_bias; a.low = low; a.norm_w = norm_w; a.state = state; a.slot_stride = slot_stride;
  a.q_cu = q_cu; a.positions = positions; a.slots = slots;
  a.heads = heads; a.dim = dim; a.vdim = vdim; a.eps = eps;
  a.n_cw = (vdim + 63) / 64;                       // waves across the value channels: 1 .. 16
  // groups of key channels: as many as fit 16 waves, no fewer rows than 8 a group, no more than 64 (the registers)
  int n_dg = 16 / a.n_cw;
  while (n_dg > 1 && (dim + n_dg - 1) / n_dg < 8) --n_dg;
  int rows = (dim + n_dg - 1) / n_dg;
  if (rows > 64) return HX_ERR_SHAPE;              // dim * ceil(vdim / 64) <= 1024
  const int dr = rows <= 8 ? 8 : rows <= 16 ? 16 : rows <= 32 ? 32 : 64;
  n_dg = (dim + dr - 1) / dr;
  a.n_dg = n_dg;
  int chunk = 16;
  auto lds_of = [&](int tc) { return (size_t)tc * (2 * (size_t)dim + (size_t)n_dg * a.n_cw * 64) * sizeof(float); };
  while (chunk > 1 && lds_of(chunk) > 96 * 1024) chunk >>= 1;
  if (lds_of(chunk) > 96 * 1024) return HX_ERR_SHAPE;
  a.chunk = chunk;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case HX_F32: return launch_recurrence<F32>(a, n_seq, dr, lds_of(chunk), s);
    case HX_BF16: return launch_recurrence<BF16>(a, n_seq, dr, lds_of(chunk), s);
    default: return HX_ERR_DTYPE;
  }
}
