// mix_rows.h — helpers of the mix library's row kernels: four consecutive elements of an activation row as four floats,
// and sums over a 256-thread workgroup.
#pragma once
#include "hx_common.h"

namespace hx {

template <typename A> struct Row4;
template <> struct Row4<F32> {
  static __device__ __forceinline__ f32x4 load(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
  static __device__ __forceinline__ void store(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
};
template <> struct Row4<BF16> {
  static __device__ __forceinline__ f32x4 load(const u16* p) {
    const u16x4 b = *reinterpret_cast<const u16x4*>(p);
    return f32x4{BF16::to_float(b[0]), BF16::to_float(b[1]), BF16::to_float(b[2]), BF16::to_float(b[3])};
  }
  static __device__ __forceinline__ void store(u16* p, f32x4 v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{BF16::from_float(v[0]), BF16::from_float(v[1]), BF16::from_float(v[2]), BF16::from_float(v[3])};
  }
};

// true if p and the row stride (elements) let a lane move four elements of type T at a time
template <typename T>
inline bool rows_by_four(const void* p, int64_t stride) {
  return (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0 && stride % 4 == 0;
}

// sums of N values over the 256 threads of the workgroup; part: 4 * N floats of LDS.  Every thread ends with the sums; part
// may be used again after the next barrier.
template <int N>
__device__ __forceinline__ void block_sums(float (&v)[N], float* part) {
#pragma unroll
  for (int n = 0; n < N; ++n) v[n] = wave_sum(v[n]);
  __syncthreads();                       // the previous use of part is over
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int n = 0; n < N; ++n) part[(threadIdx.x >> 6) * N + n] = v[n];
  }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < N; ++n) v[n] = part[n] + part[N + n] + part[2 * N + n] + part[3 * N + n];
}

// Reductions over the 16 lanes of a DPP row (lanes 16 k .. 16 k + 15) on the vector ALU alone — a shuffle goes through
// the LDS crossbar (ds_bpermute) and waits for it.  Every lane ends with the row's result.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
constexpr int kDppXor1 = 0xB1;          // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;          // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;   // lanes of each half of the row in reverse order
constexpr int kDppMirror = 0x140;       // the row in reverse order
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppMirror>(v);
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_move<kDppXor1>(v));
  v = fmaxf(v, dpp_move<kDppXor2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppMirror>(v));
  return v;
}

// A workgroup barrier that orders LDS traffic only: global loads and stores that are in flight (a prefetch for the next
// step, results on their way out) are not waited for, as __syncthreads() would.  For exchanges through LDS alone.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

}  // namespace hx
