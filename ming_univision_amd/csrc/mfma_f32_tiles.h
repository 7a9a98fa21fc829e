// mfma_f32_tiles.h — pieces shared by the attention kernels that run on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: fp32
// operands, fp32 accumulate): staging 16-row tiles through registers into LDS, the LDS-only barrier, the hardware exponential.
// Operand layouts (lane l, c = l % 16, g = l / 16): A[row c][k g], B[k g][col c], D[row 4 g + i][col c] in VGPR i.
#pragma once
#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// 16 rows x 64 NBW floats, global -> registers -> LDS (row stride LDC), zero beyond n: 16 threads per row, 16 bytes per thread and
// pass, every load of the tile in flight together.  row_ptr(j) must be readable for every j (callers clamp), row_ok(j) says whether
// row j counts.  Split in two so that the next tile's loads fly while the current tile is multiplied.
template <int NBW, typename RowPtr, typename RowOk>
__device__ __forceinline__ void load16(f32x4 (&v)[NBW], int n, int tid, RowPtr row_ptr, RowOk row_ok) {
  const int j = tid >> 4, cg = tid & 15;
  const float* src = row_ptr(j);
  const bool ok = row_ok(j);
  if ((n & 3) == 0) {
#pragma unroll
    for (int ps = 0; ps < NBW; ++ps) {
      const int d = 4 * (cg + 16 * ps);
      const f32x4 t = *reinterpret_cast<const f32x4*>(src + (d < n ? d : 0));
      v[ps] = (ok && d < n) ? t : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  } else {
#pragma unroll
    for (int ps = 0; ps < NBW; ++ps) {
      const int d = 4 * (cg + 16 * ps);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float t = src[d + e < n ? d + e : 0];
        v[ps][e] = (ok && d + e < n) ? t : 0.f;
      }
    }
  }
}
template <int NBW, int LDC>
__device__ __forceinline__ void store16(float* __restrict__ dst, const f32x4 (&v)[NBW], int tid) {
  const int j = tid >> 4, cg = tid & 15;
#pragma unroll
  for (int ps = 0; ps < NBW; ++ps) *reinterpret_cast<f32x4*>(dst + j * LDC + 4 * (cg + 16 * ps)) = v[ps];
}

// Workgroup barrier that orders LDS traffic only: the compiler's __syncthreads also drains the global loads in flight, which would
// put the prefetched tile's memory latency back on every barrier of the key walk.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
}

// exp on the hardware's base-2 exponential (one multiply + v_exp_f32, about 1e-6 relative over the softmax's range): the library
// expf is some forty instructions, and eight of them per 16-key tile in every wave were the larger part of the key walk's time
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

}  // namespace
