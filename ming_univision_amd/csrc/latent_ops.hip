// latent_ops.hip — row operators of sequence models that cache a low-rank latent instead of keys and values (mingnative.h
// section 9).  Everything here works on fp32 rows [M, n] of a step (tokens of one or several cache sequences, each sequence's
// rows consecutive) and bf16 weights; every size is an argument.
//
//   mn_affine_ln_rows        y = (x - mean) / sqrt(var + eps) * w + b                      (optional bf16 copy for an MFMA GEMM)
//   mn_gated_ln_residual     x += LN(sigmoid(g) * y) * w + b                               (gate, norm and residual add of a sublayer)
//   mn_rms_rows              y = x / sqrt(mean(x^2) + eps) * w, rows optionally scattered into a cache arena [n_seq, t_max, n]
//   mn_polynorm_rows         y = a U(z) + b U(z^2) + c U(z^3) + e,  U(v) = v / sqrt(mean(v^2) + eps)
//   mn_tap_filter_rows       y_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j) over each sequence, the taps - 1 rows before a step
//                            taken from a per-sequence state, which mn_tap_state_update then advances
//   mn_gemm_f32_batched      C = alpha * A W^T (+ bias) (* sigmoid(G)), fp32 FMA on fp32 rows x bf16 weights, batched by strides
//                            (grid.z): the true-32-bit product and the per-head absorb / expand products of latent attention
//   mn_latent_attn           causal softmax attention of per-head absorbed queries [M, H, r] against the cached latents [t, r]
//                            (keys = values = the latent, shared by all heads), online softmax in fp32, key range splittable
//   mn_softcap_rows          z = cap * tanh(z / cap)
#include "common.h"
#include "mfma_f32_tiles.h"

namespace {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------------------------------------------------------
// one wave per row: LayerNorm with weight and bias
__global__ __launch_bounds__(256) void affine_ln_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w,
                                                        const bf16_t* __restrict__ b, float eps, float* __restrict__ y, int64_t ldy,
                                                        bf16_t* __restrict__ y16, int64_t ldy16, int M, int n) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  const float* xr = x + (int64_t)row * ldx;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) s += xr[i];
  const float mean = wave_sum(s) / (float)n;
  float v = 0.f;
  for (int i = lane; i < n; i += 64) { const float d = xr[i] - mean; v += d * d; }
  const float rstd = 1.0f / sqrtf(wave_sum(v) / (float)n + eps);
  for (int i = lane; i < n; i += 64) {
    const float o = (xr[i] - mean) * rstd * bf16_to_f32(w[i]) + bf16_to_f32(b[i]);
    if (y) y[(int64_t)row * ldy + i] = o;
    if (y16) y16[(int64_t)row * ldy16 + i] = f32_to_bf16(o);
  }
}

// x[row] += LN(sigmoid(g[row]) * y[row]) * w + b
__global__ __launch_bounds__(256) void gated_ln_residual_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ g,
                                                                int64_t ldg, const float* __restrict__ yv, int64_t ldy,
                                                                const bf16_t* __restrict__ w, const bf16_t* __restrict__ b, float eps,
                                                                int M, int n) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  const float* gr = g + (int64_t)row * ldg;
  const float* yr = yv + (int64_t)row * ldy;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) s += sigmoid_f(gr[i]) * yr[i];
  const float mean = wave_sum(s) / (float)n;
  float v = 0.f;
  for (int i = lane; i < n; i += 64) { const float d = sigmoid_f(gr[i]) * yr[i] - mean; v += d * d; }
  const float rstd = 1.0f / sqrtf(wave_sum(v) / (float)n + eps);
  for (int i = lane; i < n; i += 64) {
    const float t = sigmoid_f(gr[i]) * yr[i];
    x[(int64_t)row * ldx + i] += (t - mean) * rstd * bf16_to_f32(w[i]) + bf16_to_f32(b[i]);
  }
}

// RMS norm with a plain weight; output row index = row, or row_seq[row] * t_max + row_slot[row] (append into a cache arena)
__global__ __launch_bounds__(256) void rms_rows_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, float eps,
                                                       float* __restrict__ y, int64_t ldy, bf16_t* __restrict__ y16, int64_t ldy16,
                                                       const int32_t* __restrict__ row_seq, const int32_t* __restrict__ row_slot,
                                                       int t_max, int M, int n) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  const float* xr = x + (int64_t)row * ldx;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) s += xr[i] * xr[i];
  const float r = 1.0f / sqrtf(wave_sum(s) / (float)n + eps);
  const int64_t orow = row_seq ? (int64_t)row_seq[row] * t_max + row_slot[row] : row;
  for (int i = lane; i < n; i += 64) {
    const float o = xr[i] * r * bf16_to_f32(w[i]);
    if (y) y[orow * ldy + i] = o;
    if (y16) y16[(int64_t)row * ldy16 + i] = f32_to_bf16(o);
  }
}

// one workgroup per row
__global__ __launch_bounds__(256) void polynorm_kernel(const float* __restrict__ z, int64_t ldz, const bf16_t* __restrict__ coef, float eps,
                                                       float* __restrict__ y, int64_t ldy, bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  __shared__ float red[8];
  const int row = blockIdx.x;
  const float* zr = z + (int64_t)row * ldz;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = zr[i], v2 = v * v, v3 = v2 * v;
    s2 += v2; s4 += v2 * v2; s6 += v3 * v3;
  }
  s2 = block_sum(s2, red); s4 = block_sum(s4, red); s6 = block_sum(s6, red);
  const float a = bf16_to_f32(coef[0]) / sqrtf(s2 / (float)n + eps), b = bf16_to_f32(coef[1]) / sqrtf(s4 / (float)n + eps),
              c = bf16_to_f32(coef[2]) / sqrtf(s6 / (float)n + eps), e = bf16_to_f32(coef[3]);
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = zr[i], v2 = v * v;
    const float o = a * v + b * v2 + c * (v2 * v) + e;
    if (y) y[(int64_t)row * ldy + i] = o;
    if (y16) y16[(int64_t)row * ldy16 + i] = f32_to_bf16(o);
  }
}

// One workgroup per row with the row held in registers (VPT values per thread, n <= 256 VPT): one batch of loads, the reductions,
// one batch of stores — the form for wide rows, where a single wave walking the row three times is a chain of dependent round trips.
enum { ROW_LN = 0, ROW_GATED_LN_RESIDUAL = 1, ROW_POLYNORM = 2 };
struct RowArgs {
  const float* x; int64_t ldx;          // LN / polynorm input; gated: the residual stream (updated in place)
  const float* g; int64_t ldg;          // gated: gate pre-activation
  const float* y; int64_t ldy;          // gated: sublayer result
  const bf16_t* w; const bf16_t* b;     // norm weight / bias; polynorm: w = the four coefficients
  float eps;
  float* out; int64_t ldo;
  bf16_t* out16; int64_t ldo16;
  int n;
};

template <int VPT, int MODE>
__global__ __launch_bounds__(256) void row_block_kernel(RowArgs a) {
  __shared__ float red[8];
  const int row = blockIdx.x, tid = threadIdx.x, n = a.n;
  float v[VPT];
  if (MODE == ROW_GATED_LN_RESIDUAL) {
    float gv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + 256 * i, cc = c < n ? c : 0;
      gv[i] = a.g[(int64_t)row * a.ldg + cc];
      v[i] = a.y[(int64_t)row * a.ldy + cc];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) v[i] = (tid + 256 * i < n) ? sigmoid_f(gv[i]) * v[i] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + 256 * i;
      const float t = a.x[(int64_t)row * a.ldx + (c < n ? c : 0)];
      v[i] = c < n ? t : 0.f;
    }
  }
  if (MODE == ROW_POLYNORM) {
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) { const float v2 = v[i] * v[i], v3 = v2 * v[i]; s2 += v2; s4 += v2 * v2; s6 += v3 * v3; }
    s2 = block_sum(s2, red); s4 = block_sum(s4, red); s6 = block_sum(s6, red);
    const float ca = bf16_to_f32(a.w[0]) / sqrtf(s2 / (float)n + a.eps), cb = bf16_to_f32(a.w[1]) / sqrtf(s4 / (float)n + a.eps),
                cc = bf16_to_f32(a.w[2]) / sqrtf(s6 / (float)n + a.eps), ce = bf16_to_f32(a.w[3]);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + 256 * i;
      if (c >= n) continue;
      const float v2 = v[i] * v[i], o = ca * v[i] + cb * v2 + cc * (v2 * v[i]) + ce;
      if (a.out) a.out[(int64_t)row * a.ldo + c] = o;
      if (a.out16) a.out16[(int64_t)row * a.ldo16 + c] = f32_to_bf16(o);
    }
    return;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) s += v[i];
  const float mean = block_sum(s, red) / (float)n;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) { const float d = (tid + 256 * i < n) ? v[i] - mean : 0.f; q += d * d; }
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)n + a.eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + 256 * i;
    if (c >= n) continue;
    const float o = (v[i] - mean) * rstd * bf16_to_f32(a.w[c]) + bf16_to_f32(a.b[c]);
    if (MODE == ROW_GATED_LN_RESIDUAL) {
      a.out[(int64_t)row * a.ldo + c] += o;
    } else {
      if (a.out) a.out[(int64_t)row * a.ldo + c] = o;
      if (a.out16) a.out16[(int64_t)row * a.ldo16 + c] = f32_to_bf16(o);
    }
  }
}

// rows of 512 .. 8192 values take the register form; launches it and returns true, or false for other widths
template <int MODE>
bool launch_row_block(const RowArgs& a, int M, hipStream_t st) {
  if (a.n < 512 || a.n > 8192) return false;
  const int vpt = (a.n + 255) / 256;
#define MN_RB(V_) hipLaunchKernelGGL((row_block_kernel<V_, MODE>), dim3((unsigned)M), dim3(256), 0, st, a)
  if (vpt <= 2) MN_RB(2); else if (vpt <= 4) MN_RB(4); else if (vpt <= 8) MN_RB(8); else if (vpt <= 16) MN_RB(16); else MN_RB(32);
#undef MN_RB
  return true;
}

// y[m, c] = x[m, c] + sum_k w[c, taps - 1 - k] * (the sequence's input k positions back); grid (ceil(n / 256), M)
__global__ __launch_bounds__(256) void tap_filter_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int taps,
                                                         const float* __restrict__ state, const int32_t* __restrict__ row_seq,
                                                         const int32_t* __restrict__ row_slot, const int32_t* __restrict__ row_back,
                                                         float* __restrict__ y, int64_t ldy, bf16_t* __restrict__ y16, int64_t ldy16, int n,
                                                         float self_w) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const int seq = row_seq[m], slot = row_slot[m], back = row_back[m];
  const float cur = x[(int64_t)m * ldx + c];
  float acc = self_w * cur;                         // 1: the input is added to its filter, 0: the filter alone
  for (int k = 0; k < taps; ++k) {
    float v = 0.f;
    if (k <= back) v = x[(int64_t)(m - k) * ldx + c];
    else if (slot - k >= 0) v = state[((int64_t)seq * (taps - 1) + (k - back - 1)) * n + c];
    acc += bf16_to_f32(w[(int64_t)c * taps + (taps - 1 - k)]) * v;
  }
  if (y) y[(int64_t)m * ldy + c] = acc;
  if (y16) y16[(int64_t)m * ldy16 + c] = f32_to_bf16(acc);
}

// state[seq][i] = the sequence's input i positions before its next one; only the LAST row of a sequence in the step works
__global__ __launch_bounds__(256) void tap_state_kernel(const float* __restrict__ x, int64_t ldx, int taps, float* __restrict__ state,
                                                        const int32_t* __restrict__ row_seq, const int32_t* __restrict__ row_back, int M,
                                                        int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  if (m + 1 < M && row_back[m + 1] != 0) return;
  const int cnt = row_back[m] + 1;                  // rows of this sequence in the step, ending at m
  float* st = state + (int64_t)row_seq[m] * (taps - 1) * n + c;
  for (int i = taps - 2; i >= 0; --i)               // descending: the old entries that move are read before they are overwritten
    st[(int64_t)i * n] = (i < cnt) ? x[(int64_t)(m - i) * ldx + c] : st[(int64_t)(i - cnt) * n];
}

__global__ void softcap_kernel(float* __restrict__ z, int64_t ld, int n, float cap) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) { float* p = z + (int64_t)blockIdx.y * ld + i; *p = cap * tanhf(*p / cap); }
}

// ---------------------------------------------------------------------------------------------------------------------------
// fp32 FMA GEMM: C[z][m, n] = alpha * sum_k A[z][m, k] W[z][n, k] (+ bias[n]) (* sigmoid(G[z][m, n])).  BM x 64 tiles, 16 x 16 threads.
struct GemmF32 {
  const float* A; int64_t lda, a_bs;
  const bf16_t* W; int64_t ldw, w_bs;
  const bf16_t* bias;
  float* C; int64_t ldc, c_bs;
  bf16_t* C16; int64_t ldc16, c16_bs;
  const float* G; int64_t ldg, g_bs;
  int M, N, K;
  float alpha;
};

template <int TM>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmF32 a) {
  constexpr int BM = 16 * TM, BN = 64, BK = 16;
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int z = blockIdx.z, tid = threadIdx.x;
  const float* A = a.A + (int64_t)z * a.a_bs;
  const bf16_t* W = a.W + (int64_t)z * a.w_bs;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tx = tid & 15, ty = tid >> 4;
  float acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    for (int e = tid; e < BM * BK; e += 256) {
      const int r = e / BK, k = e % BK;
      const int gm = m0 + r, gk = k0 + k;
      As[k][r] = (gm < a.M && gk < a.K) ? A[(int64_t)gm * a.lda + gk] : 0.f;
    }
    for (int e = tid; e < BN * BK; e += 256) {
      const int r = e / BK, k = e % BK;
      const int gn = n0 + r, gk = k0 + k;
      Ws[k][r] = (gn < a.N && gk < a.K) ? bf16_to_f32(W[(int64_t)gn * a.ldw + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[TM], wv[4];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = As[k][ty * TM + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int gm = m0 + ty * TM + i;
    if (gm >= a.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= a.N) continue;
      float v = acc[i][j] * a.alpha;
      if (a.bias) v += bf16_to_f32(a.bias[gn]);
      if (a.G) v *= sigmoid_f(a.G[(int64_t)z * a.g_bs + (int64_t)gm * a.ldg + gn]);
      if (a.C) a.C[(int64_t)z * a.c_bs + (int64_t)gm * a.ldc + gn] = v;
      if (a.C16) a.C16[(int64_t)z * a.c16_bs + (int64_t)gm * a.ldc16 + gn] = f32_to_bf16(v);
    }
  }
}

// Decode rows (every row alone in its sequence), one workgroup per row, the row in registers, up to three stages in one launch:
//   1 (g given)  x += LN(sigmoid(g) * y; wa, ba)          the previous sublayer's gate, norm and residual add
//   2            n  = LN(x; wb, bb)                        this sublayer's input norm
//   3 (h given)  h  = n + taps filter over the sequence's last inputs (from its state), and the state moves on by this row
struct FusedRowArgs {
  float* x; int64_t ldx;
  const float* g; int64_t ldg;
  const float* y; int64_t ldy;
  const bf16_t *wa, *ba, *wb, *bb;
  float eps;
  float* n_out; int64_t ldn;
  const bf16_t* taps_w; int taps;
  float* state; const int32_t* row_seq; const int32_t* row_slot;
  float* h; int64_t ldh;
  int n;
};

constexpr int FUSED_MAX_TAPS = 8;

template <int VPT, bool FILTER>
__global__ __launch_bounds__(256) void row_fused_kernel(FusedRowArgs a) {
  __shared__ float red[8];
  const int row = blockIdx.x, tid = threadIdx.x, n = a.n;
  float xv[VPT];
  // everything the row needs from memory is requested before the first store: the state is float like the outputs, so a load
  // placed after a store would wait its turn, one round trip per value
  float sv[FILTER ? VPT : 1][FUSED_MAX_TAPS - 1];
  const int seq = FILTER ? a.row_seq[row] : 0, slot = FILTER ? a.row_slot[row] : 0;
  float* const st0 = FILTER ? a.state + (int64_t)seq * (a.taps - 1) * n : nullptr;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + 256 * i, cc = c < n ? c : 0;
    const float t = a.x[(int64_t)row * a.ldx + cc];
    xv[i] = c < n ? t : 0.f;
    if (FILTER) {
#pragma unroll
      for (int k = 1; k < FUSED_MAX_TAPS; ++k) sv[i][k - 1] = (k < a.taps) ? st0[(int64_t)(k - 1) * n + cc] : 0.f;
    }
  }
  if (a.g) {
    float t[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + 256 * i, cc = c < n ? c : 0;
      const float gv = a.g[(int64_t)row * a.ldg + cc], yv = a.y[(int64_t)row * a.ldy + cc];
      t[i] = c < n ? sigmoid_f(gv) * yv : 0.f;
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) s += t[i];
    const float mean = block_sum(s, red) / (float)n;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) { const float d = (tid + 256 * i < n) ? t[i] - mean : 0.f; q += d * d; }
    const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)n + a.eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + 256 * i;
      if (c >= n) continue;
      xv[i] += (t[i] - mean) * rstd * bf16_to_f32(a.wa[c]) + bf16_to_f32(a.ba[c]);
      a.x[(int64_t)row * a.ldx + c] = xv[i];
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) s += xv[i];
  const float mean = block_sum(s, red) / (float)n;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) { const float d = (tid + 256 * i < n) ? xv[i] - mean : 0.f; q += d * d; }
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)n + a.eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + 256 * i;
    if (c >= n) continue;
    const float nv = (xv[i] - mean) * rstd * bf16_to_f32(a.wb[c]) + bf16_to_f32(a.bb[c]);
    a.n_out[(int64_t)row * a.ldn + c] = nv;
    if (FILTER) {
      const bf16_t* tw = a.taps_w + (int64_t)c * a.taps;
      float acc = nv + bf16_to_f32(tw[a.taps - 1]) * nv;
#pragma unroll
      for (int k = 1; k < FUSED_MAX_TAPS; ++k)
        if (k < a.taps && slot - k >= 0) acc += bf16_to_f32(tw[a.taps - 1 - k]) * sv[i][k - 1];
      a.h[(int64_t)row * a.ldh + c] = acc;
      float* st = st0 + c;
#pragma unroll
      for (int k = FUSED_MAX_TAPS - 2; k >= 1; --k)
        if (k < a.taps - 1) st[(int64_t)k * n] = sv[i][k - 1];
      if (a.taps > 1) st[0] = nv;
    }
  }
}

// C[z][m, n] = alpha * A[z][m, :] . W[z][n, :] (+ bias) (* sigmoid(G)) for few rows: one wave per output column and MM rows, lanes over K
template <int MM>
__global__ __launch_bounds__(256) void gemv_f32_kernel(GemmF32 a) {
  const int z = blockIdx.z, n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= a.N) return;
  const int m0 = blockIdx.y * MM;                       // this workgroup's rows: m0 .. m0 + MM - 1
  a.M -= m0;
  a.A += (int64_t)m0 * a.lda;
  if (a.C) a.C += (int64_t)m0 * a.ldc;
  if (a.C16) a.C16 += (int64_t)m0 * a.ldc16;
  if (a.G) a.G += (int64_t)m0 * a.ldg;
  const float* A = a.A + (int64_t)z * a.a_bs;
  const bf16_t* Wr = a.W + (int64_t)z * a.w_bs + (int64_t)n * a.ldw;
  float acc[MM];
#pragma unroll
  for (int m = 0; m < MM; ++m) acc[m] = 0.f;
#pragma unroll 4
  for (int k = lane; k < a.K; k += 64) {
    const float w = bf16_to_f32(Wr[k]);
#pragma unroll
    for (int m = 0; m < MM; ++m)
      if (m < a.M) acc[m] = fmaf(A[(int64_t)m * a.lda + k], w, acc[m]);
  }
#pragma unroll
  for (int m = 0; m < MM; ++m) {
    if (m >= a.M) break;
    float v = wave_sum(acc[m]) * a.alpha;
    if (lane != 0) continue;
    if (a.bias) v += bf16_to_f32(a.bias[n]);
    if (a.G) v *= sigmoid_f(a.G[(int64_t)z * a.g_bs + (int64_t)m * a.ldg + n]);
    if (a.C) a.C[(int64_t)z * a.c_bs + (int64_t)m * a.ldc + n] = v;
    if (a.C16) a.C16[(int64_t)z * a.c16_bs + (int64_t)m * a.ldc16 + n] = f32_to_bf16(v);
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Latent attention.  One wave per query vector (row, head); the waves of a workgroup share the staged latent tile (all heads and up
// to 4 consecutive rows of one sequence see the same keys).  Phase A: lane = key, dot over r; phase B: lane = latent component,
// sum over keys.  Running maximum / sum / accumulator in fp32 registers.
template <int RCH>
__global__ __launch_bounds__(1024) void latent_attn_kernel(const float* __restrict__ qabs, const float* __restrict__ arena,
                                                           const int32_t* __restrict__ row_seq, const int32_t* __restrict__ row_len,
                                                           const int32_t* __restrict__ blk_tab, int H, int r, int t_max, int KT,
                                                           int tiles_per_split, float* __restrict__ lat, float* __restrict__ part_acc,
                                                           float* __restrict__ part_ml, int KS, int M) {
  extern __shared__ float lds_c[];                 // [KT][r + 1]
  const int row0 = blk_tab[2 * blockIdx.x], nrows = blk_tab[2 * blockIdx.x + 1];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, NW = blockDim.x >> 6;
  const int qv = blockIdx.y * NW + wave;
  const bool active = qv < nrows * H;
  const int ri = active ? qv / H : 0, h = active ? qv % H : 0, m = row0 + ri;
  const int64_t seq = row_seq[row0];
  const int len_max = row_len[row0 + nrows - 1];
  const int my_len = active ? row_len[m] : 0;
  float q[RCH], acc[RCH];
#pragma unroll
  for (int i = 0; i < RCH; ++i) {
    const int d = lane + 64 * i;
    q[i] = (active && d < r) ? qabs[((int64_t)m * H + h) * r + d] : 0.f;
    acc[i] = 0.f;
  }
  float mrun = -INFINITY, l = 0.f;
  const int n_tiles = (len_max + KT - 1) / KT;
  const int t0 = blockIdx.z * tiles_per_split, t1 = min(t0 + tiles_per_split, n_tiles);
  const int ldc = r + 1;
  for (int tile = t0; tile < t1; ++tile) {
    const int key0 = tile * KT;
    __syncthreads();
    for (int j = wave; j < KT; j += NW) {            // a wave copies whole latent rows: consecutive lanes, consecutive components
      const bool in = key0 + j < len_max;
      const float* src = arena + (seq * t_max + key0 + j) * r;
      for (int d = lane; d < r; d += 64) lds_c[j * ldc + d] = in ? src[d] : 0.f;
    }
    __syncthreads();
    if (!active || key0 >= my_len) continue;
    // every lane runs the dot product (lanes beyond the tile or the row's length on a clamped key, masked afterwards): the
    // cross-lane reads of q below then never sit in divergent control flow
    float dot = 0.f;
    {
      const float* cj = lds_c + min(lane, KT - 1) * ldc;
#pragma unroll
      for (int i = 0; i < RCH; ++i) {
        const int dn = min(64, r - 64 * i);
        for (int dd = 0; dd < dn; ++dd) dot = fmaf(lane_f(q[i], dd), cj[64 * i + dd], dot);
      }
    }
    const float s = (lane < KT && key0 + lane < my_len) ? dot : -INFINITY;
    const float mnew = fmaxf(mrun, wave_max(s));       // finite: key0 < my_len
    const float p = (s == -INFINITY) ? 0.f : expf(s - mnew);
    const float corr = (mrun == -INFINITY) ? 0.f : expf(mrun - mnew);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < RCH; ++i) acc[i] *= corr;
    const int jn = min(KT, my_len - key0);
    for (int j = 0; j < jn; ++j) {
      const float pj = lane_f(p, j);
#pragma unroll
      for (int i = 0; i < RCH; ++i) {
        const int d = lane + 64 * i;
        if (d < r) acc[i] = fmaf(pj, lds_c[j * ldc + d], acc[i]);
      }
    }
    mrun = mnew;
  }
  if (!active) return;
  const int64_t o = ((int64_t)m * H + h);
  if (KS == 1) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < RCH; ++i) {
      const int d = lane + 64 * i;
      if (d < r) lat[o * r + d] = acc[i] * inv;
    }
  } else {
    const int64_t po = (int64_t)blockIdx.z * M * H + o;
#pragma unroll
    for (int i = 0; i < RCH; ++i) {
      const int d = lane + 64 * i;
      if (d < r) part_acc[po * r + d] = acc[i];
    }
    if (lane == 0) { part_ml[po * 2] = mrun; part_ml[po * 2 + 1] = l; }
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Latent attention on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: fp32 operands, fp32 accumulate — scores and weights stay
// 32-bit).  A workgroup of 4 waves owns 16 query vectors (row, head) of one run of rows and walks the sequence's latents in tiles
// of 16 keys staged in LDS:
//   scores   S[16 q, 16 keys] = Q C^T: every wave multiplies its quarter of the latent components (its slice of Q stays in
//            registers), the partial tiles are summed through LDS, so all four waves hold the same scores and keep the same
//            running maximum / sum without talking
//   values   O[16 q, r] += P C: the weights go through LDS into the A-operand layout, wave w owns the 16-column blocks w, w + 4, ..
// Operand layouts (lane l, c = l % 16, g = l / 16): A[row c][k g], B[k g][col c], D[row 4 g + i][col c] in VGPR i.
// (f32x4, load16 / store16, lds_barrier, fast_exp: mfma_f32_tiles.h)

template <int NBW>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(const float* __restrict__ qabs, const float* __restrict__ arena,
                                                               const int32_t* __restrict__ row_seq, const int32_t* __restrict__ row_len,
                                                               const int32_t* __restrict__ blk_tab, int H, int r, int t_max,
                                                               int tiles_per_split, float* __restrict__ lat, float* __restrict__ part_acc,
                                                               float* __restrict__ part_ml, int KS, int M) {
  // the latent is padded with zeros to RP = 64 NBW components: every loop below has a compile-time trip count
  constexpr int KT = 16, LDP = 20, LDS_S = 17, RP = 64 * NBW, LDC = RP + 4, DQ = RP / 4;
  extern __shared__ float lds[];
  const int row0 = blk_tab[2 * blockIdx.x], nrows = blk_tab[2 * blockIdx.x + 1];
  const int nqv = nrows * H, qv0 = blockIdx.y * 16;
  if (qv0 >= nqv) return;
  float* Cl = lds;                       // [16 keys][LDC]
  float* Sp = Cl + KT * LDC;             // [4 waves][16 q][LDS_S] partial scores
  float* Pl = Sp + 4 * 16 * LDS_S;       // [16 q][LDP] weights
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c16 = lane & 15, g4 = lane >> 4;
  const int64_t seq = row_seq[row0];
  const int len_max = row_len[row0 + nrows - 1];
  f32x4 v[NBW];
  // the A operands of this wave's score products stay in registers for the whole key walk: query c16, components wave DQ + 4 it + g4
  float qreg[DQ / 4];
  {
    const int qv = min(qv0 + c16, nqv - 1);
    const float* src = qabs + ((int64_t)(row0 + qv / H) * H + qv % H) * r;
#pragma unroll
    for (int it = 0; it < DQ / 4; ++it) {
      const int d = wave * DQ + 4 * it + g4;
      const float t = src[d < r ? d : 0];
      qreg[it] = (qv0 + c16 < nqv && d < r) ? t : 0.f;
    }
  }
  int mylen[4];
  float mrun[4], lrun[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int qv = qv0 + 4 * g4 + i;
    mylen[i] = qv < nqv ? row_len[row0 + qv / H] : 0;
    mrun[i] = -INFINITY;
    lrun[i] = 0.f;
  }
  f32x4 acc[NBW];
#pragma unroll
  for (int b = 0; b < NBW; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int n_tiles = (len_max + KT - 1) / KT;
  const int t0 = blockIdx.z * tiles_per_split, t1 = min(t0 + tiles_per_split, n_tiles);
  const float* abase = arena + seq * t_max * r;
  auto fetch = [&](int tile) {
    const int k0 = tile * KT;
    load16<NBW>(v, r, tid, [&](int j) { return abase + (int64_t)min(k0 + j, len_max - 1) * r; }, [&](int j) { return k0 + j < len_max; });
  };
  if (t0 < t1) fetch(t0);
  for (int tile = t0; tile < t1; ++tile) {
    const int key0 = tile * KT;
    lds_barrier();                                             // the previous tile's latents and weights are consumed
    store16<NBW, LDC>(Cl, v, tid);
    if (tile + 1 < t1) fetch(tile + 1);                          // in flight while this tile is multiplied
    lds_barrier();
    {                                                            // partial scores over this wave's quarter of the components
      f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f}, s2 = f32x4{0.f, 0.f, 0.f, 0.f};      // two chains: a product does not wait for the one before it
      const float* cb = Cl + c16 * LDC + wave * DQ + g4;
#pragma unroll
      for (int it = 0; it < DQ / 4; it += 2) {
        s = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[it], cb[4 * it], s, 0, 0, 0);
        s2 = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[it + 1], cb[4 * it + 4], s2, 0, 0, 0);
      }
      s += s2;
#pragma unroll
      for (int i = 0; i < 4; ++i) Sp[(wave * 16 + 4 * g4 + i) * LDS_S + c16] = s[i];
    }
    lds_barrier();
    float p[4], corr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int o = (4 * g4 + i) * LDS_S + c16;
      float sc = (Sp[o] + Sp[16 * LDS_S + o]) + (Sp[32 * LDS_S + o] + Sp[48 * LDS_S + o]);
      if (key0 + c16 >= mylen[i]) sc = -INFINITY;
      const float mnew = fmaxf(mrun[i], row16_max(sc));
      p[i] = (sc == -INFINITY) ? 0.f : fast_exp(sc - mnew);
      corr[i] = (mrun[i] == -INFINITY) ? 0.f : fast_exp(mrun[i] - mnew);
      lrun[i] = lrun[i] * corr[i] + row16_sum(p[i]);
      mrun[i] = mnew;
      if (wave == 0) Pl[(4 * g4 + i) * LDP + c16] = p[i];
    }
#pragma unroll
    for (int b = 0; b < NBW; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[b][i] *= corr[i];
    lds_barrier();
    // step t multiplies keys t, t + 4, t + 8, t + 12 (lane group g4 holds key t + 4 g4): with the row stride 4 mod 32 their rows
    // start 16 banks apart pairwise, so the 64 lanes' reads spread two per bank — consecutive keys would pile four on some
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float pa = Pl[c16 * LDP + t + 4 * g4];
      const float* cb = Cl + (t + 4 * g4) * LDC + 16 * wave + c16;
#pragma unroll
      for (int b = 0; b < NBW; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa, cb[64 * b], acc[b], 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int qv = qv0 + 4 * g4 + i;
    if (qv >= nqv) continue;
    const int64_t o = (int64_t)(row0 + qv / H) * H + qv % H;
    const float inv = 1.0f / lrun[i];
#pragma unroll
    for (int b = 0; b < NBW; ++b) {
      const int d = 16 * (wave + 4 * b) + c16;
      if (d >= r) continue;
      if (KS == 1) lat[o * r + d] = acc[b][i] * inv;
      else part_acc[((int64_t)blockIdx.z * M * H + o) * r + d] = acc[b][i];
    }
    if (KS > 1 && wave == 0 && c16 == 0) {
      const int64_t po = (int64_t)blockIdx.z * M * H + o;
      part_ml[po * 2] = mrun[i];
      part_ml[po * 2 + 1] = lrun[i];
    }
  }
}

// one wave per (row, head) and 64 latent components: combine the key splits (lane s holds split s's maximum and sum; KS <= 64)
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, int KS,
                                                           int MH, int r, float* __restrict__ lat) {
  const int o = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, d = blockIdx.y * 64 + lane;
  if (o >= MH) return;
  const float ms = lane < KS ? part_ml[((int64_t)lane * MH + o) * 2] : -INFINITY;
  const float ls = lane < KS ? part_ml[((int64_t)lane * MH + o) * 2 + 1] : 0.f;
  const float mx = wave_max(ms);
  const float w = (ms == -INFINITY) ? 0.f : expf(ms - mx);
  const float inv = 1.0f / wave_sum(w * ls);
  const int dc = d < r ? d : r - 1;
  float a = 0.f;
#pragma unroll 16
  for (int s = 0; s < KS; ++s) a = fmaf(lane_f(w, s), part_acc[((int64_t)s * MH + o) * r + dc], a);
  if (d < r) lat[(int64_t)o * r + d] = a * inv;
}

}  // namespace

// ---- C entry points ----------------------------------------------------------------------------------------------------------
extern "C" int mn_affine_ln_rows(const float* x, int64_t ldx, const uint16_t* w, const uint16_t* b, float eps, float* y, int64_t ldy,
                                 uint16_t* y16, int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && b && (y || y16) && M >= 1 && n >= 1, "mn_affine_ln_rows: bad args");
  const RowArgs ra{x, ldx, nullptr, 0, nullptr, 0, w, b, eps, y, ldy, y16, ldy16, n};
  if (!launch_row_block<ROW_LN>(ra, M, mn_stream(stream)))
    hipLaunchKernelGGL(affine_ln_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), x, ldx, w, b, eps, y, ldy, y16, ldy16,
                       M, n);
  MN_CHECK_LAUNCH("mn_affine_ln_rows");
  return MN_OK;
}

extern "C" int mn_gated_ln_residual(float* x, int64_t ldx, const float* g, int64_t ldg, const float* y, int64_t ldy, const uint16_t* w,
                                    const uint16_t* b, float eps, int M, int n, void* stream) {
  MN_CHECK_ARG(x && g && y && w && b && M >= 1 && n >= 1, "mn_gated_ln_residual: bad args");
  const RowArgs ra{nullptr, 0, g, ldg, y, ldy, w, b, eps, x, ldx, nullptr, 0, n};
  if (!launch_row_block<ROW_GATED_LN_RESIDUAL>(ra, M, mn_stream(stream)))
    hipLaunchKernelGGL(gated_ln_residual_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), x, ldx, g, ldg, y, ldy, w, b,
                       eps, M, n);
  MN_CHECK_LAUNCH("mn_gated_ln_residual");
  return MN_OK;
}

extern "C" int mn_rms_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16,
                           const int32_t* row_seq, const int32_t* row_slot, int t_max, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && (y || y16) && M >= 1 && n >= 1 && (!row_seq || (row_slot && t_max >= 1)), "mn_rms_rows: bad args");
  hipLaunchKernelGGL(rms_rows_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), x, ldx, w, eps, y, ldy, y16, ldy16,
                     row_seq, row_slot, t_max, M, n);
  MN_CHECK_LAUNCH("mn_rms_rows");
  return MN_OK;
}

extern "C" int mn_polynorm_rows(const float* z, int64_t ldz, const uint16_t* coef, float eps, float* y, int64_t ldy, uint16_t* y16,
                                int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(z && coef && (y || y16) && M >= 1 && n >= 1, "mn_polynorm_rows: bad args");
  const RowArgs ra{z, ldz, nullptr, 0, nullptr, 0, coef, nullptr, eps, y, ldy, y16, ldy16, n};
  if (!launch_row_block<ROW_POLYNORM>(ra, M, mn_stream(stream)))
    hipLaunchKernelGGL(polynorm_kernel, dim3((unsigned)M), dim3(256), 0, mn_stream(stream), z, ldz, coef, eps, y, ldy, y16, ldy16, n);
  MN_CHECK_LAUNCH("mn_polynorm_rows");
  return MN_OK;
}

extern "C" int mn_tap_filter_rows(const float* x, int64_t ldx, const uint16_t* w, int taps, const float* state, const int32_t* row_seq,
                                  const int32_t* row_slot, const int32_t* row_back, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16,
                                  int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && taps >= 1 && (state || taps == 1) && row_seq && row_slot && row_back && (y || y16) && M >= 1 && n >= 1,
               "mn_tap_filter_rows: bad args");
  MN_CHECK_ARG(M <= 65535, "mn_tap_filter_rows: at most 65535 rows per call");
  hipLaunchKernelGGL(tap_filter_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, w, taps, state,
                     row_seq, row_slot, row_back, y, ldy, y16, ldy16, n, 1.0f);
  MN_CHECK_LAUNCH("mn_tap_filter_rows");
  return MN_OK;
}

extern "C" int mn_tap_conv_rows(const float* x, int64_t ldx, const uint16_t* w, int taps, const float* state, const int32_t* row_seq,
                                const int32_t* row_slot, const int32_t* row_back, float* y, int64_t ldy, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && taps >= 1 && (state || taps == 1) && row_seq && row_slot && row_back && y && M >= 1 && M <= 65535 && n >= 1,
               "mn_tap_conv_rows: bad args");
  hipLaunchKernelGGL(tap_filter_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, w, taps, state,
                     row_seq, row_slot, row_back, y, ldy, (bf16_t*)nullptr, (int64_t)0, n, 0.0f);
  MN_CHECK_LAUNCH("mn_tap_conv_rows");
  return MN_OK;
}

extern "C" int mn_tap_state_update(const float* x, int64_t ldx, int taps, float* state, const int32_t* row_seq, const int32_t* row_back,
                                   int M, int n, void* stream) {
  MN_CHECK_ARG(x && taps >= 1 && row_seq && row_back && M >= 1 && M <= 65535 && n >= 1, "mn_tap_state_update: bad args");
  if (taps == 1) return MN_OK;
  MN_CHECK_ARG(state, "mn_tap_state_update: null state");
  hipLaunchKernelGGL(tap_state_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, taps, state,
                     row_seq, row_back, M, n);
  MN_CHECK_LAUNCH("mn_tap_state_update");
  return MN_OK;
}

extern "C" int mn_gated_norm_filter_rows(float* x, int64_t ldx, const float* g, int64_t ldg, const float* y, int64_t ldy, const uint16_t* wa,
                                         const uint16_t* ba, const uint16_t* wb, const uint16_t* bb, float eps, float* n_out, int64_t ldn,
                                         const uint16_t* taps_w, int taps, float* state, const int32_t* row_seq, const int32_t* row_slot,
                                         float* h, int64_t ldh, int M, int n, void* stream) {
  MN_CHECK_ARG(x && wb && bb && n_out && M >= 1 && n >= 1 && n <= 4096, "mn_gated_norm_filter_rows: bad args (rows of at most 4096 values)");
  MN_CHECK_ARG(!g || (y && wa && ba), "mn_gated_norm_filter_rows: the gated stage needs y and its norm");
  MN_CHECK_ARG(!h || (taps_w && taps >= 1 && taps <= FUSED_MAX_TAPS && (state || taps == 1) && row_seq && row_slot),
               "mn_gated_norm_filter_rows: the filter stage needs its state and at most %d taps", FUSED_MAX_TAPS);
  const FusedRowArgs a{x, ldx, g, ldg, y, ldy, wa, ba, wb, bb, eps, n_out, ldn, taps_w, taps, state, row_seq, row_slot, h, ldh, n};
  const int vpt = (n + 255) / 256;
  hipStream_t st = mn_stream(stream);
#define MN_RF(V_)                                                                                                    \
  do {                                                                                                               \
    if (h) hipLaunchKernelGGL((row_fused_kernel<V_, true>), dim3((unsigned)M), dim3(256), 0, st, a);                 \
    else hipLaunchKernelGGL((row_fused_kernel<V_, false>), dim3((unsigned)M), dim3(256), 0, st, a);                  \
  } while (0)
  if (vpt <= 1) MN_RF(1); else if (vpt <= 2) MN_RF(2); else if (vpt <= 4) MN_RF(4); else if (vpt <= 8) MN_RF(8); else MN_RF(16);
#undef MN_RF
  MN_CHECK_LAUNCH("mn_gated_norm_filter_rows");
  return MN_OK;
}

extern "C" int mn_softcap_rows(float* z, int64_t ld, int M, int n, float cap, void* stream) {
  MN_CHECK_ARG(z && M >= 1 && M <= 65535 && n >= 1 && cap > 0.f, "mn_softcap_rows: bad args");
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), z, ld, n, cap);
  MN_CHECK_LAUNCH("mn_softcap_rows");
  return MN_OK;
}

extern "C" int mn_gemm_f32_batched(const float* A, int64_t lda, int64_t a_bs, const uint16_t* W, int64_t ldw, int64_t w_bs,
                                   const uint16_t* bias, float* C, int64_t ldc, int64_t c_bs, uint16_t* C16, int64_t ldc16, int64_t c16_bs,
                                   const float* G, int64_t ldg, int64_t g_bs, int M, int N, int K, int batch, float alpha, void* stream) {
  MN_CHECK_ARG(A && W && (C || C16) && M >= 1 && N >= 1 && K >= 1 && batch >= 1 && batch <= 65535, "mn_gemm_f32_batched: bad args");
  GemmF32 a{A, lda, a_bs, W, ldw, w_bs, bias, C, ldc, c_bs, C16, ldc16, c16_bs, G, ldg, g_bs, M, N, K, alpha};
  hipStream_t st = mn_stream(stream);
  if (M <= 64) {                                         // decode-sized steps: the weights of a head are a few hundred KiB, rows in groups of 8
    if (M <= 2) hipLaunchKernelGGL((gemv_f32_kernel<2>), dim3((unsigned)mn_cdiv(N, 4), 1, (unsigned)batch), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemv_f32_kernel<8>), dim3((unsigned)mn_cdiv(N, 4), (unsigned)mn_cdiv(M, 8), (unsigned)batch), dim3(256), 0, st, a);
  } else if (M <= 16) {
    hipLaunchKernelGGL((gemm_f32_kernel<1>), dim3((unsigned)mn_cdiv(N, 64), 1, (unsigned)batch), dim3(256), 0, st, a);
  } else {
    MN_CHECK_ARG(mn_cdiv(M, 64) <= 65535, "mn_gemm_f32_batched: too many rows");
    hipLaunchKernelGGL((gemm_f32_kernel<4>), dim3((unsigned)mn_cdiv(N, 64), (unsigned)mn_cdiv(M, 64), (unsigned)batch), dim3(256), 0, st, a);
  }
  MN_CHECK_LAUNCH("mn_gemm_f32_batched");
  return MN_OK;
}

// rows of a workgroup (consecutive rows of one sequence) and the key-tile length for latent size r
extern "C" int mn_latent_attn_block_rows(void) { return 4; }
static inline int latent_kt(int r, int variant) { return variant == MN_LATENT_ATTN_VALU ? (r <= 256 ? 64 : r <= 512 ? 32 : 16) : 16; }   // VALU: the tile [KT][r + 1] fp32 stays below 66 KiB

extern "C" int mn_latent_attn_splits(int n_blk, int max_len, int r) {
  const int tiles = (int)mn_cdiv(max_len > 0 ? max_len : 1, 16);
  int ks = (int)mn_cdiv(2 * (int64_t)mn_num_cus(), n_blk > 0 ? n_blk : 1);
  const int cap = (int)mn_cdiv(tiles, 4);              // a split works on at least 64 keys
  if (ks > cap) ks = cap;
  if (ks > 64) ks = 64;
  (void)r;
  return ks < 1 ? 1 : ks;
}

extern "C" size_t mn_latent_attn_workspace_bytes(int M, int H, int r, int ks) {
  return ks <= 1 ? 0 : (size_t)ks * M * H * (r + 2) * sizeof(float);
}

extern "C" int mn_latent_attn_ex(const float* qabs, const float* arena, const int32_t* row_seq, const int32_t* row_len,
                                 const int32_t* blk_tab, int n_blk, int M, int H, int r, int t_max, int max_len, int ks, float* lat, void* ws,
                                 size_t ws_bytes, int variant, void* stream) {
  MN_CHECK_ARG(qabs && arena && row_seq && row_len && blk_tab && lat && n_blk >= 1 && M >= 1 && H >= 1 && r >= 1 && t_max >= 1,
               "mn_latent_attn: bad args");
  MN_CHECK_ARG(r <= 1024, "mn_latent_attn: latent size %d above 1024 is not supported", r);
  MN_CHECK_ARG(max_len >= 1 && max_len <= t_max && ks >= 1 && ks <= 64, "mn_latent_attn: bad max_len=%d / ks=%d (1 .. 64 key splits)", max_len, ks);
  MN_CHECK_ARG(ws_bytes >= mn_latent_attn_workspace_bytes(M, H, r, ks) && (ks == 1 || ws), "mn_latent_attn: workspace too small");
  MN_CHECK_ARG(variant == MN_LATENT_ATTN_MFMA || variant == MN_LATENT_ATTN_VALU, "mn_latent_attn: unknown variant %d", variant);
  const int KT = latent_kt(r, variant), RB = mn_latent_attn_block_rows();
  const int tiles = (int)mn_cdiv(max_len, KT), tps = (int)mn_cdiv(tiles, ks);
  float* pacc = reinterpret_cast<float*>(ws);
  float* pml = pacc ? pacc + (size_t)ks * M * H * r : nullptr;
  hipStream_t st = mn_stream(stream);
  if (variant == MN_LATENT_ATTN_MFMA) {
    const int nbw = (int)mn_cdiv(r, 64);
    const int inst = nbw <= 4 ? nbw : nbw <= 6 ? 6 : nbw <= 8 ? 8 : nbw <= 12 ? 12 : 16;      // instantiated paddings: 64 .. 256, 384, 512, 768, 1024
    const size_t lds = ((size_t)16 * (64 * inst + 4) + 4 * 16 * 17 + 16 * 20) * sizeof(float);
    const dim3 grid((unsigned)n_blk, (unsigned)mn_cdiv(RB * H, 16), (unsigned)ks);
    MN_CHECK_ARG(grid.y <= 65535 && ks <= 64, "mn_latent_attn: too many heads or key splits");
#define MN_LM(N_)                                                                                                                   \
  do {                                                                                                                              \
    static bool attr_set = false;                                                                                                   \
    if (!attr_set) {                                                                                                                \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(latent_attn_mfma_kernel<N_>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                144 * 1024);                                                                                        \
      attr_set = true;                                                                                                              \
    }                                                                                                                               \
    hipLaunchKernelGGL((latent_attn_mfma_kernel<N_>), grid, dim3(256), lds, st, qabs, arena, row_seq, row_len, blk_tab, H, r, t_max, tps, \
                       lat, pacc, pml, ks, M);                                                                                      \
  } while (0)
    switch (inst) {
      case 1: MN_LM(1); break; case 2: MN_LM(2); break; case 3: MN_LM(3); break; case 4: MN_LM(4); break;
      case 6: MN_LM(6); break; case 8: MN_LM(8); break; case 12: MN_LM(12); break; default: MN_LM(16); break;
    }
#undef MN_LM
  } else {
    const int nw = RB * H < 16 ? RB * H : 16;
    const dim3 grid((unsigned)n_blk, (unsigned)mn_cdiv(RB * H, nw), (unsigned)ks), block((unsigned)(64 * nw));
    MN_CHECK_ARG(grid.y <= 65535, "mn_latent_attn: too many heads");
    const size_t lds = (size_t)KT * (r + 1) * sizeof(float);
#define MN_LA(R_)                                                                                                                   \
  do {                                                                                                                              \
    static bool attr_set = false;                                                                                                   \
    if (!attr_set) {                                                                                                                \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(latent_attn_kernel<R_>), hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024); \
      attr_set = true;                                                                                                              \
    }                                                                                                                               \
    hipLaunchKernelGGL((latent_attn_kernel<R_>), grid, block, lds, st, qabs, arena, row_seq, row_len, blk_tab, H, r, t_max, KT, tps, lat, \
                       pacc, pml, ks, M);                                                                                           \
  } while (0)
    if (r <= 64) MN_LA(1); else if (r <= 128) MN_LA(2); else if (r <= 256) MN_LA(4); else if (r <= 512) MN_LA(8); else MN_LA(16);
#undef MN_LA
  }
  MN_CHECK_LAUNCH("mn_latent_attn");
  if (ks > 1) {
    hipLaunchKernelGGL(latent_merge_kernel, dim3((unsigned)mn_cdiv((int64_t)M * H, 4), (unsigned)mn_cdiv(r, 64)), dim3(256), 0, st, pacc, pml, ks, M * H, r,
                       lat);
    MN_CHECK_LAUNCH("mn_latent_attn(merge)");
  }
  return MN_OK;
}

extern "C" int mn_latent_attn(const float* qabs, const float* arena, const int32_t* row_seq, const int32_t* row_len, const int32_t* blk_tab,
                              int n_blk, int M, int H, int r, int t_max, int max_len, int ks, float* lat, void* ws, size_t ws_bytes,
                              void* stream) {
  return mn_latent_attn_ex(qabs, arena, row_seq, row_len, blk_tab, n_blk, M, H, r, t_max, max_len, ks, lat, ws, ws_bytes,
                           MN_LATENT_ATTN_MFMA, stream);
}
