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

// y[m, c] = x[m, c] + sum_k w[c, taps - 1 - k] * (the sequence's input k positions back); grid (ceil(n / 256), M)
__global__ __launch_bounds__(256) void tap_filter_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int taps,
                                                         const float* __restrict__ state, const int32_t* __restrict__ row_seq,
                                                         const int32_t* __restrict__ row_slot, const int32_t* __restrict__ row_back,
                                                         float* __restrict__ y, int64_t ldy, bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const int seq = row_seq[m], slot = row_slot[m], back = row_back[m];
  const float cur = x[(int64_t)m * ldx + c];
  float acc = cur;
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

// one wave per (row, head): combine the key splits
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, int KS,
                                                           int MH, int r, float* __restrict__ lat) {
  const int o = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (o >= MH) return;
  float mx = -INFINITY;
  for (int s = 0; s < KS; ++s) mx = fmaxf(mx, part_ml[((int64_t)s * MH + o) * 2]);
  float L = 0.f;
  for (int s = 0; s < KS; ++s) {
    const float ms = part_ml[((int64_t)s * MH + o) * 2];
    if (ms != -INFINITY) L += expf(ms - mx) * part_ml[((int64_t)s * MH + o) * 2 + 1];
  }
  for (int d = lane; d < r; d += 64) {
    float a = 0.f;
    for (int s = 0; s < KS; ++s) {
      const float ms = part_ml[((int64_t)s * MH + o) * 2];
      if (ms != -INFINITY) a += expf(ms - mx) * part_acc[((int64_t)s * MH + o) * r + d];
    }
    lat[(int64_t)o * r + d] = a / L;
  }
}

}  // namespace

// ---- C entry points ----------------------------------------------------------------------------------------------------------
extern "C" int mn_affine_ln_rows(const float* x, int64_t ldx, const uint16_t* w, const uint16_t* b, float eps, float* y, int64_t ldy,
                                 uint16_t* y16, int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && b && (y || y16) && M >= 1 && n >= 1, "mn_affine_ln_rows: bad args");
  hipLaunchKernelGGL(affine_ln_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), x, ldx, w, b, eps, y, ldy, y16, ldy16,
                     M, n);
  MN_CHECK_LAUNCH("mn_affine_ln_rows");
  return MN_OK;
}

extern "C" int mn_gated_ln_residual(float* x, int64_t ldx, const float* g, int64_t ldg, const float* y, int64_t ldy, const uint16_t* w,
                                    const uint16_t* b, float eps, int M, int n, void* stream) {
  MN_CHECK_ARG(x && g && y && w && b && M >= 1 && n >= 1, "mn_gated_ln_residual: bad args");
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
                     row_seq, row_slot, row_back, y, ldy, y16, ldy16, n);
  MN_CHECK_LAUNCH("mn_tap_filter_rows");
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
  if (M <= 16) {
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
static inline int latent_kt(int r) { return r <= 256 ? 64 : r <= 512 ? 32 : 16; }   // the tile [KT][r + 1] fp32 stays below 66 KiB

extern "C" int mn_latent_attn_splits(int n_blk, int max_len, int r) {
  const int KT = latent_kt(r);
  const int tiles = (int)mn_cdiv(max_len > 0 ? max_len : 1, KT);
  int ks = (int)mn_cdiv(2 * (int64_t)mn_num_cus(), n_blk > 0 ? n_blk : 1);
  const int cap = (int)mn_cdiv(tiles, 2);              // a split works on at least 2 key tiles
  if (ks > cap) ks = cap;
  if (ks > 64) ks = 64;
  return ks < 1 ? 1 : ks;
}

extern "C" size_t mn_latent_attn_workspace_bytes(int M, int H, int r, int ks) {
  return ks <= 1 ? 0 : (size_t)ks * M * H * (r + 2) * sizeof(float);
}

extern "C" int mn_latent_attn(const float* qabs, const float* arena, const int32_t* row_seq, const int32_t* row_len, const int32_t* blk_tab,
                              int n_blk, int M, int H, int r, int t_max, int max_len, int ks, float* lat, void* ws, size_t ws_bytes,
                              void* stream) {
  MN_CHECK_ARG(qabs && arena && row_seq && row_len && blk_tab && lat && n_blk >= 1 && M >= 1 && H >= 1 && r >= 1 && t_max >= 1,
               "mn_latent_attn: bad args");
  MN_CHECK_ARG(r <= 1024, "mn_latent_attn: latent size %d above 1024 is not supported", r);
  MN_CHECK_ARG(max_len >= 1 && max_len <= t_max && ks >= 1 && ks <= 65535, "mn_latent_attn: bad max_len=%d / ks=%d", max_len, ks);
  MN_CHECK_ARG(ws_bytes >= mn_latent_attn_workspace_bytes(M, H, r, ks) && (ks == 1 || ws), "mn_latent_attn: workspace too small");
  const int KT = latent_kt(r), RB = mn_latent_attn_block_rows();
  const int tiles = (int)mn_cdiv(max_len, KT), tps = (int)mn_cdiv(tiles, ks);
  const int nw = RB * H < 16 ? RB * H : 16;
  const dim3 grid((unsigned)n_blk, (unsigned)mn_cdiv(RB * H, nw), (unsigned)ks), block((unsigned)(64 * nw));
  MN_CHECK_ARG(grid.y <= 65535, "mn_latent_attn: too many heads");
  const size_t lds = (size_t)KT * (r + 1) * sizeof(float);
  float* pacc = reinterpret_cast<float*>(ws);
  float* pml = pacc ? pacc + (size_t)ks * M * H * r : nullptr;
  hipStream_t st = mn_stream(stream);
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
  MN_CHECK_LAUNCH("mn_latent_attn");
  if (ks > 1) {
    hipLaunchKernelGGL(latent_merge_kernel, dim3((unsigned)mn_cdiv((int64_t)M * H, 4)), dim3(256), 0, st, pacc, pml, ks, M * H, r, lat);
    MN_CHECK_LAUNCH("mn_latent_attn(merge)");
  }
  return MN_OK;
}
