// latent_engine.hip — the step function of latent-cache sequence models (mingnative.h section 9): one pass of the layer stack
// over the rows of a step as a chain of launches on the caller's stream.  Matrix products are routed per call:
//   M <= 8 rows                      mn_skinny_gemm (weight streaming, fp32 FMA) — the decode route of the other decoder too
//   MN_SEQ_ARITH_BF16, 9 .. 64 rows  mn_skinny_gemm's weight-streaming MFMA route on bf16 hi/lo rows (fp32-class products)
//   MN_SEQ_ARITH_BF16, M > 64        mn_gemm_bf16 on the bf16 copy the producing kernel wrote (MFMA, fp32 accumulate)
//   MN_SEQ_ARITH_F32, or a K that is no multiple of 8 / an unaligned weight: mn_gemm_f32_batched (fp32 FMA tiles)
// The per-head absorb (q W_uk) and expand (latent W_uv^T) products are batched over heads on the fp32 FMA kernel in both modes.
#include "seq_linear.h"

extern "C" size_t mn_sizeof_seq_layer(void) { return sizeof(mn_seq_layer); }
extern "C" size_t mn_sizeof_seq_model(void) { return sizeof(mn_seq_model); }
extern "C" size_t mn_sizeof_seq_state(void) { return sizeof(mn_seq_state); }

namespace {

struct Dims {
  int n_in, hd, hv, hr, q_rank, ff;
};

Dims layer_dims(const mn_seq_layer& l) {
  Dims d;
  d.hd = l.heads * l.dim; d.hv = l.heads * l.vdim; d.hr = l.heads * l.kv_rank;
  d.q_rank = l.kind == MN_SEQ_MIX_LATENT_Q ? l.q_rank : 0;
  d.n_in = (l.kind == MN_SEQ_MIX_LATENT_Q ? l.q_rank : d.hd + d.hv) + (l.writes_arena ? l.kv_rank : 0);
  d.ff = l.ff;
  return d;
}

struct Plan {
  int n_in = 1, hd = 1, hv = 1, hr = 1, q_rank = 1, ff = 1;
  size_t attn_ws = 0, gemm_ws = 0;
};

Plan make_plan(const mn_seq_model* m, int M, int max_len) {
  Plan p;
  const int RB = mn_latent_attn_block_rows();
  for (int i = 0; i < m->n_layers; ++i) {
    const mn_seq_layer& l = m->layers[i];
    const Dims d = layer_dims(l);
    if (d.n_in > p.n_in) p.n_in = d.n_in;
    if (d.hd > p.hd) p.hd = d.hd;
    if (d.hv > p.hv) p.hv = d.hv;
    if (d.hr > p.hr) p.hr = d.hr;
    if (d.q_rank > p.q_rank) p.q_rank = d.q_rank;
    if (d.ff > p.ff) p.ff = d.ff;
    // the workspace covers the finest cut of the rows (one run per row) and the most key splits that cut can ask for
    const int ks = mn_latent_attn_splits((int)mn_cdiv(M, RB), max_len, l.kv_rank);
    const size_t w = mn_latent_attn_workspace_bytes(M, l.heads, l.kv_rank, ks);
    if (w > p.attn_ws) p.attn_ws = w;
    if (m->arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64) {       // scratch of the weight-streaming MFMA route: the largest product of the stack
      const int W = m->width;
      const int shapes[6][2] = {{W, W}, {d.n_in, W}, {d.hd, d.q_rank}, {W, d.hv}, {W + d.ff, W}, {W, d.ff}};
      for (const auto& nk : shapes) {
        if (nk[0] < 1 || nk[1] < 8 || (nk[1] % 8) != 0) continue;
        const size_t g = mn_skinny_workspace_bytes(M, nk[0], nk[1], MN_EPI_NONE);
        if (g > p.gemm_ws) p.gemm_ws = g;
      }
    }
  }
  return p;
}

}  // namespace

extern "C" size_t mn_seq_workspace_bytes(const mn_seq_model* m, int M, int max_len) {
  if (!m || !m->layers || M < 1) return 0;
  const Plan p = make_plan(m, M, max_len);
  const size_t W = m->width, R = (size_t)M;
  size_t n = 0;
  n += al(R * W * 4);                       // residual
  n += al(R * W * 4) + al(R * W * 2);       // normed rows + bf16
  n += al(R * W * 4);                       // gate pre-activation of the mixer
  n += al(R * W * 4) + al(R * W * 2);       // filtered rows + bf16
  n += al(R * p.n_in * 4);                  // stacked input projections
  n += al(R * p.q_rank * 4) + al(R * p.q_rank * 2);
  n += al(R * p.hd * 4);                    // queries
  n += 2 * al(R * p.hr * 4);                // absorbed queries, attended latents
  n += al(R * p.hv * 4) + al(R * p.hv * 2); // expanded heads + bf16
  n += al(R * W * 4);                       // sublayer result
  n += al(R * (W + p.ff) * 4);              // [gate pre-activation ; up] of the feed-forward
  n += al(R * p.ff * 4) + al(R * p.ff * 2); // activation + bf16
  n += al(p.attn_ws) + al(p.gemm_ws);
  return n;
}

extern "C" int mn_seq_step(const mn_seq_model* m, const mn_seq_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                           const int32_t* row_slot, const int32_t* row_back, const int32_t* row_len, const int32_t* blk_tab, int n_blk,
                           int max_len, int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(m && st && m->layers && st->latent && x && row_seq && row_slot && row_back && row_len && blk_tab && out && workspace,
               "mn_seq_step: null pointer");
  MN_CHECK_ARG(M >= 1 && M <= 65535 && n_blk >= 1 && n_blk <= M && m->width >= 1 && m->n_layers >= 1 && m->taps >= 1,
               "mn_seq_step: bad sizes (M=%d n_blk=%d)", M, n_blk);
  MN_CHECK_ARG(max_len >= 1 && max_len <= st->t_max, "mn_seq_step: max_len=%d outside the arena (t_max=%d)", max_len, st->t_max);
  MN_CHECK_ARG(m->taps == 1 || st->taps, "mn_seq_step: null filter state");
  MN_CHECK_ARG(workspace_bytes >= mn_seq_workspace_bytes(m, M, max_len), "mn_seq_step: workspace too small");
  const Plan p = make_plan(m, M, max_len);
  const int W = m->width, arith = m->arith;
  const size_t R = (size_t)M;
  const bool want16 = arith == MN_SEQ_ARITH_BF16 && M > 64;       // bf16 copies feed the tiled MFMA GEMM only
  char* wp = reinterpret_cast<char*>(workspace);
  auto take = [&](size_t bytes) { char* q = wp; wp += al(bytes); return q; };
  float* xr = (float*)take(R * W * 4);
  float* n1 = (float*)take(R * W * 4);
  uint16_t* n1h = (uint16_t*)take(R * W * 2);
  float* g1 = (float*)take(R * W * 4);
  float* hf = (float*)take(R * W * 4);
  uint16_t* hh = (uint16_t*)take(R * W * 2);
  float* pin = (float*)take(R * p.n_in * 4);
  float* cq = (float*)take(R * p.q_rank * 4);
  uint16_t* cqh = (uint16_t*)take(R * p.q_rank * 2);
  float* qf = (float*)take(R * p.hd * 4);
  float* qabs = (float*)take(R * p.hr * 4);
  float* lat = (float*)take(R * p.hr * 4);
  float* att = (float*)take(R * p.hv * 4);
  uint16_t* atth = (uint16_t*)take(R * p.hv * 2);
  float* yf = (float*)take(R * W * 4);
  float* fin = (float*)take(R * (W + p.ff) * 4);
  float* af = (float*)take(R * p.ff * 4);
  uint16_t* afh = (uint16_t*)take(R * p.ff * 2);
  void* attn_ws = p.attn_ws ? take(p.attn_ws) : nullptr;
  void* gws = p.gemm_ws ? take(p.gemm_ws) : nullptr;
  const size_t gwb = p.gemm_ws;
  if (!want16) n1h = hh = cqh = atth = afh = nullptr;
  hipStream_t hs = mn_stream(stream);
  int rc;
#define MN_TRY(call) do { rc = (call); if (rc != MN_OK) return rc; } while (0)
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, x, ldx, xr, W);
  MN_CHECK_LAUNCH("mn_seq_step(copy)");
  const size_t taps_layer = (size_t)st->n_seq * (m->taps - 1) * W;
  // A sublayer ends with x += LN(sigmoid(g) y) and the next one starts with LN(x) (+ the tap filter in front of a mixer).  On decode
  // steps (MN_SEQ_ROWS_DISTINCT, no bf16 copies wanted) the end of one and the start of the next are ONE launch; otherwise the
  // operators run one by one.  `pend` is a sublayer end that has not been applied to x yet.
  const bool fuse = (flags & MN_SEQ_ROWS_DISTINCT) && !want16 && W <= 4096 && m->taps <= 8 && !trace;
  struct Pending { const float* g = nullptr; int64_t ldg = 0; const uint16_t *w = nullptr, *b = nullptr; } pend;
  // n_out = LN(x; wb, bb) after applying `pend`; with tstate / h_out also h = n + filter(n) and the state update
  auto norm_stage = [&](const uint16_t* wb, const uint16_t* bb, float* n_out, uint16_t* n16, const uint16_t* taps_w, float* tstate,
                        float* h_out, uint16_t* h16) -> int {
    if (fuse) {
      const int rc2 = mn_gated_norm_filter_rows(xr, W, pend.g, pend.ldg, yf, W, pend.w, pend.b, wb, bb, m->eps, n_out, W, taps_w, m->taps, tstate,
                                                row_seq, row_slot, h_out, W, M, W, stream);
      pend = Pending();
      return rc2;
    }
    int rc2 = MN_OK;
    if (pend.g) rc2 = mn_gated_ln_residual(xr, W, pend.g, pend.ldg, yf, W, pend.w, pend.b, m->eps, M, W, stream);
    pend = Pending();
    if (rc2 == MN_OK) rc2 = mn_affine_ln_rows(xr, W, wb, bb, m->eps, n_out, W, n16, W, M, W, stream);
    if (rc2 == MN_OK && h_out) rc2 = mn_tap_filter_rows(n_out, W, taps_w, m->taps, tstate, row_seq, row_slot, row_back, h_out, W, h16, W, M, W, stream);
    if (rc2 == MN_OK && h_out) rc2 = mn_tap_state_update(n_out, W, m->taps, tstate, row_seq, row_back, M, W, stream);
    return rc2;
  };
  for (int li = 0; li < m->n_layers; ++li) {
    const mn_seq_layer& l = m->layers[li];
    const Dims d = layer_dims(l);
    MN_CHECK_ARG(l.heads >= 1 && l.dim >= 1 && l.vdim >= 1 && l.kv_rank >= 1 && (l.kind == MN_SEQ_MIX_LATENT_Q || l.kind == MN_SEQ_MIX_GATED),
                 "mn_seq_step: layer %d: bad mixer", li);
    float* arena = st->latent[l.arena];
    float* tstate = st->taps ? st->taps + (size_t)li * taps_layer : nullptr;
    // ---- mixer sublayer ----
    MN_TRY(norm_stage(l.norm1_w, l.norm1_b, n1, n1h, l.taps_w, tstate, hf, hh));
    MN_TRY(linear(arith, M, n1, W, n1h, W, l.rg1_w, W, W, l.rg1_b, g1, W, gws, gwb, stream));
    MN_TRY(linear(arith, M, hf, W, hh, W, l.w_in, d.n_in, W, nullptr, pin, d.n_in, gws, gwb, stream));
    const float* qp; int64_t ldq; const float* gp = nullptr; int kv_off;
    if (l.kind == MN_SEQ_MIX_LATENT_Q) {
      MN_TRY(mn_rms_rows(pin, d.n_in, l.q_norm, m->eps, cq, l.q_rank, cqh, l.q_rank, nullptr, nullptr, 0, M, l.q_rank, stream));
      MN_TRY(linear(arith, M, cq, l.q_rank, cqh, l.q_rank, l.w_uq, d.hd, l.q_rank, nullptr, qf, d.hd, gws, gwb, stream));
      qp = qf; ldq = d.hd; kv_off = l.q_rank;
    } else {
      qp = pin; ldq = d.n_in; gp = pin + d.hd; kv_off = d.hd + d.hv;
    }
    if (l.writes_arena)
      MN_TRY(mn_rms_rows(pin + kv_off, d.n_in, l.kv_norm, m->eps, arena, l.kv_rank, nullptr, 0, row_seq, row_slot, st->t_max, M, l.kv_rank,
                         stream));
    // absorb: qabs[m, h, :] = scale * q[m, h, :] W_uk[h]   (W_ukT[h] is [kv_rank, dim])
    MN_TRY(mn_gemm_f32_batched(qp, ldq, l.dim, l.w_ukT, l.dim, (int64_t)l.kv_rank * l.dim, nullptr, qabs, d.hr, l.kv_rank, nullptr, 0, 0,
                               nullptr, 0, 0, M, l.kv_rank, l.dim, l.heads, l.scale, stream));
    const int ks = mn_latent_attn_splits(n_blk, max_len, l.kv_rank);
    MN_TRY(mn_latent_attn(qabs, arena, row_seq, row_len, blk_tab, n_blk, M, l.heads, l.kv_rank, st->t_max, max_len, ks, lat, attn_ws,
                          p.attn_ws, stream));
    // expand: att[m, h, :] = W_uv[h] lat[m, h, :]  (* sigmoid(gate))
    MN_TRY(mn_gemm_f32_batched(lat, d.hr, l.kv_rank, l.w_uv, l.kv_rank, (int64_t)l.vdim * l.kv_rank, nullptr, att, d.hv, l.vdim, atth, d.hv,
                               l.vdim, gp, d.n_in, l.vdim, M, l.vdim, l.kv_rank, l.heads, 1.0f, stream));
    MN_TRY(linear(arith, M, att, d.hv, atth, d.hv, l.w_o, W, d.hv, nullptr, yf, W, gws, gwb, stream));
    pend.g = g1; pend.ldg = W; pend.w = l.norm1b_w; pend.b = l.norm1b_b;
    // ---- feed-forward sublayer ----
    if (l.ff > 0) {
      const int nf = W + l.ff;
      MN_TRY(norm_stage(l.norm2_w, l.norm2_b, n1, n1h, nullptr, nullptr, nullptr, nullptr));
      MN_TRY(linear(arith, M, n1, W, n1h, W, l.w_ff_in, nf, W, l.b_ff_in, fin, nf, gws, gwb, stream));
      MN_TRY(mn_polynorm_rows(fin + W, nf, l.act, m->eps, af, l.ff, afh, l.ff, M, l.ff, stream));
      MN_TRY(linear(arith, M, af, l.ff, afh, l.ff, l.w_down, W, l.ff, nullptr, yf, W, gws, gwb, stream));
      pend.g = fin; pend.ldg = nf; pend.w = l.norm2b_w; pend.b = l.norm2b_b;
    }
    if (trace) {                                       // the trace wants x after the whole layer: apply the layer's last sublayer end now
      MN_TRY(mn_gated_ln_residual(xr, W, pend.g, pend.ldg, yf, W, pend.w, pend.b, m->eps, M, W, stream));
      pend = Pending();
      const hipError_t e = hipMemcpyAsync(trace + (size_t)li * R * W, xr, R * W * 4, hipMemcpyDeviceToDevice, hs);
      if (e != hipSuccess) { mn_set_error("mn_seq_step: trace copy: %s", hipGetErrorString(e)); return MN_ELAUNCH; }
    }
  }
  MN_TRY(norm_stage(m->final_w, m->final_b, out, nullptr, nullptr, nullptr, nullptr, nullptr));
#undef MN_TRY
  return MN_OK;
}

extern "C" int mn_seq_logits(const float* hidden, int64_t ldh, int M, const uint16_t* Wt, int V, int K, float cap, int arith, float* out,
                             int64_t ldo, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(hidden && Wt && out && M >= 1 && V >= 1 && K >= 1, "mn_seq_logits: bad args");
  const uint16_t* h16 = nullptr;
  if (arith == MN_SEQ_ARITH_BF16 && M > 8 && mfma_ok(Wt, K) && workspace && workspace_bytes >= (size_t)M * K * 2 && ldh == K &&
      (((uintptr_t)workspace) & 15) == 0) {
    const int rc = mn_f32_to_bf16(hidden, (uint16_t*)workspace, (int64_t)M * K, stream);
    if (rc != MN_OK) return rc;
    h16 = (const uint16_t*)workspace;
  }
  int rc = linear(arith, M, hidden, ldh, h16, K, Wt, V, K, nullptr, out, ldo, nullptr, 0, stream);
  if (rc != MN_OK) return rc;
  if (cap > 0.f) rc = mn_softcap_rows(out, ldo, M, V, cap, stream);
  return rc;
}
