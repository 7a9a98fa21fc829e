// pmix_engine.hip — the step function of parallel-mixer sequence models (mingnative.h section 10): one pass of the layer runs over
// the rows of a step as a chain of launches on the caller's stream.  Matrix products go through the routing of seq_linear.h; the
// experts of a mixture-of-experts feed-forward run
//   MN_SEQ_ARITH_BF16, M > 8    sorted by expert on a grouped bf16 MFMA GEMM: the 256 x 256-tile kernel over the list of live row tiles
//                               (mn_moe_sort_tiles, mn_gemm256_grouped_tiles: rows gathered while staging, SwiGLU in the gate / up
//                               epilogue) when width and expert width are multiples of 64, else the 128-tile kernel
//                               (mn_moe_sort, mn_gather_rows_bf16, mn_gemm_bf16_grouped) when they are multiples of 8
//   otherwise                   one (row, pick) pair at a time against the weights its index names (mn_gemv_f32_indexed, fp32 FMA)
#include "seq_linear.h"

extern "C" size_t mn_sizeof_pmix_layer(void) { return sizeof(mn_pmix_layer); }
extern "C" size_t mn_sizeof_pmix_model(void) { return sizeof(mn_pmix_model); }
extern "C" size_t mn_sizeof_pmix_state(void) { return sizeof(mn_pmix_state); }

namespace {

struct PDims {
  int cq, ck, cv, cqkv, n_in, n_cat, n_ff_in, pairs_cols;
};

PDims pdims(const mn_pmix_layer& l) {
  PDims d;
  d.cq = l.heads * l.dim; d.ck = l.kv_heads * l.dim; d.cv = l.kv_heads * l.vdim;
  d.cqkv = d.cq + d.ck + d.cv;
  d.n_in = d.cqkv + 3 * l.gru;
  d.n_cat = l.heads * l.vdim + l.gru;
  d.n_ff_in = l.experts > 0 ? (2 * l.shared_ff + l.experts + (l.shared_ff > 0 ? 1 : 0) + 7) / 8 * 8 : 0;    // zero rows pad the stack to a multiple of 8
  return d;
}

struct PPlan {
  int n_in = 1, cqkv = 1, cq = 1, n_cat = 1, n_ff_in = 1, sff = 1, top = 1, ff = 1, experts = 1;
  size_t gemm_ws = 0, attn_ws = 0, gru_ws = 0;
};

enum { EXPERTS_INDEXED = 0, EXPERTS_GROUPED = 1, EXPERTS_TILES = 2 };
int expert_route(const mn_pmix_model* m, const mn_pmix_layer& l, int M) {
  if (m->arith != MN_SEQ_ARITH_BF16 || M <= 8 || l.experts > 128 || (int64_t)M * l.top > 65536 ||
      ((((uintptr_t)l.w_gate_up) | ((uintptr_t)l.w_down)) & 15) != 0)
    return EXPERTS_INDEXED;
  const int64_t W = m->width, ff = l.ff;
  if ((W % 64) == 0 && (ff % 64) == 0 && 2 * ff * W * 2 < ((int64_t)1 << 32) && (int64_t)M * l.top * (W > ff ? W : ff) * 2 < ((int64_t)1 << 32))
    return EXPERTS_TILES;
  if ((W % 8) == 0 && (ff % 8) == 0) return EXPERTS_GROUPED;
  return EXPERTS_INDEXED;
}

PPlan make_plan(const mn_pmix_model* m, int M) {
  PPlan p;
  for (int i = 0; i < m->n_layers; ++i) {
    const mn_pmix_layer& l = m->layers[i];
    const PDims d = pdims(l);
    if (d.n_in > p.n_in) p.n_in = d.n_in;
    if (d.cqkv > p.cqkv) p.cqkv = d.cqkv;
    if (d.cq > p.cq) p.cq = d.cq;
    if (d.n_cat > p.n_cat) p.n_cat = d.n_cat;
    if (d.n_ff_in > p.n_ff_in) p.n_ff_in = d.n_ff_in;
    if (l.shared_ff > p.sff) p.sff = l.shared_ff;
    if (l.top > p.top) p.top = l.top;
    if (l.ff > p.ff) p.ff = l.ff;
    if (l.experts > p.experts) p.experts = l.experts;
    // key splits are chosen so that a launch has about two workgroups per compute unit: (runs x heads x splits) stays below four
    const size_t aw = (size_t)4 * mn_num_cus() * 16 * (2 + (size_t)l.vdim) * sizeof(float);
    if (aw > p.attn_ws) p.attn_ws = aw;
    const size_t gw = mn_mingru_scan_workspace_bytes(M, l.gru);
    if (gw > p.gru_ws) p.gru_ws = gw;
    if (m->arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64) {       // scratch of the weight-streaming MFMA route: the largest product of the stack
      const int W = m->width;
      const int shapes[4][2] = {{d.n_in, W}, {W, d.n_cat}, {d.n_ff_in, W}, {W, l.shared_ff}};
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

extern "C" size_t mn_pmix_workspace_bytes(const mn_pmix_model* m, int M) {
  if (!m || !m->layers || M < 1) return 0;
  const PPlan p = make_plan(m, M);
  const size_t W = m->width, R = (size_t)M, Z = R * p.top;
  size_t n = 0;
  n += al(R * W * 4);                                  // residual
  n += al(R * W * 4);                                  // normed rows
  n += al(R * W * 4) + al(R * W * 2);                  // sublayer input + bf16
  n += al(R * p.n_in * 4);                             // stacked input projections
  n += al(R * p.cqkv * 4);                             // filtered q / k / v
  n += al(R * p.cq * 4);                               // queries
  n += al(R * p.n_cat * 4) + al(R * p.n_cat * 2);      // [attention | recurrence] + bf16
  n += al(R * W * 4);                                  // sublayer result
  n += al(R * p.n_ff_in * 4);                          // [shared gate ; shared up ; router ; shared gate logit]
  n += al(R * p.sff * 4) + al(R * p.sff * 2);          // shared activation + bf16
  n += al(R * W * 4);                                  // shared result
  n += 2 * al(Z * 4);                                  // chosen experts, weights
  n += al(Z * 2 * p.ff * 4);                           // [gate ; up] of the pairs
  n += al(Z * p.ff * 4) + al(Z * p.ff * 2);            // their activation + bf16
  n += al(Z * W * 4);                                  // their results
  n += al(Z * W * 2);                                  // gathered bf16 rows
  n += 2 * al(((size_t)p.experts + 1) * 4) + 2 * al(Z * 4);   // counts, offsets, perm, slot_of
  n += 2 * al((Z / 256 + p.experts + 1) * 4) + al(4);         // live row tiles of the grouped products, their count
  n += al(p.gemm_ws) + al(p.attn_ws) + al(p.gru_ws);
  return n;
}

extern "C" int mn_pmix_step(const mn_pmix_model* m, const mn_pmix_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                            const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk, int max_len, int flags,
                            float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(m && st && m->layers && m->run_layer && m->run_readd && m->final_w && x && row_seq && row_slot && row_back && out && workspace,
               "mn_pmix_step: null pointer");
  MN_CHECK_ARG(st->k && st->v && st->pk && st->pv && st->canon && st->conv && st->gru, "mn_pmix_step: null state table");
  MN_CHECK_ARG(M >= 1 && M <= 65535 && m->width >= 1 && m->n_layers >= 1 && m->n_runs >= 1 && m->taps >= 0,
               "mn_pmix_step: bad sizes (M=%d)", M);
  MN_CHECK_ARG(workspace_bytes >= mn_pmix_workspace_bytes(m, M), "mn_pmix_step: workspace too small");
  const bool one_row = (flags & MN_SEQ_ROWS_DISTINCT) != 0;
  MN_CHECK_ARG(one_row || (blk_tab && n_blk >= 1 && n_blk <= M), "mn_pmix_step: rows that share sequences need the table of their runs");
  MN_CHECK_ARG(max_len >= 1 && max_len <= st->t_max, "mn_pmix_step: max_len=%d outside the cache (t_max=%d)", max_len, st->t_max);
  if (one_row) n_blk = M;
  const PPlan p = make_plan(m, M);
  const int W = m->width, arith = m->arith;
  const size_t R = (size_t)M, Zmax = R * p.top;
  MN_CHECK_ARG(Zmax <= 65535, "mn_pmix_step: %d rows x %d picks exceed 65535 (row, expert) pairs per step", M, p.top);
  const bool want16 = arith == MN_SEQ_ARITH_BF16 && M > 64;       // bf16 copies feed the tiled MFMA GEMMs only
  char* wp = reinterpret_cast<char*>(workspace);
  auto take = [&](size_t bytes) { char* q = wp; wp += al(bytes); return q; };
  float* xr = (float*)take(R * W * 4);
  float* n1 = (float*)take(R * W * 4);
  float* hf = (float*)take(R * W * 4);
  uint16_t* hh = (uint16_t*)take(R * W * 2);
  float* pin = (float*)take(R * p.n_in * 4);
  float* qkvc = (float*)take(R * p.cqkv * 4);
  float* qf = (float*)take(R * p.cq * 4);
  float* cat = (float*)take(R * p.n_cat * 4);
  uint16_t* cath = (uint16_t*)take(R * p.n_cat * 2);
  float* yf = (float*)take(R * W * 4);
  float* fin = (float*)take(R * p.n_ff_in * 4);
  float* sa = (float*)take(R * p.sff * 4);
  uint16_t* sah = (uint16_t*)take(R * p.sff * 2);
  float* sh = (float*)take(R * W * 4);
  int32_t* tidx = (int32_t*)take(Zmax * 4);
  float* tw = (float*)take(Zmax * 4);
  float* gu = (float*)take(Zmax * 2 * p.ff * 4);
  float* ea = (float*)take(Zmax * p.ff * 4);
  uint16_t* eah = (uint16_t*)take(Zmax * p.ff * 2);
  float* ye = (float*)take(Zmax * W * 4);
  uint16_t* xg = (uint16_t*)take(Zmax * W * 2);
  int32_t* counts = (int32_t*)take(((size_t)p.experts + 1) * 4);
  int32_t* offsets = (int32_t*)take(((size_t)p.experts + 1) * 4);
  int32_t* perm = (int32_t*)take(Zmax * 4);
  int32_t* slot_of = (int32_t*)take(Zmax * 4);
  int32_t* tile_g = (int32_t*)take((Zmax / 256 + p.experts + 1) * 4);
  int32_t* tile_m0 = (int32_t*)take((Zmax / 256 + p.experts + 1) * 4);
  int32_t* n_tiles = (int32_t*)take(4);
  uint16_t* const hh_buf = hh;
  void* gws = p.gemm_ws ? take(p.gemm_ws) : nullptr;
  const size_t gwb = p.gemm_ws;
  void* aws = take(p.attn_ws);
  void* gruws = take(p.gru_ws);
  if (!want16) hh = cath = sah = nullptr;
  hipStream_t hs = mn_stream(stream);
  int rc;
#define MN_TRY(call) do { rc = (call); if (rc != MN_OK) return rc; } while (0)
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, x, ldx, xr, W);
  MN_CHECK_LAUNCH("mn_pmix_step(copy)");
  // A mixer sublayer ends with x += mult * y and the next sublayer starts with RMS(x) and its input filter.  On decode steps
  // (MN_SEQ_ROWS_DISTINCT, no bf16 copies wanted) these are ONE launch; otherwise the operators run one by one.  `pend` is a
  // sublayer result that has not been added to x yet.
  const bool fuse = (flags & MN_SEQ_ROWS_DISTINCT) && !want16 && W <= 8192 && m->taps <= 8;
  const float* pend = nullptr;
  // h_out = RMS(x; w) + its filter after adding `pend`; returns through *h / *h16 where the sublayer's input lies
  auto norm_stage = [&](const uint16_t* w, const uint16_t* taps_w, float* tstate, const float** h, const uint16_t** h16) -> int {
    const bool filt = m->taps >= 1 && taps_w;
    int rc2;
    if (fuse) {
      rc2 = mn_axpy_rms_filter_rows(xr, W, pend, W, m->mult, w, m->eps, filt ? taps_w : nullptr, m->taps, tstate, row_seq, row_slot, hf, W,
                                    M, W, stream);
      pend = nullptr; *h = hf; *h16 = nullptr;
      return rc2;
    }
    if (!filt) {
      rc2 = mn_axpy_rms_rows(xr, W, pend, W, m->mult, w, m->eps, hf, W, hh, W, M, W, stream);
      pend = nullptr; *h = hf; *h16 = hh;
      return rc2;
    }
    rc2 = mn_axpy_rms_rows(xr, W, pend, W, m->mult, w, m->eps, n1, W, nullptr, 0, M, W, stream);
    pend = nullptr;
    if (rc2 == MN_OK) rc2 = mn_tap_filter_rows(n1, W, taps_w, m->taps, tstate, row_seq, row_slot, row_back, hf, W, hh, W, M, W, stream);
    if (rc2 == MN_OK) rc2 = mn_tap_state_update(n1, W, m->taps, tstate, row_seq, row_back, M, W, stream);
    *h = hf; *h16 = hh;
    return rc2;
  };
  auto flush = [&]() -> int {
    if (!pend) return MN_OK;
    const int rc2 = mn_axpy_rms_rows(xr, W, pend, W, m->mult, nullptr, m->eps, nullptr, 0, nullptr, 0, M, W, stream);
    pend = nullptr;
    return rc2;
  };
  const size_t canon_half = m->taps > 1 ? (size_t)st->n_seq * (m->taps - 1) * W : 0;
  for (int ri = 0; ri < m->n_runs; ++ri) {
    const int li = m->run_layer[ri];
    MN_CHECK_ARG(li >= 0 && li < m->n_layers, "mn_pmix_step: run %d names layer %d", ri, li);
    const mn_pmix_layer& l = m->layers[li];
    const PDims d = pdims(l);
    MN_CHECK_ARG(l.heads >= 1 && l.kv_heads >= 1 && (l.heads % l.kv_heads) == 0 && l.dim >= 1 && l.vdim >= 1 && l.gru >= 1 && l.conv >= 0 &&
                     l.window >= 0 && l.pool >= 0 && l.experts >= 0 && (l.experts == 0 || (l.top >= 1 && l.top <= l.experts && l.ff >= 1)),
                 "mn_pmix_step: layer %d: bad sizes", li);
    MN_CHECK_ARG(st->k[ri] && st->v[ri] && st->gru[ri] && (l.pool == 0 || (st->pk[ri] && st->pv[ri])) && (l.conv <= 1 || st->conv[ri]) &&
                     (m->taps <= 1 || st->canon[ri]), "mn_pmix_step: run %d: null state", ri);
    if (m->run_readd[ri]) {                           // a repeated pass: the step's input rows are added once more
      MN_TRY(flush());
      MN_TRY(mn_axpy_rms_rows(xr, W, x, ldx, 1.0f, nullptr, m->eps, nullptr, 0, nullptr, 0, M, W, stream));
    }
    const float* h; const uint16_t* h16;
    // ---- mixer sublayer ----
    MN_TRY(norm_stage(l.norm1, l.canon1, st->canon[ri], &h, &h16));
    MN_TRY(linear(arith, M, h, W, h16, W, l.w_in, d.n_in, W, l.b_in, pin, d.n_in, gws, gwb, stream));
    const bool gru_in_rows = one_row && !cath;      // decode rows without bf16 copies: the recurrence rides the launch below
    if (one_row) {        // decode rows: channel filter + state, rotation, unit norm, append and block means in one launch
      MN_TRY(mn_filter_rope_append_rows(pin, d.n_in, M, l.heads, l.kv_heads, l.dim, l.vdim, l.w_conv, l.conv, st->conv[ri], l.rot_dims, l.rot_freq,
                                        l.rot_mag, l.unit_qk, m->eps, l.scale, row_seq, row_slot, qf, d.cq, st->k[ri], st->v[ri], st->t_max,
                                        st->pk[ri], st->pv[ri], st->n_pool_max, l.pool, pin + d.cqkv, d.n_in, pin + d.cqkv + 2 * l.gru, d.n_in,
                                        st->gru[ri], gru_in_rows ? l.gru : 0, l.right_scale, cat + l.heads * l.vdim, d.n_cat, stream));
    } else {
      const float* qkv = pin; int64_t ldqkv = d.n_in;
      if (l.conv >= 1) {
        MN_TRY(mn_tap_conv_rows(pin, d.n_in, l.w_conv, l.conv, st->conv[ri], row_seq, row_slot, row_back, qkvc, d.cqkv, M, d.cqkv, stream));
        MN_TRY(mn_tap_state_update(pin, d.n_in, l.conv, st->conv[ri], row_seq, row_back, M, d.cqkv, stream));
        qkv = qkvc; ldqkv = d.cqkv;
      }
      MN_TRY(mn_rope_unit_append(qkv, ldqkv, M, l.heads, l.kv_heads, l.dim, l.vdim, l.rot_dims, l.rot_freq, l.rot_mag, l.unit_qk, m->eps, l.scale,
                                 row_seq, row_slot, qf, d.cq, st->k[ri], st->v[ri], st->t_max, stream));
      if (l.pool > 0)
        MN_TRY(mn_pool_blocks_update(st->k[ri], st->v[ri], st->t_max, st->pk[ri], st->pv[ri], st->n_pool_max, l.pool, d.ck, d.cv, row_seq,
                                     row_slot, M, stream));
    }
    {
      const int rb = one_row ? 1 : mn_window_attn_block_rows();
      int max_keys = max_len;
      if (l.window > 0) {
        max_keys = l.window + rb - 1 < max_len ? l.window + rb - 1 : max_len;
        if (l.pool > 0) max_keys += max_len / l.pool;
      }
      int ns = mn_window_attn_splits(n_blk, l.heads, l.kv_heads, one_row, max_keys);
      while (ns > 1 && mn_window_attn_workspace_bytes(n_blk, l.heads, l.kv_heads, l.vdim, one_row, ns) > p.attn_ws) --ns;
      MN_TRY(mn_window_pool_attn_blocks(qf, d.cq, st->k[ri], st->v[ri], st->pk[ri], st->pv[ri], row_seq, row_slot, blk_tab, n_blk, one_row,
                                        l.heads, l.kv_heads, l.dim, l.vdim, st->t_max, st->n_pool_max, l.window, l.pool, l.left_scale, cat,
                                        d.n_cat, cath, d.n_cat, ns, aws, p.attn_ws, stream));
    }
    const int hv = l.heads * l.vdim;
    if (gru_in_rows) {
      // done with the filter / rotation launch above
    } else if (M >= 2 * 32 && !one_row)                     // many rows: the recurrence as a chunked scan instead of one thread per channel walking them all
      MN_TRY(mn_mingru_rows_scan(pin + d.cqkv, d.n_in, pin + d.cqkv + 2 * l.gru, d.n_in, st->gru[ri], row_seq, row_slot, row_back, l.right_scale,
                                 cat + hv, d.n_cat, cath ? cath + hv : nullptr, d.n_cat, M, l.gru, gruws, p.gru_ws, stream));
    else
      MN_TRY(mn_mingru_rows(pin + d.cqkv, d.n_in, pin + d.cqkv + 2 * l.gru, d.n_in, st->gru[ri], row_seq, row_slot, row_back, l.right_scale,
                            cat + hv, d.n_cat, cath ? cath + hv : nullptr, d.n_cat, M, l.gru, stream));
    MN_TRY(linear(arith, M, cat, d.n_cat, cath, d.n_cat, l.w_out, W, d.n_cat, nullptr, yf, W, gws, gwb, stream));
    pend = yf;
    // ---- feed-forward sublayer ----
    if (l.experts > 0) {
      const int fs = l.shared_ff, E = l.experts, top = l.top, ff = l.ff, Z = M * top;
      MN_TRY(norm_stage(l.norm2, l.canon2, st->canon[ri] ? st->canon[ri] + canon_half : nullptr, &h, &h16));
      MN_TRY(linear(arith, M, h, W, h16, W, l.w_ff_in, d.n_ff_in, W, l.b_ff_in, fin, d.n_ff_in, gws, gwb, stream));
      if (fs > 0 && !sah) {          // few rows (no bf16 copy wanted): the router's pick and the shared activation in one launch
        MN_TRY(mn_router_topk_silu_rows(fin + 2 * fs, d.n_ff_in, M, E, top, tidx, tw, fin, d.n_ff_in, sa, fs, fs, stream));
      } else {
        MN_TRY(mn_router_topk_rows(fin + 2 * fs, d.n_ff_in, M, E, top, tidx, tw, stream));
        if (fs > 0) MN_TRY(mn_silu_mul_rows(fin, d.n_ff_in, sa, fs, sah, fs, M, fs, stream));
      }
      if (fs > 0) {
        MN_TRY(linear(arith, M, sa, fs, sah, fs, l.w_shared_down, W, fs, nullptr, sh, W, gws, gwb, stream));
      }
      const int32_t* so = nullptr;
      const int route = expert_route(m, l, M);
      if (route != EXPERTS_INDEXED && !h16) {          // few rows: the sublayer input was written in fp32 only
        MN_TRY(mn_f32_to_bf16(h, hh_buf, (int64_t)M * W, stream));
        h16 = hh_buf;
      }
      if (route == EXPERTS_TILES) {
        const int max_mtiles = Z / 256 + E;
        MN_TRY(mn_moe_sort_tiles(tidx, M, top, E, counts, offsets, perm, slot_of, 256, tile_g, tile_m0, n_tiles, stream));
        MN_TRY(mn_gemm256_grouped_tiles(h16, W, 0, M, perm, l.w_gate_up, W, (int64_t)2 * ff * W, offsets, counts, E, tile_g, tile_m0, n_tiles,
                                        max_mtiles, eah, ff, 0, ff, W, 6, stream));
        MN_TRY(mn_gemm256_grouped_tiles(eah, ff, 0, Z, nullptr, l.w_down, ff, (int64_t)W * ff, offsets, counts, E, tile_g, tile_m0, n_tiles,
                                        max_mtiles, ye, W, 0, W, ff, 0, stream));
        so = slot_of;
      } else if (route == EXPERTS_GROUPED) {
        MN_TRY(mn_moe_sort(tidx, M, top, E, counts, offsets, perm, slot_of, stream));
        MN_TRY(mn_gather_rows_bf16(h16, W, perm, xg, W, Z, W, stream));
        MN_TRY(mn_gemm_bf16_grouped(xg, W, l.w_gate_up, W, (int64_t)2 * ff * W, offsets, counts, E, gu, 2 * ff, M, 2 * ff, W, MN_GEMM_F32, stream));
        MN_TRY(mn_silu_mul_rows(gu, 2 * ff, nullptr, 0, eah, ff, Z, ff, stream));
        MN_TRY(mn_gemm_bf16_grouped(eah, ff, l.w_down, ff, (int64_t)W * ff, offsets, counts, E, ye, W, M, W, ff, MN_GEMM_F32, stream));
        so = slot_of;
      } else {
        MN_TRY(mn_gemv_f32_indexed(h, W, top, l.w_gate_up, W, (int64_t)2 * ff * W, tidx, gu, 2 * ff, Z, 2 * ff, W, stream));
        MN_TRY(mn_silu_mul_rows(gu, 2 * ff, ea, ff, nullptr, 0, Z, ff, stream));
        MN_TRY(mn_gemv_f32_indexed(ea, ff, 1, l.w_down, ff, (int64_t)W * ff, tidx, ye, W, Z, W, ff, stream));
      }
      MN_TRY(mn_moe_combine_residual(xr, W, ye, W, so, tw, top, fs > 0 ? sh : nullptr, W, fs > 0 ? fin + 2 * fs + E : nullptr, d.n_ff_in,
                                     m->mult, M, W, stream));
    }
    if (trace) {
      MN_TRY(flush());
      hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, xr, (int64_t)W,
                         trace + (size_t)ri * R * W, W);
      MN_CHECK_LAUNCH("mn_pmix_step(trace)");
    }
  }
  MN_TRY(mn_axpy_rms_rows(xr, W, pend, W, m->mult, m->final_w, m->eps, out, W, nullptr, 0, M, W, stream));
#undef MN_TRY
  return MN_OK;
}
