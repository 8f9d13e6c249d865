// hybrid_engine.hip — the step function of hybrid-mixer sequence models (mingnative.h section 11): one pass of the layer runs over the
// rows of a step as a chain of launches on the caller's stream.  A run is
//   h = RMS(x) w                                   (fused with the previous run's residual add: mn_axpy_rms_rows)
//   [q ; k ; v ; (gate) ; up ; router] = W_in h    ONE product for the mixer's and the feed-forward's input projections
//   mixer    attention: head norms + temperature + append, then the block attention with the heads' sinks
//            lightning: the recurrence (row by row, one decode row cut over many workgroups, or the chunked scan), RMS x sigmoid gate
//   x += [mixer | relu(up)^2] [W_o | W_down]^T     ONE product for the mixer's output and the dense / shared expert's down projection
//   experts of a mixture: as in pmix_engine.hip (sorted by expert on the grouped MFMA GEMMs, or pair by pair on fp32 FMA); picks that
//            stand for the input itself get no product: they sort behind the last expert and the combine adds w * h for them.
// Matrix products go through the routing of seq_linear.h.
#include "seq_linear.h"

extern "C" size_t mn_sizeof_hyb_layer(void) { return sizeof(mn_hyb_layer); }
extern "C" size_t mn_sizeof_hyb_model(void) { return sizeof(mn_hyb_model); }
extern "C" size_t mn_sizeof_hyb_state(void) { return sizeof(mn_hyb_state); }

namespace {

struct HDims {
  int cq, ck, cv, cg, n_up, n_router, off_g, off_up, off_router, n_in, hv, n_cat;
};

HDims hdims(const mn_hyb_layer& l) {
  HDims d;
  const int G = l.kind == MN_HYB_LIGHTNING ? l.heads : l.kv_heads;
  d.cq = l.heads * l.dim; d.ck = G * l.dim; d.cv = G * l.vdim;
  d.cg = l.kind == MN_HYB_LIGHTNING ? l.heads * l.vdim : 0;
  d.n_up = l.ff_kind == MN_HYB_FF_NONE ? 0 : l.ff;
  d.n_router = l.ff_kind == MN_HYB_FF_MOE ? l.experts + l.pass : 0;
  d.off_g = d.cq + d.ck + d.cv;
  d.off_up = d.off_g + d.cg;
  d.off_router = d.off_up + d.n_up;
  d.n_in = (d.off_router + d.n_router + 7) / 8 * 8;             // zero rows pad the stack to a multiple of 8
  d.hv = l.heads * l.vdim;
  d.n_cat = d.hv + d.n_up;
  return d;
}

struct HPlan {
  int n_in = 1, cq = 1, hv = 1, n_cat = 1, top = 1, eff = 1, experts = 1;
  size_t gemm_ws = 0, attn_ws = 0;
  int64_t lin = 0;                                               // largest heads x dim x vdim of a recurrence
};

enum { EXPERTS_INDEXED = 0, EXPERTS_GROUPED = 1, EXPERTS_TILES = 2 };
int expert_route(const mn_hyb_model* m, const mn_hyb_layer& l, int M) {
  if (m->arith != MN_SEQ_ARITH_BF16 || M <= 8 || l.experts + 1 > 128 || (int64_t)M * l.top > 65536 ||
      ((((uintptr_t)l.w_up) | ((uintptr_t)l.w_down)) & 15) != 0)
    return EXPERTS_INDEXED;
  const int64_t W = m->width, ff = l.expert_ff;
  if ((W % 64) == 0 && (ff % 64) == 0 && ff * W * 2 < ((int64_t)1 << 32) && (int64_t)M * l.top * (W > ff ? W : ff) * 2 < ((int64_t)1 << 32))
    return EXPERTS_TILES;
  if ((W % 8) == 0 && (ff % 8) == 0) return EXPERTS_GROUPED;
  return EXPERTS_INDEXED;
}

HPlan make_plan(const mn_hyb_model* m, int M) {
  HPlan p;
  for (int i = 0; i < m->n_layers; ++i) {
    const mn_hyb_layer& l = m->layers[i];
    const HDims d = hdims(l);
    if (d.n_in > p.n_in) p.n_in = d.n_in;
    if (d.cq > p.cq) p.cq = d.cq;
    if (d.hv > p.hv) p.hv = d.hv;
    if (d.n_cat > p.n_cat) p.n_cat = d.n_cat;
    if (l.ff_kind == MN_HYB_FF_MOE) {
      if (l.top > p.top) p.top = l.top;
      if (l.expert_ff > p.eff) p.eff = l.expert_ff;
      if (l.experts > p.experts) p.experts = l.experts;
    }
    if (l.kind == MN_HYB_ATTENTION) {
      const size_t aw = (size_t)4 * mn_num_cus() * 16 * (2 + (size_t)l.vdim) * sizeof(float);
      if (aw > p.attn_ws) p.attn_ws = aw;
    } else {
      const int64_t s = (int64_t)l.heads * l.dim * l.vdim;
      if (s > p.lin) p.lin = s;
    }
    if (m->arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64) {       // scratch of the weight-streaming MFMA route: the largest product of the stack
      const int W = m->width;
      const int shapes[2][2] = {{d.n_in, W}, {W, d.n_cat}};
      for (const auto& nk : shapes) {
        if (nk[0] < 1 || nk[1] < 8 || (nk[1] % 8) != 0) continue;
        const size_t g = mn_skinny_workspace_bytes(M, nk[0], nk[1], MN_EPI_NONE);
        if (g > p.gemm_ws) p.gemm_ws = g;
      }
    }
  }
  return p;
}

// chunk states the scan of a step may hold: full chunks plus one ragged chunk for each of up to 64 sequences; steps too short for the
// scan hold none
inline size_t scan_bytes(const HPlan& p, int M) {
  const int c = mn_lightning_chunk_rows();
  return M >= 2 * c ? (size_t)(mn_cdiv(M, c) + 64) * (size_t)p.lin * sizeof(float) : 0;
}

}  // namespace

extern "C" size_t mn_hyb_workspace_bytes(const mn_hyb_model* m, int M) {
  if (!m || !m->layers || M < 1) return 0;
  const HPlan p = make_plan(m, M);
  const size_t W = m->width, R = (size_t)M, Z = R * p.top;
  size_t n = 0;
  n += al(R * W * 4);                                  // residual
  n += al(R * W * 4) + al(R * W * 2);                  // normed rows + bf16
  n += al(R * p.n_in * 4);                             // stacked input projections
  n += al(R * p.cq * 4);                               // queries
  n += al(R * p.hv * 4);                               // the recurrence's heads before their norm
  n += al(R * p.n_cat * 4) + al(R * p.n_cat * 2);      // [mixer | activation] + bf16
  n += al(R * W * 4);                                  // their joined output product
  n += 2 * al(Z * 4);                                  // chosen experts, weights
  n += al(Z * p.eff * 4);                              // up of the pairs
  n += al(Z * p.eff * 4) + al(Z * p.eff * 2);          // their activation + bf16
  n += al(Z * W * 4);                                  // their results
  n += al(Z * W * 2);                                  // gathered bf16 rows
  n += 2 * al(((size_t)p.experts + 2) * 4) + 2 * al(Z * 4);   // counts, offsets, perm, slot_of
  n += 2 * al((Z / 256 + p.experts + 2) * 4) + al(4);         // live row tiles of the grouped products, their count
  n += al(p.gemm_ws) + al(p.attn_ws);
  n += al(scan_bytes(p, M));                           // chunk states of the recurrence's scan
  return n;
}

extern "C" int mn_hyb_step(const mn_hyb_model* m, const mn_hyb_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                           const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk, const int32_t* chunk_tab,
                           int n_chunks, int max_len, int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(m && st && m->layers && m->run_layer && m->final_w && x && row_seq && row_slot && row_back && out && workspace,
               "mn_hyb_step: null pointer");
  MN_CHECK_ARG(st->k && st->v && st->lin, "mn_hyb_step: null state table");
  MN_CHECK_ARG(M >= 1 && M <= 65535 && m->width >= 1 && m->n_layers >= 1 && m->n_runs >= 1, "mn_hyb_step: bad sizes (M=%d)", M);
  MN_CHECK_ARG(workspace_bytes >= mn_hyb_workspace_bytes(m, M), "mn_hyb_step: workspace too small");
  const bool one_row = (flags & MN_SEQ_ROWS_DISTINCT) != 0;
  MN_CHECK_ARG(one_row || (blk_tab && n_blk >= 1 && n_blk <= M), "mn_hyb_step: rows that share sequences need the table of their runs");
  MN_CHECK_ARG(max_len >= 1 && max_len <= st->t_max, "mn_hyb_step: max_len=%d outside the cache (t_max=%d)", max_len, st->t_max);
  if (one_row) n_blk = M;
  const HPlan p = make_plan(m, M);
  const int W = m->width, arith = m->arith;
  const size_t R = (size_t)M, Zmax = R * p.top;
  MN_CHECK_ARG(Zmax <= 65535, "mn_hyb_step: %d rows x %d picks exceed 65535 (row, expert) pairs per step", M, p.top);
  const bool want16 = arith == MN_SEQ_ARITH_BF16 && M > 64;       // bf16 copies feed the tiled MFMA GEMMs only
  char* wp = reinterpret_cast<char*>(workspace);
  auto take = [&](size_t bytes) { char* q = wp; wp += al(bytes); return q; };
  float* xr = (float*)take(R * W * 4);
  float* hf = (float*)take(R * W * 4);
  uint16_t* hh = (uint16_t*)take(R * W * 2);
  float* pin = (float*)take(R * p.n_in * 4);
  float* qf = (float*)take(R * p.cq * 4);
  float* lo = (float*)take(R * p.hv * 4);
  float* cat = (float*)take(R * p.n_cat * 4);
  uint16_t* cath = (uint16_t*)take(R * p.n_cat * 2);
  float* yf = (float*)take(R * W * 4);
  int32_t* tidx = (int32_t*)take(Zmax * 4);
  float* tw = (float*)take(Zmax * 4);
  float* gu = (float*)take(Zmax * p.eff * 4);
  float* ea = (float*)take(Zmax * p.eff * 4);
  uint16_t* eah = (uint16_t*)take(Zmax * p.eff * 2);
  float* ye = (float*)take(Zmax * W * 4);
  uint16_t* xg = (uint16_t*)take(Zmax * W * 2);
  int32_t* counts = (int32_t*)take(((size_t)p.experts + 2) * 4);
  int32_t* offsets = (int32_t*)take(((size_t)p.experts + 2) * 4);
  int32_t* perm = (int32_t*)take(Zmax * 4);
  int32_t* slot_of = (int32_t*)take(Zmax * 4);
  int32_t* tile_g = (int32_t*)take((Zmax / 256 + p.experts + 2) * 4);
  int32_t* tile_m0 = (int32_t*)take((Zmax / 256 + p.experts + 2) * 4);
  int32_t* n_tiles = (int32_t*)take(4);
  uint16_t* const hh_buf = hh;
  void* gws = p.gemm_ws ? take(p.gemm_ws) : nullptr;
  const size_t gwb = p.gemm_ws;
  void* aws = take(p.attn_ws);
  const size_t scan_cap = scan_bytes(p, M);
  void* scanws = take(scan_cap);
  if (!want16) hh = cath = nullptr;
  hipStream_t hs = mn_stream(stream);
  int rc;
#define MN_TRY(call) do { rc = (call); if (rc != MN_OK) return rc; } while (0)
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, x, ldx, xr, W);
  MN_CHECK_LAUNCH("mn_hyb_step(copy)");
  const float* pend = nullptr;                      // a sublayer result that has not been added to x yet
  // decode rows without bf16 copies: residual add + norm as one workgroup per row with the row in registers (the launch the
  // parallel-mixer step uses for its decode rows, here without a filter)
  const bool fuse = one_row && !want16 && W <= 8192;
  for (int ri = 0; ri < m->n_runs; ++ri) {
    const int li = m->run_layer[ri];
    MN_CHECK_ARG(li >= 0 && li < m->n_layers, "mn_hyb_step: run %d names layer %d", ri, li);
    const mn_hyb_layer& l = m->layers[li];
    const HDims d = hdims(l);
    const bool attn = l.kind == MN_HYB_ATTENTION, moe = l.ff_kind == MN_HYB_FF_MOE;
    MN_CHECK_ARG((attn || l.kind == MN_HYB_LIGHTNING) && l.heads >= 1 && l.dim >= 1 && l.vdim >= 1 &&
                     (!attn || (l.kv_heads >= 1 && (l.heads % l.kv_heads) == 0)) && l.ff_kind >= MN_HYB_FF_NONE && l.ff_kind <= MN_HYB_FF_MOE &&
                     (l.ff_kind != MN_HYB_FF_DENSE || l.ff >= 1) &&
                     (!moe || (l.experts >= 1 && l.pass >= 0 && l.top >= 1 && l.top <= l.experts + l.pass && l.expert_ff >= 1 && l.ff >= 0 &&
                               l.w_up && l.w_down)) && l.norm1 && l.w_in && l.w_out && (attn || (l.decay && l.mix_norm)),
                 "mn_hyb_step: layer %d: bad sizes or null weights", li);
    MN_CHECK_ARG(attn ? (st->k[ri] && st->v[ri]) : st->lin[ri] != nullptr, "mn_hyb_step: run %d: null state", ri);
    // ---- the input both sublayers read, and their stacked projections ----
    if (fuse) MN_TRY(mn_axpy_rms_filter_rows(xr, W, pend, W, 1.0f, l.norm1, m->eps, nullptr, 0, nullptr, row_seq, row_slot, hf, W, M, W, stream));
    else MN_TRY(mn_axpy_rms_rows(xr, W, pend, W, 1.0f, l.norm1, m->eps, hf, W, hh, W, M, W, stream));
    pend = nullptr;
    MN_TRY(linear(arith, M, hf, W, hh, W, l.w_in, d.n_in, W, nullptr, pin, d.n_in, gws, gwb, stream));
    // ---- mixer ----
    if (attn) {
      MN_TRY(mn_head_norm_temp_append(pin, d.n_in, M, l.heads, l.kv_heads, l.dim, l.vdim, l.q_norm, l.k_norm, m->eps, l.scale, l.temp_coef,
                                      l.temp_every, row_seq, row_slot, qf, d.cq, st->k[ri], st->v[ri], st->t_max, stream));
      int ns = mn_window_attn_splits(n_blk, l.heads, l.kv_heads, one_row, max_len);
      while (ns > 1 && mn_window_attn_workspace_bytes(n_blk, l.heads, l.kv_heads, l.vdim, one_row, ns) > p.attn_ws) --ns;
      MN_TRY(mn_window_pool_attn_blocks_sink(qf, d.cq, st->k[ri], st->v[ri], nullptr, nullptr, l.sink, row_seq, row_slot, blk_tab, n_blk, one_row,
                                             l.heads, l.kv_heads, l.dim, l.vdim, st->t_max, 1, 0, 0, 1.0f, cat, d.n_cat, cath, d.n_cat, ns, aws,
                                             p.attn_ws, -1, stream));
    } else {
      const size_t lds3 = mn_lightning_scan_lds_bytes(l.dim, l.vdim);
      const bool scan = !one_row && chunk_tab && n_chunks >= 1 && M >= 2 * mn_lightning_chunk_rows() && lds3 <= 64 * 1024 &&
                        mn_lightning_scan_workspace_bytes(n_chunks, l.heads, l.dim, l.vdim) <= scan_cap;
      if (scan)
        MN_TRY(mn_lightning_rows_scan(pin, d.n_in, M, l.heads, l.dim, l.vdim, l.decay, st->lin[ri], row_seq, row_slot, row_back, chunk_tab,
                                      n_chunks, lo, d.hv, scanws, scan_cap, stream));
      else
        MN_TRY(mn_lightning_rows(pin, d.n_in, M, l.heads, l.dim, l.vdim, l.decay, st->lin[ri], row_seq, row_slot, row_back,
                                 one_row ? MN_SEQ_ROWS_DISTINCT : 0, lo, d.hv, stream));
      MN_TRY(mn_rms_sigmoid_gate_rows(lo, d.hv, l.mix_norm, m->eps, pin + d.off_g, d.n_in, cat, d.n_cat, cath, d.n_cat, M, d.hv, stream));
    }
    // ---- the feed-forward's activation and router; the joined output product ----
    const int E = l.experts, top = l.top, eff = l.expert_ff, Z = M * top;
    if (moe) {
      const bool ride = d.n_up > 0 && !cath;           // few rows: the shared expert's activation rides the router's launch
      MN_TRY(mn_router_softmax_topk_rows(pin + d.off_router, d.n_in, M, d.n_router, E, top, l.correction, tidx, tw, ride ? pin + d.off_up : nullptr,
                                         d.n_in, ride ? cat + d.hv : nullptr, d.n_cat, ride ? d.n_up : 0, stream));
      if (d.n_up > 0 && !ride) MN_TRY(mn_relu2_rows(pin + d.off_up, d.n_in, cat + d.hv, d.n_cat, cath + d.hv, d.n_cat, M, d.n_up, stream));
    } else if (d.n_up > 0) {
      MN_TRY(mn_relu2_rows(pin + d.off_up, d.n_in, cat + d.hv, d.n_cat, cath ? cath + d.hv : nullptr, d.n_cat, M, d.n_up, stream));
    }
    MN_TRY(linear(arith, M, cat, d.n_cat, cath, d.n_cat, l.w_out, W, d.n_cat, nullptr, yf, W, gws, gwb, stream));
    if (!moe) {
      pend = yf;
    } else {
      const uint16_t* h16 = hh;
      const int32_t* so = nullptr;
      const int route = expert_route(m, l, M);
      if (route != EXPERTS_INDEXED && !h16) {          // few rows: the input was written in fp32 only
        MN_TRY(mn_f32_to_bf16(hf, hh_buf, (int64_t)M * W, stream));
        h16 = hh_buf;
      }
      if (route == EXPERTS_TILES) {                    // group E (the picks that pass the input through) gets no tiles
        const int max_mtiles = Z / 256 + E;
        MN_TRY(mn_ep_dispatch(tidx, M, top, E + 1, 0, E, counts, offsets, perm, slot_of, 256, tile_g, tile_m0, n_tiles, stream));
        MN_TRY(mn_gemm256_grouped_tiles(h16, W, 0, M, perm, l.w_up, W, (int64_t)eff * W, offsets, counts, E, tile_g, tile_m0, n_tiles, max_mtiles,
                                        eah, eff, 0, eff, W, 7, stream));          // the squared relu in the epilogue
        MN_TRY(mn_gemm256_grouped_tiles(eah, eff, 0, Z, nullptr, l.w_down, eff, (int64_t)W * eff, offsets, counts, E, tile_g, tile_m0, n_tiles,
                                        max_mtiles, ye, W, 0, W, eff, 0, stream));
        so = slot_of;
      } else if (route == EXPERTS_GROUPED) {
        MN_TRY(mn_moe_sort(tidx, M, top, E + 1, counts, offsets, perm, slot_of, stream));
        MN_TRY(mn_gather_rows_bf16(h16, W, perm, xg, W, Z, W, stream));
        MN_TRY(mn_gemm_bf16_grouped(xg, W, l.w_up, W, (int64_t)eff * W, offsets, counts, E, gu, eff, M, eff, W, MN_GEMM_F32, stream));
        MN_TRY(mn_relu2_rows(gu, eff, nullptr, 0, eah, eff, Z, eff, stream));
        MN_TRY(mn_gemm_bf16_grouped(eah, eff, l.w_down, eff, (int64_t)W * eff, offsets, counts, E, ye, W, M, W, eff, MN_GEMM_F32, stream));
        so = slot_of;
      } else {
        MN_TRY(mn_gemv_f32_indexed_upto(hf, W, top, l.w_up, W, (int64_t)eff * W, tidx, E, gu, eff, Z, eff, W, stream));
        MN_TRY(mn_relu2_rows(gu, eff, ea, eff, nullptr, 0, Z, eff, stream));
        MN_TRY(mn_gemv_f32_indexed_upto(ea, eff, 1, l.w_down, eff, (int64_t)W * eff, tidx, E, ye, W, Z, W, eff, stream));
      }
      MN_TRY(mn_moe_combine_pass_residual(xr, W, ye, W, so, tidx, tw, top, E, hf, W, yf, W, M, W, stream));
    }
    if (trace) {
      if (pend) {
        MN_TRY(mn_axpy_rms_rows(xr, W, pend, W, 1.0f, nullptr, m->eps, nullptr, 0, nullptr, 0, M, W, stream));
        pend = nullptr;
      }
      hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, xr, (int64_t)W,
                         trace + (size_t)ri * R * W, W);
      MN_CHECK_LAUNCH("mn_hyb_step(trace)");
    }
  }
  if (fuse) MN_TRY(mn_axpy_rms_filter_rows(xr, W, pend, W, 1.0f, m->final_w, m->eps, nullptr, 0, nullptr, row_seq, row_slot, out, W, M, W, stream));
  else MN_TRY(mn_axpy_rms_rows(xr, W, pend, W, 1.0f, m->final_w, m->eps, out, W, nullptr, 0, M, W, stream));
#undef MN_TRY
  return MN_OK;
}
