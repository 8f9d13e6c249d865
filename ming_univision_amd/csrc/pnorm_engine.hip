// pnorm_engine.hip — the step function of post-norm mixed-mixer sequence models (mingnative.h section 12): one pass of the layers over
// the rows of a step as a chain of launches on the caller's stream.  A layer is
//   stack = W_in x (+ bias)                         ONE product for everything the mixer projects from the residual stream
//   mixer   attention: whole-projection norms + rotation + append, the block attention (soft cap, window), a sigmoid gate per head
//           latent:    normed latent + rotated key part appended to ONE arena; the queries mapped into latent space head by head
//                      (absorbed W_uk); the block attention with all heads on one key/value head whose values are a view of the
//                      keys' first `kv_rank` columns; the attended latents expanded per head (W_uv)
//           delta:     filters + silu + unit norms + write strengths and decays, the recurrence, per-head RMS x silu gate
//   x += w1 rms(W_o mixer)                          mn_rms_scale_add_rows (writes the bf16 copy the next product reads)
//   x += w2 rms(W_down (gelu(gate) * up))           [gate ; up] = ONE product
//   x += ws rms(P (gelu(G x) * e_token))            the per-layer token input
// Matrix products go through the routing of seq_linear.h.
#include "seq_linear.h"

extern "C" size_t mn_sizeof_pn_layer(void) { return sizeof(mn_pn_layer); }
extern "C" size_t mn_sizeof_pn_model(void) { return sizeof(mn_pn_model); }
extern "C" size_t mn_sizeof_pn_state(void) { return sizeof(mn_pn_state); }
extern "C" int mn_pn_latent_ld(int rank, int rot) { return (rank + rot + 3) / 4 * 4; }

namespace {

inline int pad8(int n) { return (n + 7) / 8 * 8; }

struct PDims {
  int n_in;          // rows of the stacked input projection
  int nq;            // floats of a row's prepared queries (attention: H dim; latent: H (rank + rot); delta: q + k + v channels)
  int nmid;          // latent: H rank (attended latents); delta: H vdim (the recurrence's heads before their norm)
  int hv;            // H vdim: what W_o reads
  int off_g;         // attention: the gates' column; delta: the gate's first column
  int off_b, off_a;  // delta
  int akd, avd;      // key / value size of the attention kernel's heads
};

PDims pdims(const mn_pn_layer& l) {
  PDims d{};
  d.hv = l.heads * l.vdim;
  if (l.kind == MN_PN_ATTENTION) {
    const int cq = l.heads * l.dim, ck = l.kv_heads * l.dim, cv = l.kv_heads * l.vdim;
    d.off_g = cq + ck + cv;
    d.n_in = pad8(d.off_g + (l.has_gate ? l.heads : 0));
    d.nq = cq;
    d.akd = l.dim; d.avd = l.vdim;
  } else if (l.kind == MN_PN_LATENT) {
    d.n_in = pad8(l.heads * (l.dim + l.rot) + l.kv_rank + l.rot);
    d.nq = l.heads * (l.kv_rank + l.rot);
    d.nmid = l.heads * l.kv_rank;
    d.akd = l.kv_rank + l.rot; d.avd = l.kv_rank;
  } else {
    const int c = 2 * l.kv_heads * l.dim + l.heads * l.vdim;
    d.off_b = c; d.off_a = c + l.heads; d.off_g = c + 2 * l.heads;
    d.n_in = pad8(d.off_g + d.hv);
    d.nq = c;
    d.nmid = d.hv;
  }
  return d;
}

struct PPlan {
  int n_in = 8, nq = 1, nmid = 1, hv = 1, ff = 1, side = 8, heads = 1;
  size_t gemm_ws = 0, attn_ws = 0;
};

PPlan make_plan(const mn_pn_model* m, int M) {
  PPlan p;
  auto up = [](int& a, int b) { if (b > a) a = b; };
  for (int i = 0; i < m->n_layers; ++i) {
    const mn_pn_layer& l = m->layers[i];
    const PDims d = pdims(l);
    up(p.n_in, d.n_in); up(p.nq, d.nq); up(p.nmid, d.nmid); up(p.hv, d.hv); up(p.ff, l.ff); up(p.side, pad8(l.side)); up(p.heads, l.heads);
    if (l.kind != MN_PN_DELTA) {
      const size_t aw = (size_t)4 * mn_num_cus() * 16 * (2 + (size_t)d.avd) * sizeof(float);
      if (aw > p.attn_ws) p.attn_ws = aw;
    }
    if (m->arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64) {       // scratch of the weight-streaming MFMA route: the largest product of the stack
      const int W = m->width;
      const int shapes[6][2] = {{d.n_in, W}, {W, d.hv}, {2 * l.ff, W}, {W, l.ff}, {pad8(l.side), W}, {W, l.side}};
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

extern "C" size_t mn_pn_workspace_bytes(const mn_pn_model* m, int M) {
  if (!m || !m->layers || M < 1) return 0;
  const PPlan p = make_plan(m, M);
  const size_t W = m->width, R = (size_t)M;
  size_t n = 0;
  n += al(R * W * 4) + al(R * W * 2);                  // residual + bf16
  n += al(R * p.n_in * 4);                             // stacked input projections
  n += al(R * p.nq * 4);                               // prepared queries / recurrence inputs
  n += al(R * p.nmid * 4);                             // attended latents / the recurrence's heads
  n += al(R * 2 * p.heads * 4);                        // write strengths and decays
  n += al(R * p.hv * 4) + al(R * p.hv * 2);            // what W_o reads + bf16
  n += al(R * W * 4);                                  // a sublayer's result
  n += al(R * 2 * p.ff * 4);                           // [gate ; up]
  n += al(R * p.ff * 4) + al(R * p.ff * 2);            // their product + bf16
  n += 2 * al(R * p.side * 4);                         // the token input's gate and its product with the table rows
  n += al(p.gemm_ws) + al(p.attn_ws);
  return n;
}

extern "C" int mn_pn_step(const mn_pn_model* m, const mn_pn_state* st, const float* x, int64_t ldx, int M, const int32_t* row_tok,
                          const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk,
                          int max_len, int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(m && st && m->layers && m->final_w && x && row_seq && row_slot && row_back && out && workspace, "mn_pn_step: null pointer");
  MN_CHECK_ARG(st->k && st->v && st->conv && st->lin, "mn_pn_step: null state table");
  MN_CHECK_ARG(M >= 1 && M <= 65535 && m->width >= 1 && m->n_layers >= 1, "mn_pn_step: bad sizes (M=%d)", M);
  MN_CHECK_ARG(workspace_bytes >= mn_pn_workspace_bytes(m, M), "mn_pn_step: workspace too small");
  const bool one_row = (flags & MN_SEQ_ROWS_DISTINCT) != 0;
  MN_CHECK_ARG(one_row || (blk_tab && n_blk >= 1 && n_blk <= M), "mn_pn_step: rows that share sequences need the table of their runs");
  MN_CHECK_ARG(max_len >= 1 && max_len <= st->t_max, "mn_pn_step: max_len=%d outside the cache (t_max=%d)", max_len, st->t_max);
  if (one_row) n_blk = M;
  const PPlan p = make_plan(m, M);
  const int W = m->width, arith = m->arith;
  const size_t R = (size_t)M;
  const bool want16 = arith == MN_SEQ_ARITH_BF16 && M > 64;       // bf16 copies feed the tiled MFMA GEMMs only
  char* wp = reinterpret_cast<char*>(workspace);
  auto take = [&](size_t bytes) { char* q = wp; wp += al(bytes); return q; };
  float* xr = (float*)take(R * W * 4);
  uint16_t* xh = (uint16_t*)take(R * W * 2);
  float* pin = (float*)take(R * p.n_in * 4);
  float* qf = (float*)take(R * p.nq * 4);
  float* mid = (float*)take(R * p.nmid * 4);
  float* bd = (float*)take(R * 2 * p.heads * 4);
  float* cat = (float*)take(R * p.hv * 4);
  uint16_t* cath = (uint16_t*)take(R * p.hv * 2);
  float* yf = (float*)take(R * W * 4);
  float* gu = (float*)take(R * 2 * p.ff * 4);
  float* act = (float*)take(R * p.ff * 4);
  uint16_t* acth = (uint16_t*)take(R * p.ff * 2);
  float* sg = (float*)take(R * p.side * 4);
  float* sa = (float*)take(R * p.side * 4);
  void* gws = p.gemm_ws ? take(p.gemm_ws) : nullptr;
  const size_t gwb = p.gemm_ws;
  void* aws = take(p.attn_ws);
  if (!want16) xh = cath = acth = nullptr;
  hipStream_t hs = mn_stream(stream);
  int rc;
#define MN_TRY(call) do { rc = (call); if (rc != MN_OK) return rc; } while (0)
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, x, ldx, xr, W);
  MN_CHECK_LAUNCH("mn_pn_step(copy)");
  if (xh) MN_TRY(mn_f32_to_bf16(xr, xh, (int64_t)M * W, stream));
  for (int li = 0; li < m->n_layers; ++li) {
    const mn_pn_layer& l = m->layers[li];
    const PDims d = pdims(l);
    const bool attn = l.kind == MN_PN_ATTENTION, latent = l.kind == MN_PN_LATENT, delta = l.kind == MN_PN_DELTA;
    MN_CHECK_ARG((attn || latent || delta) && l.heads >= 1 && l.dim >= 1 && l.vdim >= 1 && l.ff >= 0 && l.side >= 0 && l.window >= 0 && l.norm1 &&
                     l.w_in && l.w_o && (l.ff == 0 || (l.norm2 && l.w_gate_up && l.w_down)) &&
                     (l.side == 0 || (l.side_norm && l.w_side_gate && l.w_side_proj && l.side_table && row_tok)),
                 "mn_pn_step: layer %d: bad sizes or null weights", li);
    MN_CHECK_ARG(!attn || (l.kv_heads >= 1 && (l.heads % l.kv_heads) == 0 && st->k[li] && st->v[li] && (l.rot_dims == 0 || l.rot_freq)),
                 "mn_pn_step: layer %d: attention: bad head counts, null arenas or no frequencies", li);
    MN_CHECK_ARG(!latent || (l.kv_rank >= 1 && l.rot >= 0 && l.k_norm && l.w_ukT && l.w_uv && st->k[li] && (l.rot_dims == 0 || l.rot_freq)),
                 "mn_pn_step: layer %d: latent attention: bad sizes, null weights or arena", li);
    MN_CHECK_ARG(!delta || (l.kv_heads >= 1 && (l.heads % l.kv_heads) == 0 && l.conv >= 1 && l.w_conv && l.mix_norm && l.a_log && l.dt_bias &&
                            st->lin[li] && (l.conv == 1 || st->conv[li])),
                 "mn_pn_step: layer %d: delta rule: bad sizes, null weights or states", li);
    // ---- the mixer's stacked projections of the residual stream ----
    MN_TRY(linear(arith, M, xr, W, xh, W, l.w_in, d.n_in, W, l.b_in, pin, d.n_in, gws, gwb, stream));
    if (attn || latent) {
      const int H = l.heads, G = attn ? l.kv_heads : 1;
      const float* karena = st->k[li];
      const float* varena = attn ? st->v[li] : st->k[li];
      int64_t ldk = 0, ldv = 0;
      float* att = attn ? cat : mid;                     // attention writes what W_o reads; latent attention the attended latents
      const int64_t ldatt = attn ? d.hv : d.nmid;
      if (attn) {
        MN_TRY(mn_proj_norm_rope_append(pin, d.n_in, M, H, G, l.dim, l.vdim, l.q_norm, l.k_norm, m->eps, l.rot_dims, l.rot_interleaved, l.rot_freq,
                                        l.scale, row_seq, row_slot, qf, d.nq, st->k[li], (int64_t)G * l.dim, st->v[li], (int64_t)G * l.vdim,
                                        st->t_max, stream));
      } else {
        ldk = ldv = mn_pn_latent_ld(l.kv_rank, l.rot);
        MN_TRY(mn_latent_rope_append(pin, d.n_in, M, H, l.dim, l.rot, l.kv_rank, l.k_norm, m->eps, l.rot_dims, l.rot_interleaved, l.rot_freq,
                                     l.scale, row_seq, row_slot, qf, d.nq, st->k[li], ldk, st->t_max, stream));
        // the plain part of every head's query mapped into latent space: q_lat[h] = scale * W_uk[h]^T q[h]
        MN_TRY(mn_gemm_f32_batched(pin, d.n_in, l.dim + l.rot, l.w_ukT, l.dim, (int64_t)l.kv_rank * l.dim, nullptr, qf, d.nq, l.kv_rank + l.rot,
                                   nullptr, 0, 0, nullptr, 0, 0, M, l.kv_rank, l.dim, H, l.scale, stream));
      }
      int keys = max_len;
      if (l.window > 0 && l.window + 3 < keys) keys = l.window + 3;
      // latent attention's decode rows run on the matrix-core kernel (all heads of a row in one workgroup): its key tiles hold 16 keys
      int ns = mn_window_attn_splits_tile(n_blk, H, G, one_row, keys, latent && one_row ? 16 : 64);
      if (latent && one_row && (int64_t)ns * d.avd > 16384) ns = 16384 / d.avd > 1 ? 16384 / d.avd : 1;   // the merge reads ns x 16 x avd partial sums a row
      while (ns > 1 && mn_window_attn_workspace_bytes(n_blk, H, G, d.avd, one_row, ns) > p.attn_ws) --ns;
      const bool gate = attn && l.has_gate;
      MN_TRY(mn_window_pool_attn_blocks_cap(qf, d.nq, karena, ldk, varena, ldv, nullptr, nullptr, nullptr, l.softcap, row_seq, row_slot, blk_tab,
                                            n_blk, one_row, H, G, d.akd, d.avd, st->t_max, 1, l.window, 0, 1.0f, att, ldatt,
                                            (attn && !gate) ? cath : nullptr, d.hv, ns, aws, p.attn_ws, -1, stream));
      if (gate) MN_TRY(mn_head_sigmoid_gate_rows(cat, d.hv, pin + d.off_g, d.n_in, cath, d.hv, M, H, l.vdim, stream));
      if (latent)                                        // every head's value = W_uv[h] (its attended latent)
        MN_TRY(mn_gemm_f32_batched(mid, d.nmid, l.kv_rank, l.w_uv, l.kv_rank, (int64_t)l.vdim * l.kv_rank, nullptr, cat, d.hv, l.vdim, cath, d.hv,
                                   l.vdim, nullptr, 0, 0, M, l.vdim, l.kv_rank, H, 1.0f, stream));
    } else {
      const int chan = d.nq;
      // decode rows move their filter state on inside the preparation launch
      MN_TRY(mn_delta_prep_rows(pin, d.n_in, M, l.heads, l.kv_heads, l.dim, l.vdim, d.off_b, d.off_a, l.w_conv, l.conv, st->conv[li], one_row ? 1 : 0,
                                l.a_log, l.dt_bias, l.unit_eps, 1.0f / sqrtf((float)l.dim), row_seq, row_slot, row_back, qf, chan, bd,
                                2 * l.heads, stream));
      if (l.conv > 1 && !one_row) MN_TRY(mn_tap_state_update(pin, d.n_in, l.conv, st->conv[li], row_seq, row_back, M, chan, stream));
      MN_TRY(mn_gated_delta_rows(qf, chan, bd, 2 * l.heads, M, l.heads, l.kv_heads, l.dim, l.vdim, st->lin[li], row_seq, row_slot, row_back,
                                 one_row ? MN_SEQ_ROWS_DISTINCT : 0, mid, d.nmid, stream));
      MN_TRY(mn_head_rms_silu_gate_rows(mid, d.nmid, l.mix_norm, m->eps, pin + d.off_g, d.n_in, cat, d.hv, cath, d.hv, M, l.heads, l.vdim,
                                        stream));
    }
    MN_TRY(linear(arith, M, cat, d.hv, cath, d.hv, l.w_o, W, d.hv, l.b_o, yf, W, gws, gwb, stream));
    MN_TRY(mn_rms_scale_add_rows(xr, W, yf, W, l.norm1, m->eps, xh, W, M, W, stream));
    // ---- feed-forward ----
    if (l.ff > 0) {
      bool fused = false;                                // few rows: the gelu product rides the weight-streaming product's epilogue
      if (!acth) MN_TRY(linear_geglu(arith, M, xr, W, l.w_gate_up, l.ff, W, act, l.ff, gws, gwb, stream, &fused));
      if (!fused) {
        MN_TRY(linear(arith, M, xr, W, xh, W, l.w_gate_up, 2 * l.ff, W, nullptr, gu, 2 * l.ff, gws, gwb, stream));
        MN_TRY(mn_gelu_mul_rows(gu, 2 * l.ff, gu + l.ff, 2 * l.ff, nullptr, 0, nullptr, act, l.ff, acth, l.ff, M, l.ff, stream));
      }
      MN_TRY(linear(arith, M, act, l.ff, acth, l.ff, l.w_down, W, l.ff, nullptr, yf, W, gws, gwb, stream));
      MN_TRY(mn_rms_scale_add_rows(xr, W, yf, W, l.norm2, m->eps, xh, W, M, W, stream));
    }
    // ---- the per-layer token input ----
    if (l.side > 0) {
      const int sp = pad8(l.side);
      MN_TRY(linear(arith, M, xr, W, xh, W, l.w_side_gate, sp, W, nullptr, sg, sp, gws, gwb, stream));
      MN_TRY(mn_gelu_mul_rows(sg, sp, nullptr, 0, l.side_table, m->side_ld, row_tok, sa, l.side, nullptr, 0, M, l.side, stream));
      MN_TRY(linear(arith, M, sa, l.side, nullptr, 0, l.w_side_proj, W, l.side, nullptr, yf, W, gws, gwb, stream));
      MN_TRY(mn_rms_scale_add_rows(xr, W, yf, W, l.side_norm, m->eps, xh, W, M, W, stream));
    }
    if (trace) {
      hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)mn_cdiv(W, 256), (unsigned)M), dim3(256), 0, hs, xr, (int64_t)W,
                         trace + (size_t)li * R * W, W);
      MN_CHECK_LAUNCH("mn_pn_step(trace)");
    }
  }
  // decode rows: the one-workgroup-per-row launch with the row in registers (the other step functions' launch, here without a filter)
  if (one_row && W <= 8192) MN_TRY(mn_axpy_rms_filter_rows(xr, W, nullptr, W, 1.0f, m->final_w, m->eps, nullptr, 0, nullptr, row_seq, row_slot, out, W, M, W, stream));
  else MN_TRY(mn_axpy_rms_rows(xr, W, nullptr, W, 1.0f, m->final_w, m->eps, out, W, nullptr, 0, M, W, stream));
#undef MN_TRY
  return MN_OK;
}
