// pnorm_ops.hip — operators of the post-norm mixed-mixer sequence models (mingnative.h section 12).  Everything here is fp32: the
// residual sum, norms, angles, gates, decays and the recurrent state.
//   mn_rms_scale_add_rows         x += y / sqrt(mean(y^2) + eps) * w   (the norm sits on the sublayer's RESULT)
//   mn_gelu_mul_rows              y = gelu_tanh(a) * b, b a second row or a slice of a bf16 table row chosen by an index per row
//   mn_proj_norm_rope_append      RMS norm over the WHOLE q and k projections, rotary pairs (interleaved or half-split), append to arenas
//   mn_latent_rope_append         normed latent + one rotated key part into a latent arena; the queries' rotated parts
//   mn_head_sigmoid_gate_rows     one sigmoid gate per head
//   mn_delta_prep_rows            short causal conv + silu of q / k / v, unit-length q and k heads, write strengths and decays
//   mn_gated_delta_rows           the gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
//   mn_head_rms_silu_gate_rows    per-head RMS norm with a weight shared by the heads, times silu(gate)
#include <math.h>

#include "common.h"
#include "mfma_f32_tiles.h"

extern "C" int mn_rotary_frequencies_scaled_host(int dims, double base, double factor, double low, double high, double original, float* freq) {
  MN_CHECK_ARG(freq && dims >= 2 && (dims % 2) == 0 && base > 0.0 && factor >= 0.0, "mn_rotary_frequencies_scaled_host: bad args");
  MN_CHECK_ARG(factor == 0.0 || (high > low && original > 0.0 && low > 0.0), "mn_rotary_frequencies_scaled_host: scaling needs 0 < low < high, original > 0");
  const double two_pi = 6.283185307179586476925286766559;
  for (int i = 0; i < dims / 2; ++i) {
    double f = pow(base, -2.0 * (double)i / (double)dims);
    if (factor > 0.0) {
      const double wave = two_pi / f;
      if (wave > original / low) f = f / factor;
      else if (!(wave < original / high)) {
        const double s = (original / wave - low) / (high - low);
        f = (1.0 - s) * f / factor + s * f;
      }
    }
    freq[i] = (float)f;
  }
  return MN_OK;
}

namespace {

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_x(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rms_scale_add_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y, int64_t ldy,
                                                            const bf16_t* __restrict__ w, float eps, bf16_t* __restrict__ x16, int64_t ldx16,
                                                            int n) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  const float* yr = y + (int64_t)m * ldy;
  float ss = 0.f;
  for (int c = tid; c < n; c += 256) { const float v = yr[c]; ss = fmaf(v, v, ss); }
  ss = block_sum(ss, red);
  const float den = sqrtf(ss / (float)n + eps);
  for (int c = tid; c < n; c += 256) {
    const float t = x[(int64_t)m * ldx + c] + yr[c] / den * bf16_to_f32(w[c]);
    x[(int64_t)m * ldx + c] = t;
    if (x16) x16[(int64_t)m * ldx16 + c] = f32_to_bf16(t);
  }
}

// the same with the row in registers (rows of at most 256 VPT values): every load is issued before the reduction
template <int VPT>
__global__ __launch_bounds__(256) void rms_scale_add_reg_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y, int64_t ldy,
                                                                const bf16_t* __restrict__ w, float eps, bf16_t* __restrict__ x16, int64_t ldx16,
                                                                int n) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  float yv[VPT], xv[VPT], wv[VPT];
#pragma unroll
  for (int t = 0; t < VPT; ++t) {
    const int c = tid + 256 * t;
    yv[t] = c < n ? y[(int64_t)m * ldy + c] : 0.f;
    xv[t] = c < n ? x[(int64_t)m * ldx + c] : 0.f;
    wv[t] = c < n ? bf16_to_f32(w[c]) : 0.f;
  }
  float ss = 0.f;
#pragma unroll
  for (int t = 0; t < VPT; ++t) ss = fmaf(yv[t], yv[t], ss);
  ss = block_sum(ss, red);
  const float den = sqrtf(ss / (float)n + eps);
#pragma unroll
  for (int t = 0; t < VPT; ++t) {
    const int c = tid + 256 * t;
    if (c < n) {
      const float v = xv[t] + yv[t] / den * wv[t];
      x[(int64_t)m * ldx + c] = v;
      if (x16) x16[(int64_t)m * ldx16 + c] = f32_to_bf16(v);
    }
  }
}

__global__ __launch_bounds__(256) void gelu_mul_kernel(const float* __restrict__ a, int64_t lda, const float* __restrict__ b, int64_t ldb,
                                                       const bf16_t* __restrict__ table, int64_t ldt, const int32_t* __restrict__ idx,
                                                       float* __restrict__ y, int64_t ldy, bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const float other = table ? bf16_to_f32(table[(int64_t)idx[m] * ldt + c]) : b[(int64_t)m * ldb + c];
  const float v = gelu_tanh_f(a[(int64_t)m * lda + c]) * other;
  if (y) y[(int64_t)m * ldy + c] = v;
  if (y16) y16[(int64_t)m * ldy16 + c] = f32_to_bf16(v);
}

// ---------------------------------------------------------------------------------------------------------------------------
// Rotation of value d of a head (d < rot_dims) at position pos.  interleaved: pairs (2i, 2i + 1); else pairs (i, i + rot_dims / 2).
// `at(j)` returns value j of the same head (already normed).
template <typename At>
__device__ __forceinline__ float rotate_value(At at, int d, int rot_dims, int interleaved, const float* __restrict__ freq, int pos) {
  const int half = rot_dims >> 1;
  const bool first = interleaved ? (d & 1) == 0 : d < half;
  const int i = interleaved ? (d >> 1) : (first ? d : d - half);
  const int partner = interleaved ? (d ^ 1) : (first ? d + half : d - half);
  const float ang = (float)pos * freq[i];
  const float c = cosf(ang), s = sinf(ang);
  const float v = at(d), p = at(partner);
  return first ? v * c - p * s : v * c + p * s;
}

struct ProjNormArgs {
  const float* qkv; int64_t ld;
  int H, G, dim, vdim, rot_dims, interleaved, t_max;
  const bf16_t *q_norm, *k_norm;
  const float* freq;
  float eps, q_scale;
  const int32_t *row_seq, *row_slot;
  float* q_out; int64_t ldq;
  float* k_arena; int64_t ldk;
  float* v_arena; int64_t ldv;
};

__global__ __launch_bounds__(256) void proj_norm_rope_append_kernel(ProjNormArgs a) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  const int nq = a.H * a.dim, nk = a.G * a.dim, nv = a.G * a.vdim;
  const float* row = a.qkv + (int64_t)m * a.ld;
  const int seq = a.row_seq[m], pos = a.row_slot[m];
  float rq = 1.0f, rk = 1.0f;
  if (a.q_norm) {
    float ss = 0.f;
    for (int e = tid; e < nq; e += 256) ss = fmaf(row[e], row[e], ss);
    rq = 1.0f / sqrtf(block_sum(ss, red) / (float)nq + a.eps);
  }
  if (a.k_norm) {
    float ss = 0.f;
    for (int e = tid; e < nk; e += 256) ss = fmaf(row[nq + e], row[nq + e], ss);
    rk = 1.0f / sqrtf(block_sum(ss, red) / (float)nk + a.eps);
  }
  for (int e = tid; e < nq; e += 256) {
    const int d = e % a.dim, e0 = e - d;
    auto at = [&](int j) { return row[e0 + j] * rq * (a.q_norm ? bf16_to_f32(a.q_norm[e0 + j]) : 1.0f); };
    const float v = d < a.rot_dims ? rotate_value(at, d, a.rot_dims, a.interleaved, a.freq, pos) : at(d);
    a.q_out[(int64_t)m * a.ldq + e] = v * a.q_scale;
  }
  float* kd = a.k_arena + ((int64_t)seq * a.t_max + pos) * a.ldk;
  for (int e = tid; e < nk; e += 256) {
    const int d = e % a.dim, e0 = e - d;
    auto at = [&](int j) { return row[nq + e0 + j] * rk * (a.k_norm ? bf16_to_f32(a.k_norm[e0 + j]) : 1.0f); };
    kd[e] = d < a.rot_dims ? rotate_value(at, d, a.rot_dims, a.interleaved, a.freq, pos) : at(d);
  }
  float* vd = a.v_arena + ((int64_t)seq * a.t_max + pos) * a.ldv;
  for (int e = tid; e < nv; e += 256) vd[e] = row[nq + nk + e];
}

struct LatentRopeArgs {
  const float* qd; int64_t ld;               // per row [q: H x (dim + rot) ; down projection: rank + rot]
  int H, dim, rot, rank, rot_dims, interleaved, t_max;
  const bf16_t* c_norm;                      // [rank]
  const float* freq;
  float eps, q_scale;
  const int32_t *row_seq, *row_slot;
  float* q_out; int64_t ldq;                 // [M, H x (rank + rot)]: the rotated parts land at columns rank .. rank + rot of every head
  float* arena; int64_t lda;                 // [n_seq, t_max, lda >= rank + rot]
};

__global__ __launch_bounds__(256) void latent_rope_append_kernel(LatentRopeArgs a) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  const int hq = a.dim + a.rot;
  const float* row = a.qd + (int64_t)m * a.ld;
  const float* dk = row + (int64_t)a.H * hq;
  const int seq = a.row_seq[m], pos = a.row_slot[m];
  float ss = 0.f;
  for (int e = tid; e < a.rank; e += 256) ss = fmaf(dk[e], dk[e], ss);
  const float den = sqrtf(block_sum(ss, red) / (float)a.rank + a.eps);
  float* dst = a.arena + ((int64_t)seq * a.t_max + pos) * a.lda;
  for (int e = tid; e < a.rank; e += 256) dst[e] = dk[e] / den * bf16_to_f32(a.c_norm[e]);
  for (int d = tid; d < a.rot; d += 256) {
    auto at = [&](int j) { return dk[a.rank + j]; };
    dst[a.rank + d] = d < a.rot_dims ? rotate_value(at, d, a.rot_dims, a.interleaved, a.freq, pos) : at(d);
  }
  for (int e = tid; e < a.H * a.rot; e += 256) {
    const int h = e / a.rot, d = e - h * a.rot;
    const float* src = row + (int64_t)h * hq + a.dim;
    auto at = [&](int j) { return src[j]; };
    const float v = d < a.rot_dims ? rotate_value(at, d, a.rot_dims, a.interleaved, a.freq, pos) : at(d);
    a.q_out[(int64_t)m * a.ldq + (int64_t)h * (a.rank + a.rot) + a.rank + d] = v * a.q_scale;
  }
}

__global__ __launch_bounds__(256) void head_sigmoid_gate_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ g, int64_t ldg,
                                                                bf16_t* __restrict__ x16, int64_t ldx16, int H, int vdim) {
  const int m = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
  if (e >= H * vdim) return;
  const float v = x[(int64_t)m * ldx + e] * sigmoid_f(g[(int64_t)m * ldg + e / vdim]);
  x[(int64_t)m * ldx + e] = v;
  if (x16) x16[(int64_t)m * ldx16 + e] = f32_to_bf16(v);
}

// ---------------------------------------------------------------------------------------------------------------------------
// Gated delta rule, preparation of a row: channels [q: G dim ; k: G dim ; v: H vdim] of the raw projections go through their causal
// filter (earlier inputs from the rows before it in this call, then from the sequence's state) and silu; q and k heads become unit
// vectors (q also times q_scale); beta = sigmoid(b), decay = exp(-exp(a_log) softplus(a + dt_bias)).
struct DeltaPrepArgs {
  const float* proj; int64_t ld;             // raw [q ; k ; v] at column 0, b at off_b, a at off_a
  int H, G, dim, vdim, taps, off_b, off_a;
  const bf16_t* w_conv;                      // [2 G dim + H vdim, taps], the last tap multiplies the current row
  float* state;                              // [n_seq, taps - 1, channels]
  int advance;                               // 1: every row is alone in its sequence and moves the state on by itself
  const float *a_log, *dt_bias;              // device fp32 [H]
  float unit_eps, q_scale;
  const int32_t *row_seq, *row_slot, *row_back;
  float* qkv; int64_t ldo;                   // [M, channels]
  float* bd; int64_t ldbd;                   // [M, 2 H]: beta, decay
};

__device__ __forceinline__ float conv_silu(const DeltaPrepArgs& a, int m, int c, int n, int seq, int slot, int back) {
  float acc = 0.f;
  for (int k = 0; k < a.taps; ++k) {
    float v = 0.f;
    if (k <= back) v = a.proj[(int64_t)(m - k) * a.ld + c];
    else if (slot - k >= 0) v = a.state[((int64_t)seq * (a.taps - 1) + (k - back - 1)) * n + c];
    acc = fmaf(bf16_to_f32(a.w_conv[(int64_t)c * a.taps + (a.taps - 1 - k)]), v, acc);
  }
  if (a.advance && a.taps > 1) {                // a one-row sequence: entry i becomes entry i - 1, entry 0 this row's input
    float* st = a.state + (int64_t)seq * (a.taps - 1) * n + c;
    for (int i = a.taps - 2; i >= 1; --i) st[(int64_t)i * n] = st[(int64_t)(i - 1) * n];
    st[0] = a.proj[(int64_t)m * a.ld + c];
  }
  return silu_x(acc);
}

// grid (M, ceil(units / 4)): a wave takes one unit of a row — a q or k head (its unit norm is a wave's reduction) or 256 value channels
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaPrepArgs a) {
  const int m = blockIdx.x, tid = threadIdx.x, lane = tid & 63, unit = blockIdx.y * 4 + (tid >> 6);
  const int nqk = 2 * a.G * a.dim, nv = a.H * a.vdim, n = nqk + nv;
  const int seq = a.row_seq[m], slot = a.row_slot[m], back = a.row_back[m];
  float* out = a.qkv + (int64_t)m * a.ldo;
  if (unit < 2 * a.G) {
    const int c0 = unit * a.dim;
    float ss = 0.f;
    for (int d = lane; d < a.dim; d += 64) {
      const float v = conv_silu(a, m, c0 + d, n, seq, slot, back);
      out[c0 + d] = v;
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    const float r = (unit < a.G ? a.q_scale : 1.0f) / sqrtf(ss + a.unit_eps);
    for (int d = lane; d < a.dim; d += 64) out[c0 + d] *= r;      // the lane rereads what it wrote itself
  } else {
    const int e0 = (unit - 2 * a.G) * 256;
    for (int e = e0 + lane; e < min(nv, e0 + 256); e += 64) out[nqk + e] = conv_silu(a, m, nqk + e, n, seq, slot, back);
  }
  if (blockIdx.y == 0) {
    for (int h = tid; h < a.H; h += 256) {
      const float* row = a.proj + (int64_t)m * a.ld;
      a.bd[(int64_t)m * a.ldbd + h] = sigmoid_f(row[a.off_b + h]);
      a.bd[(int64_t)m * a.ldbd + a.H + h] = expf(-expf(a.a_log[h]) * softplus_f(row[a.off_a + h] + a.dt_bias[h]));
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// The recurrence.  Every value column of a head's state is a recurrence of its own: with s = S[:, c],
//   s <- g s;  u = beta (v_c - s . k);  s <- s + k u;  o_c = s . q     i.e.  o_c = g (s_old . q) + u (k . q),  u = beta (v_c - g (s_old . k))
// so both dot products are taken on the OLD column and reduced together.
struct DeltaArgs {
  const float* qkv; int64_t ld;              // per row [q: G dim ; k: G dim ; v: H vdim], prepared
  const float* bd; int64_t ldbd;             // per row [beta: H ; decay: H]
  int H, G, dim, vdim;
  float* state;                              // [n_seq, H, dim, vdim]
  const int32_t *row_seq, *row_slot, *row_back;
  float* out; int64_t ldo;                   // [M, H vdim]
  int M;
};

__device__ __forceinline__ float sum8(float v) {                    // over the 8 lanes of an aligned group; every lane gets the sum
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  return v;
}

// Rows of sequences (a prompt portion): grid (M, H, ceil(vdim / 32)); the workgroup of a sequence's FIRST row in the call walks that
// sequence's rows.  A workgroup owns 32 value columns; 8 lanes share a column, lane s of them holds the state rows s, s + 8, ... in
// registers (NR of them; NR = 0: the column stays in the arena, any dim).  The rows are taken in batches of DB: a batch's q, k, v,
// write strengths and decays go global -> registers (while the previous batch is computed) -> LDS, k . q of every row is summed once
// per workgroup, and the DB steps of the recurrence then run from LDS and registers alone — a step is two partial dot products, one
// reduction over the 8 lanes and the update, with no barrier and no memory latency between steps.
constexpr int DB = 16;
template <int NR>
__global__ __launch_bounds__(256) void delta_rows_kernel(DeltaArgs a) {
  extern __shared__ float lds[];             // [DB][2 dim] q, k; [DB][32] v; [DB] beta, decay, k . q
  const int m0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, s = tid & 7, cl = tid >> 3, c = blockIdx.z * 32 + cl;
  if (a.row_back[m0] != 0) return;
  const int d = a.dim, kvh = h / (a.H / a.G);
  const bool on = c < a.vdim;
  // rows of this sequence in the call: they are consecutive, so the rows that continue it form a prefix of every 256 looked at
  int n = 1;
  for (;;) {
    const int m = m0 + n + tid;
    const int cnt = __syncthreads_count(m < a.M && a.row_back[m] == m - m0);
    n += cnt;
    if (cnt < 256) break;
  }
  float* sp = a.state + (((int64_t)a.row_seq[m0] * a.H + h) * d) * a.vdim + (on ? c : 0);
  const bool fresh = a.row_slot[m0] == 0;
  constexpr int NS = NR > 0 ? NR : 1;
  float S[NS];
  if (NR > 0) {
#pragma unroll
    for (int j = 0; j < NS; ++j) { const int i = s + 8 * j; S[j] = (on && !fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f; }
  } else if (fresh && on) {
    for (int i = s; i < d; i += 8) sp[(int64_t)i * a.vdim] = 0.f;
  }
  float* qk = lds;                           // row r: q at r * 2 d, k at r * 2 d + d
  float* vs = qk + DB * 2 * d;               // [DB][32]
  float* bs = vs + DB * 32;                  // [DB] beta, [DB] decay, [DB] k . q
  constexpr int NQ = 32;                     // staged q / k values per thread and batch: DB * 2 dim / 256 <= 32 for dim <= 256
  const int per = 2 * d * DB;
  float rq[NQ], rv[2], rb = 0.f;
  auto fetch = [&](int b0) {                 // batch rows b0 .. b0 + DB of the sequence into registers
    const int rows = min(DB, n - b0);
#pragma unroll
    for (int t = 0; t < NQ; ++t) {
      const int e = tid + 256 * t;
      if (e < per) {
        const int r = e / (2 * d), i = e - r * 2 * d;
        rq[t] = r < rows ? a.qkv[(int64_t)(m0 + b0 + r) * a.ld + (i < d ? 0 : a.G * d) + (int64_t)kvh * d + (i < d ? i : i - d)] : 0.f;
      }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int e = tid + 256 * t, r = e >> 5, cc = blockIdx.z * 32 + (e & 31);
      rv[t] = (r < rows && cc < a.vdim) ? a.qkv[(int64_t)(m0 + b0 + r) * a.ld + 2 * a.G * d + (int64_t)h * a.vdim + cc] : 0.f;
    }
    if (tid < 2 * DB) {
      const int r = tid % DB;
      rb = r < rows ? a.bd[(int64_t)(m0 + b0 + r) * a.ldbd + (tid < DB ? 0 : a.H) + h] : 0.f;
    }
  };
  fetch(0);
  for (int b0 = 0; b0 < n; b0 += DB) {
    const int rows = min(DB, n - b0);
    __syncthreads();                         // the previous batch's steps have read their rows
    if (NR > 0 || d <= 256) {
#pragma unroll
      for (int t = 0; t < NQ; ++t) { const int e = tid + 256 * t; if (e < per) qk[e] = rq[t]; }
    } else {                                 // larger heads than the registers stage: straight from memory
      for (int e = tid; e < per; e += 256) {
        const int r = e / (2 * d), i = e - r * 2 * d;
        qk[e] = r < rows ? a.qkv[(int64_t)(m0 + b0 + r) * a.ld + (i < d ? 0 : a.G * d) + (int64_t)kvh * d + (i < d ? i : i - d)] : 0.f;
      }
    }
    vs[tid] = rv[0]; vs[tid + 256] = rv[1];
    if (tid < 2 * DB) bs[tid] = rb;
    __syncthreads();
    if (b0 + DB < n) fetch(b0 + DB);         // in flight while this batch is computed
    {                                        // k . q of every row: 16 threads a row
      const int r = tid >> 4, l = tid & 15;
      float t = 0.f;
      for (int i = l; i < d; i += 16) t = fmaf(qk[r * 2 * d + i], qk[r * 2 * d + d + i], t);
      t = row16_sum(t);
      if (l == 0) bs[2 * DB + r] = t;
    }
    lds_barrier();                           // orders LDS only: the next batch's loads stay in flight
    for (int r = 0; r < rows; ++r) {
      const float* q = qk + r * 2 * d;
      const float* k = q + d;
      const float v = vs[r * 32 + cl], beta = bs[r], g = bs[DB + r], kq = bs[2 * DB + r];
      float pk = 0.f, pq = 0.f;
      if (NR > 0) {
#pragma unroll
        for (int j = 0; j < NS; ++j) {
          const int i = s + 8 * j;
          if (i < d) { pk = fmaf(S[j], k[i], pk); pq = fmaf(S[j], q[i], pq); }
        }
      } else {
        for (int i = s; i < d; i += 8) {
          const float sv = on ? sp[(int64_t)i * a.vdim] : 0.f;
          pk = fmaf(sv, k[i], pk); pq = fmaf(sv, q[i], pq);
        }
      }
      pk = sum8(pk); pq = sum8(pq);
      const float u = beta * (v - g * pk);
      if (NR > 0) {
#pragma unroll
        for (int j = 0; j < NS; ++j) { const int i = s + 8 * j; if (i < d) S[j] = fmaf(g, S[j], k[i] * u); }
      } else if (on) {
        for (int i = s; i < d; i += 8) sp[(int64_t)i * a.vdim] = fmaf(g, sp[(int64_t)i * a.vdim], k[i] * u);
      }
      if (on && s == 0) a.out[(int64_t)(m0 + b0 + r) * a.ldo + (int64_t)h * a.vdim + c] = fmaf(g, pq, u * kq);
    }
  }
  if (NR > 0 && on) {
#pragma unroll
    for (int j = 0; j < NS; ++j) { const int i = s + 8 * j; if (i < d) sp[(int64_t)i * a.vdim] = S[j]; }
  }
}

// The same walk for heads of at most 256 state rows, without a branch in the step: grid (H * ceil(vdim / CPB), M) — the workgroups that
// work (those of a sequence's first row) are neighbours in the launch order and land on different CUs.  LPC lanes share a value column
// (CPB = 256 / LPC columns a workgroup); a lane holds the state rows 4 (s + LPC jj) + t, t < 4, jj < NS / 4, so that q and k come from
// LDS in 16-byte reads; LDS rows are padded with zeros to DP = NS * LPC values, under which the padded state rows stay zero.
template <int NS, int LPC, int DBT>
__global__ __launch_bounds__(256) void delta_rows_fast_kernel(DeltaArgs a) {
  constexpr int CPB = 256 / LPC, DP = NS * LPC, NQ = DBT * 2 * DP / 256, NV = (DBT * CPB + 255) / 256;
  extern __shared__ float lds[];             // [DBT][2 DP] q, k; [DBT][CPB] v; [DBT] beta, decay, k . q; [DBT][CPB] outputs
  const int m0 = blockIdx.y, ncb = (a.vdim + CPB - 1) / CPB, h = blockIdx.x / ncb, cb = blockIdx.x - h * ncb;
  const int tid = threadIdx.x, s = tid % LPC, cl = tid / LPC, c = cb * CPB + cl;
  if (a.row_back[m0] != 0) return;
  const int d = a.dim, kvh = h / (a.H / a.G);
  const bool on = c < a.vdim;
  int n = 1;
  for (;;) {
    const int m = m0 + n + tid;
    const int cnt = __syncthreads_count(m < a.M && a.row_back[m] == m - m0);
    n += cnt;
    if (cnt < 256) break;
  }
  float* sp = a.state + (((int64_t)a.row_seq[m0] * a.H + h) * d) * a.vdim + (on ? c : 0);
  const bool fresh = a.row_slot[m0] == 0;
  float S[NS];
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const int i = 4 * (s + LPC * (j >> 2)) + (j & 3);
    S[j] = (on && !fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f;
  }
  float* qk = lds;                           // row r: q at r * 2 DP, k at r * 2 DP + DP
  float* vs = qk + DBT * 2 * DP;
  float* bs = vs + DBT * CPB;
  float* os = bs + 3 * DBT;                   // [DBT][CPB] the batch's outputs
  float rq[NQ], rv[NV], rb = 0.f;
  // element e of a batch's q / k block: row e / (2 DP), value e % (2 DP) (q below DP, k from DP on)
  auto fetch = [&](int b0) {
    const int rows = min(DBT, n - b0);
#pragma unroll
    for (int t = 0; t < NQ; ++t) {
      const int e = tid + 256 * t, r = e / (2 * DP), i = e % (2 * DP), ii = i % DP;
      rq[t] = (r < rows && ii < d) ? a.qkv[(int64_t)(m0 + b0 + r) * a.ld + (i < DP ? 0 : a.G * d) + (int64_t)kvh * d + ii] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      const int e = tid + 256 * t, r = e / CPB, cc = cb * CPB + e % CPB;
      rv[t] = (r < rows && cc < a.vdim) ? a.qkv[(int64_t)(m0 + b0 + r) * a.ld + 2 * a.G * d + (int64_t)h * a.vdim + cc] : 0.f;
    }
    if (tid < 2 * DBT) {
      const int r = tid % DBT;
      rb = r < rows ? a.bd[(int64_t)(m0 + b0 + r) * a.ldbd + (tid < DBT ? 0 : a.H) + h] : 0.f;
    }
  };
  fetch(0);
  for (int b0 = 0; b0 < n; b0 += DBT) {
    const int rows = min(DBT, n - b0);
    lds_barrier();                           // the previous batch's steps have read their rows
#pragma unroll
    for (int t = 0; t < NQ; ++t) qk[tid + 256 * t] = rq[t];
#pragma unroll
    for (int t = 0; t < NV; ++t) { const int e = tid + 256 * t; if (e < DBT * CPB) vs[e] = rv[t]; }
    if (tid < 2 * DBT) bs[tid] = rb;
    lds_barrier();
    if (b0 + DBT < n) fetch(b0 + DBT);         // in flight while this batch is computed
    for (int r = tid >> 4; r < DBT; r += 16) {   // k . q of every row: 16 threads a row
      const int l = tid & 15;
      float t = 0.f;
#pragma unroll
      for (int i = l; i < DP; i += 16) t = fmaf(qk[r * 2 * DP + i], qk[r * 2 * DP + DP + i], t);
      t = row16_sum(t);
      if (l == 0) bs[2 * DBT + r] = t;
    }
    lds_barrier();                           // orders LDS only: the next batch's loads stay in flight
    // the operands of step r + 1 are read from LDS before step r is computed: they do not depend on the state
    float kk[NS], qq[NS], v, beta, g, kq;
    auto load_row = [&](int r, float (&k_)[NS], float (&q_)[NS], float& v_, float& b_, float& g_, float& kq_) {
      const float* q = qk + r * 2 * DP + 4 * s;
#pragma unroll
      for (int jj = 0; jj < NS / 4; ++jj) {
        const float4 k4 = *reinterpret_cast<const float4*>(q + DP + 4 * LPC * jj), q4 = *reinterpret_cast<const float4*>(q + 4 * LPC * jj);
        k_[4 * jj] = k4.x; k_[4 * jj + 1] = k4.y; k_[4 * jj + 2] = k4.z; k_[4 * jj + 3] = k4.w;
        q_[4 * jj] = q4.x; q_[4 * jj + 1] = q4.y; q_[4 * jj + 2] = q4.z; q_[4 * jj + 3] = q4.w;
      }
      v_ = vs[r * CPB + cl]; b_ = bs[r]; g_ = bs[DBT + r]; kq_ = bs[2 * DBT + r];
    };
    load_row(0, kk, qq, v, beta, g, kq);
#pragma unroll 2
    for (int r = 0; r < rows; ++r) {
      float kn[NS], qn[NS], vn, bn, gn, kqn;
      load_row(min(r + 1, DBT - 1), kn, qn, vn, bn, gn, kqn);
      float pk = 0.f, pq = 0.f, pk2 = 0.f, pq2 = 0.f;
#pragma unroll
      for (int j = 0; j < NS; j += 2) {
        pk = fmaf(S[j], kk[j], pk); pk2 = fmaf(S[j + 1], kk[j + 1], pk2);
        pq = fmaf(S[j], qq[j], pq); pq2 = fmaf(S[j + 1], qq[j + 1], pq2);
      }
      pk += pk2; pq += pq2;
      if (LPC == 16) { pk = row16_sum(pk); pq = row16_sum(pq); } else { pk = sum8(pk); pq = sum8(pq); }
      const float u = beta * (v - g * pk);
#pragma unroll
      for (int j = 0; j < NS; ++j) S[j] = fmaf(g, S[j], kk[j] * u);
      if (s == 0) os[r * CPB + cl] = fmaf(g, pq, u * kq);
#pragma unroll
      for (int j = 0; j < NS; ++j) { kk[j] = kn[j]; qq[j] = qn[j]; }
      v = vn; beta = bn; g = gn; kq = kqn;
    }
    lds_barrier();
#pragma unroll
    for (int t = 0; t < NV; ++t) {           // the batch's outputs, a row's columns side by side
      const int e = tid + 256 * t, r = e / CPB, cc = cb * CPB + e % CPB;
      if (r < rows && cc < a.vdim) a.out[(int64_t)(m0 + b0 + r) * a.ldo + (int64_t)h * a.vdim + cc] = os[e];
    }
  }
  if (on) {
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      const int i = 4 * (s + LPC * (j >> 2)) + (j & 3);
      if (i < d) sp[(int64_t)i * a.vdim] = S[j];
    }
  }
}

// Decode rows (every row alone in its sequence): grid (M, H, ceil(vdim / 32)); a workgroup owns 32 value columns of one head's
// state, its 8 groups of 32 threads split the state's rows, the partial dot products meet in LDS, then every thread updates its rows.
__global__ __launch_bounds__(256) void delta_step_kernel(DeltaArgs a) {
  extern __shared__ float lds[];             // [2 dim] q, k; [3][8][32] partial sums
  const int m = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, cl = tid & 31, sub = tid >> 5, c = blockIdx.z * 32 + cl;
  const int d = a.dim, kvh = h / (a.H / a.G);
  const float* row = a.qkv + (int64_t)m * a.ld;
  float* q = lds;
  float* k = lds + d;
  float* part = lds + 2 * d;
  for (int i = tid; i < 2 * d; i += 256) lds[i] = row[(i < d ? 0 : a.G * d) + (int64_t)kvh * d + (i < d ? i : i - d)];
  const bool on = c < a.vdim;
  const float v = on ? row[2 * a.G * d + (int64_t)h * a.vdim + c] : 0.f;
  const float beta = a.bd[(int64_t)m * a.ldbd + h], g = a.bd[(int64_t)m * a.ldbd + a.H + h];
  const bool fresh = a.row_slot[m] == 0;
  float* sp = a.state + (((int64_t)a.row_seq[m] * a.H + h) * d) * a.vdim + (on ? c : 0);
  __syncthreads();
  float pk = 0.f, pq = 0.f, kq = 0.f;
  constexpr int PRE = 8;
  for (int i0 = sub; i0 < d; i0 += 8 * PRE) {
    float sv[PRE];
#pragma unroll
    for (int t = 0; t < PRE; ++t) { const int i = i0 + 8 * t; sv[t] = (on && !fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f; }
#pragma unroll
    for (int t = 0; t < PRE; ++t) {
      const int i = i0 + 8 * t;
      if (i < d) { pk = fmaf(sv[t], k[i], pk); pq = fmaf(sv[t], q[i], pq); kq = fmaf(k[i], q[i], kq); }
    }
  }
  part[sub * 32 + cl] = pk; part[256 + sub * 32 + cl] = pq; part[512 + sub * 32 + cl] = kq;
  __syncthreads();
  pk = pq = kq = 0.f;
#pragma unroll
  for (int t = 0; t < 8; ++t) { pk += part[t * 32 + cl]; pq += part[256 + t * 32 + cl]; kq += part[512 + t * 32 + cl]; }
  const float u = beta * (v - g * pk);
  if (on) {
    if (sub == 0) a.out[(int64_t)m * a.ldo + (int64_t)h * a.vdim + c] = fmaf(g, pq, u * kq);
    for (int i0 = sub; i0 < d; i0 += 8 * PRE) {
      float sv[PRE];
#pragma unroll
      for (int t = 0; t < PRE; ++t) { const int i = i0 + 8 * t; sv[t] = (!fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f; }
#pragma unroll
      for (int t = 0; t < PRE; ++t) { const int i = i0 + 8 * t; if (i < d) sp[(int64_t)i * a.vdim] = fmaf(g, sv[t], k[i] * u); }
    }
  }
}

// grid (ceil(H / 4), M): one wave per head
__global__ __launch_bounds__(256) void head_rms_silu_gate_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, float eps,
                                                                 const float* __restrict__ g, int64_t ldg, float* __restrict__ y, int64_t ldy,
                                                                 bf16_t* __restrict__ y16, int64_t ldy16, int H, int vdim) {
  const int m = blockIdx.y, h = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (h >= H) return;
  const float* xr = x + (int64_t)m * ldx + (int64_t)h * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += 64) ss = fmaf(xr[c], xr[c], ss);
  const float den = sqrtf(wave_sum(ss) / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) {
    const float v = xr[c] / den * bf16_to_f32(w[c]) * silu_x(g[(int64_t)m * ldg + (int64_t)h * vdim + c]);
    if (y) y[(int64_t)m * ldy + (int64_t)h * vdim + c] = v;
    if (y16) y16[(int64_t)m * ldy16 + (int64_t)h * vdim + c] = f32_to_bf16(v);
  }
}

}  // namespace

extern "C" int mn_rms_scale_add_rows(float* x, int64_t ldx, const float* y, int64_t ldy, const uint16_t* w, float eps, uint16_t* x16,
                                     int64_t ldx16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && y && w && M >= 1 && n >= 1, "mn_rms_scale_add_rows: bad args");
  hipStream_t st = mn_stream(stream);
#define MN_RSA(V_) hipLaunchKernelGGL((rms_scale_add_reg_kernel<V_>), dim3((unsigned)M), dim3(256), 0, st, x, ldx, y, ldy, w, eps, x16, ldx16, n)
  if (n <= 1024) MN_RSA(4); else if (n <= 2048) MN_RSA(8); else if (n <= 4096) MN_RSA(16); else if (n <= 8192) MN_RSA(32);
  else hipLaunchKernelGGL(rms_scale_add_kernel, dim3((unsigned)M), dim3(256), 0, st, x, ldx, y, ldy, w, eps, x16, ldx16, n);
#undef MN_RSA
  MN_CHECK_LAUNCH("mn_rms_scale_add_rows");
  return MN_OK;
}

extern "C" int mn_gelu_mul_rows(const float* a, int64_t lda, const float* b, int64_t ldb, const uint16_t* table, int64_t ldt,
                                const int32_t* idx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(a && (b || (table && idx)) && (y || y16) && M >= 1 && M <= 65535 && n >= 1, "mn_gelu_mul_rows: bad args");
  hipLaunchKernelGGL(gelu_mul_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), a, lda, b, ldb,
                     b ? nullptr : table, ldt, idx, y, ldy, y16, ldy16, n);
  MN_CHECK_LAUNCH("mn_gelu_mul_rows");
  return MN_OK;
}

extern "C" int mn_proj_norm_rope_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* q_norm,
                                        const uint16_t* k_norm, float eps, int rot_dims, int interleaved, const float* freq, float q_scale,
                                        const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena,
                                        int64_t ldk, float* v_arena, int64_t ldv, int t_max, void* stream) {
  MN_CHECK_ARG(qkv && row_seq && row_slot && q_out && k_arena && v_arena && M >= 1 && H >= 1 && G >= 1 && dim >= 1 && vdim >= 1 && t_max >= 1 &&
                   rot_dims >= 0 && rot_dims <= dim && (rot_dims % 2) == 0 && (rot_dims == 0 || freq) && ldk >= (int64_t)G * dim &&
                   ldv >= (int64_t)G * vdim,
               "mn_proj_norm_rope_append: bad args (rot_dims=%d of dim=%d)", rot_dims, dim);
  ProjNormArgs a{qkv, ldqkv, H, G, dim, vdim, rot_dims, interleaved ? 1 : 0, t_max, q_norm, k_norm, freq, eps, q_scale, row_seq, row_slot,
                 q_out, ldq, k_arena, ldk, v_arena, ldv};
  hipLaunchKernelGGL(proj_norm_rope_append_kernel, dim3((unsigned)M), dim3(256), 0, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_proj_norm_rope_append");
  return MN_OK;
}

extern "C" int mn_latent_rope_append(const float* qd, int64_t ld, int M, int H, int dim, int rot, int rank, const uint16_t* c_norm, float eps,
                                     int rot_dims, int interleaved, const float* freq, float q_scale, const int32_t* row_seq,
                                     const int32_t* row_slot, float* q_out, int64_t ldq, float* arena, int64_t lda, int t_max, void* stream) {
  MN_CHECK_ARG(qd && c_norm && row_seq && row_slot && q_out && arena && M >= 1 && H >= 1 && dim >= 0 && rot >= 0 && rank >= 1 && t_max >= 1 &&
                   rot_dims >= 0 && rot_dims <= rot && (rot_dims % 2) == 0 && (rot_dims == 0 || freq) && lda >= (int64_t)rank + rot,
               "mn_latent_rope_append: bad args (rot_dims=%d of rot=%d)", rot_dims, rot);
  LatentRopeArgs a{qd, ld, H, dim, rot, rank, rot_dims, interleaved ? 1 : 0, t_max, c_norm, freq, eps, q_scale, row_seq, row_slot, q_out, ldq,
                   arena, lda};
  hipLaunchKernelGGL(latent_rope_append_kernel, dim3((unsigned)M), dim3(256), 0, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_latent_rope_append");
  return MN_OK;
}

extern "C" int mn_head_sigmoid_gate_rows(float* x, int64_t ldx, const float* g, int64_t ldg, uint16_t* x16, int64_t ldx16, int M, int H,
                                         int vdim, void* stream) {
  MN_CHECK_ARG(x && g && M >= 1 && M <= 65535 && H >= 1 && vdim >= 1, "mn_head_sigmoid_gate_rows: bad args");
  hipLaunchKernelGGL(head_sigmoid_gate_kernel, dim3((unsigned)mn_cdiv((int64_t)H * vdim, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x,
                     ldx, g, ldg, x16, ldx16, H, vdim);
  MN_CHECK_LAUNCH("mn_head_sigmoid_gate_rows");
  return MN_OK;
}

extern "C" int mn_delta_prep_rows(const float* proj, int64_t ld, int M, int H, int G, int dim, int vdim, int off_b, int off_a,
                                  const uint16_t* w_conv, int taps, float* state, int advance_state, const float* a_log,
                                  const float* dt_bias, float unit_eps, float q_scale, const int32_t* row_seq, const int32_t* row_slot,
                                  const int32_t* row_back, float* qkv, int64_t ldo, float* bd, int64_t ldbd, void* stream) {
  MN_CHECK_ARG(proj && w_conv && a_log && dt_bias && row_seq && row_slot && row_back && qkv && bd && M >= 1 && H >= 1 && G >= 1 && (H % G) == 0 &&
                   dim >= 1 && vdim >= 1 && taps >= 1 && (taps == 1 || state) && ldbd >= 2 * (int64_t)H,
               "mn_delta_prep_rows: bad args");
  DeltaPrepArgs a{proj, ld, H, G, dim, vdim, taps, off_b, off_a, w_conv, state, advance_state ? 1 : 0, a_log, dt_bias, unit_eps, q_scale, row_seq, row_slot, row_back,
                  qkv, ldo, bd, ldbd};
  const int64_t units = 2 * (int64_t)G + mn_cdiv((int64_t)H * vdim, 256);
  MN_CHECK_ARG(M <= 65535 * 32 && mn_cdiv(units, 4) <= 65535, "mn_delta_prep_rows: too many rows or channels");
  hipLaunchKernelGGL(delta_prep_kernel, dim3((unsigned)M, (unsigned)mn_cdiv(units, 4)), dim3(256), 0, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_delta_prep_rows");
  return MN_OK;
}

extern "C" int mn_gated_delta_rows(const float* qkv, int64_t ld, const float* bd, int64_t ldbd, int M, int H, int G, int dim, int vdim,
                                   float* state, const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, int flags,
                                   float* out, int64_t ldo, void* stream) {
  const bool distinct = (flags & MN_SEQ_ROWS_DISTINCT) != 0;
  MN_CHECK_ARG(qkv && bd && state && row_seq && row_slot && (row_back || distinct) && out && M >= 1 && M <= 65535 && H >= 1 && H <= 65535 &&
                   G >= 1 && (H % G) == 0 && dim >= 1 && dim <= 512 && vdim >= 1 && mn_cdiv(vdim, 32) <= 65535,
               "mn_gated_delta_rows: bad args (dim=%d: at most 512)", dim);
  DeltaArgs a{qkv, ld, bd, ldbd, H, G, dim, vdim, state, row_seq, row_slot, row_back, out, ldo, M};
  hipStream_t st = mn_stream(stream);
  const dim3 grid((unsigned)M, (unsigned)H, (unsigned)mn_cdiv(vdim, 32));
  if (distinct) {
    hipLaunchKernelGGL(delta_step_kernel, grid, dim3(256), ((size_t)2 * dim + 768) * sizeof(float), st, a);
    MN_CHECK_LAUNCH("mn_gated_delta_rows(step)");
    return MN_OK;
  }
  if (dim <= 256) {
    MN_CHECK_ARG(M <= 65535 && (int64_t)H * mn_cdiv(vdim, 16) < ((int64_t)1 << 31), "mn_gated_delta_rows: too many rows or columns");
#define MN_DF(NS_, LPC_, DB_)                                                                                                                 \
  hipLaunchKernelGGL((delta_rows_fast_kernel<NS_, LPC_, DB_>), dim3((unsigned)(H * mn_cdiv(vdim, 256 / LPC_)), (unsigned)M), dim3(256),  \
                     ((size_t)DB_ * 2 * NS_ * LPC_ + 2 * DB_ * (256 / LPC_) + 3 * DB_) * sizeof(float), st, a)
    if (dim <= 32) MN_DF(4, 8, 32); else if (dim <= 64) MN_DF(4, 16, 32); else if (dim <= 128) MN_DF(8, 16, 32); else MN_DF(16, 16, 16);
#undef MN_DF
  } else {
    const size_t lds = ((size_t)DB * 2 * dim + DB * 32 + 3 * DB) * sizeof(float);    // 16 rows of q and k: 64 KiB at dim 512
    if (lds > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&delta_rows_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      MN_CHECK_ARG(e == hipSuccess, "mn_gated_delta_rows: %zu bytes of LDS refused (dim=%d)", lds, dim);
    }
    hipLaunchKernelGGL((delta_rows_kernel<0>), grid, dim3(256), lds, st, a);
  }
  MN_CHECK_LAUNCH("mn_gated_delta_rows");
  return MN_OK;
}

extern "C" int mn_head_rms_silu_gate_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, const float* g, int64_t ldg, float* y,
                                          int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int H, int vdim, void* stream) {
  MN_CHECK_ARG(x && w && g && (y || y16) && M >= 1 && M <= 65535 && H >= 1 && vdim >= 1, "mn_head_rms_silu_gate_rows: bad args");
  hipLaunchKernelGGL(head_rms_silu_gate_kernel, dim3((unsigned)mn_cdiv(H, 4), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, w, eps, g,
                     ldg, y, ldy, y16, ldy16, H, vdim);
  MN_CHECK_LAUNCH("mn_head_rms_silu_gate_rows");
  return MN_OK;
}
