// pmix_ops.hip — row operators of parallel-mixer sequence models (mingnative.h section 10): a windowed softmax attention with
// pooled far blocks beside a minGRU recurrence, RMS pre-norms, a mixture-of-experts feed-forward.  Everything works on fp32 rows
// [M, n] of a step (tokens of one or several cache sequences, each sequence's rows consecutive) and bf16 weights; every size and
// constant is an argument.
//
//   mn_axpy_rms_rows           x += mult * y;  n = x / sqrt(mean(x^2) + eps) * w
//   mn_axpy_rms_filter_rows    the same for decode rows, with the sublayer-input filter and its state update in the launch
//   mn_rope_unit_append        rotary (frequency table) + unit-RMS per head on q and k, q scaled, k / v appended to their arenas
//   mn_pool_blocks_update      mean key / value of the blocks a step completes
//   mn_filter_rope_append_rows decode rows: the q / k / v channel filter with its state, the rotation and append, the block means — one launch
//   mn_window_pool_attn        softmax over the window's tokens and the block means before it, online softmax in fp32
//   mn_window_pool_attn_blocks the same, tiled: runs of rows and query heads share key tiles, key splits with a merge launch
//   mn_mingru_rows             S = (1 - z) S + z c over each sequence's rows, gated output (mn_mingru_rows_scan: as a chunked scan)
//   mn_router_topk_rows        top-k of the router logits, softmax over the chosen
//   mn_silu_mul_rows           silu(gate) * up
//   mn_gemv_f32_indexed        one row against the weight block an index names (experts of few rows, and the fp32 path)
//   mn_moe_combine_residual    x += mult * (sum_j w_j y_j + sigmoid(sg) shared)
#include <math.h>

#include "common.h"
#include "mfma_f32_tiles.h"

extern "C" int mn_rotary_frequencies_host(int dims, double base, double factor, double original, double fast, double slow, float* freq,
                                          float* mag) {
  MN_CHECK_ARG(dims >= 2 && (dims % 2) == 0 && base > 1.0 && freq && mag, "mn_rotary_frequencies_host: bad args (dims=%d)", dims);
  const int half = dims / 2;
  const double two_pi = 6.283185307179586476925286766559;
  double lo = 0, hi = 0;
  if (factor > 0) {
    MN_CHECK_ARG(original > 0 && fast > 0 && slow > 0, "mn_rotary_frequencies_host: bad scaling");
    auto dim_of = [&](double turns) { return dims * log(original / (two_pi * turns)) / (2.0 * log(base)); };
    lo = floor(dim_of(fast)); if (lo < 0) lo = 0;
    hi = ceil(dim_of(slow)); if (hi > dims - 1) hi = dims - 1;
  }
  for (int i = 0; i < half; ++i) {
    const double f = pow(base, -2.0 * i / dims);
    double v = f;
    if (factor > 0) {
      double den = hi - lo; if (den < 0.001) den = 0.001;
      double ramp = (i - lo) / den; if (ramp < 0) ramp = 0; if (ramp > 1) ramp = 1;
      v = f / factor * ramp + f * (1.0 - ramp);
    }
    freq[i] = (float)v;
  }
  *mag = factor > 0 ? (float)(0.1 * log(factor) + 1.0) : 1.0f;
  return MN_OK;
}

namespace {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------------------------------------------------------
// one wave per row: x += mult * y, then RMS norm with a weight
__global__ __launch_bounds__(256) void axpy_rms_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y, int64_t ldy,
                                                       float mult, const bf16_t* __restrict__ w, float eps, float* __restrict__ nout,
                                                       int64_t ldn, bf16_t* __restrict__ n16, int64_t ldn16, int M, int n) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  float* xr = x + (int64_t)row * ldx;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) {
    float v = xr[i];
    if (y) { v += mult * y[(int64_t)row * ldy + i]; xr[i] = v; }
    s += v * v;
  }
  if (!nout && !n16) return;
  const float r = 1.0f / sqrtf(wave_sum(s) / (float)n + eps);
  for (int i = lane; i < n; i += 64) {
    const float o = xr[i] * r * bf16_to_f32(w[i]);
    if (nout) nout[(int64_t)row * ldn + i] = o;
    if (n16) n16[(int64_t)row * ldn16 + i] = f32_to_bf16(o);
  }
}

// Decode rows, one workgroup per row, the row in registers: x += mult * y; n = RMS(x) w; h = n + filter(n, state); state moves on.
constexpr int FUSED_MAX_TAPS = 8;
struct AxpyRmsFilterArgs {
  float* x; int64_t ldx;
  const float* y; int64_t ldy; float mult;
  const bf16_t* w; float eps;
  const bf16_t* taps_w; int taps;
  float* state; const int32_t* row_seq; const int32_t* row_slot;
  float* h; int64_t ldh;
  int n;
};

// MT: the most taps this instance holds in registers (4 or 8)
template <int VPT, int MT>
__global__ __launch_bounds__(256) void axpy_rms_filter_kernel(AxpyRmsFilterArgs a) {
  __shared__ float red[8];
  const int row = blockIdx.x, tid = threadIdx.x, n = a.n;
  const bool filter = a.taps_w != nullptr && a.taps >= 1;
  const int seq = filter ? a.row_seq[row] : 0, slot = filter ? a.row_slot[row] : 0;
  float* const st0 = (filter && a.taps > 1) ? a.state + (int64_t)seq * (a.taps - 1) * n : nullptr;
  float xv[VPT], sv[VPT][MT - 1], wv[VPT], tv[VPT][MT];
  const float* sbase = st0 ? st0 : a.x + (int64_t)row * a.ldx;         // without a state: any readable row, stride 0
  const int64_t sstr = st0 ? n : 0;
  const int ns = st0 ? a.taps - 1 : 1;                                  // state entries
  const bf16_t* tbase = filter ? a.taps_w : a.w;                        // without a filter: the norm weight, stride 0
  const int tstr = filter ? a.taps : 0, nt = filter ? a.taps : 1;
  // every load of the row — inputs, state, norm weight, filter taps — is issued before the reduction, and before the first store
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + 256 * i, cc = c < n ? c : 0;
    float t = a.x[(int64_t)row * a.ldx + cc];
    if (a.y) t += a.mult * a.y[(int64_t)row * a.ldy + cc];
    xv[i] = c < n ? t : 0.f;
    wv[i] = bf16_to_f32(a.w[cc]);
    // unconditional loads at clamped (always valid) addresses, the unused ones zeroed afterwards: a load under a branch would wait
    // for its value before the next branch, one round trip per tap
#pragma unroll
    for (int k = 1; k < MT; ++k) {
      const float v = sbase[(int64_t)(min(k, ns) - 1) * sstr + cc];
      sv[i][k - 1] = (st0 && k < a.taps) ? v : 0.f;
    }
#pragma unroll
    for (int k = 0; k < MT; ++k) {
      const float v = bf16_to_f32(tbase[(int64_t)cc * tstr + max(nt - 1 - k, 0)]);
      tv[i][k] = (filter && k < a.taps) ? v : 0.f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) s += xv[i] * xv[i];
  const float r = 1.0f / sqrtf(block_sum(s, red) / (float)n + a.eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + 256 * i;
    if (c >= n) continue;
    if (a.y) a.x[(int64_t)row * a.ldx + c] = xv[i];
    const float nv = xv[i] * r * wv[i];
    float acc = nv;
    if (filter) {
      acc += tv[i][0] * nv;                              // tv[k]: the tap on the input k positions back
#pragma unroll
      for (int k = 1; k < MT; ++k)
        if (k < a.taps && slot - k >= 0) acc += tv[i][k] * sv[i][k - 1];
      if (st0) {
        float* st = st0 + c;
#pragma unroll
        for (int k = MT - 2; k >= 1; --k)
          if (k < a.taps - 1) st[(int64_t)k * n] = sv[i][k - 1];
        st[0] = nv;
      }
    }
    a.h[(int64_t)row * a.ldh + c] = acc;
  }
}

// The same with 16-byte accesses: a thread owns NV groups of four consecutive channels (rows of n % 4 == 0 values at 16-byte aligned
// addresses, at most 4 taps): a row of 2 048 values is 16 loads per thread instead of 80.
template <int NV>
__global__ __launch_bounds__(256) void axpy_rms_filter_vec_kernel(AxpyRmsFilterArgs a) {
  __shared__ float red[8];
  constexpr int MT = 4;
  const int row = blockIdx.x, tid = threadIdx.x, n = a.n, ng = n / 4;
  const bool filter = a.taps_w != nullptr && a.taps >= 1;
  const int seq = filter ? a.row_seq[row] : 0, slot = filter ? a.row_slot[row] : 0;
  float* const st0 = (filter && a.taps > 1) ? a.state + (int64_t)seq * (a.taps - 1) * n : nullptr;
  const float* sbase = st0 ? st0 : a.x + (int64_t)row * a.ldx;
  const int64_t sstr = st0 ? n : 0;
  const int ns = st0 ? a.taps - 1 : 1;
  float4 xv[NV], sv[NV][MT - 1];
  float wv[NV][4], tv[NV][4][MT];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int gi = tid + 256 * i, gg = gi < ng ? gi : 0, c0 = 4 * gg;
    float4 t = *reinterpret_cast<const float4*>(a.x + (int64_t)row * a.ldx + c0);
    if (a.y) {
      const float4 yv = *reinterpret_cast<const float4*>(a.y + (int64_t)row * a.ldy + c0);
      t.x += a.mult * yv.x; t.y += a.mult * yv.y; t.z += a.mult * yv.z; t.w += a.mult * yv.w;
    }
    xv[i] = gi < ng ? t : make_float4(0.f, 0.f, 0.f, 0.f);
    const uint2 wq = *reinterpret_cast<const uint2*>(a.w + c0);
    wv[i][0] = bf16lo_to_f32(wq.x); wv[i][1] = bf16hi_to_f32(wq.x); wv[i][2] = bf16lo_to_f32(wq.y); wv[i][3] = bf16hi_to_f32(wq.y);
#pragma unroll
    for (int k = 1; k < MT; ++k) {
      const float4 v = *reinterpret_cast<const float4*>(sbase + (int64_t)(min(k, ns) - 1) * sstr + c0);
      sv[i][k - 1] = (st0 && k < a.taps) ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (filter && a.taps == 4 && (((uintptr_t)a.taps_w) & 15) == 0) {      // four channels x four taps: 32 contiguous bytes
      const uint4* tp = reinterpret_cast<const uint4*>(a.taps_w + (int64_t)c0 * 4);
      const uint4 ta = tp[0], tb = tp[1];
      const uint32_t wd[8] = {ta.x, ta.y, ta.z, ta.w, tb.x, tb.y, tb.z, tb.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {                        // tv[.][k]: the tap on the input k positions back = weight 3 - k
        tv[i][e][3] = bf16lo_to_f32(wd[2 * e]); tv[i][e][2] = bf16hi_to_f32(wd[2 * e]);
        tv[i][e][1] = bf16lo_to_f32(wd[2 * e + 1]); tv[i][e][0] = bf16hi_to_f32(wd[2 * e + 1]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int k = 0; k < MT; ++k) {
          const float v = filter ? bf16_to_f32(a.taps_w[(int64_t)(c0 + e) * a.taps + max(a.taps - 1 - k, 0)]) : 0.f;
          tv[i][e][k] = k < a.taps ? v : 0.f;
        }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) s += xv[i].x * xv[i].x + xv[i].y * xv[i].y + xv[i].z * xv[i].z + xv[i].w * xv[i].w;
  const float r = 1.0f / sqrtf(block_sum(s, red) / (float)n + a.eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int gi = tid + 256 * i, c0 = 4 * gi;
    if (gi >= ng) continue;
    if (a.y) *reinterpret_cast<float4*>(a.x + (int64_t)row * a.ldx + c0) = xv[i];
    const float xe[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
    float nv[4], hv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      nv[e] = xe[e] * r * wv[i][e];
      hv[e] = nv[e];
      if (filter) {
        hv[e] += tv[i][e][0] * nv[e];
#pragma unroll
        for (int k = 1; k < MT; ++k) {
          const float4 q = sv[i][k - 1];
          const float se = e == 0 ? q.x : (e == 1 ? q.y : (e == 2 ? q.z : q.w));
          if (k < a.taps && slot - k >= 0) hv[e] += tv[i][e][k] * se;
        }
      }
    }
    if (st0) {
#pragma unroll
      for (int k = MT - 2; k >= 1; --k)
        if (k < a.taps - 1) *reinterpret_cast<float4*>(st0 + (int64_t)k * n + c0) = sv[i][k - 1];
      *reinterpret_cast<float4*>(st0 + c0) = make_float4(nv[0], nv[1], nv[2], nv[3]);
    }
    *reinterpret_cast<float4*>(a.h + (int64_t)row * a.ldh + c0) = make_float4(hv[0], hv[1], hv[2], hv[3]);
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// One wave per (row, head vector): q heads 0 .. H - 1, k heads H .. H + G - 1, v heads after them.  A lane holds the pairs
// (i, i + half) for i = lane, lane + 64, ... and the values past rot_dims: at most 8 of each (dim <= 512).
struct RopeArgs {
  const float* qkv; int64_t ldqkv;
  int H, G, dim, vdim, rot_dims;
  const float* freq; float mag; int unit; float eps, q_scale;
  const int32_t* row_seq; const int32_t* row_slot;
  float* q_out; int64_t ldq;
  float* k_arena; float* v_arena; int t_max;
  // decode rows only (ROW): the channel filter in front with its state, and the block means behind
  const bf16_t* w_conv; int conv; float* conv_state;
  float* pk; float* pv; int n_pool_max, pool;
  // ... and the minGRU of the same rows, in extra workgroups of the launch (gru_n 0: none)
  const float* zx; int64_t ldzx; const float* gg; int64_t ldgg; float* gru_state; int gru_n; float gru_scale; float* gru_out; int64_t ldgo;
};

// ROW: every row is alone in its sequence (a decode step).  The kernel then reads its channels through the short causal filter
// (taps from w_conv, the sequence's earlier inputs from conv_state, which it moves on) and, when the row completes a block of
// `pool` slots, writes the block's mean key / value too: mn_tap_conv_rows + mn_tap_state_update + the rotation + mn_pool_blocks_update
// of such a row in one launch.  Every channel is read by exactly one lane.
template <bool ROW>
__global__ __launch_bounds__(256) void rope_unit_append_kernel(RopeArgs a, int M) {
  const int hv = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, m = blockIdx.y;
  const int nh = a.H + 2 * a.G;
  if (ROW && a.gru_n > 0 && (int)blockIdx.x >= (nh + 3) / 4) {      // the recurrence of this row: one thread per channel
    const int c = ((int)blockIdx.x - (nh + 3) / 4) * 256 + threadIdx.x;
    if (c >= a.gru_n) return;
    float* sp = a.gru_state + (int64_t)a.row_seq[m] * a.gru_n + c;
    const float S0 = a.row_slot[m] == 0 ? 0.f : *sp;
    const float z = sigmoid_f(a.zx[(int64_t)m * a.ldzx + c]);
    const float u = a.zx[(int64_t)m * a.ldzx + a.gru_n + c];
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    const float S = (1.0f - z) * S0 + z * cand;
    a.gru_out[(int64_t)m * a.ldgo + c] = a.gru_scale * S * silu_f(a.gg[(int64_t)m * a.ldgg + c]);
    *sp = S;
    return;
  }
  if (hv >= nh) return;
  const float* row = a.qkv + (int64_t)m * a.ldqkv;
  const int seq = a.row_seq[m], slot = a.row_slot[m];
  const int64_t crow = (int64_t)seq * a.t_max + slot;
  const int C = (a.H + a.G) * a.dim + a.G * a.vdim;
  const bool do_pool = ROW && a.pool > 0 && (slot % a.pool) == a.pool - 1 && slot / a.pool < a.n_pool_max;
  auto ld = [&](int ch) -> float {
    const float cur = row[ch];
    if (!ROW || a.conv < 1) return cur;
    const bf16_t* w = a.w_conv + (int64_t)ch * a.conv;
    float acc = bf16_to_f32(w[a.conv - 1]) * cur;
    if (a.conv > 1) {
      float* st = a.conv_state + (int64_t)seq * (a.conv - 1) * C + ch;
      for (int k = 1; k < a.conv; ++k)
        if (slot - k >= 0) acc += bf16_to_f32(w[a.conv - 1 - k]) * st[(int64_t)(k - 1) * C];
      for (int k = a.conv - 2; k >= 1; --k) st[(int64_t)k * C] = st[(int64_t)(k - 1) * C];
      st[0] = cur;
    }
    return acc;
  };
  auto put = [&](float* arena, float* parena, int n_ch, int c, float val) {      // append, and the block's mean when this row completes it
    arena[crow * n_ch + c] = val;
    if (do_pool) {
      const int b = slot / a.pool;
      const float* src = arena + ((int64_t)seq * a.t_max + (int64_t)b * a.pool) * n_ch + c;
      float s = 0.f;
      for (int j = 0; j < a.pool - 1; ++j) s += src[(int64_t)j * n_ch];
      s += val;
      parena[((int64_t)seq * a.n_pool_max + b) * n_ch + c] = s / (float)a.pool;
    }
  };
  if (hv >= a.H + a.G) {                                         // a value head: into its arena
    const int g = hv - a.H - a.G;
    for (int i = lane; i < a.vdim; i += 64) put(a.v_arena, a.pv, a.G * a.vdim, g * a.vdim + i, ld((a.H + a.G) * a.dim + g * a.vdim + i));
    return;
  }
  const bool is_q = hv < a.H;
  const int ch0 = hv * a.dim;
  float* qdst = a.q_out + (int64_t)m * a.ldq + (int64_t)hv * a.dim;
  const int kc0 = (hv - a.H) * a.dim;
  const int half = a.rot_dims / 2;
  const float pos = (float)slot;
  float lo[4], hi[4], rest[8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    lo[j] = hi[j] = 0.f;
    if (i < half) {
      const float u = ld(ch0 + i), v = ld(ch0 + i + half);
      const float ang = pos * a.freq[i];
      const float c = cosf(ang) * a.mag, s = sinf(ang) * a.mag;
      lo[j] = u * c - v * s;
      hi[j] = v * c + u * s;
      ss += lo[j] * lo[j] + hi[j] * hi[j];
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = a.rot_dims + lane + 64 * j;
    rest[j] = 0.f;
    if (i < a.dim) { rest[j] = ld(ch0 + i); ss += rest[j] * rest[j]; }
  }
  float r = 1.0f;
  if (a.unit) r = 1.0f / sqrtf(wave_sum(ss) / (float)a.dim + a.eps);
  if (is_q) r *= a.q_scale;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    if (i < half) {
      if (is_q) { qdst[i] = lo[j] * r; qdst[i + half] = hi[j] * r; }
      else { put(a.k_arena, a.pk, a.G * a.dim, kc0 + i, lo[j] * r); put(a.k_arena, a.pk, a.G * a.dim, kc0 + i + half, hi[j] * r); }
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = a.rot_dims + lane + 64 * j;
    if (i < a.dim) {
      if (is_q) qdst[i] = rest[j] * r;
      else put(a.k_arena, a.pk, a.G * a.dim, kc0 + i, rest[j] * r);
    }
  }
}

// grid (ceil((Gd + Gv) / 256), M): a row that completes a block writes the block's means (slots summed in ascending order)
__global__ __launch_bounds__(256) void pool_blocks_kernel(const float* __restrict__ k_arena, const float* __restrict__ v_arena, int t_max,
                                                          float* __restrict__ pk, float* __restrict__ pv, int n_pool_max, int pool, int Gd,
                                                          int Gv, const int32_t* __restrict__ row_seq, const int32_t* __restrict__ row_slot) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const int slot = row_slot[m];
  if ((slot % pool) != pool - 1 || c >= Gd + Gv) return;
  const int b = slot / pool, seq = row_seq[m];
  if (b >= n_pool_max) return;
  const bool is_k = c < Gd;
  const int cc = is_k ? c : c - Gd, n = is_k ? Gd : Gv;
  const float* src = (is_k ? k_arena : v_arena) + ((int64_t)seq * t_max + (int64_t)b * pool) * n + cc;
  float s = 0.f;
  for (int j = 0; j < pool; ++j) s += src[(int64_t)j * n];
  (is_k ? pk : pv)[((int64_t)seq * n_pool_max + b) * n + cc] = s / (float)pool;
}

// ---------------------------------------------------------------------------------------------------------------------------
// Attention, plain form: one workgroup per (row, key/value head, chunk of <= 8 query heads of its group).  Keys are walked in
// tiles of 256 (block means first, then the window's tokens): a thread scores one key for the chunk's heads, the tile's softmax
// statistics are merged into the running ones, then the threads turn to output columns and add the tile's weighted values.
constexpr int ATT_R = 8, ATT_TILE = 256, ATT_NOUT = 8;
struct AttnArgs {
  const float* q; int64_t ldq;
  const float *k, *v, *pk, *pv;
  const int32_t* row_seq; const int32_t* row_slot;
  int H, G, dim, vdim, t_max, n_pool_max, window, pool;
  float out_scale;
  float* out; int64_t ldo; bf16_t* out16; int64_t ldo16;
};

__global__ __launch_bounds__(256) void window_pool_attn_kernel(AttnArgs a) {
  extern __shared__ float lds[];
  const int m = blockIdx.x, tid = threadIdx.x;
  const int rep = a.H / a.G, chunks = (rep + ATT_R - 1) / ATT_R;
  const int g = blockIdx.y / chunks, h0 = g * rep + (blockIdx.y % chunks) * ATT_R;
  const int R = min(ATT_R, g * rep + rep - h0);
  float* qs = lds;                              // [R][dim]
  float* sc = qs + ATT_R * a.dim;               // [R][ATT_TILE]
  float* stat = sc + ATT_R * ATT_TILE;          // [R] running max, [R] running sum, [R] rescale of this tile
  const int seq = a.row_seq[m], pos = a.row_slot[m];
  int t0 = 0, nb = 0;
  if (a.window > 0) {
    t0 = max(0, pos - a.window + 1);
    if (a.pool > 0 && pos - a.window + 1 >= 0) nb = (pos - a.window + 1) / a.pool;
  }
  const int nk = nb + (pos - t0 + 1);
  for (int e = tid; e < R * a.dim; e += 256) qs[e] = a.q[(int64_t)m * a.ldq + (int64_t)h0 * a.dim + e];
  if (tid < ATT_R) { stat[tid] = -INFINITY; stat[ATT_R + tid] = 0.f; }
  const int Gd = a.G * a.dim, Gv = a.G * a.vdim;
  const float* kb = a.k + ((int64_t)seq * a.t_max + t0) * Gd + (int64_t)g * a.dim;
  const float* vb = a.v + ((int64_t)seq * a.t_max + t0) * Gv + (int64_t)g * a.vdim;
  const float* pkb = a.pk ? a.pk + (int64_t)seq * a.n_pool_max * Gd + (int64_t)g * a.dim : nullptr;
  const float* pvb = a.pv ? a.pv + (int64_t)seq * a.n_pool_max * Gv + (int64_t)g * a.vdim : nullptr;
  const int n_out = R * a.vdim;
  float acc[ATT_NOUT];
#pragma unroll
  for (int o = 0; o < ATT_NOUT; ++o) acc[o] = 0.f;
  __syncthreads();
  for (int j0 = 0; j0 < nk; j0 += ATT_TILE) {
    const int nt = min(ATT_TILE, nk - j0);
    // scores of this thread's key
    if (tid < nt) {
      const int j = j0 + tid;
      const float* kp = j < nb ? pkb + (int64_t)j * Gd : kb + (int64_t)(j - nb) * Gd;
      float s[ATT_R];
#pragma unroll
      for (int r = 0; r < ATT_R; ++r) s[r] = 0.f;
      for (int d = 0; d < a.dim; ++d) {
        const float kv = kp[d];
#pragma unroll
        for (int r = 0; r < ATT_R; ++r)
          if (r < R) s[r] = fmaf(qs[r * a.dim + d], kv, s[r]);
      }
#pragma unroll
      for (int r = 0; r < ATT_R; ++r)
        if (r < R) sc[r * ATT_TILE + tid] = s[r];
    }
    __syncthreads();
    // statistics: wave w owns heads w, w + 4
    for (int r = tid >> 6; r < R; r += 4) {
      const int lane = tid & 63;
      float mx = -INFINITY;
      for (int i = lane; i < nt; i += 64) mx = fmaxf(mx, sc[r * ATT_TILE + i]);
      mx = wave_max(mx);
      const float m_old = stat[r], m_new = fmaxf(m_old, mx);
      float sum = 0.f;
      for (int i = lane; i < nt; i += 64) {
        const float p = expf(sc[r * ATT_TILE + i] - m_new);
        sc[r * ATT_TILE + i] = p;
        sum += p;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float alpha = expf(m_old - m_new);          // first tile: exp(-inf) = 0
        stat[r] = m_new;
        stat[ATT_R + r] = stat[ATT_R + r] * alpha + sum;
        stat[2 * ATT_R + r] = alpha;
      }
    }
    __syncthreads();
    // weighted values: thread -> output columns o = tid + 256 i of [R][vdim]
#pragma unroll
    for (int o = 0; o < ATT_NOUT; ++o) {
      const int e = tid + 256 * o;
      if (e >= n_out) break;
      const int r = e / a.vdim, c = e - r * a.vdim;
      float t = acc[o] * stat[2 * ATT_R + r];
      const float* pr = sc + r * ATT_TILE;
      for (int i = 0; i < nt; ++i) {
        const int j = j0 + i;
        const float* vp = j < nb ? pvb + (int64_t)j * Gv : vb + (int64_t)(j - nb) * Gv;
        t = fmaf(pr[i], vp[c], t);
      }
      acc[o] = t;
    }
    __syncthreads();
  }
#pragma unroll
  for (int o = 0; o < ATT_NOUT; ++o) {
    const int e = tid + 256 * o;
    if (e >= n_out) break;
    const int r = e / a.vdim;
    const float val = acc[o] / stat[ATT_R + r] * a.out_scale;
    const int64_t col = (int64_t)h0 * a.vdim + e;
    if (a.out) a.out[(int64_t)m * a.ldo + col] = val;
    if (a.out16) a.out16[(int64_t)m * a.ldo16 + col] = f32_to_bf16(val);
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Attention, tiled form: one workgroup per (run of <= RB consecutive rows of one sequence, key/value head, chunk of query heads,
// key split) holds AQ query vectors (rows x heads) in LDS and walks its share of the run's keys in tiles of 64 (block means first,
// then the tokens from the first row's window start to the last row's position; what a row may not see is masked per (row, key)).
// Scores: four threads per key, each a quarter of the head's values, all AQ vectors against the key in registers.  The tile's
// softmax statistics are merged into the running ones by one wave per vector.  Values: a thread owns one output column (and a
// share of the tile's keys when the head has fewer than 256 columns) for all AQ vectors.  With key splits the unnormalised sums
// and statistics go to a workspace and a second launch merges them.
constexpr int AKT = 64;
struct AttnTArgs {
  const float* q; int64_t ldq;
  const float *k, *v, *pk, *pv;
  const int32_t *row_seq, *row_slot, *blk_tab;
  int H, G, dim, vdim, t_max, n_pool_max, window, pool, rows_per_blk, hpc, nsplit;
  float out_scale;
  float* out; int64_t ldo; bf16_t* out16; int64_t ldo16;
  float* part;
  const float* sink;    // optional fp32 [H]: exp(sink[h]) joins the softmax's denominator of head h (no key, no value)
  float cap;            // > 0: every score s becomes cap * tanh(s / cap) before the softmax
  int64_t ldk, ldv;     // row strides of the key and value arenas (>= G * dim, G * vdim): a value arena may be a view into the key arena
};

__device__ __forceinline__ float soft_cap(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// 1 / (the softmax's normaliser) of a vector with running maximum m and sum l (of exp(score - m)), the head's sink included:
// numerator and denominator are both taken relative to max(m, sink)
__device__ __forceinline__ float softmax_inv(float m, float l, const float* sink, int h) {
  if (!sink) return 1.0f / l;
  const float sk = sink[h], mm = fmaxf(m, sk);
  const float f = expf(m - mm);
  return f / (l * f + expf(sk - mm));
}

__device__ __forceinline__ int win_t0(int pos, int window) { return window > 0 ? max(0, pos - window + 1) : 0; }
__device__ __forceinline__ int win_nb(int pos, int window, int pool) {
  return (window > 0 && pool > 0 && pos - window + 1 >= 0) ? (pos - window + 1) / pool : 0;
}

template <int AQ, bool VEC>
__global__ __launch_bounds__(256) void window_attn_tiled_kernel(AttnTArgs a) {
  extern __shared__ float lds[];
  const int tid = threadIdx.x, b = blockIdx.x, gy = blockIdx.y, sp = blockIdx.z;
  const int rep = a.H / a.G, chunks = (rep + a.hpc - 1) / a.hpc;
  const int g = gy / chunks, h0 = g * rep + (gy % chunks) * a.hpc;
  const int Rc = min(a.hpc, g * rep + rep - h0);
  const int r0 = a.blk_tab ? a.blk_tab[2 * b] : b;
  const int nr = a.blk_tab ? min(a.blk_tab[2 * b + 1], a.rows_per_blk) : 1;
  const int nqv = nr * Rc;
  const int seq = a.row_seq[r0], pos0 = a.row_slot[r0], posL = pos0 + nr - 1;
  const int nbL = win_nb(posL, a.window, a.pool), tF = win_t0(pos0, a.window);
  const int nk = nbL + (posL - tF + 1);
  const int ntile = (nk + AKT - 1) / AKT, tps = (ntile + a.nsplit - 1) / a.nsplit;
  const int tile0 = sp * tps, tile1 = min(ntile, tile0 + tps);
  float* qs = lds;                          // [AQ][dim]
  float* sc = qs + AQ * a.dim;              // [AQ][AKT]
  float* pT = sc + AQ * AKT;                // [AKT][AQ]
  float* st_m = pT + AKT * AQ;              // [AQ] running max, [AQ] running sum, [AQ] rescale of this tile
  float* st_l = st_m + AQ;
  float* st_a = st_l + AQ;
  float* red = st_a + AQ;                   // [256 / cw][AQ][cw]
  for (int e = tid; e < AQ * a.dim; e += 256) {
    const int qv = e / a.dim, d = e - qv * a.dim;
    qs[e] = qv < nqv ? a.q[(int64_t)(r0 + qv / Rc) * a.ldq + (int64_t)(h0 + qv % Rc) * a.dim + d] : 0.f;
  }
  if (tid < AQ) { st_m[tid] = -INFINITY; st_l[tid] = 0.f; st_a[tid] = 0.f; }
  const int Gd = a.G * a.dim, Gv = a.G * a.vdim;
  const float* kb = a.k + ((int64_t)seq * a.t_max + tF) * a.ldk + (int64_t)g * a.dim;
  const float* vb = a.v + ((int64_t)seq * a.t_max + tF) * a.ldv + (int64_t)g * a.vdim;
  const float* pkb = a.pk ? a.pk + (int64_t)seq * a.n_pool_max * Gd + (int64_t)g * a.dim : nullptr;
  const float* pvb = a.pv ? a.pv + (int64_t)seq * a.n_pool_max * Gv + (int64_t)g * a.vdim : nullptr;
  constexpr int NCB = 2;                    // column blocks of 256: vdim <= 512
  constexpr int PRE = AQ == 4 ? 8 : 2;      // loads in flight per thread: deep for the few vectors of decode rows, where latency is all there is
  float acc[NCB][AQ];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
    for (int i = 0; i < AQ; ++i) acc[cb][i] = 0.f;
  __syncthreads();
  for (int tile = tile0; tile < tile1; ++tile) {
    const int j0 = tile * AKT, nt = min(AKT, nk - j0);
    {  // ---- scores ----
      const int key = tid >> 2, part = tid & 3, j = j0 + key;
      const bool valid = key < nt;
      const float* kp = !valid ? kb : (j < nbL ? pkb + (int64_t)j * Gd : kb + (int64_t)(j - nbL) * a.ldk);
      float s[AQ];
#pragma unroll
      for (int i = 0; i < AQ; ++i) s[i] = 0.f;
      if (valid) {
        if (VEC) {
          const int nf = a.dim / 4;
          for (int f0 = part; f0 < nf; f0 += 4 * PRE) {   // PRE 16-byte pieces of the key in flight before the first product
            float4 kv[PRE];
#pragma unroll
            for (int u = 0; u < PRE; ++u) {
              const int f = f0 + 4 * u;
              kv[u] = f < nf ? *reinterpret_cast<const float4*>(kp + 4 * f) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < PRE; ++u) {
              const int f = f0 + 4 * u;
              if (f >= nf) break;
#pragma unroll
              for (int i = 0; i < AQ; ++i) {
                const float4 qq = *reinterpret_cast<const float4*>(qs + i * a.dim + 4 * f);
                s[i] = fmaf(qq.x, kv[u].x, s[i]); s[i] = fmaf(qq.y, kv[u].y, s[i]); s[i] = fmaf(qq.z, kv[u].z, s[i]); s[i] = fmaf(qq.w, kv[u].w, s[i]);
              }
            }
          }
        } else {
          for (int d = part; d < a.dim; d += 4) {
            const float kv = kp[d];
#pragma unroll
            for (int i = 0; i < AQ; ++i) s[i] = fmaf(qs[i * a.dim + d], kv, s[i]);
          }
        }
      }
      const int t = tF + (j - nbL);          // the token a non-pooled key index stands for
#pragma unroll
      for (int i = 0; i < AQ; ++i) {
        float v = s[i];
        v += __shfl_xor(v, 1);
        v += __shfl_xor(v, 2);
        if ((i & 3) == part) {
          const int pos = pos0 + i / Rc;
          const bool see = valid && i < nqv && (j < nbL ? j < win_nb(pos, a.window, a.pool) : (t >= win_t0(pos, a.window) && t <= pos));
          sc[i * AKT + key] = see ? soft_cap(v, a.cap) : -INFINITY;
        }
      }
    }
    __syncthreads();
    // ---- statistics: wave w owns the vectors w, w + 4, ... ----
    for (int i = tid >> 6; i < AQ; i += 4) {
      const int lane = tid & 63;
      const float x = sc[i * AKT + lane];
      const float m_old = st_m[i], m_new = fmaxf(m_old, wave_max(x));
      const float p = m_new == -INFINITY ? 0.f : expf(x - m_new);
      const float sum = wave_sum(p);
      pT[lane * AQ + i] = p;
      if (lane == 0) {
        const float alpha = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
        st_m[i] = m_new;
        st_l[i] = st_l[i] * alpha + sum;
        st_a[i] = alpha;
      }
    }
    __syncthreads();
    // ---- weighted values ----
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      const int c0 = cb * 256;
      if (c0 >= a.vdim) break;
      const int cw = min(256, a.vdim - c0), nsub = 256 / cw, c = tid % cw, ksub = tid / cw;
      if (ksub < nsub) {
#pragma unroll
        for (int i = 0; i < AQ; ++i) acc[cb][i] *= st_a[i];
        for (int jj0 = ksub; jj0 < nt; jj0 += PRE * nsub) {  // PRE values of the column in flight before the first product
          float vv[PRE];
#pragma unroll
          for (int u = 0; u < PRE; ++u) {
            const int jj = jj0 + u * nsub, j = j0 + jj;
            vv[u] = jj < nt ? (j < nbL ? pvb + (int64_t)j * Gv : vb + (int64_t)(j - nbL) * a.ldv)[c0 + c] : 0.f;
          }
#pragma unroll
          for (int u = 0; u < PRE; ++u) {
            const int jj = jj0 + u * nsub;
            if (jj >= nt) break;
            const float* pr = pT + jj * AQ;
#pragma unroll
            for (int i = 0; i < AQ; i += 4) {
              const float4 pp = *reinterpret_cast<const float4*>(pr + i);
              acc[cb][i] = fmaf(pp.x, vv[u], acc[cb][i]); acc[cb][i + 1] = fmaf(pp.y, vv[u], acc[cb][i + 1]);
              acc[cb][i + 2] = fmaf(pp.z, vv[u], acc[cb][i + 2]); acc[cb][i + 3] = fmaf(pp.w, vv[u], acc[cb][i + 3]);
            }
          }
        }
      }
    }
    __syncthreads();
  }
  // ---- the key shares of a column meet in LDS; then the result, or this split's part of it ----
  float* part_out = a.nsplit > 1 ? a.part + (((int64_t)b * gridDim.y + gy) * a.nsplit + sp) * ((int64_t)AQ * (2 + a.vdim)) : nullptr;
  if (part_out && tid < AQ) { part_out[tid] = st_m[tid]; part_out[AQ + tid] = st_l[tid]; }
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c0 = cb * 256;
    if (c0 >= a.vdim) break;
    const int cw = min(256, a.vdim - c0), nsub = 256 / cw, c = tid % cw, ksub = tid / cw;
    if (ksub < nsub) {
#pragma unroll
      for (int i = 0; i < AQ; ++i) red[(ksub * AQ + i) * cw + c] = acc[cb][i];
    }
    __syncthreads();
    for (int e = tid; e < nqv * cw; e += 256) {
      const int i = e / cw, cc = e - i * cw;
      float t = 0.f;
      for (int u = 0; u < nsub; ++u) t += red[(u * AQ + i) * cw + cc];
      if (part_out) {
        part_out[2 * AQ + (int64_t)i * a.vdim + c0 + cc] = t;
      } else {
        const float val = t * softmax_inv(st_m[i], st_l[i], a.sink, h0 + i % Rc) * a.out_scale;
        const int64_t col = (int64_t)(h0 + i % Rc) * a.vdim + c0 + cc;
        const int row = r0 + i / Rc;
        if (a.out) a.out[(int64_t)row * a.ldo + col] = val;
        if (a.out16) a.out16[(int64_t)row * a.ldo16 + col] = f32_to_bf16(val);
      }
    }
    __syncthreads();
  }
}

// Attention on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: scores and weights stay 32-bit), for runs of rows.  A workgroup of
// 4 waves owns the same 16 query vectors as the tiled form (<= 4 rows x <= 4 heads of one key/value head) and walks its keys —
// block means, then tokens — in tiles of 16, keys AND values staged through registers into LDS while the previous tile is multiplied:
//   scores   S[16 q, 16 keys] = Q K^T: every wave multiplies its quarter of the head's values (its slice of Q stays in registers),
//            the partial tiles are summed through LDS, so all four waves hold the same scores, apply the same per-(row, key)
//            visibility and keep the same running maximum / sum
//   values   O[16 q, vdim] += P V: the weights go through LDS into the A-operand layout, wave w owns the 16-column blocks w, w + 4, ..
// NBD / NBV: 64-value blocks of a key / a value (zero padded).  Key splits write the same partial layout as the tiled form.
// VK: the values are the first columns of the keys (one key/value head whose value arena is a view of the key arena — latent
// attention): the staged key tile serves both products and no value tile is loaded; NBV <= NBD.  Without a table of runs (decode
// rows) workgroup b takes row b and its up to 16 query heads.
template <int NBD, int NBV, bool VK = false>
__global__ __launch_bounds__(256) void window_attn_mfma_kernel(AttnTArgs a) {
  constexpr int KT = 16, LDP = 20, LDS_S = 17, DP = 64 * NBD, VP = 64 * NBV, LDK = DP + 4, LDV = VK ? LDK : VP + 4, DQ = DP / 4, AQ = 16;
  extern __shared__ float lds[];
  const int tid = threadIdx.x, b = blockIdx.x, gy = blockIdx.y, sp = blockIdx.z;
  const int rep = a.H / a.G, chunks = (rep + a.hpc - 1) / a.hpc;
  const int g = gy / chunks, h0 = g * rep + (gy % chunks) * a.hpc;
  const int Rc = min(a.hpc, g * rep + rep - h0);
  const int r0 = a.blk_tab ? a.blk_tab[2 * b] : b;
  const int nr = a.blk_tab ? min(a.blk_tab[2 * b + 1], a.rows_per_blk) : 1;
  const int nqv = nr * Rc;
  const int seq = a.row_seq[r0], pos0 = a.row_slot[r0], posL = pos0 + nr - 1;
  const int nbL = win_nb(posL, a.window, a.pool), tF = win_t0(pos0, a.window);
  const int nk = nbL + (posL - tF + 1);
  const int ntile = (nk + KT - 1) / KT, tps = (ntile + a.nsplit - 1) / a.nsplit;
  const int t0 = sp * tps, t1 = min(ntile, t0 + tps);
  float* Kl = lds;                       // [16 keys][LDK]
  float* Vl = VK ? Kl : Kl + KT * LDK;   // [16 keys][LDV]
  float* Sp = VK ? Kl + KT * LDK : Vl + KT * LDV;   // [4 waves][16 q][LDS_S] partial scores
  float* Pl = Sp + 4 * 16 * LDS_S;       // [16 q][LDP] weights
  const int wave = tid >> 6, lane = tid & 63, c16 = lane & 15, g4 = lane >> 4;
  // the A operands of this wave's score products stay in registers for the whole key walk: query c16, values wave DQ + 4 it + g4
  float qreg[DQ / 4];
  {
    const int qv = min(c16, nqv - 1);
    const float* src = a.q + (int64_t)(r0 + qv / Rc) * a.ldq + (int64_t)(h0 + qv % Rc) * a.dim;
#pragma unroll
    for (int it = 0; it < DQ / 4; ++it) {
      const int d = wave * DQ + 4 * it + g4;
      const float t = src[d < a.dim ? d : 0];
      qreg[it] = (c16 < nqv && d < a.dim) ? t : 0.f;
    }
  }
  int mypos[4], my_nb[4], my_t0[4];
  float mrun[4], lrun[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int qv = 4 * g4 + i;
    mypos[i] = qv < nqv ? pos0 + qv / Rc : -1;              // -1: no such vector, it sees nothing
    my_nb[i] = qv < nqv ? win_nb(mypos[i], a.window, a.pool) : 0;
    my_t0[i] = qv < nqv ? win_t0(mypos[i], a.window) : 0;
    mrun[i] = -INFINITY;
    lrun[i] = 0.f;
  }
  f32x4 acc[NBV];
#pragma unroll
  for (int c = 0; c < NBV; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int Gd = a.G * a.dim, Gv = a.G * a.vdim;
  const float* kb = a.k + ((int64_t)seq * a.t_max + tF) * a.ldk + (int64_t)g * a.dim;
  const float* vb = a.v + ((int64_t)seq * a.t_max + tF) * a.ldv + (int64_t)g * a.vdim;
  const float* pkb = a.pk ? a.pk + (int64_t)seq * a.n_pool_max * Gd + (int64_t)g * a.dim : nullptr;
  const float* pvb = a.pv ? a.pv + (int64_t)seq * a.n_pool_max * Gv + (int64_t)g * a.vdim : nullptr;
  f32x4 vk[NBD], vv[NBV];
  auto fetch = [&](int tile) {
    const int k0 = tile * KT;
    load16<NBD>(vk, a.dim, tid, [&](int j) { const int jj = min(k0 + j, nk - 1); return jj < nbL ? pkb + (int64_t)jj * Gd : kb + (int64_t)(jj - nbL) * a.ldk; },
                [&](int j) { return k0 + j < nk; });
    if (!VK) load16<NBV>(vv, a.vdim, tid, [&](int j) { const int jj = min(k0 + j, nk - 1); return jj < nbL ? pvb + (int64_t)jj * Gv : vb + (int64_t)(jj - nbL) * a.ldv; },
                [&](int j) { return k0 + j < nk; });
  };
  if (t0 < t1) fetch(t0);
  for (int tile = t0; tile < t1; ++tile) {
    const int key0 = tile * KT;
    lds_barrier();                                             // the previous tile's keys, values and weights are consumed
    store16<NBD, LDK>(Kl, vk, tid);
    if (!VK) store16<NBV, LDV>(Vl, vv, tid);
    if (tile + 1 < t1) fetch(tile + 1);                          // in flight while this tile is multiplied
    lds_barrier();
    {                                                            // partial scores over this wave's quarter of the head's values
      f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f}, s2 = f32x4{0.f, 0.f, 0.f, 0.f};
      const float* cb = Kl + c16 * LDK + wave * DQ + g4;
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
    float corr[4];
    const int j = key0 + c16, tok = tF + (j - nbL);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int o = (4 * g4 + i) * LDS_S + c16;
      float sc = soft_cap((Sp[o] + Sp[16 * LDS_S + o]) + (Sp[32 * LDS_S + o] + Sp[48 * LDS_S + o]), a.cap);
      const bool see = j < nk && (j < nbL ? j < my_nb[i] : (tok >= my_t0[i] && tok <= mypos[i]));
      if (!see) sc = -INFINITY;
      const float mnew = fmaxf(mrun[i], row16_max(sc));
      const float p = (sc == -INFINITY) ? 0.f : fast_exp(sc - mnew);
      corr[i] = (mrun[i] == -INFINITY) ? 0.f : fast_exp(mrun[i] - mnew);
      lrun[i] = lrun[i] * corr[i] + row16_sum(p);
      mrun[i] = mnew;
      if (wave == 0) Pl[(4 * g4 + i) * LDP + c16] = p;
    }
#pragma unroll
    for (int c = 0; c < NBV; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[c][i] *= corr[i];
    lds_barrier();
    // step t multiplies keys t, t + 4, t + 8, t + 12 (lane group g4 holds key t + 4 g4): with the row stride 4 mod 32 their rows
    // start 16 banks apart pairwise
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float pa = Pl[c16 * LDP + t + 4 * g4];
      const float* cb = Vl + (t + 4 * g4) * LDV + 16 * wave + c16;
#pragma unroll
      for (int c = 0; c < NBV; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa, cb[64 * c], acc[c], 0, 0, 0);
    }
  }
  float* part_out = a.nsplit > 1 ? a.part + (((int64_t)b * gridDim.y + gy) * a.nsplit + sp) * ((int64_t)AQ * (2 + a.vdim)) : nullptr;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int qv = 4 * g4 + i;
    if (qv >= nqv) continue;
    const int row = r0 + qv / Rc;
    const int64_t col0 = (int64_t)(h0 + qv % Rc) * a.vdim;
    const float inv = a.out_scale * softmax_inv(mrun[i], lrun[i], a.sink, h0 + qv % Rc);
#pragma unroll
    for (int c = 0; c < NBV; ++c) {
      const int d = 16 * (wave + 4 * c) + c16;
      if (d >= a.vdim) continue;
      if (part_out) {
        part_out[2 * AQ + (int64_t)qv * a.vdim + d] = acc[c][i];
      } else {
        const float val = acc[c][i] * inv;
        if (a.out) a.out[(int64_t)row * a.ldo + col0 + d] = val;
        if (a.out16) a.out16[(int64_t)row * a.ldo16 + col0 + d] = f32_to_bf16(val);
      }
    }
    if (part_out && wave == 0 && c16 == 0) { part_out[qv] = mrun[i]; part_out[AQ + qv] = lrun[i]; }
  }
}

// grid (n_blk, G * chunks, ceil(vdim / MERGE_COLS)): the splits' statistics and sums of every vector become its result; a workgroup
// takes a slice of the value columns (one workgroup a run left the merge of a single decode row on one CU)
constexpr int MERGE_COLS = 64;
template <int AQ>
__global__ __launch_bounds__(256) void window_attn_merge_kernel(AttnTArgs a) {
  const int tid = threadIdx.x, b = blockIdx.x, gy = blockIdx.y;
  const int rep = a.H / a.G, chunks = (rep + a.hpc - 1) / a.hpc;
  const int g = gy / chunks, h0 = g * rep + (gy % chunks) * a.hpc;
  const int Rc = min(a.hpc, g * rep + rep - h0);
  const int r0 = a.blk_tab ? a.blk_tab[2 * b] : b;
  const int nr = a.blk_tab ? min(a.blk_tab[2 * b + 1], a.rows_per_blk) : 1;
  const int nqv = nr * Rc;
  const int64_t stride = (int64_t)AQ * (2 + a.vdim);
  const float* base = a.part + ((int64_t)b * gridDim.y + gy) * a.nsplit * stride;
  // the weight of every (vector, split) once per workgroup: exp(its maximum - the overall maximum), and the vectors' normalisers
  __shared__ float wgt[AQ * 64];
  __shared__ float Ls[AQ], Ms[AQ];
  for (int i = tid >> 6; i < AQ; i += 4) {            // one wave per vector, one lane per split (at most 64)
    const int lane = tid & 63;
    const bool on = lane < a.nsplit;
    const float ms = on ? base[lane * stride + i] : -INFINITY;
    const float ls = on ? base[lane * stride + AQ + i] : 0.f;
    const float mx = wave_max(ms);
    const float w = ms == -INFINITY ? 0.f : expf(ms - mx);
    wgt[i * 64 + lane] = w;
    const float L = wave_sum(ls * w);
    if (lane == 0) { Ls[i] = L; Ms[i] = mx; }
  }
  __syncthreads();
  const int c0 = blockIdx.z * MERGE_COLS, cw = min(MERGE_COLS, a.vdim - c0);     // this workgroup's slice of the value columns
  for (int e = tid; e < nqv * cw; e += 256) {
    const int i = e / cw, c = c0 + e - i * cw;
    const float* src = base + 2 * AQ + (int64_t)i * a.vdim + c;
    float t = 0.f;
#pragma unroll 4
    for (int s = 0; s < a.nsplit; ++s) t = fmaf(src[s * stride], wgt[i * 64 + s], t);
    const float val = t * softmax_inv(Ms[i], Ls[i], a.sink, h0 + i % Rc) * a.out_scale;
    const int64_t col = (int64_t)(h0 + i % Rc) * a.vdim + c;
    const int row = r0 + i / Rc;
    if (a.out) a.out[(int64_t)row * a.ldo + col] = val;
    if (a.out16) a.out16[(int64_t)row * a.ldo16 + col] = f32_to_bf16(val);
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// minGRU: grid (ceil(n / 256), M); the workgroup of a sequence's FIRST row in the step walks that sequence's rows
__global__ __launch_bounds__(256) void mingru_kernel(const float* __restrict__ zx, int64_t ldzx, const float* __restrict__ g, int64_t ldg,
                                                     float* __restrict__ state, const int32_t* __restrict__ row_seq,
                                                     const int32_t* __restrict__ row_slot, const int32_t* __restrict__ row_back,
                                                     float out_scale, float* __restrict__ out, int64_t ldo, bf16_t* __restrict__ out16,
                                                     int64_t ldo16, int M, int n) {
  const int m0 = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (row_back[m0] != 0 || c >= n) return;
  float* sp = state + (int64_t)row_seq[m0] * n + c;
  float S = row_slot[m0] == 0 ? 0.f : *sp;
  for (int m = m0; m < M && row_back[m] == m - m0; ++m) {
    const float z = sigmoid_f(zx[(int64_t)m * ldzx + c]);
    const float u = zx[(int64_t)m * ldzx + n + c];
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    const float o = out_scale * S * silu_f(g[(int64_t)m * ldg + c]);
    if (out) out[(int64_t)m * ldo + c] = o;
    if (out16) out16[(int64_t)m * ldo16 + c] = f32_to_bf16(o);
  }
  *sp = S;
}

// minGRU as a chunked scan, for steps of many rows.  Over ALL rows of the step the recurrence is S_m = a_m S_(m-1) + b_m with
// a = 1 - z, b = z * candidate, where a sequence's first row in the step takes a = 0 and b = (1 - z) S_start + z * candidate
// (S_start: the sequence's stored state, zero at position 0).  Pass 1: every chunk of MG_CH rows -> (product of a, scan from zero),
// and S_start of the first rows parked in their output rows.  Pass 2: one thread per channel carries S over the chunks.  Pass 3:
// every chunk again from its carried S, writing the outputs and, at a sequence's last row, its state.
constexpr int MG_CH = 32;
struct MinGruArgs {
  const float* zx; int64_t ldzx;
  const float* g; int64_t ldg;
  float* state; const int32_t *row_seq, *row_slot, *row_back;
  float out_scale;
  float* out; int64_t ldo; bf16_t* out16; int64_t ldo16;
  float* ws;            // [n_chunks][2][n]
  int M, n;
};

__device__ __forceinline__ void mingru_ab(const MinGruArgs& a, int m, int c, float s_start, float& av, float& bv) {
  const float z = sigmoid_f(a.zx[(int64_t)m * a.ldzx + c]);
  const float u = a.zx[(int64_t)m * a.ldzx + a.n + c];
  const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
  av = 1.0f - z;
  bv = z * cand;
  if (a.row_back[m] == 0) { bv = av * s_start + bv; av = 0.f; }
}

__global__ __launch_bounds__(256) void mingru_pass1_kernel(MinGruArgs a) {
  const int ch = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= a.n) return;
  const int m0 = ch * MG_CH, m1 = min(a.M, m0 + MG_CH);
  float A = 1.f, B = 0.f;
  for (int m = m0; m < m1; ++m) {
    float s_start = 0.f;
    if (a.row_back[m] == 0) {
      s_start = a.row_slot[m] == 0 ? 0.f : a.state[(int64_t)a.row_seq[m] * a.n + c];
      a.out[(int64_t)m * a.ldo + c] = s_start;
    }
    float av, bv;
    mingru_ab(a, m, c, s_start, av, bv);
    A *= av;
    B = av * B + bv;
  }
  a.ws[((int64_t)ch * 2) * a.n + c] = A;
  a.ws[((int64_t)ch * 2 + 1) * a.n + c] = B;
}

__global__ __launch_bounds__(256) void mingru_pass2_kernel(MinGruArgs a, int n_chunks) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= a.n) return;
  float S = 0.f;
  for (int ch = 0; ch < n_chunks; ++ch) {
    const float A = a.ws[((int64_t)ch * 2) * a.n + c], B = a.ws[((int64_t)ch * 2 + 1) * a.n + c];
    a.ws[((int64_t)ch * 2) * a.n + c] = S;               // the chunk's carried-in state replaces its product
    S = A * S + B;
  }
}

__global__ __launch_bounds__(256) void mingru_pass3_kernel(MinGruArgs a) {
  const int ch = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= a.n) return;
  const int m0 = ch * MG_CH, m1 = min(a.M, m0 + MG_CH);
  float S = a.ws[((int64_t)ch * 2) * a.n + c];
  for (int m = m0; m < m1; ++m) {
    const float s_start = a.row_back[m] == 0 ? a.out[(int64_t)m * a.ldo + c] : 0.f;
    float av, bv;
    mingru_ab(a, m, c, s_start, av, bv);
    S = av * S + bv;
    const float o = a.out_scale * S * silu_f(a.g[(int64_t)m * a.ldg + c]);
    a.out[(int64_t)m * a.ldo + c] = o;
    if (a.out16) a.out16[(int64_t)m * a.ldo16 + c] = f32_to_bf16(o);
    if (m + 1 == a.M || a.row_back[m + 1] == 0) a.state[(int64_t)a.row_seq[m] * a.n + c] = S;
  }
}

// one wave per row: `top` rounds of arg-max (ties: the lower index), then the softmax over the chosen logits.  Lane l owns the
// logits l, l + 64, ... and a bit per owned logit that says it has been chosen (E <= 4096).
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits, int64_t ld, int M, int E, int top,
                                                          int32_t* __restrict__ idx, float* __restrict__ w, const float* __restrict__ sx,
                                                          int64_t ldsx, float* __restrict__ sy, int64_t ldsy, int sn) {
  const int nb = (M + 3) / 4;
  if ((int)blockIdx.x >= nb) {                          // extra workgroups: sy[m, c] = silu(sx[m, c]) * sx[m, sn + c]
    const int per_row = (sn + 255) / 256, e = (int)blockIdx.x - nb, m = e / per_row, c = (e % per_row) * 256 + threadIdx.x;
    if (c < sn) sy[(int64_t)m * ldsy + c] = silu_f(sx[(int64_t)m * ldsx + c]) * sx[(int64_t)m * ldsx + sn + c];
    return;
  }
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  const float* z = logits + (int64_t)row * ld;
  int32_t* ir = idx + (int64_t)row * top;
  float* wr = w + (int64_t)row * top;
  uint64_t taken = 0;
  float first = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, i = 0; e < E; e += 64, ++i) {
      const float v = z[e];
      if (!((taken >> i) & 1) && (v > best || (v == best && e < bi) || bi == 0x7fffffff)) { best = v; bi = e; }
    }
    for (int off = 32; off >= 1; off >>= 1) {
      const float ob = __shfl_xor(best, off);
      const int oi = __shfl_xor(bi, off);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > best || (ob == best && oi < bi))) { best = ob; bi = oi; }
    }
    if ((bi & 63) == lane) taken |= (uint64_t)1 << (bi >> 6);
    if (k == 0) first = best;
    const float p = expf(best - first);
    sum += p;
    if (lane == 0) { ir[k] = bi; wr[k] = p; }
  }
  // lane 0 wrote the unnormalised weights and is the one that scales them
  if (lane == 0)
    for (int k = 0; k < top; ++k) wr[k] = wr[k] / sum;
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ x, int64_t ldx, float* __restrict__ y, int64_t ldy,
                                                       bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const float o = silu_f(x[(int64_t)m * ldx + c]) * x[(int64_t)m * ldx + n + c];
  if (y) y[(int64_t)m * ldy + c] = o;
  if (y16) y16[(int64_t)m * ldy16 + c] = f32_to_bf16(o);
}

// one wave per output value: grid (ceil(N / 4), Z).  VEC: rows of K % 8 == 0 values at 16-byte aligned addresses, 8 weights per load
template <bool VEC>
__global__ __launch_bounds__(256) void gemv_indexed_kernel(const float* __restrict__ A, int64_t lda, int a_div, const bf16_t* __restrict__ W,
                                                           int64_t ldw, int64_t w_bs, const int32_t* __restrict__ w_idx,
                                                           float* __restrict__ C, int64_t ldc, int N, int K, int n_idx) {
  const int z = blockIdx.y, n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N || (unsigned)w_idx[z] >= (unsigned)n_idx) return;      // an index that names no weight block: the row is left as it is
  const float* ar = A + (int64_t)(z / a_div) * lda;
  const bf16_t* wr = W + (int64_t)w_idx[z] * w_bs + (int64_t)n * ldw;
  float acc = 0.f;
  if (VEC) {
    for (int k = lane * 8; k < K; k += 512) {
      const uint4 wv = *reinterpret_cast<const uint4*>(wr + k);
      const float4 a0 = *reinterpret_cast<const float4*>(ar + k), a1 = *reinterpret_cast<const float4*>(ar + k + 4);
      acc = fmaf(a0.x, bf16lo_to_f32(wv.x), acc); acc = fmaf(a0.y, bf16hi_to_f32(wv.x), acc);
      acc = fmaf(a0.z, bf16lo_to_f32(wv.y), acc); acc = fmaf(a0.w, bf16hi_to_f32(wv.y), acc);
      acc = fmaf(a1.x, bf16lo_to_f32(wv.z), acc); acc = fmaf(a1.y, bf16hi_to_f32(wv.z), acc);
      acc = fmaf(a1.z, bf16lo_to_f32(wv.w), acc); acc = fmaf(a1.w, bf16hi_to_f32(wv.w), acc);
    }
  } else {
    for (int k = lane; k < K; k += 64) acc = fmaf(ar[k], bf16_to_f32(wr[k]), acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) C[(int64_t)z * ldc + n] = acc;
}

__global__ __launch_bounds__(256) void moe_combine_residual_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y,
                                                                   int64_t ldy, const int32_t* __restrict__ slot_of,
                                                                   const float* __restrict__ w, int top, const float* __restrict__ shared,
                                                                   int64_t lds, const float* __restrict__ sg, int64_t ldsg, float mult,
                                                                   int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  float acc = 0.f;
  for (int j = 0; j < top; ++j) {
    const int z = m * top + j;
    const int64_t r = slot_of ? slot_of[z] : z;
    acc = fmaf(w[z], y[r * ldy + c], acc);
  }
  if (shared) acc += (sg ? sigmoid_f(sg[(int64_t)m * ldsg]) : 1.0f) * shared[(int64_t)m * lds + c];
  x[(int64_t)m * ldx + c] += mult * acc;
}

}  // namespace

extern "C" int mn_axpy_rms_rows(float* x, int64_t ldx, const float* y, int64_t ldy, float mult, const uint16_t* w, float eps, float* n_out,
                                int64_t ldn, uint16_t* n16, int64_t ldn16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && M >= 1 && n >= 1 && (w || (!n_out && !n16)), "mn_axpy_rms_rows: bad args");
  hipLaunchKernelGGL(axpy_rms_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), x, ldx, y, ldy, mult, w, eps, n_out,
                     ldn, n16, ldn16, M, n);
  MN_CHECK_LAUNCH("mn_axpy_rms_rows");
  return MN_OK;
}

extern "C" int mn_axpy_rms_filter_rows(float* x, int64_t ldx, const float* y, int64_t ldy, float mult, const uint16_t* w, float eps,
                                       const uint16_t* taps_w, int taps, float* state, const int32_t* row_seq, const int32_t* row_slot,
                                       float* h, int64_t ldh, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && h && M >= 1 && n >= 1 && n <= 8192, "mn_axpy_rms_filter_rows: bad args (n=%d: at most 8192)", n);
  MN_CHECK_ARG(!taps_w || (taps >= 1 && taps <= FUSED_MAX_TAPS && row_seq && row_slot && (taps == 1 || state)),
               "mn_axpy_rms_filter_rows: bad filter (taps=%d: at most %d)", taps, FUSED_MAX_TAPS);
  AxpyRmsFilterArgs a{x, ldx, y, ldy, mult, w, eps, taps_w, taps_w ? taps : 0, state, row_seq, row_slot, h, ldh, n};
  const int vpt = (n + 255) / 256;
  hipStream_t st = mn_stream(stream);
  const bool vec = (n % 4) == 0 && a.taps <= 4 && (ldx % 4) == 0 && (ldh % 4) == 0 && (!y || (ldy % 4) == 0) &&
                   ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)h) | ((uintptr_t)state)) & 15) == 0 && (((uintptr_t)w) & 7) == 0;
  if (vec) {
    const int nvg = (n / 4 + 255) / 256;
    if (nvg <= 1) hipLaunchKernelGGL((axpy_rms_filter_vec_kernel<1>), dim3((unsigned)M), dim3(256), 0, st, a);
    else if (nvg <= 2) hipLaunchKernelGGL((axpy_rms_filter_vec_kernel<2>), dim3((unsigned)M), dim3(256), 0, st, a);
    else if (nvg <= 4) hipLaunchKernelGGL((axpy_rms_filter_vec_kernel<4>), dim3((unsigned)M), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((axpy_rms_filter_vec_kernel<8>), dim3((unsigned)M), dim3(256), 0, st, a);
    MN_CHECK_LAUNCH("mn_axpy_rms_filter_rows");
    return MN_OK;
  }
#define MN_RB(V_)                                                                                                   \
  do {                                                                                                              \
    if (a.taps <= 4) hipLaunchKernelGGL((axpy_rms_filter_kernel<V_, 4>), dim3((unsigned)M), dim3(256), 0, st, a); \
    else hipLaunchKernelGGL((axpy_rms_filter_kernel<V_, 8>), dim3((unsigned)M), dim3(256), 0, st, a);             \
  } while (0)
  if (vpt <= 1) MN_RB(1); else if (vpt <= 2) MN_RB(2); else if (vpt <= 4) MN_RB(4); else if (vpt <= 8) MN_RB(8);
  else if (vpt <= 16) MN_RB(16); else MN_RB(32);
#undef MN_RB
  MN_CHECK_LAUNCH("mn_axpy_rms_filter_rows");
  return MN_OK;
}

extern "C" int mn_rope_unit_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, int rot_dims, const float* freq,
                                   float mag, int unit, float eps, float q_scale, const int32_t* row_seq, const int32_t* row_slot,
                                   float* q_out, int64_t ldq, float* k_arena, float* v_arena, int t_max, void* stream) {
  MN_CHECK_ARG(qkv && row_seq && row_slot && q_out && k_arena && v_arena && M >= 1 && M <= 65535 && H >= 1 && G >= 1 && t_max >= 1,
               "mn_rope_unit_append: bad args");
  MN_CHECK_ARG(dim >= 1 && dim <= 512 && vdim >= 1 && rot_dims >= 0 && rot_dims <= dim && (rot_dims % 2) == 0 && (rot_dims == 0 || freq),
               "mn_rope_unit_append: dim=%d (at most 512), rot_dims=%d (even, at most dim)", dim, rot_dims);
  RopeArgs a{qkv, ldqkv, H, G, dim, vdim, rot_dims, freq, mag, unit, eps, q_scale, row_seq, row_slot, q_out, ldq, k_arena, v_arena, t_max,
             nullptr, 0, nullptr, nullptr, nullptr, 0, 0, nullptr, 0, nullptr, 0, nullptr, 0, 0.f, nullptr, 0};
  hipLaunchKernelGGL((rope_unit_append_kernel<false>), dim3((unsigned)mn_cdiv(H + 2 * G, 4), (unsigned)M), dim3(256), 0, mn_stream(stream), a, M);
  MN_CHECK_LAUNCH("mn_rope_unit_append");
  return MN_OK;
}

extern "C" int mn_filter_rope_append_rows(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* w_conv, int conv,
                                          float* conv_state, int rot_dims, const float* freq, float mag, int unit, float eps, float q_scale,
                                          const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena,
                                          float* v_arena, int t_max, float* pk, float* pv, int n_pool_max, int pool, const float* zx,
                                          int64_t ldzx, const float* g, int64_t ldg, float* gru_state, int gru_n, float gru_scale, float* gru_out,
                                          int64_t ldgo, void* stream) {
  MN_CHECK_ARG(gru_n == 0 || (gru_n > 0 && zx && g && gru_state && gru_out), "mn_filter_rope_append_rows: bad recurrence args");
  MN_CHECK_ARG(qkv && row_seq && row_slot && q_out && k_arena && v_arena && M >= 1 && M <= 65535 && H >= 1 && G >= 1 && t_max >= 1,
               "mn_filter_rope_append_rows: bad args");
  MN_CHECK_ARG(dim >= 1 && dim <= 512 && vdim >= 1 && rot_dims >= 0 && rot_dims <= dim && (rot_dims % 2) == 0 && (rot_dims == 0 || freq),
               "mn_filter_rope_append_rows: dim=%d (at most 512), rot_dims=%d (even, at most dim)", dim, rot_dims);
  MN_CHECK_ARG(conv >= 0 && (conv == 0 || w_conv) && (conv <= 1 || conv_state) && pool >= 0 && (pool == 0 || (pk && pv && n_pool_max >= 1)),
               "mn_filter_rope_append_rows: bad filter or block arenas");
  RopeArgs a{qkv, ldqkv, H, G, dim, vdim, rot_dims, freq, mag, unit, eps, q_scale, row_seq, row_slot, q_out, ldq, k_arena, v_arena, t_max,
             w_conv, conv, conv_state, pk, pv, n_pool_max, pool, zx, ldzx, g, ldg, gru_state, gru_n, gru_scale, gru_out, ldgo};
  hipLaunchKernelGGL((rope_unit_append_kernel<true>), dim3((unsigned)(mn_cdiv(H + 2 * G, 4) + mn_cdiv(gru_n, 256)), (unsigned)M), dim3(256), 0,
                     mn_stream(stream), a, M);
  MN_CHECK_LAUNCH("mn_filter_rope_append_rows");
  return MN_OK;
}

extern "C" int mn_pool_blocks_update(const float* k_arena, const float* v_arena, int t_max, float* pk, float* pv, int n_pool_max, int pool,
                                     int Gd, int Gv, const int32_t* row_seq, const int32_t* row_slot, int M, void* stream) {
  MN_CHECK_ARG(k_arena && v_arena && pk && pv && row_seq && row_slot && pool >= 1 && n_pool_max >= 1 && Gd >= 1 && Gv >= 1 && M >= 1 &&
                   M <= 65535, "mn_pool_blocks_update: bad args");
  hipLaunchKernelGGL(pool_blocks_kernel, dim3((unsigned)mn_cdiv(Gd + Gv, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), k_arena,
                     v_arena, t_max, pk, pv, n_pool_max, pool, Gd, Gv, row_seq, row_slot);
  MN_CHECK_LAUNCH("mn_pool_blocks_update");
  return MN_OK;
}

extern "C" int mn_window_pool_attn(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk, const float* pv,
                                   const int32_t* row_seq, const int32_t* row_slot, int M, int H, int G, int dim, int vdim, int t_max,
                                   int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                                   int64_t ldo16, void* stream) {
  MN_CHECK_ARG(q && k_arena && v_arena && row_seq && row_slot && (out || out16) && M >= 1 && H >= 1 && G >= 1 && (H % G) == 0 && dim >= 1 &&
                   vdim >= 1 && t_max >= 1 && window >= 0 && pool >= 0, "mn_window_pool_attn: bad args");
  MN_CHECK_ARG(pool == 0 || (window > 0 && pk && pv && n_pool_max >= 1), "mn_window_pool_attn: pooled blocks need a window and their arenas");
  const int rep = H / G, chunks = (rep + ATT_R - 1) / ATT_R;
  MN_CHECK_ARG((rep < ATT_R ? rep : ATT_R) * vdim <= ATT_NOUT * 256, "mn_window_pool_attn: vdim=%d too large", vdim);
  const size_t lds = ((size_t)ATT_R * dim + ATT_R * ATT_TILE + 3 * ATT_R) * sizeof(float);
  MN_CHECK_ARG(lds <= 64 * 1024, "mn_window_pool_attn: dim=%d too large", dim);
  AttnArgs a{q, ldq, k_arena, v_arena, pool ? pk : nullptr, pool ? pv : nullptr, row_seq, row_slot, H, G, dim, vdim, t_max, n_pool_max, window,
             pool, out_scale, out, ldo, out16, ldo16};
  hipLaunchKernelGGL(window_pool_attn_kernel, dim3((unsigned)M, (unsigned)(G * chunks)), dim3(256), lds, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_window_pool_attn");
  return MN_OK;
}

extern "C" int mn_window_attn_block_rows(void) { return 4; }

namespace {
struct AttnShape { int aq, rows, hpc, chunks; };
AttnShape attn_shape(int H, int G, int one_row) {
  AttnShape s;
  const int rep = H / G;
  s.rows = one_row ? 1 : 4;
  s.aq = (one_row && rep <= 4) ? 4 : 16;
  s.hpc = s.aq / s.rows;
  s.chunks = (rep + s.hpc - 1) / s.hpc;
  return s;
}
}  // namespace

extern "C" int mn_window_attn_splits(int n_blk, int H, int G, int one_row, int max_keys) {
  return mn_window_attn_splits_tile(n_blk, H, G, one_row, max_keys, AKT);
}

extern "C" int mn_window_attn_splits_tile(int n_blk, int H, int G, int one_row, int max_keys, int key_tile) {
  if (n_blk < 1 || H < 1 || G < 1 || (H % G) != 0 || max_keys < 1 || key_tile < 1) return 1;
  const AttnShape sh = attn_shape(H, G, one_row);
  const int64_t wgs = (int64_t)n_blk * G * sh.chunks, tiles = mn_cdiv(max_keys, key_tile);
  int64_t ns = mn_cdiv(2 * (int64_t)mn_num_cus(), wgs);
  if (ns > tiles) ns = tiles;
  if (ns > 64) ns = 64;
  return ns < 1 ? 1 : (int)ns;
}

extern "C" size_t mn_window_attn_workspace_bytes(int n_blk, int H, int G, int vdim, int one_row, int nsplit) {
  if (nsplit <= 1 || n_blk < 1 || H < 1 || G < 1 || (H % G) != 0) return 0;
  const AttnShape sh = attn_shape(H, G, one_row);
  return (size_t)n_blk * G * sh.chunks * nsplit * sh.aq * (2 + (size_t)vdim) * sizeof(float);
}

extern "C" int mn_window_pool_attn_blocks(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                          const float* pv, const int32_t* row_seq, const int32_t* row_slot, const int32_t* blk_tab, int n_blk,
                                          int one_row, int H, int G, int dim, int vdim, int t_max, int n_pool_max, int window, int pool,
                                          float out_scale, float* out, int64_t ldo, uint16_t* out16, int64_t ldo16, int nsplit, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  // runs of rows with heads of at most 256 values go to the matrix cores, decode rows and larger heads to the fp32 FMA kernel
  const int variant = (!one_row && dim <= 256 && vdim <= 256) ? MN_WINDOW_ATTN_MFMA : MN_WINDOW_ATTN_VALU;
  return mn_window_pool_attn_blocks_ex(q, ldq, k_arena, v_arena, pk, pv, row_seq, row_slot, blk_tab, n_blk, one_row, H, G, dim, vdim, t_max,
                                       n_pool_max, window, pool, out_scale, out, ldo, out16, ldo16, nsplit, workspace, workspace_bytes, variant,
                                       stream);
}

extern "C" int mn_window_pool_attn_blocks_ex(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                             const float* pv, const int32_t* row_seq, const int32_t* row_slot, const int32_t* blk_tab, int n_blk,
                                             int one_row, int H, int G, int dim, int vdim, int t_max, int n_pool_max, int window, int pool,
                                             float out_scale, float* out, int64_t ldo, uint16_t* out16, int64_t ldo16, int nsplit, void* workspace,
                                             size_t workspace_bytes, int variant, void* stream) {
  return mn_window_pool_attn_blocks_sink(q, ldq, k_arena, v_arena, pk, pv, nullptr, row_seq, row_slot, blk_tab, n_blk, one_row, H, G, dim, vdim,
                                         t_max, n_pool_max, window, pool, out_scale, out, ldo, out16, ldo16, nsplit, workspace, workspace_bytes,
                                         variant, stream);
}

extern "C" int mn_window_pool_attn_blocks_sink(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                               const float* pv, const float* sink, const int32_t* row_seq, const int32_t* row_slot,
                                               const int32_t* blk_tab, int n_blk, int one_row, int H, int G, int dim, int vdim, int t_max,
                                               int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                                               int64_t ldo16, int nsplit, void* workspace, size_t workspace_bytes, int variant, void* stream) {
  return mn_window_pool_attn_blocks_cap(q, ldq, k_arena, 0, v_arena, 0, pk, pv, sink, 0.0f, row_seq, row_slot, blk_tab, n_blk, one_row, H, G, dim,
                                        vdim, t_max, n_pool_max, window, pool, out_scale, out, ldo, out16, ldo16, nsplit, workspace,
                                        workspace_bytes, variant, stream);
}

extern "C" int mn_window_pool_attn_blocks_cap(const float* q, int64_t ldq, const float* k_arena, int64_t ldk, const float* v_arena, int64_t ldv,
                                              const float* pk, const float* pv, const float* sink, float softcap, const int32_t* row_seq,
                                              const int32_t* row_slot, const int32_t* blk_tab, int n_blk, int one_row, int H, int G, int dim,
                                              int vdim, int t_max, int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo,
                                              uint16_t* out16, int64_t ldo16, int nsplit, void* workspace, size_t workspace_bytes, int variant,
                                              void* stream) {
  if (ldk <= 0) ldk = (int64_t)G * dim;
  if (ldv <= 0) ldv = (int64_t)G * vdim;
  MN_CHECK_ARG(ldk >= (int64_t)G * dim && ldv >= (int64_t)G * vdim && ((dim % 4) != 0 || (ldk % 4) == 0) && ((vdim % 4) != 0 || (ldv % 4) == 0) &&
                   softcap >= 0.0f,
               "mn_window_pool_attn_blocks: arena row strides below a row, or no multiple of 4 under heads that are; or a negative soft cap");
  const bool variant_auto = variant < 0;
  MN_CHECK_ARG(q && k_arena && v_arena && row_seq && row_slot && (out || out16) && n_blk >= 1 && H >= 1 && G >= 1 && (H % G) == 0 && dim >= 1 &&
                   vdim >= 1 && vdim <= 512 && t_max >= 1 && window >= 0 && pool >= 0 && nsplit >= 1 && nsplit <= 64,
               "mn_window_pool_attn_blocks: bad args (vdim=%d: at most 512; nsplit=%d: at most 64)", vdim, nsplit);
  MN_CHECK_ARG(pool == 0 || (window > 0 && pk && pv && n_pool_max >= 1), "mn_window_pool_attn_blocks: pooled blocks need a window and their arenas");
  MN_CHECK_ARG(one_row || blk_tab, "mn_window_pool_attn_blocks: runs of several rows need their table");
  const AttnShape sh = attn_shape(H, G, one_row);
  MN_CHECK_ARG((int64_t)G * sh.chunks <= 65535, "mn_window_pool_attn_blocks: too many heads");
  MN_CHECK_ARG(nsplit == 1 || (workspace && workspace_bytes >= mn_window_attn_workspace_bytes(n_blk, H, G, vdim, one_row, nsplit)),
               "mn_window_pool_attn_blocks: workspace too small");
  AttnTArgs a{q, ldq, k_arena, v_arena, pool ? pk : nullptr, pool ? pv : nullptr, row_seq, row_slot, one_row ? nullptr : blk_tab, H, G, dim, vdim,
              t_max, n_pool_max, window, pool, sh.rows, sh.hpc, nsplit, out_scale, out, ldo, out16, ldo16, (float*)workspace, sink, softcap, ldk, ldv};
  // values that are a view of the keys (one key/value head, the same arena and stride): the matrix-core kernel stages one tile for both
  const bool vk = G == 1 && k_arena == v_arena && ldk == ldv && vdim <= dim && !pool;
  const bool mfma_fits = vk ? (dim <= 640 && sh.aq == 16) : (!one_row && dim <= 256 && vdim <= 256);
  if (variant_auto) variant = mfma_fits ? MN_WINDOW_ATTN_MFMA : MN_WINDOW_ATTN_VALU;
  MN_CHECK_ARG(variant == MN_WINDOW_ATTN_VALU || (variant == MN_WINDOW_ATTN_MFMA && mfma_fits),
               "mn_window_pool_attn_blocks: the matrix-core kernel takes runs of rows with dim, vdim <= 256, or values inside keys of dim <= 640");
  if (variant == MN_WINDOW_ATTN_MFMA) {
    const dim3 gridm((unsigned)n_blk, (unsigned)(G * sh.chunks), (unsigned)nsplit);
    hipStream_t stm = mn_stream(stream);
    if (vk) {
      const int nb = dim <= 256 ? (dim + 63) / 64 : (dim <= 320 ? 5 : (dim <= 384 ? 6 : (dim <= 512 ? 8 : 10)));
      const size_t ldsm = ((size_t)16 * (64 * nb + 4) + 4 * 16 * 17 + 16 * 20) * sizeof(float);
#define MN_WK(D_) hipLaunchKernelGGL((window_attn_mfma_kernel<D_, D_, true>), gridm, dim3(256), ldsm, stm, a)
      switch (nb) {
        case 1: MN_WK(1); break;
        case 2: MN_WK(2); break;
        case 3: MN_WK(3); break;
        case 4: MN_WK(4); break;
        case 5: MN_WK(5); break;
        case 6: MN_WK(6); break;
        case 8: MN_WK(8); break;
        default: MN_WK(10); break;
      }
#undef MN_WK
    } else {
      const int nbd = dim <= 64 ? 1 : (dim <= 128 ? 2 : 4), nbv = vdim <= 64 ? 1 : (vdim <= 128 ? 2 : 4);
      const size_t ldsm = ((size_t)16 * (64 * nbd + 4) + (size_t)16 * (64 * nbv + 4) + 4 * 16 * 17 + 16 * 20) * sizeof(float);
#define MN_WM(D_, V_) hipLaunchKernelGGL((window_attn_mfma_kernel<D_, V_>), gridm, dim3(256), ldsm, stm, a)
      if (nbd == 1) { if (nbv == 1) MN_WM(1, 1); else if (nbv == 2) MN_WM(1, 2); else MN_WM(1, 4); }
      else if (nbd == 2) { if (nbv == 1) MN_WM(2, 1); else if (nbv == 2) MN_WM(2, 2); else MN_WM(2, 4); }
      else { if (nbv == 1) MN_WM(4, 1); else if (nbv == 2) MN_WM(4, 2); else MN_WM(4, 4); }
#undef MN_WM
    }
    MN_CHECK_LAUNCH("mn_window_pool_attn_blocks(mfma)");
    if (nsplit > 1) {
      hipLaunchKernelGGL((window_attn_merge_kernel<16>), dim3((unsigned)n_blk, (unsigned)(G * sh.chunks), (unsigned)mn_cdiv(vdim, MERGE_COLS)), dim3(256), 0, stm, a);
      MN_CHECK_LAUNCH("mn_window_pool_attn_blocks(merge)");
    }
    return MN_OK;
  }
  const size_t lds = ((size_t)sh.aq * dim + 2 * (size_t)sh.aq * AKT + 3 * sh.aq + (size_t)sh.aq * 256) * sizeof(float);
  MN_CHECK_ARG(lds <= 64 * 1024, "mn_window_pool_attn_blocks: dim=%d too large", dim);
  const bool vec = (dim % 4) == 0 && (ldq % 4) == 0 && (ldk % 4) == 0 && (((uintptr_t)q | (uintptr_t)k_arena | (uintptr_t)pk) & 15) == 0;
  const dim3 grid((unsigned)n_blk, (unsigned)(G * sh.chunks), (unsigned)nsplit);
  hipStream_t st = mn_stream(stream);
  if (sh.aq == 4) {
    if (vec) hipLaunchKernelGGL((window_attn_tiled_kernel<4, true>), grid, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((window_attn_tiled_kernel<4, false>), grid, dim3(256), lds, st, a);
  } else {
    if (vec) hipLaunchKernelGGL((window_attn_tiled_kernel<16, true>), grid, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((window_attn_tiled_kernel<16, false>), grid, dim3(256), lds, st, a);
  }
  MN_CHECK_LAUNCH("mn_window_pool_attn_blocks");
  if (nsplit > 1) {
    const dim3 mg((unsigned)n_blk, (unsigned)(G * sh.chunks), (unsigned)mn_cdiv(vdim, MERGE_COLS));
    if (sh.aq == 4) hipLaunchKernelGGL((window_attn_merge_kernel<4>), mg, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((window_attn_merge_kernel<16>), mg, dim3(256), 0, st, a);
    MN_CHECK_LAUNCH("mn_window_pool_attn_blocks(merge)");
  }
  return MN_OK;
}

extern "C" int mn_mingru_rows(const float* zx, int64_t ldzx, const float* g, int64_t ldg, float* state, const int32_t* row_seq,
                              const int32_t* row_slot, const int32_t* row_back, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                              int64_t ldo16, int M, int n, void* stream) {
  MN_CHECK_ARG(zx && g && state && row_seq && row_slot && row_back && (out || out16) && M >= 1 && M <= 65535 && n >= 1,
               "mn_mingru_rows: bad args");
  hipLaunchKernelGGL(mingru_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), zx, ldzx, g, ldg, state,
                     row_seq, row_slot, row_back, out_scale, out, ldo, out16, ldo16, M, n);
  MN_CHECK_LAUNCH("mn_mingru_rows");
  return MN_OK;
}

extern "C" size_t mn_mingru_scan_workspace_bytes(int M, int n) {
  return M < 1 || n < 1 ? 0 : (size_t)mn_cdiv(M, MG_CH) * 2 * n * sizeof(float);
}

extern "C" int mn_mingru_rows_scan(const float* zx, int64_t ldzx, const float* g, int64_t ldg, float* state, const int32_t* row_seq,
                                   const int32_t* row_slot, const int32_t* row_back, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                                   int64_t ldo16, int M, int n, void* workspace, size_t workspace_bytes, void* stream) {
  MN_CHECK_ARG(zx && g && state && row_seq && row_slot && row_back && out && M >= 1 && n >= 1 && mn_cdiv(M, MG_CH) <= 65535,
               "mn_mingru_rows_scan: bad args");
  MN_CHECK_ARG(workspace && workspace_bytes >= mn_mingru_scan_workspace_bytes(M, n), "mn_mingru_rows_scan: workspace too small");
  MinGruArgs a{zx, ldzx, g, ldg, state, row_seq, row_slot, row_back, out_scale, out, ldo, out16, ldo16, (float*)workspace, M, n};
  const int n_chunks = (int)mn_cdiv(M, MG_CH);
  const dim3 grid((unsigned)mn_cdiv(n, 256), (unsigned)n_chunks);
  hipStream_t st = mn_stream(stream);
  hipLaunchKernelGGL(mingru_pass1_kernel, grid, dim3(256), 0, st, a);
  hipLaunchKernelGGL(mingru_pass2_kernel, dim3(grid.x), dim3(256), 0, st, a, n_chunks);
  hipLaunchKernelGGL(mingru_pass3_kernel, grid, dim3(256), 0, st, a);
  MN_CHECK_LAUNCH("mn_mingru_rows_scan");
  return MN_OK;
}

extern "C" int mn_router_topk_rows(const float* logits, int64_t ld, int M, int E, int top, int32_t* idx, float* w, void* stream) {
  MN_CHECK_ARG(logits && idx && w && M >= 1 && E >= 1 && E <= 4096 && top >= 1 && top <= E, "mn_router_topk_rows: bad args (E=%d top=%d)", E, top);
  hipLaunchKernelGGL(router_topk_kernel, dim3((unsigned)mn_cdiv(M, 4)), dim3(256), 0, mn_stream(stream), logits, ld, M, E, top, idx, w,
                     (const float*)nullptr, (int64_t)0, (float*)nullptr, (int64_t)0, 0);
  MN_CHECK_LAUNCH("mn_router_topk_rows");
  return MN_OK;
}

extern "C" int mn_router_topk_silu_rows(const float* logits, int64_t ld, int M, int E, int top, int32_t* idx, float* w, const float* x,
                                        int64_t ldx, float* y, int64_t ldy, int n, void* stream) {
  MN_CHECK_ARG(logits && idx && w && x && y && M >= 1 && E >= 1 && E <= 4096 && top >= 1 && top <= E && n >= 1 &&
                   mn_cdiv(M, 4) + (int64_t)M * mn_cdiv(n, 256) <= 0x7fffffff, "mn_router_topk_silu_rows: bad args (E=%d top=%d)", E, top);
  hipLaunchKernelGGL(router_topk_kernel, dim3((unsigned)(mn_cdiv(M, 4) + (int64_t)M * mn_cdiv(n, 256))), dim3(256), 0, mn_stream(stream), logits,
                     ld, M, E, top, idx, w, x, ldx, y, ldy, n);
  MN_CHECK_LAUNCH("mn_router_topk_silu_rows");
  return MN_OK;
}

extern "C" int mn_silu_mul_rows(const float* x, int64_t ldx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n,
                                void* stream) {
  MN_CHECK_ARG(x && (y || y16) && M >= 1 && M <= 65535 && n >= 1, "mn_silu_mul_rows: bad args");
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, y, ldy, y16,
                     ldy16, n);
  MN_CHECK_LAUNCH("mn_silu_mul_rows");
  return MN_OK;
}

extern "C" int mn_gemv_f32_indexed(const float* A, int64_t lda, int a_div, const uint16_t* W, int64_t ldw, int64_t w_bs,
                                   const int32_t* w_idx, float* C, int64_t ldc, int Z, int N, int K, void* stream) {
  return mn_gemv_f32_indexed_upto(A, lda, a_div, W, ldw, w_bs, w_idx, 0x7fffffff, C, ldc, Z, N, K, stream);
}

extern "C" int mn_gemv_f32_indexed_upto(const float* A, int64_t lda, int a_div, const uint16_t* W, int64_t ldw, int64_t w_bs,
                                        const int32_t* w_idx, int n_idx, float* C, int64_t ldc, int Z, int N, int K, void* stream) {
  MN_CHECK_ARG(A && W && w_idx && C && a_div >= 1 && Z >= 1 && Z <= 65535 && N >= 1 && K >= 1 && n_idx >= 1,
               "mn_gemv_f32_indexed: bad args (Z=%d)", Z);
  const bool vec = (K % 8) == 0 && (ldw % 8) == 0 && (w_bs % 8) == 0 && (lda % 4) == 0 && (((uintptr_t)W | (uintptr_t)A) & 15) == 0;
  const dim3 grid((unsigned)mn_cdiv(N, 4), (unsigned)Z);
  if (vec) hipLaunchKernelGGL((gemv_indexed_kernel<true>), grid, dim3(256), 0, mn_stream(stream), A, lda, a_div, W, ldw, w_bs, w_idx, C, ldc, N, K, n_idx);
  else hipLaunchKernelGGL((gemv_indexed_kernel<false>), grid, dim3(256), 0, mn_stream(stream), A, lda, a_div, W, ldw, w_bs, w_idx, C, ldc, N, K, n_idx);
  MN_CHECK_LAUNCH("mn_gemv_f32_indexed");
  return MN_OK;
}

extern "C" int mn_moe_combine_residual(float* x, int64_t ldx, const float* y, int64_t ldy, const int32_t* slot_of, const float* w, int top,
                                       const float* shared, int64_t lds, const float* sg, int64_t ldsg, float mult, int M, int n,
                                       void* stream) {
  MN_CHECK_ARG(x && y && w && top >= 1 && M >= 1 && M <= 65535 && n >= 1, "mn_moe_combine_residual: bad args");
  hipLaunchKernelGGL(moe_combine_residual_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, y,
                     ldy, slot_of, w, top, shared, lds, sg, ldsg, mult, n);
  MN_CHECK_LAUNCH("mn_moe_combine_residual");
  return MN_OK;
}
