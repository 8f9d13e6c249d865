// hybrid_ops.hip — operators of hybrid-mixer sequence models (mingnative.h section 11): per-head weighted RMS norm of queries and
// keys with a position-dependent query temperature and the cache append, the decayed linear-attention recurrence ("lightning"
// attention) with its fp32 state, the RMS-norm x sigmoid-gate of its joined heads, the squared-relu activation, a router that scores
// by softmax over every output, picks by score + correction and passes some picks through, and the expert combine that knows them.
// Rows are fp32, weights bf16; everything here is fp32 arithmetic.
#include "mfma_f32_tiles.h"

namespace {

__device__ __forceinline__ float sigm32(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu32(float x) { return x / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------------------------------------------------------
// One wave per (row, head vector): q heads 0 .. H - 1, k heads H .. H + G - 1, v heads after them; a lane holds values lane, lane + 64, ..
// (dim <= 512).  q and k heads: x / sqrt(mean(x^2) + eps) * w; q further times q_scale * (1 + coef ln(floor((pos + 1) / every) + 1)).
struct HeadNormArgs {
  const float* qkv; int64_t ldqkv;
  int H, G, dim, vdim;
  const bf16_t *qw, *kw;
  float eps, q_scale, temp_coef; int temp_every;
  const int32_t *row_seq, *row_slot;
  float* q_out; int64_t ldq;
  float *k_arena, *v_arena; int t_max;
};

__global__ __launch_bounds__(256) void head_norm_temp_append_kernel(HeadNormArgs a) {
  const int hv = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, m = blockIdx.y;
  const int nh = a.H + 2 * a.G;
  if (hv >= nh) return;
  const float* row = a.qkv + (int64_t)m * a.ldqkv;
  const int seq = a.row_seq[m], slot = a.row_slot[m];
  const int64_t crow = (int64_t)seq * a.t_max + slot;
  if (hv >= a.H + a.G) {
    const int g = hv - a.H - a.G;
    const float* src = row + (a.H + a.G) * a.dim + g * a.vdim;
    float* dst = a.v_arena + crow * ((int64_t)a.G * a.vdim) + (int64_t)g * a.vdim;
    for (int i = lane; i < a.vdim; i += 64) dst[i] = src[i];
    return;
  }
  const bool is_q = hv < a.H;
  const float* src = row + (int64_t)hv * a.dim;
  float v[8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = lane + 64 * j;
    v[j] = i < a.dim ? src[i] : 0.f;
    ss += v[j] * v[j];
  }
  float r = 1.0f / sqrtf(wave_sum(ss) / (float)a.dim + a.eps);
  const bf16_t* w = is_q ? a.qw : a.kw;
  float* dst = is_q ? a.q_out + (int64_t)m * a.ldq + (int64_t)hv * a.dim
                    : a.k_arena + crow * ((int64_t)a.G * a.dim) + (int64_t)(hv - a.H) * a.dim;
  float f = 1.0f;
  if (is_q) {
    f = a.q_scale;
    if (a.temp_every > 0 && a.temp_coef != 0.f) f *= 1.0f + a.temp_coef * logf((float)((slot + 1) / a.temp_every) + 1.0f);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = lane + 64 * j;
    if (i < a.dim) {
      float o = v[j] * r;
      if (w) o *= bf16_to_f32(w[i]);
      dst[i] = o * f;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Decayed linear-attention recurrence, one thread per (head, value column): S[:, c] = decay S[:, c] + k v[c], o[c] = S[:, c] . q, with
// q, k, v = silu of the projected rows.  The workgroup of a sequence's FIRST row in the step walks that sequence's rows; q and k of
// a token are staged through LDS (two buffers: one barrier per token).  NB > 0: the state column (dim <= 32 NB values) lives in
// registers; NB == 0: it stays in the state arena (any dim).
struct LightArgs {
  const float* qkv; int64_t ldqkv;           // per row [q (H dim) ; k (H dim) ; v (H vdim)] before the activation
  int H, dim, vdim;
  const float* decay;                        // device fp32 [H]
  float* state;                              // [n_seq, H, dim, vdim]
  const int32_t *row_seq, *row_slot, *row_back;
  float* out; int64_t ldo;                   // [M, H vdim]
  int M;
};

template <int NB>
__global__ __launch_bounds__(256) void lightning_rows_kernel(LightArgs a) {
  extern __shared__ float lds[];             // [2][2 dim]
  const int m0 = blockIdx.x, h = blockIdx.y, c = blockIdx.z * 256 + threadIdx.x, tid = threadIdx.x;
  if (a.row_back[m0] != 0) return;
  const int d = a.dim;
  const bool on = c < a.vdim;
  const float lam = a.decay[h];
  float* sp = a.state + (((int64_t)a.row_seq[m0] * a.H + h) * d) * a.vdim + (on ? c : 0);
  const bool fresh = a.row_slot[m0] == 0;
  constexpr int NR = NB > 0 ? 32 * NB : 1;
  float S[NR];
  if (NB > 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i) S[i] = (on && !fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f;
  } else if (fresh && on) {
    for (int i = 0; i < d; ++i) sp[(int64_t)i * a.vdim] = 0.f;
  }
  int buf = 0;
  for (int m = m0; m < a.M && a.row_back[m] == m - m0; ++m, buf ^= 1) {
    const float* row = a.qkv + (int64_t)m * a.ldqkv;
    float* qk = lds + buf * 2 * d;
    for (int i = tid; i < 2 * d; i += 256) qk[i] = silu32(row[(int64_t)(i < d ? 0 : a.H * d) + (int64_t)h * d + (i < d ? i : i - d)]);
    const float v = on ? silu32(row[(int64_t)2 * a.H * d + (int64_t)h * a.vdim + c]) : 0.f;
    __syncthreads();
    float o = 0.f;
    if (NB > 0) {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        if (i < d) {
          S[i] = fmaf(lam, S[i], qk[d + i] * v);
          o = fmaf(S[i], qk[i], o);
        }
      }
    } else if (on) {
      for (int i = 0; i < d; ++i) {
        const float s = fmaf(lam, sp[(int64_t)i * a.vdim], qk[d + i] * v);
        sp[(int64_t)i * a.vdim] = s;
        o = fmaf(s, qk[i], o);
      }
    }
    if (on) a.out[(int64_t)m * a.ldo + (int64_t)h * a.vdim + c] = o;
  }
  if (NB > 0 && on) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (i < d) sp[(int64_t)i * a.vdim] = S[i];
  }
}

// Decode rows: grid (M, H, ceil(vdim / 32)); a workgroup owns 32 value columns of one head's state, its 8 groups of 32 threads
// split the rows of the state (dim / 8 each), and the partial sums of a column meet in LDS.
__global__ __launch_bounds__(256) void lightning_step_kernel(LightArgs a) {
  extern __shared__ float lds[];             // [2 dim] q, k; [8][32] partial outputs
  const int m = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, cl = tid & 31, sub = tid >> 5, c = blockIdx.z * 32 + cl;
  const int d = a.dim;
  const float* row = a.qkv + (int64_t)m * a.ldqkv;
  float* qk = lds;
  float* part = lds + 2 * d;
  for (int i = tid; i < 2 * d; i += 256) qk[i] = silu32(row[(int64_t)(i < d ? 0 : a.H * d) + (int64_t)h * d + (i < d ? i : i - d)]);
  const bool on = c < a.vdim;
  const float v = on ? silu32(row[(int64_t)2 * a.H * d + (int64_t)h * a.vdim + c]) : 0.f;
  const float lam = a.decay[h];
  const bool fresh = a.row_slot[m] == 0;
  float* sp = a.state + (((int64_t)a.row_seq[m] * a.H + h) * d) * a.vdim + (on ? c : 0);
  __syncthreads();
  float o = 0.f;
  if (on) {
    constexpr int PRE = 8;                   // state values in flight per thread
    for (int i0 = sub; i0 < d; i0 += 8 * PRE) {
      float s[PRE];
#pragma unroll
      for (int u = 0; u < PRE; ++u) {
        const int i = i0 + 8 * u;
        s[u] = (!fresh && i < d) ? sp[(int64_t)i * a.vdim] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < PRE; ++u) {
        const int i = i0 + 8 * u;
        if (i < d) {
          const float t = fmaf(lam, s[u], qk[d + i] * v);
          sp[(int64_t)i * a.vdim] = t;
          o = fmaf(t, qk[i], o);
        }
      }
    }
  }
  part[sub * 32 + cl] = o;
  __syncthreads();
  if (sub == 0 && on) {
    float t = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) t += part[u * 32 + cl];
    a.out[(int64_t)m * a.ldo + (int64_t)h * a.vdim + c] = t;
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// The recurrence as a chunked scan.  With n the rows of a chunk, lam the head's decay and S0 the state at the chunk's start:
//   own sum   KV = sum_j lam^(n-1-j) k_j v_j^T                               (pass 1, every chunk and head by itself)
//   carry     S0 of the next chunk = lam^n S0 + KV, along each sequence       (pass 2, one thread per state value)
//   outputs   o_i = lam^(i+1) S0^T q_i + sum_(j<=i) lam^(i-j) (q_i . k_j) v_j  (pass 3, every chunk and head by itself)
constexpr int LCH = 32;
struct LightScanArgs {
  LightArgs b;
  const int32_t* chunk_tab; int n_chunks;
  float* ws;                                 // [n_chunks, H, dim, vdim]
};
__device__ __forceinline__ float powi32(float lam, float loglam, int p) { return p == 0 ? 1.0f : (lam > 0.f ? expf((float)p * loglam) : 0.f); }

// CV value columns per thread (4: 16-byte loads of the values and the carried state; needs vdim % 4 == 0), the rows of the result
// split over the thread groups that share a column group
template <int CV>
__device__ __forceinline__ void ld_cols(const float* p, float (&v)[CV]) {
  if constexpr (CV == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    v[0] = *p;
  }
}

template <int CV>
__global__ __launch_bounds__(256) void light_scan_kv_kernel(LightScanArgs s) {
  extern __shared__ float lds[];             // k [LCH][dim] (decayed), v [LCH][vdim]
  const LightArgs& a = s.b;
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, d = a.dim, e = a.vdim;
  const int r0 = s.chunk_tab[2 * ch], n = s.chunk_tab[2 * ch + 1];
  float* kl = lds;
  float* vl = lds + LCH * d;
  const float lam = a.decay[h], ll = lam > 0.f ? logf(lam) : 0.f;
  for (int x = tid; x < n * d; x += 256) {
    const int j = x / d, i = x - j * d;
    kl[x] = silu32(a.qkv[(int64_t)(r0 + j) * a.ldqkv + (int64_t)a.H * d + (int64_t)h * d + i]) * powi32(lam, ll, n - 1 - j);
  }
  for (int x = tid; x < n * e; x += 256) {
    const int j = x / e, c = x - j * e;
    vl[x] = silu32(a.qkv[(int64_t)(r0 + j) * a.ldqkv + (int64_t)2 * a.H * d + (int64_t)h * e + c]);
  }
  __syncthreads();
  float* dst = s.ws + ((int64_t)ch * a.H + h) * d * e;
  constexpr int R = 8;
  const int ncg = e / CV;
  for (int g0 = 0; g0 < ncg; g0 += 256) {
    const int cw = min(256, ncg - g0), nsub = 256 / cw, c = CV * (g0 + tid % cw), sub = tid / cw;
    if (sub >= nsub) continue;
    for (int ib = 0; ib < d; ib += R * nsub) {
      float acc[R][CV];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int q = 0; q < CV; ++q) acc[r][q] = 0.f;
      for (int j = 0; j < n; ++j) {
        float vv[CV];
        ld_cols<CV>(vl + j * e + c, vv);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int i = ib + sub + r * nsub;
          const float kk = kl[j * d + (i < d ? i : 0)];
#pragma unroll
          for (int q = 0; q < CV; ++q) acc[r][q] = fmaf(kk, vv[q], acc[r][q]);
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int i = ib + sub + r * nsub;
        if (i >= d) continue;
#pragma unroll
        for (int q = 0; q < CV; ++q) dst[(int64_t)i * e + c + q] = acc[r][q];
      }
    }
  }
}

// grid (ceil(dim vdim / 256), H, n_chunks): the workgroup of a sequence's first chunk in the step walks that sequence's chunks
__global__ __launch_bounds__(256) void light_scan_carry_kernel(LightScanArgs s) {
  const LightArgs& a = s.b;
  const int x = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y, c0 = blockIdx.z, de = a.dim * a.vdim;
  const int r0 = s.chunk_tab[2 * c0];
  if (a.row_back[r0] != 0 || x >= de) return;
  const float lam = a.decay[h], ll = lam > 0.f ? logf(lam) : 0.f;
  float* sp = a.state + ((int64_t)a.row_seq[r0] * a.H + h) * de + x;
  float S = a.row_slot[r0] == 0 ? 0.f : *sp;
  for (int ch = c0; ch < s.n_chunks; ++ch) {
    if (ch > c0 && a.row_back[s.chunk_tab[2 * ch]] == 0) break;      // the next sequence starts here
    float* w = s.ws + ((int64_t)ch * a.H + h) * de + x;
    const float kv = *w;
    *w = S;
    S = fmaf(powi32(lam, ll, s.chunk_tab[2 * ch + 1]), S, kv);
  }
  *sp = S;
}

template <int CV>
__global__ __launch_bounds__(256) void light_scan_out_kernel(LightScanArgs s) {
  extern __shared__ float lds[];             // q [LCH][dim + 1], k [LCH][dim + 1], v [LCH][vdim], P [LCH][LCH + 1]
  const LightArgs& a = s.b;
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, d = a.dim, e = a.vdim, dp = d + 1;   // odd row stride: the score loop walks rows
  const int r0 = s.chunk_tab[2 * ch], n = s.chunk_tab[2 * ch + 1];
  float* ql = lds;
  float* kl = ql + LCH * dp;
  float* vl = kl + LCH * dp + (4 - (2 * LCH * dp) % 4) % 4;      // 16-byte aligned rows of values
  float* P = vl + LCH * e;
  const float lam = a.decay[h], ll = lam > 0.f ? logf(lam) : 0.f;
  for (int x = tid; x < n * d; x += 256) {
    const int j = x / d, i = x - j * d;
    const float* row = a.qkv + (int64_t)(r0 + j) * a.ldqkv + (int64_t)h * d + i;
    ql[j * dp + i] = silu32(row[0]);
    kl[j * dp + i] = silu32(row[(int64_t)a.H * d]);
  }
  for (int x = tid; x < n * e; x += 256) {
    const int j = x / e, c = x - j * e;
    vl[x] = silu32(a.qkv[(int64_t)(r0 + j) * a.ldqkv + (int64_t)2 * a.H * d + (int64_t)h * e + c]);
  }
  __syncthreads();
  for (int x = tid; x < n * n; x += 256) {
    const int i = x / n, j = x - i * n;
    float t = 0.f;
    if (j <= i) {
      float t2 = 0.f;
      int u = 0;
      for (; u + 1 < d; u += 2) {
        t = fmaf(ql[i * dp + u], kl[j * dp + u], t);
        t2 = fmaf(ql[i * dp + u + 1], kl[j * dp + u + 1], t2);
      }
      if (u < d) t = fmaf(ql[i * dp + u], kl[j * dp + u], t);
      t = (t + t2) * powi32(lam, ll, i - j);
    }
    P[i * (LCH + 1) + j] = t;
  }
  __syncthreads();
  const float* S0 = s.ws + ((int64_t)ch * a.H + h) * d * e;
  constexpr int R = 4;
  const int ncg = e / CV;
  for (int g0 = 0; g0 < ncg; g0 += 256) {
    const int cw = min(256, ncg - g0), nsub = 256 / cw, c = CV * (g0 + tid % cw), sub = tid / cw;
    if (sub >= nsub) continue;
    for (int ib = 0; ib < n; ib += R * nsub) {
      float acc[R][CV];
      int qrow[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int i = ib + sub + r * nsub;
        qrow[r] = (i < n ? i : 0) * dp;
#pragma unroll
        for (int q = 0; q < CV; ++q) acc[r][q] = 0.f;
      }
      for (int u = 0; u < d; ++u) {                    // the part that comes from the chunk's start state
        float sv[CV];
        ld_cols<CV>(S0 + (int64_t)u * e + c, sv);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float qq = ql[qrow[r] + u];
#pragma unroll
          for (int q = 0; q < CV; ++q) acc[r][q] = fmaf(qq, sv[q], acc[r][q]);
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float f = powi32(lam, ll, ib + sub + r * nsub + 1);
#pragma unroll
        for (int q = 0; q < CV; ++q) acc[r][q] *= f;
      }
      for (int j = 0; j < n; ++j) {                    // the chunk's own keys
        float vv[CV];
        ld_cols<CV>(vl + j * e + c, vv);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int i = ib + sub + r * nsub;
          const float pp = P[(i < n ? i : 0) * (LCH + 1) + j];
#pragma unroll
          for (int q = 0; q < CV; ++q) acc[r][q] = fmaf(pp, vv[q], acc[r][q]);
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int i = ib + sub + r * nsub;
        if (i >= n) continue;
#pragma unroll
        for (int q = 0; q < CV; ++q) a.out[(int64_t)(r0 + i) * a.ldo + (int64_t)h * e + c + q] = acc[r][q];
      }
    }
  }
}

// Pass 3 on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: fp32 operands and accumulation; operand layouts in mfma_f32_tiles.h).  A
// workgroup of 4 waves owns one (chunk, head): q, k (rows of ldq floats) and v (rows of ldv floats) of the chunk's <= 32 rows are staged
// activated and zero padded; waves 0 .. 2 multiply the three 16 x 16 score tiles on or below the diagonal and park them, decayed and
// masked, in LDS; then wave w owns the 16-column tiles w, w + 4, .. of the result, both row tiles at once: Q S0 with the carried state
// read straight from the workspace (8 loads in flight), times lam^(i + 1) by rows, plus P V.
__global__ __launch_bounds__(256) void light_scan_out_mfma_kernel(LightScanArgs s, int ldq, int ldv) {
  extern __shared__ float lds[];             // q [32][ldq], k [32][ldq], v [32][ldv], P [32][36]
  constexpr int LDP = 36;
  const LightArgs& a = s.b;
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, d = a.dim, e = a.vdim;
  const int r0 = s.chunk_tab[2 * ch], n = s.chunk_tab[2 * ch + 1];
  const int wave = tid >> 6, lane = tid & 63, c16 = lane & 15, g4 = lane >> 4;
  float* ql = lds;
  float* kl = ql + LCH * ldq;
  float* vl = kl + LCH * ldq;
  float* P = vl + LCH * ldv;
  const float lam = a.decay[h], ll = lam > 0.f ? logf(lam) : 0.f;
  for (int x = tid; x < LCH * ldq; x += 256) {
    const int j = x / ldq, i = x - j * ldq;
    float qv = 0.f, kv = 0.f;
    if (j < n && i < d) {
      const float* row = a.qkv + (int64_t)(r0 + j) * a.ldqkv + (int64_t)h * d + i;
      qv = silu32(row[0]);
      kv = silu32(row[(int64_t)a.H * d]);
    }
    ql[x] = qv;
    kl[x] = kv;
  }
  for (int x = tid; x < LCH * ldv; x += 256) {
    const int j = x / ldv, c = x - j * ldv;
    vl[x] = (j < n && c < e) ? silu32(a.qkv[(int64_t)(r0 + j) * a.ldqkv + (int64_t)2 * a.H * d + (int64_t)h * e + c]) : 0.f;
  }
  __syncthreads();
  const int ksteps = (d + 3) / 4;            // ldq >= 4 ksteps, the padding is zero
  if (wave < 3) {                            // score tiles (0, 0), (1, 0), (1, 1)
    const int ti = wave == 0 ? 0 : 1, tj = wave == 2 ? 1 : 0;
    f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f}, sc2 = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* ap = ql + (16 * ti + c16) * ldq + g4;
    const float* bp = kl + (16 * tj + c16) * ldq + g4;
    int it = 0;
    for (; it + 1 < ksteps; it += 2) {
      sc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[4 * it], bp[4 * it], sc, 0, 0, 0);
      sc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[4 * it + 4], bp[4 * it + 4], sc2, 0, 0, 0);
    }
    if (it < ksteps) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[4 * it], bp[4 * it], sc, 0, 0, 0);
    sc += sc2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * ti + 4 * g4 + i, col = 16 * tj + c16;
      P[row * LDP + col] = col <= row ? sc[i] * powi32(lam, ll, row - col) : 0.f;
    }
  } else {                                   // the tile above the diagonal
    for (int x = lane; x < 256; x += 64) P[(x >> 4) * LDP + 16 + (x & 15)] = 0.f;
  }
  __syncthreads();
  const float* S0 = s.ws + ((int64_t)ch * a.H + h) * d * e;
  float rowf[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) rowf[t][i] = powi32(lam, ll, 16 * t + 4 * g4 + i + 1);
  const int ntile = (e + 15) / 16;
  for (int ct = wave; ct < ntile; ct += 4) {
    const int col = 16 * ct + c16;
    const bool col_ok = col < e;
    const float* sp = S0 + (col_ok ? col : 0);
    f32x4 acc0 = f32x4{0.f, 0.f, 0.f, 0.f}, acc1 = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* a0 = ql + c16 * ldq + g4;
    const float* a1 = ql + (16 + c16) * ldq + g4;
    for (int it0 = 0; it0 < ksteps; it0 += 8) {
      float b[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = 4 * (it0 + u) + g4;
        const float t = sp[(int64_t)(k < d ? k : 0) * e];
        b[u] = (col_ok && k < d) ? t : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (it0 + u < ksteps) {
          acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[4 * (it0 + u)], b[u], acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[4 * (it0 + u)], b[u], acc1, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) { acc0[i] *= rowf[0][i]; acc1[i] *= rowf[1][i]; }
    const float* p0 = P + c16 * LDP + g4;
    const float* p1 = P + (16 + c16) * LDP + g4;
    const float* vb = vl + g4 * ldv + 16 * ct + c16;
#pragma unroll
    for (int it = 0; it < LCH / 4; ++it) {
      const float bv = vb[4 * it * ldv];
      if (it < 4) acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(p0[4 * it], bv, acc0, 0, 0, 0);      // row tile 0 sees keys 0 .. 15 only
      acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(p1[4 * it], bv, acc1, 0, 0, 0);
    }
    if (col_ok) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ra = 4 * g4 + i, rb = 16 + ra;
        if (ra < n) a.out[(int64_t)(r0 + ra) * a.ldo + (int64_t)h * e + col] = acc0[i];
        if (rb < n) a.out[(int64_t)(r0 + rb) * a.ldo + (int64_t)h * e + col] = acc1[i];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------------
// one workgroup per row: y = x / sqrt(mean(x^2) + eps) * w * sigmoid(g)
__global__ __launch_bounds__(256) void rms_sigmoid_gate_kernel(const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, float eps,
                                                               const float* __restrict__ g, int64_t ldg, float* __restrict__ y, int64_t ldy,
                                                               bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (int64_t)m * ldx;
  float ss = 0.f;
  for (int i = tid; i < n; i += 256) ss += xr[i] * xr[i];
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)n + eps);
  for (int i = tid; i < n; i += 256) {
    const float o = xr[i] * r * bf16_to_f32(w[i]) * sigm32(g[(int64_t)m * ldg + i]);
    if (y) y[(int64_t)m * ldy + i] = o;
    if (y16) y16[(int64_t)m * ldy16 + i] = f32_to_bf16(o);
  }
}

__global__ __launch_bounds__(256) void relu2_kernel(const float* __restrict__ x, int64_t ldx, float* __restrict__ y, int64_t ldy,
                                                    bf16_t* __restrict__ y16, int64_t ldy16, int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const float t = fmaxf(x[(int64_t)m * ldx + c], 0.f), o = t * t;
  if (y) y[(int64_t)m * ldy + c] = o;
  if (y16) y16[(int64_t)m * ldy16 + c] = f32_to_bf16(o);
}

// ---------------------------------------------------------------------------------------------------------------------------
// Router, one wave per row (n <= 512 outputs, 8 per lane): s = softmax(logits) over all n; the `top` largest of s + correction (ties: the
// lower index); weights = their s / (sum of their s + 1e-20).  Outputs at or past n_real stand for "pass the input through": every
// such pick is written as index n_real.  With relu_x the launch's other workgroups write relu(x)^2 of the same rows.
struct RouterArgs {
  const float* logits; int64_t ld;
  int M, n, n_real, top;
  const float* corr;
  int32_t* idx; float* w;
  const float* rx; int64_t ldrx; float* ry; int64_t ldry; int rn;
};

__global__ __launch_bounds__(256) void router_softmax_topk_kernel(RouterArgs a) {
  const int nrb = (a.M + 3) / 4;
  if ((int)blockIdx.x >= nrb) {               // the activation riding this launch
    const int e = ((int)blockIdx.x - nrb) * 256 + threadIdx.x;
    if (e >= a.M * a.rn) return;
    const int m = e / a.rn, c = e - m * a.rn;
    const float t = fmaxf(a.rx[(int64_t)m * a.ldrx + c], 0.f);
    a.ry[(int64_t)m * a.ldry + c] = t * t;
    return;
  }
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (m >= a.M) return;
  const float* z = a.logits + (int64_t)m * a.ld;
  float s[8], ch[8];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = lane + 64 * j;
    s[j] = i < a.n ? z[i] : -INFINITY;
    mx = fmaxf(mx, s[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    s[j] = (lane + 64 * j) < a.n ? expf(s[j] - mx) : 0.f;
    sum += s[j];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = lane + 64 * j;
    s[j] = s[j] / sum;
    ch[j] = i < a.n ? s[j] + (a.corr ? a.corr[i] : 0.f) : -INFINITY;
  }
  float wsum = 0.f, mine = 0.f;
  int mine_i = 0;
  for (int t = 0; t < a.top; ++t) {
    float bv = -INFINITY; int bi = 0x7fffffff; float bs = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = lane + 64 * j;
      if (ch[j] > bv) { bv = ch[j]; bi = i; bs = s[j]; }      // ascending i within a lane: the first of equals stays
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(bi, o);
      const float os = __shfl_xor(bs, o);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; bs = os; }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (lane + 64 * j == bi) ch[j] = -INFINITY;
    wsum += bs;
    if (lane == t % 64) { mine = bs; mine_i = bi; }
    if (t % 64 == 63 || t == a.top - 1) {                      // lanes 0 .. t % 64 hold the picks 64 (t / 64) ..
      // weights need the whole sum: park them until the last pick
      if (lane <= t % 64) { a.idx[(int64_t)m * a.top + (t / 64) * 64 + lane] = mine_i < a.n_real ? mine_i : a.n_real; a.w[(int64_t)m * a.top + (t / 64) * 64 + lane] = mine; }
    }
  }
  __builtin_amdgcn_wave_barrier();
  const float inv = 1.0f / (wsum + 1e-20f);
  for (int t = lane; t < a.top; t += 64) a.w[(int64_t)m * a.top + t] *= inv;
}

// x[m] += add[m] + sum_j w[m, j] * (idx[m, j] < n_real ? y[r(m, j)] : h[m])
__global__ __launch_bounds__(256) void moe_combine_pass_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y, int64_t ldy,
                                                               const int32_t* __restrict__ slot_of, const int32_t* __restrict__ idx,
                                                               const float* __restrict__ w, int top, int n_real, const float* __restrict__ h,
                                                               int64_t ldh, const float* __restrict__ add, int64_t ldadd, int n) {
  const int m = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  float acc = 0.f, pass = 0.f;
  for (int j = 0; j < top; ++j) {
    const int z = m * top + j;
    if (idx[z] < n_real) {
      const int64_t r = slot_of ? slot_of[z] : z;
      acc = fmaf(w[z], y[r * ldy + c], acc);
    } else {
      pass += w[z];
    }
  }
  if (pass != 0.f) acc = fmaf(pass, h[(int64_t)m * ldh + c], acc);
  if (add) acc += add[(int64_t)m * ldadd + c];
  x[(int64_t)m * ldx + c] += acc;
}

}  // namespace

extern "C" int mn_head_norm_temp_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* q_norm,
                                        const uint16_t* k_norm, float eps, float q_scale, float temp_coef, int temp_every,
                                        const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena,
                                        float* v_arena, int t_max, void* stream) {
  MN_CHECK_ARG(qkv && row_seq && row_slot && q_out && k_arena && v_arena && M >= 1 && M <= 65535 && H >= 1 && G >= 1 && dim >= 1 && dim <= 512 &&
                   vdim >= 1 && t_max >= 1, "mn_head_norm_temp_append: bad args (dim=%d: at most 512)", dim);
  HeadNormArgs a{qkv, ldqkv, H, G, dim, vdim, q_norm, k_norm, eps, q_scale, temp_coef, temp_every, row_seq, row_slot, q_out, ldq, k_arena, v_arena,
                 t_max};
  hipLaunchKernelGGL(head_norm_temp_append_kernel, dim3((unsigned)mn_cdiv(H + 2 * G, 4), (unsigned)M), dim3(256), 0, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_head_norm_temp_append");
  return MN_OK;
}

extern "C" int mn_lightning_rows(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                                 const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, int flags, float* out, int64_t ldo,
                                 void* stream) {
  const bool distinct = (flags & MN_SEQ_ROWS_DISTINCT) != 0;
  MN_CHECK_ARG(qkv && decay && state && row_seq && row_slot && (row_back || distinct) && out && M >= 1 && M <= 65535 && H >= 1 && H <= 65535 &&
                   dim >= 1 && dim <= 4096 && vdim >= 1, "mn_lightning_rows: bad args");
  LightArgs a{qkv, ldqkv, H, dim, vdim, decay, state, row_seq, row_slot, row_back, out, ldo, M};
  hipStream_t st = mn_stream(stream);
  if (distinct) {
    MN_CHECK_ARG(mn_cdiv(vdim, 32) <= 65535, "mn_lightning_rows: vdim=%d too large", vdim);
    hipLaunchKernelGGL(lightning_step_kernel, dim3((unsigned)M, (unsigned)H, (unsigned)mn_cdiv(vdim, 32)), dim3(256),
                       ((size_t)2 * dim + 256) * sizeof(float), st, a);
    MN_CHECK_LAUNCH("mn_lightning_rows(step)");
    return MN_OK;
  }
  const dim3 grid((unsigned)M, (unsigned)H, (unsigned)mn_cdiv(vdim, 256));
  const size_t lds = (size_t)4 * dim * sizeof(float);
  if (dim <= 32) hipLaunchKernelGGL((lightning_rows_kernel<1>), grid, dim3(256), lds, st, a);
  else if (dim <= 64) hipLaunchKernelGGL((lightning_rows_kernel<2>), grid, dim3(256), lds, st, a);
  else if (dim <= 128) hipLaunchKernelGGL((lightning_rows_kernel<4>), grid, dim3(256), lds, st, a);
  else if (dim <= 256) hipLaunchKernelGGL((lightning_rows_kernel<8>), grid, dim3(256), lds, st, a);
  else hipLaunchKernelGGL((lightning_rows_kernel<0>), grid, dim3(256), lds, st, a);
  MN_CHECK_LAUNCH("mn_lightning_rows");
  return MN_OK;
}

extern "C" int mn_lightning_chunk_rows(void) { return LCH; }

// LDS of the scan's output pass: q and k rows of dim + 1 floats, value rows, the chunk's decayed scores
extern "C" size_t mn_lightning_scan_lds_bytes(int dim, int vdim) {
  return ((size_t)LCH * (2 * (dim + 1) + vdim) + 4 + (size_t)LCH * (LCH + 1)) * sizeof(float);
}

extern "C" size_t mn_lightning_scan_workspace_bytes(int n_chunks, int H, int dim, int vdim) {
  if (n_chunks < 1 || H < 1 || dim < 1 || vdim < 1) return 0;
  return (size_t)n_chunks * H * dim * vdim * sizeof(float);
}

namespace {
// row strides of the matrix-core pass: q / k rows = 4 mod 32 floats, v rows = 16 mod 32 — the operand reads of a wave then fall two to a bank
inline int scan_ldq(int dim) { const int p = (dim + 3) / 4 * 4; return p + ((p % 32) == 0 ? 4 : ((36 - p % 32) % 32)); }
inline int scan_ldv(int vdim) { const int p = (vdim + 15) / 16 * 16; return p + ((p % 32) == 0 ? 16 : 0); }
inline size_t scan_mfma_lds(int dim, int vdim) { return ((size_t)LCH * (2 * scan_ldq(dim) + scan_ldv(vdim)) + LCH * 36) * sizeof(float); }
}  // namespace

extern "C" int mn_lightning_rows_scan(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                                      const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* chunk_tab,
                                      int n_chunks, float* out, int64_t ldo, void* workspace, size_t workspace_bytes, void* stream) {
  return mn_lightning_rows_scan_ex(qkv, ldqkv, M, H, dim, vdim, decay, state, row_seq, row_slot, row_back, chunk_tab, n_chunks, out, ldo, workspace,
                                   workspace_bytes, scan_mfma_lds(dim, vdim) <= 64 * 1024 ? MN_LIGHTNING_SCAN_MFMA : MN_LIGHTNING_SCAN_VALU, stream);
}

extern "C" int mn_lightning_rows_scan_ex(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                                         const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* chunk_tab,
                                         int n_chunks, float* out, int64_t ldo, void* workspace, size_t workspace_bytes, int variant,
                                         void* stream) {
  MN_CHECK_ARG(qkv && decay && state && row_seq && row_slot && row_back && chunk_tab && out && workspace && M >= 1 && H >= 1 && H <= 65535 &&
                   dim >= 1 && vdim >= 1 && n_chunks >= 1 && n_chunks <= 65535, "mn_lightning_rows_scan: bad args");
  MN_CHECK_ARG(workspace_bytes >= mn_lightning_scan_workspace_bytes(n_chunks, H, dim, vdim), "mn_lightning_rows_scan: workspace too small");
  MN_CHECK_ARG(variant == MN_LIGHTNING_SCAN_MFMA || variant == MN_LIGHTNING_SCAN_VALU, "mn_lightning_rows_scan: unknown variant %d", variant);
  const size_t lds3 = mn_lightning_scan_lds_bytes(dim, vdim);
  MN_CHECK_ARG(lds3 <= 64 * 1024, "mn_lightning_rows_scan: heads of %d + %d values do not fit (use mn_lightning_rows)", dim, vdim);
  LightScanArgs s{LightArgs{qkv, ldqkv, H, dim, vdim, decay, state, row_seq, row_slot, row_back, out, ldo, M}, chunk_tab, n_chunks, (float*)workspace};
  hipStream_t st = mn_stream(stream);
  // four value columns per thread where rows of values and of the state are 16-byte aligned
  const bool v4 = (vdim % 4) == 0 && (((uintptr_t)workspace) & 15) == 0;
  if (v4) hipLaunchKernelGGL((light_scan_kv_kernel<4>), dim3((unsigned)n_chunks, (unsigned)H), dim3(256), (size_t)LCH * (dim + vdim) * sizeof(float), st, s);
  else hipLaunchKernelGGL((light_scan_kv_kernel<1>), dim3((unsigned)n_chunks, (unsigned)H), dim3(256), (size_t)LCH * (dim + vdim) * sizeof(float), st, s);
  MN_CHECK_LAUNCH("mn_lightning_rows_scan(sums)");
  hipLaunchKernelGGL(light_scan_carry_kernel, dim3((unsigned)mn_cdiv((int64_t)dim * vdim, 256), (unsigned)H, (unsigned)n_chunks), dim3(256), 0, st, s);
  MN_CHECK_LAUNCH("mn_lightning_rows_scan(carry)");
  if (variant == MN_LIGHTNING_SCAN_MFMA) {
    MN_CHECK_ARG(scan_mfma_lds(dim, vdim) <= 64 * 1024, "mn_lightning_rows_scan: heads of %d + %d values do not fit the matrix-core pass", dim, vdim);
    hipLaunchKernelGGL(light_scan_out_mfma_kernel, dim3((unsigned)n_chunks, (unsigned)H), dim3(256), scan_mfma_lds(dim, vdim), st, s, scan_ldq(dim),
                       scan_ldv(vdim));
  } else if (v4) hipLaunchKernelGGL((light_scan_out_kernel<4>), dim3((unsigned)n_chunks, (unsigned)H), dim3(256), lds3, st, s);
  else hipLaunchKernelGGL((light_scan_out_kernel<1>), dim3((unsigned)n_chunks, (unsigned)H), dim3(256), lds3, st, s);
  MN_CHECK_LAUNCH("mn_lightning_rows_scan(outputs)");
  return MN_OK;
}

extern "C" int mn_rms_sigmoid_gate_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, const float* g, int64_t ldg, float* y,
                                        int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && w && g && (y || y16) && M >= 1 && n >= 1, "mn_rms_sigmoid_gate_rows: bad args");
  hipLaunchKernelGGL(rms_sigmoid_gate_kernel, dim3((unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, w, eps, g, ldg, y, ldy, y16, ldy16, n);
  MN_CHECK_LAUNCH("mn_rms_sigmoid_gate_rows");
  return MN_OK;
}

extern "C" int mn_relu2_rows(const float* x, int64_t ldx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream) {
  MN_CHECK_ARG(x && (y || y16) && M >= 1 && M <= 65535 && n >= 1, "mn_relu2_rows: bad args");
  hipLaunchKernelGGL(relu2_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, y, ldy, y16, ldy16, n);
  MN_CHECK_LAUNCH("mn_relu2_rows");
  return MN_OK;
}

extern "C" int mn_router_softmax_topk_rows(const float* logits, int64_t ld, int M, int n, int n_real, int top, const float* correction,
                                           int32_t* idx, float* w, const float* relu_x, int64_t ldrx, float* relu_y, int64_t ldry, int relu_n,
                                           void* stream) {
  MN_CHECK_ARG(logits && idx && w && M >= 1 && n >= 1 && n <= 512 && n_real >= 0 && n_real <= n && top >= 1 && top <= n,
               "mn_router_softmax_topk_rows: bad args (n=%d: at most 512 outputs)", n);
  MN_CHECK_ARG(relu_n == 0 || (relu_x && relu_y && relu_n > 0), "mn_router_softmax_topk_rows: the activation needs its rows");
  RouterArgs a{logits, ld, M, n, n_real, top, correction, idx, w, relu_x, ldrx, relu_y, ldry, relu_n};
  const int64_t blocks = mn_cdiv(M, 4) + (relu_n > 0 ? mn_cdiv((int64_t)M * relu_n, 256) : 0);
  hipLaunchKernelGGL(router_softmax_topk_kernel, dim3((unsigned)blocks), dim3(256), 0, mn_stream(stream), a);
  MN_CHECK_LAUNCH("mn_router_softmax_topk_rows");
  return MN_OK;
}

extern "C" int mn_moe_combine_pass_residual(float* x, int64_t ldx, const float* y, int64_t ldy, const int32_t* slot_of, const int32_t* idx,
                                            const float* w, int top, int n_real, const float* h, int64_t ldh, const float* add, int64_t ldadd,
                                            int M, int n, void* stream) {
  MN_CHECK_ARG(x && y && idx && w && h && top >= 1 && M >= 1 && M <= 65535 && n >= 1, "mn_moe_combine_pass_residual: bad args");
  hipLaunchKernelGGL(moe_combine_pass_kernel, dim3((unsigned)mn_cdiv(n, 256), (unsigned)M), dim3(256), 0, mn_stream(stream), x, ldx, y, ldy,
                     slot_of, idx, w, top, n_real, h, ldh, add, ldadd, n);
  MN_CHECK_LAUNCH("mn_moe_combine_pass_residual");
  return MN_OK;
}
