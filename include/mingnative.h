/*
 * mingnative.h — C ABI of libmingnative.so: the MI355X (gfx950) native hot path of
 * Ming-UniVision (MingTok-Vision tokenizer -> Bailing-MoE next-token forward ->
 * rectified-flow SwiGLU head -> MingTok decode).
 *
 * The reference has no FFI: the path is PyTorch module calls that dispatch into
 * third-party GPU kernels (cuBLAS/cuDNN/flash-attn).  Every entry
 * point below replaces one of those call sites; the reference file:line is cited
 * per function (paths relative to the reference repo root).
 *
 * Conventions
 *   - extern "C", plain pointers and sizes, no torch types.
 *   - All pointers are DEVICE pointers unless the name ends in _host.
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream).
 *   - Launchers never allocate, never synchronise, never throw: they enqueue work
 *     on `stream` and return 0, or a negative MN_E* code (see mn_last_error()).
 *   - Weights are bf16 (uint16_t bit patterns) in the reference's nn.Linear layout
 *     [out_features, in_features] row-major unless stated.  Small-row ("decode")
 *     activations are fp32; batched (MFMA) activations are bf16 with fp32 accumulate.
 */
#ifndef MINGNATIVE_H
#define MINGNATIVE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MN_VERSION 129 /* 0.1.29: post-norm mixed-mixer sequence models (section 12).  0.1.28: hybrid-mixer sequence models (section 11).  0.1.27: parallel-mixer sequence models (section 10).  0.1.26: latent-cache sequence models (section 9).  0.1.24: mn_persist_set_status_word; mn_tp_allreduce PUSH|REDUCE above the one-shot row limit implies GATHER.  0.1.23: ABI guards mn_sizeof_* / mn_struct_layout.  0.1.20: fp8 weight mode (section 7): wfmt / row-scale fields at the END of mn_skinny_args, mn_rf_head,
                          mn_llm and mn_llm_tp (zero = bf16: callers of 0.1.10 that zero-fill the structs are unchanged),
                          mn_quant_fp8_rows / mn_dequant_fp8_rows / mn_stream_mfma_w8 / mn_stream_mfma_grouped_w8 */

/* Only the entry points declared here are exported (the library is built with -fvisibility=hidden; tests/test_host_logic.py
 * holds `nm -D` to exactly this list).  The launchers keep no mutable process state: launch plans are pure functions of the
 * arguments, so calls are re-entrant per stream.  The A/B hooks of tools/ live in libmingnative_dev.so (mingnative_dev.h). */
#if defined(__GNUC__)
#define MN_API __attribute__((visibility("default")))
#else
#define MN_API
#endif

enum {
  MN_OK = 0,
  MN_EINVAL = -1,   /* bad argument (shape / alignment / enum) */
  MN_ELAUNCH = -2,  /* hip launch failure, see mn_last_error() */
  MN_ENOSPACE = -3  /* workspace too small */
};

MN_API int mn_version(void);
MN_API const char* mn_last_error(void);
/* Number of compute units of the current device (host query, cached). */
MN_API int mn_num_cus(void);

/* ABI guards (round 5): the binding side (ctypes Structures, cgo / JNI struct mirrors) can check that its layout of every struct
 * below is the library's — a field added on one side only would otherwise corrupt calls silently.  mn_sizeof_* = sizeof(the struct);
 * mn_struct_layout(which, offsets, cap) writes offsetof(every field, in declaration order) into offsets[0 .. min(n, cap)) and
 * returns the field count n (MN_EINVAL for an unknown `which`). */
enum mn_struct_id { MN_STRUCT_SKINNY_ARGS = 0, MN_STRUCT_RF_HEAD = 1, MN_STRUCT_LLM = 2, MN_STRUCT_SEMDEC = 3, MN_STRUCT_TP_COMM = 4,
                    MN_STRUCT_LLM_TP = 5, MN_STRUCT_SEQ_LAYER = 6, MN_STRUCT_SEQ_MODEL = 7, MN_STRUCT_SEQ_STATE = 8,
                    MN_STRUCT_PMIX_LAYER = 9, MN_STRUCT_PMIX_MODEL = 10, MN_STRUCT_PMIX_STATE = 11 };
MN_API size_t mn_sizeof_skinny_args(void);
MN_API size_t mn_sizeof_rf_head(void);
MN_API size_t mn_sizeof_llm(void);
MN_API size_t mn_sizeof_semdec(void);
MN_API size_t mn_sizeof_tp_comm(void);
MN_API size_t mn_sizeof_llm_tp(void);
MN_API int mn_struct_layout(int which, size_t* offsets, int cap);

/* ------------------------------------------------------------------------------------------
 * 1. Skinny GEMM (M <= 8 rows): out = epilogue( prologue(x) @ W^T + bias )
 *    Weight-streaming, HBM-bound.  Replaces every nn.Linear call with <= 8 rows on the
 *    decode path: modeling_bailing_moe.py:760,824 (query_key_value / dense), :483-484
 *    (expert / shared-expert MLPs), :1551 (lm_head), :1571-1574 (vis_head);
 *    diff_loss_rf_swiglu.py:27-34,194-198,263-266,282-286,324-326 (RF head);
 *    mingtok layers/attention.py:49-51, layers/swiglu_ffn.py:27-28 (semantic-decoder decode step);
 *    modeling_bailingmm.py:111-115 (linear_proj).
 * ------------------------------------------------------------------------------------------ */
enum mn_prologue {
  MN_PRO_NONE = 0,
  MN_PRO_SILU = 1,      /* x' = silu(x) */
  MN_PRO_ADD_SILU = 2,  /* x' = silu(x + pro_a)          (adaLN input SiLU(t_emb + c), diff_loss_rf_swiglu.py:263-266,376) */
  MN_PRO_RMSNORM = 3,   /* x' = x * rsqrt(mean(x^2)+eps) * ln_g   (BailingMoeRMSNorm, modeling_bailing_moe.py:131-136) */
  MN_PRO_LN = 4,        /* x' = LayerNorm(x; ln_g, ln_b, eps)     (nn.LayerNorm eps=1e-6) */
  MN_PRO_LN_MOD = 5     /* x' = LayerNorm(x; ln_g?, ln_b?, eps) * (1 + pro_b) + pro_a   (modulate, diff_loss_rf_swiglu.py:184-185,270,290) */
};
enum mn_epilogue {
  MN_EPI_NONE = 0,
  MN_EPI_SILU = 1,
  MN_EPI_GELU = 2,        /* exact erf GELU (nn.GELU default) */
  MN_EPI_SWIGLU = 3,      /* out[n] = silu(y[n]) * y[n + N]; W and bias hold 2N rows (chunk(2), swiglu_ffn.py:30-34) */
  MN_EPI_RESID = 4,       /* out = res + y */
  MN_EPI_RESID_GATE = 5,  /* out = res + gate * y   (ResBlock, diff_loss_rf_swiglu.py:272) */
  MN_EPI_GEGLU_TANH = 6   /* out[n] = gelu_tanh(y[n]) * y[n + N], gelu in its tanh form; W and bias hold 2N rows like MN_EPI_SWIGLU (bf16 weights only) */
};

typedef struct mn_skinny_args {
  const float* x;      int64_t ldx;    /* [M, K] fp32 (per batch entry) */
  const uint16_t* w;   int64_t ldw;    /* bf16 [N or 2N, K]; row stride ldw elements */
  const uint16_t* bias;                /* bf16 [N or 2N] or NULL */
  float* out;          int64_t ldo;    /* [M, N] fp32 */
  int32_t M, N, K;                     /* 1 <= M <= 8; K % 8 == 0 (K is per segment when nseg > 1) */
  int32_t prologue, epilogue;
  const float* pro_a;  int64_t ld_pro_a; /* ADD_SILU: addend [K] (ld 0) or [M,K]; LN_MOD: shift [M,K] */
  const float* pro_b;  int64_t ld_pro_b; /* LN_MOD: scale [M,K] */
  const uint16_t* ln_g; const uint16_t* ln_b; /* bf16 [K] norm gain / bias (NULL = none) */
  float eps;
  const float* res;    int64_t ldres;  /* RESID / RESID_GATE */
  const float* gate;   int64_t ldgate; /* RESID_GATE */
  /* Batching over independent problems that differ in weights (MoE experts):
   * entry b uses W + w_index[b]*w_batch_stride (w_index NULL -> b), x + (b / x_batch_div)*x_batch_stride,
   * out + b*out_batch_stride, res + b*res_batch_stride.  batch <= 0 means 1. */
  int32_t batch; const int32_t* w_index; int64_t w_batch_stride;
  int64_t x_batch_stride; int32_t x_batch_div; int64_t out_batch_stride; int64_t res_batch_stride;
  /* K-segments (MoE down-projection summed over the experts of one token):
   * y = sum_s seg_scale[b*nseg+s] * x[:, s*K:(s+1)*K] @ W[seg_index[b*nseg+s]]^T ; nseg <= 0 means 1. */
  int32_t nseg; const int32_t* seg_index; const float* seg_scale; int64_t seg_w_stride;
  /* Scratch for the matrix-core route (M >= 5, batched generation): such launches run as prologue (activations
   * split into bf16 hi + lo) -> weight-streaming MFMA kernel over K slices -> reduce + epilogue, and need
   * mn_skinny_workspace_bytes(M, N, K, epilogue) bytes.  May be NULL for M <= 8 (fp32-FMA kernel is used). */
  void* ws; size_t ws_bytes;
  /* fp8 weights (section 7): wfmt = MN_W_FP8_E4M3 -> `w` points to e4m3 bytes [N or 2N, K] (K % 16 == 0; strides count bytes) and
   * wscale to one fp32 scale per weight row.  M == 1 with prologue NONE and epilogue NONE / SWIGLU / RESID — the expert launches of a
   * 1- or 2-row decode step, batch and K-segment forms included — runs the one-row fp8 kernel (skinny_w8.hip): batch entry b reads its
   * scales at wscale + w_index[b] * wscale_batch_stride, segment s at + seg_index[s] * wscale_seg_stride.  Everything else (1..64
   * rows, dense weights with ldw == K, no batch / segments) takes the matrix-core route and needs ws (mn_skinny_workspace_bytes_w8). */
  int32_t wfmt; const float* wscale; int64_t wscale_batch_stride; int64_t wscale_seg_stride;
} mn_skinny_args;

/* 1 <= M <= 64 (batch / nseg forms: M <= 8). */
MN_API int mn_skinny_gemm(const mn_skinny_args* args, void* stream);
MN_API size_t mn_skinny_workspace_bytes(int M, int N, int K, int epilogue);
MN_API size_t mn_skinny_workspace_bytes_w8(int M, int N, int K, int epilogue);
MN_API size_t mn_skinny_workspace_bytes_wq(int wfmt, int M, int N, int K, int epilogue);   /* any weight format (section 7) */

/* ------------------------------------------------------------------------------------------
 * 2. MoE router: RMSNorm + gate GEMV + fp32 softmax + top-k + renormalise, with the
 *    image-gate override on rows flagged by image_mask.
 *    Replaces BailingMoeGate.forward (modeling_bailing_moe.py:505-520) and the multi-gate blend
 *    of BailingMoeSparseMoeBlock.forward (:565-592).  M <= 64, num_experts <= 64.
 *      x [M,H] fp32 (pre-norm residual stream), norm_w bf16 [H]
 *      gate_w / image_gate_w bf16 [E,H]; image_mask uint8 [M] or NULL
 *      -> x_norm [M,H] fp32 (the normalised rows, input of the experts)
 *         topk_idx int32 [M, n_slot], topk_w fp32 [M, n_slot] where
 *         n_slot = top_k + n_shared_slots; the trailing shared slots are filled with
 *         (E + j, 1.0) so that shared experts ride the same grouped GEMV.
 * ------------------------------------------------------------------------------------------ */
MN_API int mn_moe_router(const float* x, int64_t ldx, const uint16_t* norm_w, float eps,
                  const uint16_t* gate_w, const uint16_t* image_gate_w, const uint8_t* image_mask,
                  int M, int H, int E, int top_k, int norm_topk_prob, int n_shared_slots,
                  float* x_norm, int32_t* topk_idx, float* topk_w, float* logits_ws /* [2*M*E] scratch */,
                  void* ws, size_t ws_bytes /* optional: mn_skinny_workspace_bytes(M, E, H, 0) enables the MFMA route */,
                  void* stream);

/* ------------------------------------------------------------------------------------------
 * 3. RoPE + KV-cache append, and masked GQA / MHA decode attention.
 *    Replaces apply_rotary_pos_emb + DynamicCache.update + the eager/flash attention of
 *    BailingMoeAttention.forward (modeling_bailing_moe.py:428-461, 768-812) and, with
 *    rope = 0, CausalAttention.forward + cache (mingtok layers/attention.py:138-163).
 *
 *    KV cache layout: fp32 [n_seq][2 (k,v)][n_kv_heads][t_max][head_dim].
 *    qkv [M, (n_q + 2 n_kv) * hd] fp32, heads ordered q.., k.., v.. (qkv.split, :762-764); the ViT
 *    layout [3][n_heads][hd] (attention.py:140) is the same ordering with n_q == n_kv.
 *    row_seq[m]: cache sequence of row m; row_slot[m]: cache slot to write; row_pos[m]: rotary
 *    position (cumsum(mask)-1, :1905).  cos/sin tables fp32 [n_pos, hd/2].
 *    q_out [M, n_q*hd] fp32 receives rotated (and scaled by q_scale) queries.
 *    A row whose slot is outside [0, t_max) writes no K / V (the Python surface raises before a cache fills up; the kernel
 *    never stores outside the sequence's rows of the arena).
 * ------------------------------------------------------------------------------------------ */
MN_API int mn_rope_kv_append(const float* qkv, int64_t ldqkv, int M, int n_q, int n_kv, int hd,
                      int rope, const float* cos_tab, const float* sin_tab,
                      const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_pos,
                      float q_scale, float* q_out, float* kv_cache, int64_t t_max, void* stream);
/*    3D rotary variant (BailingMoe3DRotaryEmbedding :413-425 + apply_multimodal_rotary_pos_emb :463-469, the
 *    `rope_scaling.type == "3D"` branch at :780-782): row_pos is [3][M] = temporal, height, width positions; rotary
 *    frequency i (of each half of the head) follows the t stream for i < sec_t, the h stream for the next sec_h, the
 *    w stream for the rest (mrope_section [16, 24, 24] at hd = 128).  sec_t == 0 is the Legacy rotary above.  With
 *    equal t/h/w positions the result is bit-identical to Legacy. */
MN_API int mn_rope_kv_append_3d(const float* qkv, int64_t ldqkv, int M, int n_q, int n_kv, int hd,
                         int rope, const float* cos_tab, const float* sin_tab,
                         const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_pos, int sec_t, int sec_h,
                         float q_scale, float* q_out, float* kv_cache, int64_t t_max, void* stream);

/*    out[m] = softmax(q[m] . K[seq]^T + mask) V[seq] over keys j < row_len[m] with
 *    key_mask[m*ld_mask + j] != 0 (key_mask NULL = all ones).  A row with every key masked gets the mean of V over its keys
 *    [0, row_len): what the reference's additive finfo.min mask degenerates to (uniform softmax, modeling_bailing_moe.py:1466).
 *    q is pre-scaled.  out [M, n_q*hd] fp32.  The key range is split over workgroups
 *    (flash-decoding); workspace holds the per-split partials. */
MN_API size_t mn_attn_decode_workspace_bytes(int M, int n_q, int hd, int64_t t_max);
MN_API int mn_attn_decode(const float* q, int M, int n_q, int n_kv, int hd, const float* kv_cache, int64_t t_max,
                   const int32_t* row_seq, const int32_t* row_len, const uint8_t* key_mask, int64_t ld_mask,
                   float* out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * 4. Batched (MFMA) path: bf16 GEMM with fused epilogues, LayerNorm, flash attention hd=64.
 *    Replaces nn.Linear / nn.LayerNorm / flash_attn_func in the MingTok ViT blocks
 *    (layers/block.py:80-105, layers/attention.py:78-108,213-239, layers/mlp.py:34-40,
 *    layers/swiglu_ffn.py:30-34) and the step-invariant adaLN GEMM of the RF head.
 * ------------------------------------------------------------------------------------------ */
enum mn_gemm_epilogue {
  MN_GEMM_BF16 = 0,        /* C bf16 = A W^T + bias */
  MN_GEMM_BF16_GELU = 1,   /* C bf16 = gelu(A W^T + bias) */
  MN_GEMM_F32 = 2,         /* C fp32 = A W^T + bias */
  MN_GEMM_F32_RESID = 3    /* C fp32 += A W^T + bias   (residual stream accumulate) */
};
/* A bf16 [M,K] (lda), W bf16 [N,K] (ldw), bias bf16 [N] or NULL, C [M,N] (ldc). K % 32 == 0. */
MN_API int mn_gemm_bf16(const uint16_t* A, int64_t lda, const uint16_t* W, int64_t ldw, const uint16_t* bias,
                 void* C, int64_t ldc, int M, int N, int K, int epilogue, void* stream);

/* Split-K form for few-row weight-streaming problems: slice z of the K range writes partials[z][M][N] (fp32);
 * returns the number of slices used (>= 1) or a negative error. */
MN_API int mn_gemm_bf16_splitk(const uint16_t* A, int64_t lda, const uint16_t* W, int64_t ldw, float* partials,
                        int M, int N, int K, int ksplit, void* stream);

/* ---- many-token (prefill) operators of the Bailing-MoE decoder, bf16 MFMA path -------------------------------
 * Replace, for q_len > 16: BailingMoeRMSNorm (modeling_bailing_moe.py:131-136), apply_rotary_pos_emb +
 * DynamicCache.update (:428-461, :789), the flash-attn varlen prefill (:946-1007), BailingMoeGate (:505-520) and
 * moe_infer's argsort / per-expert loop / un-permute / weighted sum (:608-639). */
MN_API int mn_rmsnorm_bf16(const float* x, int64_t ldx, const uint16_t* g, float eps, uint16_t* y, int64_t ldy, int M, int D,
                    void* stream);
/* qkv fp32 [T, (n_q + 2 n_kv) hd]; token t gets rotary position pos[t] and cache slot slot0 + t of ONE sequence:
 * kv_seq fp32 [2][n_kv][t_max][hd].  q_out bf16 [T, n_q, hd] (rotated, scaled). */
MN_API int mn_rope_kv_prefill(const float* qkv, int64_t ldqkv, int T, int n_q, int n_kv, int hd, const float* cos_tab,
                       const float* sin_tab, const int32_t* pos, int slot0, float q_scale, uint16_t* q_out,
                       float* kv_seq, int64_t t_max, void* stream);
/* Flash attention, head_dim 128, GQA: query i of the T new tokens attends keys j <= past + i with
 * key_mask[j] != 0 (NULL = all).  Keys/values come from the fp32 arena of the sequence.  out bf16 [T, n_q*128]. */
MN_API int mn_attn_prefill_gqa_hd128(const uint16_t* q, const float* kv_seq, int64_t t_max, int n_q, int n_kv, int past, int T,
                              const uint8_t* key_mask, uint16_t* out, void* stream);
/* top-k routing from precomputed gate logits [T, E] (image-gate logits chosen where image_mask is set). */
MN_API int mn_moe_topk_logits(const float* logits_text, const float* logits_image, const uint8_t* image_mask, int T, int E,
                       int top_k, int norm_topk_prob, int n_shared_slots, int32_t* topk_idx, float* topk_w, void* stream);
/* Expert-sort of the (token, pick) pairs: counts[g], offsets[g+1], perm[sorted pos] = token,
 * slot_of[token * n_slot + pick] = sorted pos.  T * n_slot <= 65536, n_groups <= 128.  All device arrays. */
MN_API int mn_moe_sort(const int32_t* topk_idx, int T, int n_slot, int n_groups, int32_t* counts, int32_t* offsets,
                int32_t* perm, int32_t* slot_of, void* stream);
MN_API int mn_gather_rows_bf16(const uint16_t* x, int64_t ldx, const int32_t* perm, uint16_t* y, int64_t ldy, int n_rows, int D,
                        void* stream);
/* h[t] += sum_j w[t, j] * y[slot_of[t, j]]  (fp32) */
MN_API int mn_moe_combine(const float* y, int64_t ldy, const int32_t* slot_of, const float* w, int n_slot, float* h, int64_t ldh,
                   int T, int D, void* stream);
/* C fp32 [M,N] = (A_hi + A_lo) W^T + bias: activations split into bf16 hi and lo halves (A_lo starts a_lo_off elements
 * after A_hi, same row stride), both multiplied against the same W tiles in one launch — fp32-class products on the bf16
 * MFMA (used for the RF head's adaLN projections of all Euler steps, diff_loss_rf_swiglu.py:263-266, 283-286). */
MN_API int mn_gemm_bf16_hilo(const uint16_t* A_hi, int64_t lda, int64_t a_lo_off, const uint16_t* W, int64_t ldw,
                      const uint16_t* bias, float* C, int64_t ldc, int M, int N, int K, void* stream);
/* Grouped GEMM over experts: rows [off[g], off[g] + cnt[g]) of A / C use W + g * w_gstride.  off / cnt are device
 * arrays (from mn_moe_sort); m_max >= every cnt[g].  epilogue: MN_GEMM_BF16 or MN_GEMM_F32, no bias. */
MN_API int mn_gemm_bf16_grouped(const uint16_t* A, int64_t lda, const uint16_t* W, int64_t ldw, int64_t w_gstride,
                         const int32_t* off, const int32_t* cnt, int n_groups, void* C, int64_t ldc, int m_max, int N,
                         int K, int epilogue, void* stream);

/* ---- wide-row GEMM (gemm256.hip): 256 x 256 x 64 tiles, 8 waves, two long phases per K-tile with counted vmcnt ----------
 * The nn.Linear call sites above when hundreds of rows are in flight (lock-step generation of 128+ images: RF head
 * w12 / w3 / adaLN, diff_loss_rf_swiglu.py:54-72, 263-272, 283-292; MingTok batches; long-prompt prefill).
 * Needs K % 64 == 0, N % 4 == 0, 16-byte aligned rows and operands below 4 GiB (mn_gemm256_supported); C 16-byte (fp32) /
 * 8-byte (bf16) aligned with ldc % 4 == 0 and an 8-byte aligned bias (the epilogue stores 4 consecutive columns per lane).
 *   a_lo_off == 0: A bf16 [M,K].   a_lo_off != 0: A is a bf16 hi/lo pair (lo rows a_lo_off elements after the hi rows),
 *   the product is (A_hi + A_lo) W^T with both halves riding the same W tiles (a tile then covers 128 rows).
 * epilogue: enum mn_gemm_epilogue. */
MN_API int mn_gemm256_supported(int64_t lda, int64_t a_lo_off, int64_t ldw, int64_t w_rows, int M, int N, int K);
MN_API int mn_gemm256(const uint16_t* A, int64_t lda, int64_t a_lo_off, const uint16_t* W, int64_t ldw, const uint16_t* bias,
               void* C, int64_t ldc, int M, int N, int K, int epilogue, void* stream);
/* Split-K: slice z of the K range writes fp32 partials[z][M][N] (bias folded into slice 0); returns the slice count. */
MN_API int mn_gemm256_splitk(const uint16_t* A, int64_t lda, int64_t a_lo_off, const uint16_t* W, int64_t ldw,
                      const uint16_t* bias, float* partials, int M, int N, int K, int ksplit, void* stream);
/* SwiGLU-fused (swiglu_ffn.py:30-34, diff_loss_rf_swiglu.py:54-72): W12 bf16 [2*hidden, K] (gate rows then up rows),
 * b12 bf16 [2*hidden] or NULL.  Y receives silu(A Wg^T + bg) * (A Wu^T + bu) split into bf16 hi rows [M, hidden] (ldy)
 * and lo rows y_lo_off elements further — the operand layout of the next hi/lo GEMM. */
MN_API int mn_gemm256_swiglu_split(const uint16_t* A, int64_t lda, int64_t a_lo_off, const uint16_t* W12, int64_t ldw,
                            const uint16_t* b12, uint16_t* Y, int64_t ldy, int64_t y_lo_off, int M, int hidden, int K,
                            void* stream);

/* The same with a plain bf16 result Y [M, hidden] (batched bf16 path: MingTok SwiGLU blocks); a_lo_off = 0 for bf16 activations. */
MN_API int mn_gemm256_swiglu(const uint16_t* A, int64_t lda, int64_t a_lo_off, const uint16_t* W12, int64_t ldw, const uint16_t* b12,
                      uint16_t* Y, int64_t ldy, int M, int hidden, int K, void* stream);
/* Grouped form (MoE experts, modeling_bailing_moe.py:605-639, hundreds of rows in flight): group g multiplies row positions
 * [off[g], off[g] + cnt[g]) — position r reads A row a_rows[r] when a_rows != NULL (the gather of the expert-sorted order,
 * done while staging) — by W + g * w_gstride and writes rows off[g].. of C.  A is a bf16 hi/lo pair (a_lo_off > 0).
 *   swiglu == 0: C fp32 [*, N];   swiglu == 1: W_g holds 2N rows (gate rows, up rows), C = bf16 hi rows [*, N] (ldc) and
 *   lo rows c_lo_off elements further of silu(gate) * up.   off / cnt: device arrays (mn_moe_sort); cnt[g] <= m_max.
 *   A has a_rows_total rows (every a_rows entry is below it: bounds the 32-bit source offsets). */
MN_API int mn_gemm256_grouped(const uint16_t* A, int64_t lda, int64_t a_lo_off, int64_t a_rows_total, const int32_t* a_rows,
                              const uint16_t* W, int64_t ldw, int64_t w_gstride, const int32_t* off, const int32_t* cnt, int n_groups,
                              void* C, int64_t ldc, int64_t c_lo_off, int m_max, int N, int K, int swiglu, void* stream);

/* Operand of a hi/lo gemm256 launch from an fp32 row block: Y = act(norm(x)) as bf16 hi rows [M, D] (ldy) and lo rows y_lo_off
 * elements further (y_lo_off == 0: plain bf16, no lo rows) and / or as fp32 rows `out` (ldo); either may be NULL.  norm 0: none; 1: RMSNorm(g) (modeling_bailing_moe.py:131-136);
 * 2: LayerNorm(g, b optional) (mingtok layers/block.py:80-105).  act 1: exact-erf GELU (mlp.py:34-40).  D % 4 == 0, D <= 4096.
 * The fp32-class ("precise") form of the MingTok blocks and of linear_proj is built from this + mn_gemm256 on hi/lo operands. */
MN_API int mn_norm_act_split(const float* x, int64_t ldx, int norm, const uint16_t* g, const uint16_t* b, float eps, int act,
                             uint16_t* Y, int64_t ldy, int64_t y_lo_off, float* out, int64_t ldo, int M, int D, void* stream);

/* Tail of a split-K Linear that joins the fp32 residual stream, fused with the next LayerNorm (MingTok layers/block.py:80-105):
 * h[m] += sum_z P[z * slab + m * D + :] (bias already in slab 0, as mn_gemm256_splitk leaves it); if y != NULL:
 * y[m] = bf16(LayerNorm(h[m]; ln_g, ln_b optional, eps)), followed by exact-erf GELU when gelu != 0.  D % 4 == 0, D <= 4096. */
MN_API int mn_slab_resid_norm(const float* P, int nz, int64_t slab, float* h, int64_t ldh, const uint16_t* ln_g, const uint16_t* ln_b,
                       float eps, int gelu, uint16_t* y, int64_t ldy, int M, int D, void* stream);

/* mn_rope_kv_prefill for several prompt spans in one launch: span i = rows [r0_i, r0_i + len_i) of qkv / q_out (rotary position
 * pos[row]), appended to cache sequence seq_i from slot slot0 of kv_layer [n_seq_total, 2, n_kv, t_max, hd];
 * seq_tab: device int32 [n_spans][3] = (seq_i, r0_i, len_i). */
MN_API int mn_rope_kv_prefill_spans(const float* qkv, int64_t ldqkv, int n_q, int n_kv, int hd, const float* cos_tab, const float* sin_tab,
                             const int32_t* pos, int slot0, float q_scale, uint16_t* q_out, float* kv_layer, int64_t t_max,
                             const int32_t* seq_tab, int n_spans, int max_len, void* stream);

/* mn_moe_combine fused with the RMSNorm of the next consumer: h[t] += sum_s tw[t, s] * yg[slot_of[t, s]] (moe_infer,
 * modeling_bailing_moe.py:630-639); if y != NULL: y[t] = bf16(RMSNorm(h[t]; eps) * norm_w).  H % 4 == 0, H <= 4096. */
MN_API int mn_moe_combine_norm(const float* yg, const int32_t* slot_of, const float* tw, int n_slot, float* h, int64_t ldh,
                        const uint16_t* norm_w, float eps, uint16_t* y, int64_t ldy, int T, int H, void* stream);

/* GQA 4:1 flash attention (head dim 128, bottom-right causal; modeling_bailing_moe.py:848-1045) of several prompt spans in one
 * launch, K / V read from the fp32 KV arena of one layer (kv_layer [n_seq_total, 2, n_kv, t_max, 128]): span i = rows
 * [r0_i, r0_i + len_i) of q / out (bf16 [rows, n_q, 128], q RoPE'd and pre-scaled) against keys [0, past + len_i) of cache
 * sequence seq_i.  seq_tab: device int32 [n_spans][3] = (seq_i, r0_i, len_i); max_len >= every len_i; key_mask optional
 * uint8 [n_spans, mask_stride] (1 = attend). */
MN_API int mn_flash_prefill_gqa_hd128(const uint16_t* q, const float* kv_layer, int64_t t_max, int n_q, int n_kv, int past,
                               const int32_t* seq_tab, int n_spans, int max_len, const uint8_t* key_mask, int64_t mask_stride,
                               uint16_t* out, void* stream);
/* The fp32-class form (the attention of mn_llm_step_spans): q FP32 [rows, n_q, 128] (RoPE'd, pre-scaled), all operands as bf16 hi + lo
 * pairs (three MFMAs per product), fp32 softmax / accumulators.  span_tab: device int32 [n_spans][4] = (seq_i, r0_i, len_i, past_i)
 * — every span brings its own `past`.  out fp32 [rows, n_q * 128] and / or split bf16 hi rows, then lo rows split_lo_off elements
 * on (either may be NULL).  No key mask. */
MN_API int mn_flash_prefill_gqa_hd128_f32(const float* q, const float* kv_layer, int64_t t_max, int n_q, int n_kv, const int32_t* span_tab,
                                          int n_spans, int max_len, float* out, uint16_t* split, int64_t split_lo_off, void* stream);

/* mn_moe_sort plus the list of LIVE row tiles of the grouped GEMMs: tile t (t < *n_tiles) = rows [tile_m0[t], tile_m0[t] +
 * tile_rows) of group tile_g[t]; tile_g / tile_m0 hold up to T * n_slot / tile_rows + n_groups entries.  All device arrays.
 * (modeling_bailing_moe.py:608-616: the expert-count / argsort bookkeeping of moe_infer, without the host sync.) */
MN_API int mn_moe_sort_tiles(const int32_t* topk_idx, int T, int n_slot, int n_groups, int32_t* counts, int32_t* offsets, int32_t* perm,
                      int32_t* slot_of, int tile_rows, int32_t* tile_g, int32_t* tile_m0, int32_t* n_tiles, void* stream);

/* Grouped gemm256 over that tile list (tile_rows = 128 for a hi/lo A, 256 for a plain bf16 A with a_lo_off = 0): no workgroup
 * runs for an empty tile, whatever the split of the rows over the experts.  A has a_rows_total rows.
 *   epi 0: C fp32 [*, N];  1: C bf16 [*, N];  4: W_g holds 2N rows (gate, up), C = bf16 hi rows + lo rows c_lo_off further of
 *   silu(gate) * up;  6: the same as plain bf16;  7: C bf16 [*, N] = max(., 0)^2.   max_mtiles >= sum_g ceil(cnt[g] / tile_rows). */
MN_API int mn_gemm256_grouped_tiles(const uint16_t* A, int64_t lda, int64_t a_lo_off, int64_t a_rows_total, const int32_t* a_rows,
                             const uint16_t* W, int64_t ldw, int64_t w_gstride, const int32_t* off, const int32_t* cnt, int n_groups,
                             const int32_t* tile_g, const int32_t* tile_m0, const int32_t* n_tiles, int max_mtiles, void* C,
                             int64_t ldc, int64_t c_lo_off, int N, int K, int epi, void* stream);

/* Weight-streaming MFMA kernel behind the M >= 5 route of mn_skinny_gemm: Y bf16 [2][M][K] (activations split
 * into hi rows then lo rows), W bf16 [Ntot, K] dense, P fp32 [nz][M][Ntot] K-slice partials with
 * nz = mn_stream_mfma_slices(M, Ntot, K) (the launch plan picks slices of 256..1024 k so that every wave of the
 * chip gets the same number of 16-row weight tiles); returns nz.  M <= 64 (33..64 rows run the K-loop form: 8 x 2
 * tiles per workgroup over a long K-range, x chunks double-buffered in LDS).  HBM-bound: every weight byte is read once. */
MN_API int mn_stream_mfma(const uint16_t* Y, const uint16_t* W, float* P, int M, int Ntot, int K, void* stream);
MN_API int mn_stream_mfma_slices(int M, int Ntot, int K);
/* Grouped form (MoE experts; replaces the per-token expert loop of modeling_bailing_moe.py:605-639 for 5..32
 * rows): group g of G multiplies the x rows xrows[off[g] .. off[g+1]) (identity rows when xrows == NULL) by
 * W + g * w_stride and writes rows off[g].. of P [nz][p_rows][Ntot]; Y holds y_rows hi rows then y_rows lo rows;
 * no group may exceed max_rows (<= 64) rows.  off / xrows are device arrays.  Every distinct expert is streamed
 * once for all the rows routed to it.  Returns nz = mn_stream_mfma_grouped_slices(G, max_rows, Ntot, K). */
MN_API int mn_stream_mfma_grouped(const uint16_t* Y, int y_rows, const uint16_t* W, int64_t w_stride, float* P, int p_rows,
                           const int32_t* off, const int32_t* xrows, int G, int max_rows, int Ntot, int K,
                           void* stream);
MN_API int mn_stream_mfma_grouped_slices(int G, int max_rows, int Ntot, int K);

/* y bf16 [M,D] = LayerNorm(x fp32 [M,D]; g,b bf16, eps) ; optional GELU afterwards (encoder out layer,
 * vision_transformer.py:173-178). */
MN_API int mn_layernorm_bf16(const float* x, int64_t ldx, const uint16_t* g, const uint16_t* b, float eps,
                      uint16_t* y, int64_t ldy, int M, int D, int gelu, void* stream);

/* h bf16 [M,H] = silu(x12[:, :H]) * x12[:, H:]   (x12 bf16 [M,2H]) */
MN_API int mn_swiglu_bf16(const uint16_t* x12, int64_t ldx, uint16_t* h, int64_t ldh, int M, int H, void* stream);

/* Flash attention, head_dim 64, bf16 in/out, fp32 softmax.
 * qkv bf16 [B, T, 3, n_heads, 64] (the reshape of attention.py:83,98); out bf16 [B, T, n_heads*64].
 * causal: 0 = bidirectional (Attention / MemEffAttention), 1 = causal (MemEffCausalAttention). */
MN_API int mn_attn_prefill_hd64(const uint16_t* qkv, uint16_t* out, int B, int T, int n_heads, int causal, void* stream);
/* The same attention in the fp32-class regime (within 1e-3 of the fp32 reference path): qkv FP32
 * [B, T, 3, n_heads, 64]; operands carried as bf16 hi + lo pairs, three MFMAs per product, fp32 softmax and accumulators.
 * out fp32 [B * T, n_heads * 64] and / or split bf16 [2][B * T][n_heads * 64] (hi rows, then lo rows: the projection GEMM's
 * operand); either may be NULL. */
MN_API int mn_attn_prefill_hd64_f32(const float* qkv, float* out, uint16_t* split, int B, int T, int n_heads, int causal, void* stream);

/* Small fp32 elementwise helpers of the ViT glue (all [M, D] row-major contiguous):
 *   mn_add_bcast_f32    out[i] = a[i] + b[i % period]     (+pos-embed, vision_transformer.py:222)
 *   mn_group_mean_add   out[m,c] = y[m,c] + mean_g x[m, c*G + g], G = D/C   (encoder out shortcut, :174)
 *   mn_repeat_add       out[m,n] = y[m,n] + s[m, n / (D/C)] * scale + shift   (decoder in shortcut, :375-379)
 *   mn_clamp_f32        x = clamp(x, lo, hi) in place            (modeling_mingtok.py:194) */
MN_API int mn_add_bcast_f32(const float* a, const float* b, float* out, int64_t n, int64_t period, void* stream);
MN_API int mn_group_mean_add(const float* y, const float* x, float* out, int M, int D, int Cout, void* stream);
MN_API int mn_repeat_add(const float* y, const float* s, float* out, int M, int D, int Cin, float scale, float shift, void* stream);
MN_API int mn_clamp_f32(float* x, int64_t n, float lo, float hi, void* stream);
/* The MingTok layout shuffles as single passes that write the consumer's operand directly:
 * mn_patchify_operand: PatchEmbed's conv k = s = P as a GEMM (layers/patch_embed.py:69-82): image fp32 [B,3,Hi,Wi] -> A operand bf16
 *   [B * (Hi/P) * (Wi/P), 3 P^2] (row = patch, column = (c, py, px)); y_lo_off != 0: bf16 hi rows at Y, lo rows y_lo_off elements further.
 * mn_tokens_assemble: prepare_tokens (vision_transformer.py:218-223): out[b, n] = (n < N ? tok[b N + n] : cls) + pos[n], cls LAST.
 * mn_subtoken_rearrange: "b (h w) (x y c) -> b (h x w y) c" of forward_pixel_decoder (modeling_mingtok.py:184-188), fp32, Dp = c.
 * mn_unpatchify_clamp: unpatchify 'nhwpqc->nchpwq' (vision_transformer.py:515-527) + clamp_ (modeling_mingtok.py:195): o fp32
 *   [B * hh * ww, p * p * 3] -> image [B, 3, hh p, ww p]. */
MN_API int mn_patchify_operand(const float* image, int B, int Hi, int Wi, int P, uint16_t* Y, int64_t y_lo_off, void* stream);
MN_API int mn_tokens_assemble(const float* tok, const uint16_t* cls, const float* pos, float* out, int B, int N, int D, void* stream);
MN_API int mn_subtoken_rearrange(const float* y, float* x, int B, int h, int w, int r, int Dp, void* stream);
MN_API int mn_unpatchify_clamp(const float* o, float* image, int B, int hh, int ww, int p, float lo, float hi, void* stream);

/* fp32 <-> bf16 conversion and hi/lo split helpers (elementwise, n elements). */
MN_API int mn_f32_to_bf16(const float* x, uint16_t* y, int64_t n, void* stream);
MN_API int mn_bf16_to_f32(const uint16_t* x, float* y, int64_t n, void* stream);
/* hi = bf16(x), lo = bf16(x - hi): lets an fp32 activation go through the bf16 MFMA twice at fp32-class accuracy */
MN_API int mn_f32_split_bf16(const float* x, uint16_t* hi, uint16_t* lo, int64_t n, void* stream);

/* ------------------------------------------------------------------------------------------
 * 5. Composite device-side sequences (one C call = many launches, no host sync).
 *    See the struct comments; Python builds these tables once at load time.
 * ------------------------------------------------------------------------------------------ */

/* Rectified-flow head (RectifiedFlowLoss.sample, diff_loss_rf_swiglu.py:103-181, called from
 * forward_for_image_generation_inner, modeling_bailing_moe.py:1659-1670). */
typedef struct mn_rf_head {
  int32_t w, depth, hidden, z_dim, target, steps, llm_hidden;
  /* vis_head = Linear(llm_hidden->z) + LayerNorm(z) */
  const uint16_t *vis_w, *vis_b, *vis_ln_g, *vis_ln_b;
  const uint16_t *cond_w, *cond_b;        /* cond_embed [w, z] */
  const uint16_t *in_w, *in_b;            /* input_proj [w, target] */
  const float* temb;                      /* [steps, w] fp32: time_embed(t_s * 1000), precomputed at load */
  /* all adaLN projections stacked: rows [depth*3w + 2w, w] = blocks' (shift,scale,gate) then final (shift,scale) */
  const uint16_t *ada_w, *ada_b;
  const uint16_t* const* ln_g;  const uint16_t* const* ln_b;   /* [depth] in_ln */
  const uint16_t* const* w12;   const uint16_t* const* b12;    /* [depth] [2*hidden, w] */
  const uint16_t* const* w3;    const uint16_t* const* b3;     /* [depth] [w, hidden] */
  const uint16_t *fin_w, *fin_b;          /* final_layer.linear [target, w] */
  /* fp8 weight mode (section 7; 0 = bf16).  wfmt = MN_W_FP8_E4M3: w12[b] / w3[b] point to e4m3 BYTES in the same [out, in] layout and
   * w12_scale[b] [2*hidden] / w3_scale[b] [w] hold one fp32 scale per output row; every other tensor stays bf16.  Calls then take
   * the weight-streaming route only (rows <= 64: that route is HBM-bound, fp8 halves its bytes; mn_rf_max_rows returns 64). */
  int32_t wfmt;
  const float* const* w12_scale; const float* const* w3_scale;
  /* optional (NULL = the adaLN GEMM always reads the bf16 ada_w): the stacked adaLN matrix as e4m3 bytes [depth*3w + 2w, w] + row
   * scales.  Used when all Euler steps' rows fit one streaming launch (steps * rows <= 64, i.e. <= 4 CFG rows at 16 steps: the
   * reference's call shape); ada_w must then hold the SAME values (the exact bf16 expansion) for the larger row counts. */
  const uint8_t* ada_q; const float* ada_scale;
  /* (0.1.24) arithmetic regime of the WIDE route (> 64 rows in lock-step); 0 = fp32-class (bf16 hi/lo MFMA pairs, the parity regime).
   * MN_ARITH_FP8_MFMA (section 8; needs wfmt == MN_W_FP8_E4M3 with ada_q): the ResBlock GEMMs w12 / w3 and the adaLN GEMM multiply
   * e4m3 activations (quantised per row from the bf16 operand) by the e4m3 weight bytes on the scaled fp8 MFMA — no bf16 expansion of
   * the weights, 2.2-2.6 x the hi/lo pair's rate per GEMM — a LABELLED reduced-arithmetic regime with its own stated tolerance
   * (tests/test_gpu_fp8_mfma.py); every other Linear of the head, and every route up to 64 rows, is unchanged. */
  int32_t arith;
} mn_rf_head;
enum { MN_ARITH_FP32_CLASS = 0, MN_ARITH_FP8_MFMA = 1 };

/* hidden [rows, llm_hidden] fp32 (last hidden states of the LLM step), rows = n_images x R image-major with
 * R = 1 (no CFG), 2 ([cond, uncond]) or 3 ([cond, uncond, text_uncond]) rows per image; rows <= 64.
 * noise [n_images, target] fp32; latent_out [n_images, target] fp32 (all CFG rows of an image carry the same
 * latent).  n_images = 1 is the reference's batch-size-1 call.  Workspace: mn_rf_workspace_bytes(h, rows). */
MN_API size_t mn_rf_workspace_bytes(const mn_rf_head* h, int rows);
/* (0.1.24) At <= 2 rows the sampler runs as ONE persistent launch whose phases are separated by an in-launch grid barrier (every
 * workgroup must be resident).  A barrier wait is bounded (2 s): on expiry the result is NaN in every workgroup — and, because a
 * launcher never synchronises, the library raises the CALLER's status word so the host can tell "NaN because a co-tenant process /
 * a CU mask kept the grid from being resident" from a numerical failure: register one zero-initialised uint32 of DEVICE memory per
 * process (NULL = off; the word is the only process state the library keeps besides the launch-ordering event), read it at any host
 * sync, non-zero = a wait expired since it was last cleared (0x300; clear it yourself).  Remedy: MINGNATIVE_RF_PERSIST=0 (launch chain). */
MN_API int mn_persist_set_status_word(uint32_t* device_word);
/* Rows one call accepts: 64 (weight-streaming kernels), or 2048 when every width is a multiple of 64 — then calls with more
 * than 64 rows take the wide route (each Linear a 256 x 256-tile MFMA GEMM on bf16 hi/lo operands, gemm256.hip). */
MN_API int mn_rf_max_rows(const mn_rf_head* h);
MN_API int mn_rf_sample(const mn_rf_head* h, const float* hidden, int64_t ld_hidden, int rows, int n_images,
                 const float* noise, float temperature, float text_cfg, float image_cfg, float* latent_out,
                 void* workspace, size_t workspace_bytes, void* stream);

/* Bailing-MoE decoder stack, decode-style step for M <= 64 rows
 * (BailingMoeModel.forward, modeling_bailing_moe.py:1391-1540, with q_len rows per sequence). */
typedef struct mn_llm {
  int32_t hidden, n_layers, n_q, n_kv, head_dim, n_experts, top_k, n_shared_slots, moe_inter;
  int32_t norm_topk_prob;
  float rms_eps;
  const uint16_t* const* ln1;        /* [L] input_layernorm [H] */
  const uint16_t* const* wqkv;       /* [L] [(nq+2nkv)*hd, H] */
  const uint16_t* const* wdense;     /* [L] [H, nq*hd] */
  const uint16_t* const* ln2;        /* [L] post_attention_layernorm */
  const uint16_t* const* gate;       /* [L] [E, H] */
  const uint16_t* const* image_gate; /* [L] [E, H] or NULL entries */
  const uint16_t* const* w_gate_up;  /* [L] [E + n_shared_slots, 2*I, H]: rows 0..I-1 gate_proj, I..2I-1 up_proj */
  const uint16_t* const* w_down;     /* [L] [E + n_shared_slots, H, I] */
  const uint16_t* final_norm;        /* [H] */
  const float *cos_tab, *sin_tab;    /* [n_pos, hd/2] */
  int32_t n_pos;
  int32_t mrope_sec_t, mrope_sec_h;  /* 0, 0: Legacy rotary, row_pos [M]; else 3D rotary sections, row_pos [3][M] (t, h, w) */
  /* fp8 weight mode (section 7; 0 = bf16).  wfmt = MN_W_FP8_E4M3: w_gate_up[l] / w_down[l] point to e4m3 BYTES in the same packed
   * layout, w_gate_up_scale[l] [E + S, 2I] / w_down_scale[l] [E + S, H] hold one fp32 scale per output row of every expert;
   * attention, router and norm weights stay bf16.  Steps then take the weight-streaming route only (rows <= 64; every row count
   * runs the grouped expert kernels; mn_llm_max_rows returns 64). */
  int32_t wfmt;
  const float* const* w_gate_up_scale; const float* const* w_down_scale;
  /* (0.1.24) arithmetic regime of the WIDE route, as mn_rf_head.arith: MN_ARITH_FP8_MFMA (needs wfmt == MN_W_FP8_E4M3) runs the grouped
   * expert GEMMs (gate/up with the SwiGLU epilogue, down) on e4m3 activations x the e4m3 expert bytes (section 8) — no per-layer bf16
   * expansion of the experts; attention, router and every route up to 64 rows unchanged.  Labelled reduced arithmetic, own tolerance. */
  int32_t arith;
} mn_llm;

MN_API size_t mn_llm_workspace_bytes(const mn_llm* m, int rows, int64_t t_max);
MN_API int mn_llm_max_rows(const mn_llm* m);      /* 64, or 2048 (wide route: see mn_rf_max_rows) */
/* x fp32 in (embeddings): row m is read from x + (m / x_row_div) * ldx (ldx == 0 broadcasts one row to all M
 * rows; x_row_div = R shares one embedding between the R CFG rows of an image)
 * -> hidden_out [M,H] fp32 (after the final RMSNorm).
 * kv_cache: fp32 [n_layers][n_seq][2][n_kv][t_max][hd]; per-row int32 device arrays as in
 * mn_rope_kv_append / mn_attn_decode (row_len = row_slot + 1 is computed by the caller). */
MN_API int mn_llm_step(const mn_llm* m, const float* x, int64_t ldx, int x_row_div, int M, const uint8_t* image_mask,
                const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_pos, const int32_t* row_len,
                const uint8_t* key_mask, int64_t ld_mask, float* kv_cache, int n_seq, int64_t t_max,
                float* hidden_out, void* workspace, size_t workspace_bytes, void* stream);

/* Diagnostic (0.1.24; parity tests with teacher-forced routing): while `capture` is non-NULL every mn_llm_step* call copies each layer's
 * routing — int32 [n_layers][M][top_k + n_shared_slots]: the chosen expert ids in the path's own slot order, then the shared
 * pseudo-experts n_experts + j — to it, on the call's stream.  Process-global, not thread-safe; NULL (default) = off. */
MN_API int mn_llm_route_capture(int32_t* capture);

/* mn_llm_step with flags.  MN_STEP_DISTINCT_SEQUENCES: every row belongs to a different cache sequence and row_len == row_slot + 1
 * (a decode step of independent conversations / CFG rows — NOT a prefill chunk, whose rows attend each other's new K / V lines): the
 * rotary embedding and the K / V append then ride the attention launch (one launch fewer per layer; <= 64 rows, n_q / n_kv in
 * {1, 2, 4}).  Results are identical to mn_llm_step. */
#define MN_STEP_DISTINCT_SEQUENCES 1
MN_API int mn_llm_step_ex(const mn_llm* m, const float* x, int64_t ldx, int x_row_div, int M, const uint8_t* image_mask,
                   const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_pos, const int32_t* row_len,
                   const uint8_t* key_mask, int64_t ld_mask, float* kv_cache, int n_seq, int64_t t_max,
                   float* hidden_out, void* workspace, size_t workspace_bytes, int flags, void* stream);

/* mn_llm_step for a PREFILL chunk whose rows are whole spans of cache sequences (BailingMoeModel.forward on a prompt, :1391-1540;
 * eager / flash causal attention, :791-812, 848-1045): span i = rows [r0_i, r0_i + len_i) of x, in order the slots
 * [past_i, past_i + len_i) of cache sequence seq_i (row_seq / row_slot / row_pos / row_len describe the same rows, row_len =
 * row_slot + 1; no key mask).  span_tab: device int32 [n_spans][4] = (seq_i, r0_i, len_i, past_i); max_len >= every len_i.
 * On the wide route (> 64 rows, head dim 128, GQA 4:1) the attention then runs as tiled flash attention on bf16 hi/lo operands
 * (fp32-class like the rest of the route) instead of row by row; every other shape takes mn_llm_step's path.  Same results. */
MN_API int mn_llm_step_spans(const mn_llm* m, const float* x, int64_t ldx, int M, const uint8_t* image_mask, const int32_t* row_seq,
                             const int32_t* row_slot, const int32_t* row_pos, const int32_t* row_len, float* kv_cache, int n_seq,
                             int64_t t_max, const int32_t* span_tab, int n_spans, int max_len, float* hidden_out, void* workspace,
                             size_t workspace_bytes, void* stream);

/* a[i] += delta, b[i] += delta, c[i] += delta for i < M (any pointer may be NULL): advances the
 * device-resident row_slot / row_pos / row_len arrays between autoregressive steps without a host round trip. */
MN_API int mn_rows_advance(int32_t* a, int32_t* b, int32_t* c, int M, int delta, void* stream);

/* MingTok semantic decoder, cached causal decode step for M <= 64 rows of ONE sequence each
 * (MingTok.forward_feature_decoder, modeling_mingtok.py:165-174 -> TransformerDecoder.forward_features,
 * vision_transformer.py:382-451) followed by linear_proj (modeling_bailingmm.py:111-115). */
typedef struct mn_semdec {
  int32_t dim, depth, n_heads, hidden, in_dim, proj_dim, proj_depth;
  float mean, scale;
  const uint16_t *in_w, *in_b;
  const uint16_t* const* ln1_g; const uint16_t* const* ln1_b;
  const uint16_t* const* wqkv;  const uint16_t* const* bqkv;
  const uint16_t* const* wproj; const uint16_t* const* bproj;
  const uint16_t* const* ln2_g; const uint16_t* const* ln2_b;
  const uint16_t* const* w12;   const uint16_t* const* b12;
  const uint16_t* const* w3;    const uint16_t* const* b3;
  const uint16_t *norm_g, *norm_b;
  const uint16_t* const* proj_w; const uint16_t* const* proj_b;  /* [proj_depth] linear_proj layers */
  /* Wide-row route (M > 64, optional; NULL arrays = route unavailable): the SwiGLU hidden width zero-padded to a
   * multiple of 64 (hidden_pad): w12p [2*hidden_pad, dim] (gate rows, zero rows, up rows, zero rows), b12p [2*hidden_pad],
   * w3p [dim, hidden_pad] (zero columns) — load-time copies, results unchanged. */
  int32_t hidden_pad;
  const uint16_t* const* w12p; const uint16_t* const* b12p; const uint16_t* const* w3p;
} mn_semdec;

MN_API size_t mn_semdec_workspace_bytes(const mn_semdec* s, int rows, int64_t t_max);
MN_API int mn_semdec_max_rows(const mn_semdec* s);   /* 64, or 2048 when the padded SwiGLU weights are given */
/* latent_norm [M, in_dim] fp32 (normalised latent from the RF head) -> sem_out [M, dim] fp32 (x_norm),
 * embed_out [M, proj_dim] fp32 (linear_proj(sem)), either may be NULL.
 * kv_cache fp32 [depth][n_seq][2][n_heads][t_max][64]. */
MN_API int mn_semdec_step(const mn_semdec* s, const float* latent_norm, int M,
                   const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_len,
                   float* kv_cache, int n_seq, int64_t t_max, float* sem_out, float* embed_out,
                   void* workspace, size_t workspace_bytes, void* stream);


/* ------------------------------------------------------------------------------------------
 * 6. Tensor / expert parallelism of the decode path over one xGMI node (BASELINE configs[4]; SURVEY.md §8e — no reference
 *    counterpart: the reference runs the model on one device).  One process per GPU; every rank calls the same composites on its
 *    SHARD with the same arguments.  Partitioning, the one-shot all-reduce and the segment mechanism: csrc/tp.inl, DESIGN.md §7.
 * ------------------------------------------------------------------------------------------ */
#define MN_TP_MAX_WORLD 16

/* Communicator: every rank owns an inbox fp32 [2 (epoch parity)][world (sender)][cap] and arrival flags uint32
 * [world (sender)][rows_cap] in fine-grained device memory (mn_tp_alloc), mapped on every other rank (mn_tp_ipc_*).  inbox[p] /
 * flags[p] are the DEVICE addresses of rank p's arrays as seen from THIS rank (host arrays of `world` pointers).  epoch counts the
 * all-reduces completed on the communicator; it is advanced by the calls below, identically on every rank.  err: a local device
 * word that a bounded flag wait sets non-zero when it gives up (a dead peer / diverged launch order never hangs the GPU).  The
 * wait is bounded in WALL time — wait_ms milliseconds on the GPU's constant 100 MHz clock, 0 = the default of 30 s: host-side skew
 * between ranks (first-launch code loading, an allocator stall) is legitimate and can be long — and a row whose wait expired
 * POISONS its outputs with NaN instead of summing stale slabs: callers check err at their next host sync (TpRank does), and a
 * result can never silently miss an all-reduce. */
typedef struct mn_tp_comm {
  int32_t rank, world;
  float* const* inbox;
  uint32_t* const* flags;
  int64_t cap;          /* floats per (parity, sender) slab: >= rows * widest reduced row (3072 for the 16B-A3B RF head) */
  int32_t rows_cap;
  uint32_t epoch;
  uint32_t* err;
  uint32_t wait_ms;     /* 0 = 30 000 */
  /* Rows above which an all-reduce runs TWO-SHOT (round 5): reduce-scatter by pushing column piece j to rank j, the owner sums the
   * `world` pieces and pushes the reduced piece to every rank (all-gather) — 2 (world - 1) / world of the payload per rank instead of
   * (world - 1) x: what a many-row TP step wants; the one-shot form (one xGMI hop) stays for decode sizes.  0 = the default (16 rows);
   * < 0 = never (the relayed transport).  A two-shot all-reduce takes TWO epochs and adds one segment to the composites. */
  int32_t two_shot_rows;
} mn_tp_comm;

/* Host-side setup (these DO allocate / map; they are not launchers): fine-grained (uncached, system-coherent) device memory, its
 * IPC handle (64 bytes) for the other ranks, and the mapping of a peer's handle.  bytes for one rank's inbox = 2 * world * cap * 4,
 * flags = world * rows_cap * 4 (zero-filled by the caller). */
MN_API int mn_tp_alloc(size_t bytes, void** dptr);
MN_API int mn_tp_free(void* dptr);
MN_API int mn_tp_ipc_handle(void* dptr, void* handle_out_64);
MN_API int mn_tp_ipc_open(const void* handle_64, void** dptr);
MN_API int mn_tp_ipc_close(void* dptr);

/* out[m] = sum over the ranks of x[m]: x fp32 [M, D] (ldx == D) is this rank's partial, out fp32 [M, D] (ldo).  One-shot: the rank
 * pushes its rows into every rank's inbox over xGMI and sets their arrival flags; the reduce kernel waits on its LOCAL flags only.
 * 64 <= D <= 4096, D % 4 == 0, M <= rows_cap, M * D <= cap.  (latency-bound 4-18 KB payloads.) */
enum { MN_TP_PUSH = 1, MN_TP_REDUCE = 2, MN_TP_GATHER = 4 };   /* phase bits: all = the whole all-reduce in one call; split = work between them.
                                                                  MN_TP_GATHER (two-shot only, between the other two): the owner's reduce + all-gather push */
/* 1 or 2: how many segments (= epochs) an all-reduce of `rows` x D takes on this communicator (2 = two-shot). */
MN_API int mn_tp_allreduce_segments(const mn_tp_comm* comm, int rows, int D);
MN_API int mn_allreduce_oneshot(mn_tp_comm* comm, const float* x, int64_t ldx, float* out, int64_t ldo, int M, int D, int phase,
                                void* stream);

/* Expert parallelism, replicate-and-reduce: every rank holds all rows and the global routing (topk_idx [T, n_slot]
 * GLOBAL expert ids).  dispatch = moe_infer's count / argsort bookkeeping (modeling_bailing_moe.py:608-616) restricted to the experts
 * [expert0, expert0 + n_local) this rank owns: mn_moe_sort_tiles' outputs, the row-tile list only for those experts.
 * combine = the weighted un-permute (:630-639) across ranks: part[m] = sum over the LOCAL picks of topk_w * yg[slot_of] (+ optional
 * slabs P: the rank's slice of the shared expert), all-reduced; out[m] = h[m] + sum over ranks. */
MN_API int mn_ep_dispatch(const int32_t* topk_idx, int T, int n_slot, int n_experts, int expert0, int n_local, int32_t* counts,
                          int32_t* offsets, int32_t* perm, int32_t* slot_of, int tile_rows, int32_t* tile_g, int32_t* tile_m0,
                          int32_t* n_tiles, void* stream);
MN_API int mn_ep_combine(mn_tp_comm* comm, const float* yg, const int32_t* slot_of, const int32_t* topk_idx, const float* topk_w,
                         int n_slot, int expert0, int n_local, const float* P, int nz, int64_t slab, const float* h, int64_t ldh,
                         float* out, int64_t ldo, int M, int D, void* stream);

/* Decoder-stack step on a shard.  m describes the rank's shard as an mn_llm: n_q / n_kv = its local head counts, wqkv[l] =
 * [(n_q + 2 n_kv) * hd, H] (its q heads, then its K, then its V rows), wdense[l] = [H, n_q * hd] (its columns), n_experts = the
 * GLOBAL expert count with gate / image_gate replicated, n_shared_slots = 0, w_gate_up[l] / w_down[l] = its n_local_experts routed
 * experts; the KV arena holds its KV heads only.  tp adds the expert window and the rank's slice of the shared expert
 * (gate rows then up rows of shared_inter units, zero-padded to a multiple of 64; 0 = none).
 * Segments (mn_llm_tp_segments = 2 * n_layers + 1 with one-shot all-reduces; (that - 1) * mn_tp_allreduce_segments(comm, rows, hidden) + 1
 * in general — a two-shot all-reduce adds the owners' reduce + all-gather segment): [seg_begin, seg_end) selects the launch ranges between all-reduces; a rank
 * in production passes (0, n_segments).  Rows 1..2048; workspace mn_llm_tp_workspace_bytes.  Other arguments as mn_llm_step. */
typedef struct mn_llm_tp {
  int32_t expert0, n_local_experts;
  int32_t shared_inter;
  const uint16_t* const* ws_gate_up;   /* [L] [2 * shared_inter, H] */
  const uint16_t* const* ws_down;      /* [L] [H, shared_inter] */
  /* m->wfmt = MN_W_FP8_E4M3: ws_gate_up / ws_down are e4m3 bytes with these row scales ([2 * shared_inter] / [H] per layer) */
  const float* const* ws_gate_up_scale; const float* const* ws_down_scale;
} mn_llm_tp;
MN_API size_t mn_llm_tp_workspace_bytes(const mn_llm* m, const mn_llm_tp* tp, int rows, int64_t t_max);
MN_API int mn_llm_tp_segments(const mn_llm* m);
MN_API int mn_llm_step_tp(const mn_llm* m, const mn_llm_tp* tp, mn_tp_comm* comm, const float* x, int64_t ldx, int x_row_div, int M,
                          const uint8_t* image_mask, const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_pos,
                          const int32_t* row_len, const uint8_t* key_mask, int64_t ld_mask, float* kv_cache, int n_seq, int64_t t_max,
                          float* hidden_out, void* workspace, size_t workspace_bytes, int seg_begin, int seg_end, void* stream);

/* RectifiedFlowLoss.sample on a shard: h->hidden = the rank's share of the SwiGLU width, w12[b] = [2 * hidden, w] (its gate rows,
 * then its up rows), b12[b] likewise, w3[b] = [w, hidden] (its columns); b3 and all other tensors are the full replicated ones.
 * One all-reduce per ResBlock per Euler step; segments = steps * depth + 1.  Other arguments as mn_rf_sample; rows 1..2048. */
MN_API size_t mn_rf_tp_workspace_bytes(const mn_rf_head* h, int rows);
MN_API int mn_rf_tp_segments(const mn_rf_head* h);
MN_API int mn_rf_sample_tp(const mn_rf_head* h, mn_tp_comm* comm, const float* hidden, int64_t ld_hidden, int rows, int n_images,
                           const float* noise, float temperature, float text_cfg, float image_cfg, float* latent_out,
                           void* workspace, size_t workspace_bytes, int seg_begin, int seg_end, void* stream);

/* lm_head + greedy pick (compute_logit, modeling_bailing_moe.py:1604-1620, + the argmax of greedy decoding):
 * idx[m] = vocab_offset + argmax_v hidden[m] . W[v] (ties -> lowest index, torch.argmax's rule), val[m] = that logit (optional).
 * W bf16 [V, H]: the whole lm_head, or a rank's vocabulary slice starting at vocab_offset.  The fp32 logits [M, V] are left in the
 * first bytes of the workspace (mn_lmhead_argmax_workspace_bytes). */
MN_API size_t mn_lmhead_argmax_workspace_bytes(int M, int V, int H);
MN_API int mn_lmhead_argmax(const float* hidden, int64_t ld_hidden, int M, const uint16_t* W, int64_t ldw, int V, int H,
                            int64_t vocab_offset, int64_t* idx, float* val, void* workspace, size_t workspace_bytes, void* stream);

/* Sampled pick (the `do_sample` branch of HF GenerationMixin.generate, which the reference forwards its generate kwargs to:
 * modeling_bailingmm.py:249-262, modeling_bailing_moe.py:1769-1796; warpers in transformers/generation/logits_process.py —
 * TemperatureLogitsWarper -> TopKLogitsWarper -> TopPLogitsWarper -> softmax -> one multinomial draw):
 * idx[m] = vocab_offset + the token the inverse CDF of the warped distribution of logits[m] gives at u[m] in [0, 1), tokens ranked by
 * descending score, ties by ascending id.  top_k = 0 and top_p >= 1 switch the respective warper off.  The kernel ranks at most 2048
 * candidates: top_k > 2048 is refused (MN_EINVAL); with top_k = 0 and top_p < 1 the nucleus limit is top_p of the FULL vocabulary's
 * softmax mass and the nucleus is searched among the 2048 largest scores — HF's result exactly whenever its nucleus holds <= 2048 tokens.
 * status (optional, int32 [M], may be NULL) reports the rows where that did not hold: MN_SAMPLE_NUCLEUS_TRUNCATED (the nucleus wanted more
 * than 2048 tokens and was cut to the 2048 best) and MN_SAMPLE_TIES_TRUNCATED (more ties at the k-th score than candidates left: the lowest
 * ids were kept).  The caller owns the uniform stream (u), so a decode is reproducible from a seed.  logits fp32 [M, V], row stride ld
 * (e.g. the first bytes of mn_lmhead_argmax's workspace). */
enum { MN_SAMPLE_NUCLEUS_TRUNCATED = 1, MN_SAMPLE_TIES_TRUNCATED = 2 };
MN_API int mn_sample_logits(const float* logits, int64_t ld, int M, int V, float temperature, int top_k, float top_p, const float* u,
                            int64_t vocab_offset, int64_t* idx, int32_t* status, void* stream);

/* ------------------------------------------------------------------------------------------
 * 7. fp8 weight mode (BASELINE configs[4] "fp8").
 *    No arithmetic counterpart in the reference: its reduced-byte surface is the `dtype` switch of MingUniVisionInfer
 *    (mingunivision/mingunivisioninfer.py:46-70, int8 / int4 weight-only through quanto / bitsandbytes); the only fp8 trace is
 *    vllm/ming_lite.patch:171-190.  This mode is weight-only too: OCP e4m3fn bytes + one fp32 scale per OUTPUT ROW,
 *        W[n, k] = e4m3(Wq[n, k]) * scale[n],
 *    for the tensors that carry the bytes of the HBM-bound decode route — RF w12 / w3 and the routed + shared experts.
 *    Activations stay fp32 / bf16 hi+lo pairs and the MFMAs stay bf16: the kernels convert e4m3 -> bf16 in registers (exact)
 *    and apply the row scale to the fp32 accumulators, so the result is that of the DEQUANTISED weights to fp32 rounding —
 *    parity is defined against the oracle fed those (tests/test_gpu_fp8.py); the distance between the quantised and the bf16
 *    model is reported separately.  mn_quant_fp8_rows emits power-of-two scales, for which the dequantised weights are exactly
 *    representable in bf16 (mn_dequant_fp8_rows): the same model can be run through every bf16 route.
 * ------------------------------------------------------------------------------------------ */
enum { MN_W_BF16 = 0, MN_W_FP8_E4M3 = 1, MN_W_INT8 = 2, MN_W_NF4 = 3 };
/* MN_W_NF4 (round 5): the reference's `dtype="int4"` surface (mingunivisioninfer.py:46-58: BitsAndBytesConfig(load_in_4bit, nf4,
 * bf16 compute), i.e. bitsandbytes Linear4bit; third-party, absent here; restated in oracle/int4_ref.py) —
 *     W[n, k] = bf16_rne(NF4[code[n, k]] * absmax[n, k / 64]),   blocks of 64 consecutive k, fp32 absmax, no double quantisation.
 * Layout: `w` / Wq = rows of K / 2 bytes (two codes per byte; inside every dword the nibbles hold k 0 4 1 5 2 6 3 7 of its eight
 * consecutive k, from bit 0 up), `wscale` = the absmax table [rows][K / 64].  K % 64 == 0.  Strides of the grouped forms count
 * ELEMENTS for the codes (w_stride weights = w_stride / 2 bytes) and floats for the absmax tables.  The kernels look every block's 16
 * possible bf16 values up with v_perm_b32 (w8_codec.h) on the way into the MFMA tile; nothing is scaled afterwards.  Routes: the
 * weight-streaming launches (<= 64 rows; the experts run the grouped launch from one row on). */
MN_API int mn_quant_nf4_rows(const uint16_t* W, int64_t ldw, uint8_t* Wq, int64_t ldq, float* absmax, int64_t n_rows, int K, void* stream);
MN_API int mn_dequant_nf4_rows(const uint8_t* Wq, int64_t ldq, const float* absmax, uint16_t* W, int64_t ldw, int64_t n_rows, int K,
                               void* stream);
/* K-slice count of a dense streaming launch in format wfmt (the slab count the caller's reducing kernel sees) */
MN_API int mn_stream_mfma_wq_slices(int wfmt, int M, int Ntot, int K);
/* MN_W_INT8: the reference's `dtype="int8"` surface (mingunivisioninfer.py:59-68: HF QuantoConfig(weights="int8") = optimum-quanto qint8
 * weights; third-party, absent here; restated in oracle/int8_ref.py) — symmetric, one scale per output row, in the weight's dtype:
 *     scale[n] = bf16(amax_n / 127),  q = clamp(round(bf16(W / scale)), -128, 127),  W'[n, k] = bf16_rne(q[n, k] * scale[n]).
 * (Round 4 used power-of-two scales applied to the accumulators; round 5 follows quanto: the product is rounded to bf16 PER ELEMENT,
 * as quanto's qbytes_mm multiplies scale * weights in the activation dtype before the matmul — so the row scale rides the byte
 * conversion inside the kernels and nothing is scaled afterwards.)  Routes: the weight-streaming launches (<= 64 rows; experts on the
 * grouped launch from one row on). */
/* Row-wise quantisation at load: scale[n] = 2^ceil(log2(amax_n / 448)) (1 for an all-zero row), Wq[n, k] = e4m3_rne(W[n, k] / scale[n]).
 * W bf16 [n_rows, K] (row stride ldw), Wq bytes (row stride ldq), K % 4 == 0. */
MN_API int mn_quant_fp8_rows(const uint16_t* W, int64_t ldw, uint8_t* Wq, int64_t ldq, float* scale, int64_t n_rows, int K, void* stream);
/* W[n, k] = bf16_rne(e4m3(Wq[n, k]) * scale[n]) — exact for power-of-two scales. */
MN_API int mn_dequant_fp8_rows(const uint8_t* Wq, int64_t ldq, const float* scale, uint16_t* W, int64_t ldw, int64_t n_rows, int K,
                               void* stream);
/* mn_stream_mfma / mn_stream_mfma_grouped on fp8 weights: Wq e4m3 [Ntot, K] dense (K % 16 == 0, 16-byte aligned), wscale fp32
 * [Ntot]; grouped: group g reads Wq + g * w_stride bytes and wscale + g * s_stride floats.  Half the HBM bytes per launch. */
MN_API int mn_stream_mfma_w8(const uint16_t* Y, const uint8_t* Wq, const float* wscale, float* P, int M, int Ntot, int K, void* stream);
/* ... with the byte format as an argument (wfmt = MN_W_FP8_E4M3 | MN_W_INT8; the _w8 forms are wfmt = MN_W_FP8_E4M3) */
MN_API int mn_stream_mfma_wq(const uint16_t* Y, const uint8_t* Wq, const float* wscale, float* P, int M, int Ntot, int K, int wfmt, void* stream);
MN_API int mn_stream_mfma_grouped_wq(const uint16_t* Y, int y_rows, const uint8_t* Wq, int64_t w_stride, const float* wscale,
                                     int64_t s_stride, float* P, int p_rows, const int32_t* off, const int32_t* xrows, int G,
                                     int max_rows, int Ntot, int K, int wfmt, void* stream);
/* int8 rows by quanto's rule (above; scale 1 for an all-zero row), and back.  Arguments as the fp8 pair. */
MN_API int mn_quant_int8_rows(const uint16_t* W, int64_t ldw, uint8_t* Wq, int64_t ldq, float* scale, int64_t n_rows, int K, void* stream);
MN_API int mn_dequant_int8_rows(const uint8_t* Wq, int64_t ldq, const float* scale, uint16_t* W, int64_t ldw, int64_t n_rows, int K,
                                void* stream);
MN_API int mn_stream_mfma_w8_slices(int M, int Ntot, int K);
MN_API int mn_stream_mfma_grouped_w8(const uint16_t* Y, int y_rows, const uint8_t* Wq, int64_t w_stride, const float* wscale,
                                     int64_t s_stride, float* P, int p_rows, const int32_t* off, const int32_t* xrows, int G,
                                     int max_rows, int Ntot, int K, void* stream);

/* ------------------------------------------------------------------------------------------
 * 8. fp8-MFMA regime (0.1.24) — BASELINE.json configs[4]'s "fp8 MFMA".  A LABELLED reduced-arithmetic regime with its own tolerance,
 *    never a default: the reference has no fp8 path, the parity target is the fp32 oracle at a stated looser bar.
 *    Both GEMM operands are OCP e4m3 bytes with one fp32 scale per row (weights: the "fp8" weight format of section 7; activations:
 *    mn_quant_fp8_rows of the bf16 operand the hi/lo route would multiply), products on v_mfma_f32_16x16x128_f8f6f4 (no block
 *    scales), fp32 accumulation — the 256 x 256-tile kernel of the wide route at twice the bf16 MFMA rate per pass, one pass
 *    instead of the hi/lo pair's two.
 *    C = epilogue((A8 . a_scale)(W8 . w_scale)^T + bias): swiglu == 0 -> C fp32 [M, N] (ksplit > 1: slice z at C + z * M * N, ldc == N,
 *    returns the slice count); swiglu == 1 -> W8 holds 2N rows (gate, up), C bf16 [M, N] = silu(gate) * up (swiglu_ffn.py:30-34,
 *    diff_loss_rf_swiglu.py:54-72).  K % 128 == 0, 16-byte aligned rows and scale arrays.
 * ------------------------------------------------------------------------------------------ */
MN_API int mn_gemm256_f8(const uint8_t* A, int64_t lda, const float* a_scale, const uint8_t* W, int64_t ldw, const float* w_scale,
                         const uint16_t* bias, void* C, int64_t ldc, int M, int N, int K, int swiglu, int ksplit, void* stream);
MN_API int mn_gemm256_f8_slices(int K, int ksplit);

/* ------------------------------------------------------------------------------------------
 * 9. Latent-cache sequence models (0.1.26): decoder stacks whose attention layers cache one low-rank latent per token instead of
 *    keys and values (keys and values of every head are linear maps of it, so queries are absorbed into latent space and the
 *    attention runs against the latents themselves), with a short causal per-channel filter in front of the mixer, sigmoid-gated
 *    sublayer results that are normalised before the residual add, and a polynomial-of-unit-norms feed-forward activation.
 *    Rows are fp32, weights bf16 [out, in]; every size and constant is a field or an argument.  The residual stream, norms,
 *    gates, softmax and the cached latents are fp32 in both arithmetic modes; `arith` chooses the matrix products:
 *    MN_SEQ_ARITH_BF16 = bf16 MFMA products with fp32 accumulation for steps of more than 8 rows (fp32 FMA below),
 *    MN_SEQ_ARITH_F32 = fp32 FMA everywhere.
 * ------------------------------------------------------------------------------------------ */
MN_API int mn_affine_ln_rows(const float* x, int64_t ldx, const uint16_t* w, const uint16_t* b, float eps, float* y, int64_t ldy,
                             uint16_t* y16, int64_t ldy16, int M, int n, void* stream);
/* x += LN(sigmoid(g) * y; w, b) row by row (g holds the gate's pre-activation) */
MN_API int mn_gated_ln_residual(float* x, int64_t ldx, const float* g, int64_t ldg, const float* y, int64_t ldy, const uint16_t* w,
                                const uint16_t* b, float eps, int M, int n, void* stream);
/* y = x / sqrt(mean(x^2) + eps) * w; with row_seq / row_slot the fp32 output row of input row m is row_seq[m] * t_max + row_slot[m]
 * (append into a cache arena [n_seq, t_max, n]); y16 (optional) is a bf16 copy in input row order */
MN_API int mn_rms_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16,
                       const int32_t* row_seq, const int32_t* row_slot, int t_max, int M, int n, void* stream);
/* y = c0 U(z) + c1 U(z^2) + c2 U(z^3) + c3 with U(v) = v / sqrt(mean(v^2) + eps), powers element by element; coef bf16 [4] */
MN_API int mn_polynorm_rows(const float* z, int64_t ldz, const uint16_t* coef, float eps, float* y, int64_t ldy, uint16_t* y16,
                            int64_t ldy16, int M, int n, void* stream);
/* Causal per-channel filter over each sequence's rows, added to its input: y_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), w bf16
 * [n, taps].  Row m is position row_slot[m] of sequence row_seq[m] and has row_back[m] earlier rows of its sequence in this call
 * (directly before it); older inputs come from state fp32 [n_seq, taps - 1, n] (entry i = the input i + 1 positions before the
 * call's first row of that sequence), positions before 0 count as zero.  mn_tap_state_update moves the state past the call's rows. */
MN_API int mn_tap_filter_rows(const float* x, int64_t ldx, const uint16_t* w, int taps, const float* state, const int32_t* row_seq,
                              const int32_t* row_slot, const int32_t* row_back, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16,
                              int M, int n, void* stream);
MN_API int mn_tap_state_update(const float* x, int64_t ldx, int taps, float* state, const int32_t* row_seq, const int32_t* row_back,
                               int M, int n, void* stream);
/* Decode rows — every row ALONE in its sequence within the call — in one launch, up to three stages: (g given) x += LN(sigmoid(g) y;
 * wa, ba); n_out = LN(x; wb, bb); (h given) h = n_out + the tap filter over the sequence's state, and the state moves on by this row
 * (mn_tap_filter_rows + mn_tap_state_update for one-row sequences).  Rows of at most 4096 values, at most 8 taps. */
MN_API int mn_gated_norm_filter_rows(float* x, int64_t ldx, const float* g, int64_t ldg, const float* y, int64_t ldy, const uint16_t* wa,
                                     const uint16_t* ba, const uint16_t* wb, const uint16_t* bb, float eps, float* n_out, int64_t ldn,
                                     const uint16_t* taps_w, int taps, float* state, const int32_t* row_seq, const int32_t* row_slot,
                                     float* h, int64_t ldh, int M, int n, void* stream);
MN_API int mn_softcap_rows(float* z, int64_t ld, int M, int n, float cap, void* stream);
/* C[z] = alpha * A[z] W[z]^T (+ bias) (* sigmoid(G[z])) for z < batch, operands of batch entry z at base + z * (their _bs stride):
 * fp32 FMA, any M / N / K.  C (fp32) and C16 (bf16 copy) are both optional outputs. */
MN_API int mn_gemm_f32_batched(const float* A, int64_t lda, int64_t a_bs, const uint16_t* W, int64_t ldw, int64_t w_bs,
                               const uint16_t* bias, float* C, int64_t ldc, int64_t c_bs, uint16_t* C16, int64_t ldc16, int64_t c16_bs,
                               const float* G, int64_t ldg, int64_t g_bs, int M, int N, int K, int batch, float alpha, void* stream);
/* Attention against cached latents.  qabs fp32 [M, H, r]: the queries of every head mapped into latent space, softmax scale
 * included; arena fp32 [n_seq, t_max, r]; row m attends slots [0, row_len[m]) of sequence row_seq[m].  blk_tab int32 [n_blk, 2] =
 * (first row, rows <= mn_latent_attn_block_rows()) cuts the rows into runs of consecutive rows of ONE sequence with ascending
 * row_len.  lat fp32 [M, H, r] = softmax-weighted mean of the latents.  ks > 1 splits the key range over ks workgroups per run
 * (mn_latent_attn_splits proposes it from the launch size; workspace from mn_latent_attn_workspace_bytes).  r <= 1024. */
MN_API int mn_latent_attn_block_rows(void);
MN_API int mn_latent_attn_splits(int n_blk, int max_len, int r);
MN_API size_t mn_latent_attn_workspace_bytes(int M, int H, int r, int ks);
MN_API int mn_latent_attn(const float* qabs, const float* arena, const int32_t* row_seq, const int32_t* row_len, const int32_t* blk_tab,
                          int n_blk, int M, int H, int r, int t_max, int max_len, int ks, float* lat, void* workspace,
                          size_t workspace_bytes, void* stream);
/* The same with the kernel named: MN_LATENT_ATTN_MFMA (what mn_latent_attn runs) = scores and weighted sums on the fp32 matrix
 * cores (v_mfma_f32_16x16x4_f32: fp32 operands and accumulation), 16 query vectors per workgroup, 16-key tiles;
 * MN_LATENT_ATTN_VALU = one wave per query vector on fp32 FMA (the plain kernel the other is checked against). */
enum { MN_LATENT_ATTN_MFMA = 0, MN_LATENT_ATTN_VALU = 1 };
MN_API int mn_latent_attn_ex(const float* qabs, const float* arena, const int32_t* row_seq, const int32_t* row_len, const int32_t* blk_tab,
                             int n_blk, int M, int H, int r, int t_max, int max_len, int ks, float* lat, void* workspace,
                             size_t workspace_bytes, int variant, void* stream);

enum { MN_SEQ_ARITH_BF16 = 0, MN_SEQ_ARITH_F32 = 1 };
enum { MN_SEQ_MIX_LATENT_Q = 0,   /* queries through an RMS-normed latent (w_in rows: [q latent ; kv latent]) */
       MN_SEQ_MIX_GATED = 1 };    /* direct queries, sigmoid gate on the concatenated heads (w_in rows: [q ; gate ; kv latent]) */
typedef struct mn_seq_layer {
  int32_t kind, heads, dim, vdim, kv_rank, q_rank; /* q_rank: MN_SEQ_MIX_LATENT_Q only */
  int32_t ff;                                      /* 0: the layer has no feed-forward */
  int32_t arena;                                   /* index of the latent arena it attends */
  int32_t writes_arena;                            /* 1: w_in ends with its own kv-latent rows and it appends them; 0: it reads another layer's */
  float scale;
  const uint16_t *norm1_w, *norm1_b, *norm1b_w, *norm1b_b, *norm2_w, *norm2_b, *norm2b_w, *norm2b_b;   /* [width] each */
  const uint16_t *taps_w;                          /* [width, taps] */
  const uint16_t *rg1_w, *rg1_b;                   /* gate of the mixer's result: [width, width], [width] */
  const uint16_t *w_in;                            /* the mixer's projections of its input, stacked by rows (see kind) */
  const uint16_t *q_norm, *kv_norm;                /* [q_rank], [kv_rank] */
  const uint16_t *w_uq;                            /* [heads * dim, q_rank] */
  const uint16_t *w_ukT;                           /* [heads, kv_rank, dim]: the key expansion of every head, transposed */
  const uint16_t *w_uv;                            /* [heads * vdim, kv_rank] */
  const uint16_t *w_o;                             /* [width, heads * vdim] */
  const uint16_t *w_ff_in, *b_ff_in;               /* [width + ff, width] = [feed-forward gate ; up], bias [width + ff] (zero on the up rows) */
  const uint16_t *w_down;                          /* [width, ff] */
  const uint16_t *act;                             /* [4] */
} mn_seq_layer;
typedef struct mn_seq_model {
  int32_t width, n_layers, taps, arith;
  float eps;
  const mn_seq_layer* layers;                      /* HOST array [n_layers] */
  const uint16_t *final_w, *final_b;
} mn_seq_model;
typedef struct mn_seq_state {
  float* const* latent;                            /* HOST array of device pointers: arena a = fp32 [n_seq, t_max, its layer's kv_rank] */
  float* taps;                                     /* fp32 [n_layers, n_seq, taps - 1, width] */
  int32_t n_seq, t_max;
} mn_seq_state;
MN_API size_t mn_sizeof_seq_layer(void);
MN_API size_t mn_sizeof_seq_model(void);
MN_API size_t mn_sizeof_seq_state(void);
/* One pass of the stack over M rows (a prefill portion, decode rows of several sequences, or a mix; each sequence's rows
 * consecutive and in order).  x fp32 [M, width]: input embeddings.  Per row: row_seq (cache sequence), row_slot (its position =
 * the cache slot its latent goes to), row_back (earlier rows of its sequence in this call), row_len (= row_slot + 1: slots it
 * attends); blk_tab / n_blk as in mn_latent_attn; max_len >= every row_len.  Appends the latents, advances the filter states.
 * out fp32 [M, width]: the final norm's output.  trace (optional) fp32 [n_layers, M, width]: the residual stream after every layer. */
MN_API size_t mn_seq_workspace_bytes(const mn_seq_model* m, int M, int max_len);
enum { MN_SEQ_ROWS_DISTINCT = 1 };   /* flags: every row is alone in its sequence (a decode step): gate / norm / filter launches are fused */
MN_API int mn_seq_step(const mn_seq_model* m, const mn_seq_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                       const int32_t* row_slot, const int32_t* row_back, const int32_t* row_len, const int32_t* blk_tab, int n_blk,
                       int max_len, int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream);
/* logits fp32 [M, V] = hidden W^T by the step's product routing (arith as in mn_seq_model), then the soft cap (cap <= 0: none);
 * workspace: M * K * 2 bytes (the bf16 operand of the MFMA route) */
MN_API int mn_seq_logits(const float* hidden, int64_t ldh, int M, const uint16_t* W, int V, int K, float cap, int arith, float* out,
                         int64_t ldo, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * 10. Parallel-mixer sequence models (0.1.27): decoder stacks whose mixer is a windowed softmax attention (grouped key/value heads,
 *     short causal filters on the projected q / k / v channels, rotary positions with optional YaRN frequencies on the first
 *     `rot_dims` values of a head, unit-RMS queries and keys, a sliding window plus one mean key / value per whole block of `pool`
 *     tokens before it) running beside a minGRU recurrence on the same input, both summed with fixed scales; RMS pre-norms with a
 *     causal per-channel filter added to what each sublayer reads; a mixture-of-experts feed-forward (top-k softmax over the chosen
 *     logits, optional sigmoid-gated shared expert); `x += mult * sublayer`.  A contiguous range of layers may run several times with
 *     the same weights (each run owns its caches and states; the embedding rows are added again before every repeated pass).
 *     Rows are fp32, weights bf16 [out, in]; every size and constant is a field or an argument.  The residual stream, norms,
 *     angles, scores, softmax, router, recurrent state and cached keys / values are fp32 in both arithmetic modes (`arith` as in
 *     section 9 chooses the matrix products).
 * ------------------------------------------------------------------------------------------ */
/* y_t = sum_j w[:, j] x_(t - taps + 1 + j): mn_tap_filter_rows without the added input (state and row arrays as there) */
MN_API int mn_tap_conv_rows(const float* x, int64_t ldx, const uint16_t* w, int taps, const float* state, const int32_t* row_seq,
                            const int32_t* row_slot, const int32_t* row_back, float* y, int64_t ldy, int M, int n, void* stream);
/* x += mult * y (y may be NULL), then n_out = x / sqrt(mean(x^2) + eps) * w (n_out NULL: the add only); n16: optional bf16 copy */
MN_API int mn_axpy_rms_rows(float* x, int64_t ldx, const float* y, int64_t ldy, float mult, const uint16_t* w, float eps, float* n_out,
                            int64_t ldn, uint16_t* n16, int64_t ldn16, int M, int n, void* stream);
/* Decode rows (every row alone in its sequence) in one launch: x += mult * y; n = RMS(x) w; h = n + the tap filter over the
 * sequence's state (taps_w NULL: h = n), and the state moves on by this row.  Rows of at most 8192 values, at most 8 taps. */
MN_API int mn_axpy_rms_filter_rows(float* x, int64_t ldx, const float* y, int64_t ldy, float mult, const uint16_t* w, float eps,
                                   const uint16_t* taps_w, int taps, float* state, const int32_t* row_seq, const int32_t* row_slot,
                                   float* h, int64_t ldh, int M, int n, void* stream);
/* Rotary frequencies of the pairs (i, i + dims / 2), i < dims / 2: base^(-2i / dims), with YaRN interpolation when factor > 0
 * (ramp between the dimensions whose wavelengths make `fast` and `slow` turns over `original` positions).  HOST output freq
 * [dims / 2]; returns the factor cos and sin are multiplied by through *mag. */
MN_API int mn_rotary_frequencies_host(int dims, double base, double factor, double original, double fast, double slow, float* freq,
                                      float* mag);
/* Per row and head vector of qkv fp32 [M, (H + G) * dim + G * vdim]: rotate the first rot_dims values of every q and k head at
 * position row_slot[m] (freq device fp32 [rot_dims / 2], cos / sin times mag; rot_dims 0: none), divide q and k heads by their root
 * mean square (unit = 0: skip), write q * q_scale to q_out [M, H * dim] and append k / v to the arenas
 * k_arena [n_seq, t_max, G * dim], v_arena [n_seq, t_max, G * vdim] at (row_seq[m], row_slot[m]).  dim, vdim <= 512. */
MN_API int mn_rope_unit_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, int rot_dims, const float* freq,
                               float mag, int unit, float eps, float q_scale, const int32_t* row_seq, const int32_t* row_slot, float* q_out,
                               int64_t ldq, float* k_arena, float* v_arena, int t_max, void* stream);
/* Decode rows (every row alone in its sequence) in one launch: qkv holds the UNFILTERED projections; every channel goes through the
 * causal filter w_conv bf16 [channels, conv] over the sequence's earlier inputs in conv_state fp32 [n_seq, conv - 1, channels], which
 * moves on by this row (conv 0: no filter); then mn_rope_unit_append; then, for a row that completes a block of `pool` slots, the
 * block's mean key / value as mn_pool_blocks_update writes them (pool 0: none).  With gru_n > 0 extra workgroups of the launch run
 * mn_mingru_rows on the same rows (zx, g, gru_state, gru_scale = its out_scale, gru_out fp32 with row stride ldgo). */
MN_API int mn_filter_rope_append_rows(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* w_conv, int conv,
                                      float* conv_state, int rot_dims, const float* freq, float mag, int unit, float eps, float q_scale,
                                      const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena,
                                      float* v_arena, int t_max, float* pk, float* pv, int n_pool_max, int pool, const float* zx,
                                      int64_t ldzx, const float* g, int64_t ldg, float* gru_state, int gru_n, float gru_scale, float* gru_out,
                                      int64_t ldgo, void* stream);
/* Mean key / value of every block of `pool` slots that a row of this call completes (row_slot % pool == pool - 1):
 * pk [n_seq, n_pool_max, G * dim], pv [n_seq, n_pool_max, G * vdim], block b of a sequence = its slots [b pool, (b + 1) pool). */
MN_API int mn_pool_blocks_update(const float* k_arena, const float* v_arena, int t_max, float* pk, float* pv, int n_pool_max, int pool,
                                 int Gd, int Gv, const int32_t* row_seq, const int32_t* row_slot, int M, void* stream);
/* Softmax attention of q fp32 [M, H, dim] (scale included) for row m at position i = row_slot[m] of sequence row_seq[m] over the
 * slots j with 0 <= i - j < window (window 0: every j <= i) and, with pool > 0, over the block means b with (b + 1) pool - 1 <=
 * i - window, all in one softmax; query head h uses key / value head h / (H / G).  out[m, h * vdim + c] = out_scale * result
 * (fp32, row stride ldo; out16: optional bf16 copy).  (H / G) * vdim <= 8 * 256 per 8 heads; any dim. */
MN_API int mn_window_pool_attn(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk, const float* pv,
                               const int32_t* row_seq, const int32_t* row_slot, int M, int H, int G, int dim, int vdim, int t_max,
                               int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                               int64_t ldo16, void* stream);
/* The same attention in its tiled form (what mn_pmix_step runs; mn_window_pool_attn is the plain kernel it is checked against): a
 * workgroup takes a run of up to mn_window_attn_block_rows() consecutive rows of ONE sequence at consecutive positions (blk_tab int32
 * [n_blk, 2] = (first row, rows)), or single rows (one_row = 1: row b is block b, blk_tab unused), and shares each 64-key tile of the
 * run among its rows and query heads.  nsplit > 1 cuts a run's keys over nsplit workgroups and merges their partial softmaxes in a
 * second launch (mn_window_attn_splits proposes it from the launch size and max_keys, the most keys any run sees; workspace from
 * mn_window_attn_workspace_bytes).  vdim <= 512. */
MN_API int mn_window_attn_block_rows(void);
MN_API int mn_window_attn_splits(int n_blk, int H, int G, int one_row, int max_keys);
/* the same for a kernel whose key tiles hold key_tile keys (64: the fp32 FMA kernel, what mn_window_attn_splits assumes; 16: the
 * matrix-core kernel, which decode rows take when their values lie inside their keys) */
MN_API int mn_window_attn_splits_tile(int n_blk, int H, int G, int one_row, int max_keys, int key_tile);
MN_API size_t mn_window_attn_workspace_bytes(int n_blk, int H, int G, int vdim, int one_row, int nsplit);
MN_API int mn_window_pool_attn_blocks(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                      const float* pv, const int32_t* row_seq, const int32_t* row_slot, const int32_t* blk_tab, int n_blk,
                                      int one_row, int H, int G, int dim, int vdim, int t_max, int n_pool_max, int window, int pool,
                                      float out_scale, float* out, int64_t ldo, uint16_t* out16, int64_t ldo16, int nsplit, void* workspace,
                                      size_t workspace_bytes, void* stream);
/* The same with the kernel named: MN_WINDOW_ATTN_MFMA (what mn_window_pool_attn_blocks runs for runs of rows with dim, vdim <= 256) =
 * scores and weighted sums on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: fp32 operands and accumulation), 16-key tiles with
 * keys and values staged in LDS; MN_WINDOW_ATTN_VALU = the fp32 FMA kernel (decode rows, larger heads). */
enum { MN_WINDOW_ATTN_MFMA = 0, MN_WINDOW_ATTN_VALU = 1 };
MN_API int mn_window_pool_attn_blocks_ex(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                         const float* pv, const int32_t* row_seq, const int32_t* row_slot, const int32_t* blk_tab, int n_blk,
                                         int one_row, int H, int G, int dim, int vdim, int t_max, int n_pool_max, int window, int pool,
                                         float out_scale, float* out, int64_t ldo, uint16_t* out16, int64_t ldo16, int nsplit, void* workspace,
                                         size_t workspace_bytes, int variant, void* stream);
/* The same with a sink per query head (sink fp32 [H] on the device, or NULL): exp(sink[h]) joins the softmax's denominator of head h
 * — it has no key and no value and is not scaled.  variant < 0: the kernel mn_window_pool_attn_blocks would choose. */
MN_API int mn_window_pool_attn_blocks_sink(const float* q, int64_t ldq, const float* k_arena, const float* v_arena, const float* pk,
                                           const float* pv, const float* sink, const int32_t* row_seq, const int32_t* row_slot,
                                           const int32_t* blk_tab, int n_blk, int one_row, int H, int G, int dim, int vdim, int t_max,
                                           int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                                           int64_t ldo16, int nsplit, void* workspace, size_t workspace_bytes, int variant, void* stream);
/* minGRU over each sequence's rows: z = sigmoid(zx[m, c]), u = zx[m, n + c] (biases already added), candidate = u + 1/2 (u >= 0) or
 * sigmoid(u); S = (1 - z) S + z candidate from state fp32 [n_seq, n] (a row at slot 0 starts from zero), which is left at the
 * sequence's last row; out[m, c] = out_scale * S * silu(g[m, c]).  Rows of one sequence are consecutive (row_back as in 9). */
MN_API int mn_mingru_rows(const float* zx, int64_t ldzx, const float* g, int64_t ldg, float* state, const int32_t* row_seq,
                          const int32_t* row_slot, const int32_t* row_back, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                          int64_t ldo16, int M, int n, void* stream);
/* The same as a chunked scan (three launches: per-chunk products and sums, a carry over the chunks, the outputs): the form for steps
 * of many rows, where one thread walking all rows of a sequence is a chain of M dependent steps.  out (fp32) is required. */
MN_API size_t mn_mingru_scan_workspace_bytes(int M, int n);
MN_API int mn_mingru_rows_scan(const float* zx, int64_t ldzx, const float* g, int64_t ldg, float* state, const int32_t* row_seq,
                               const int32_t* row_slot, const int32_t* row_back, float out_scale, float* out, int64_t ldo, uint16_t* out16,
                               int64_t ldo16, int M, int n, void* workspace, size_t workspace_bytes, void* stream);
/* The `top` largest of logits[m, 0 .. E) (ties: the lower index) and the softmax over those alone: idx int32 [M, top], w fp32 [M, top] */
MN_API int mn_router_topk_rows(const float* logits, int64_t ld, int M, int E, int top, int32_t* idx, float* w, void* stream);
/* mn_router_topk_rows and y[m, c] = silu(x[m, c]) * x[m, n + c] (fp32) in one launch: the router's pick and the shared expert's
 * activation of decode rows read the same stacked projection */
MN_API int mn_router_topk_silu_rows(const float* logits, int64_t ld, int M, int E, int top, int32_t* idx, float* w, const float* x,
                                    int64_t ldx, float* y, int64_t ldy, int n, void* stream);
/* y[m, c] = silu(x[m, c]) * x[m, n + c]; y16: optional bf16 copy */
MN_API int mn_silu_mul_rows(const float* x, int64_t ldx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream);
/* C[z] fp32 [N] = A[z / a_div] . W[w_idx[z]]^T for z < Z: one input row against the weight block its index names (fp32 FMA; A row
 * stride lda, weight block stride w_bs, C row stride ldc). */
MN_API int mn_gemv_f32_indexed(const float* A, int64_t lda, int a_div, const uint16_t* W, int64_t ldw, int64_t w_bs, const int32_t* w_idx,
                               float* C, int64_t ldc, int Z, int N, int K, void* stream);
/* The same where only indices in [0, n_idx) name a weight block: rows with any other index are left untouched */
MN_API int mn_gemv_f32_indexed_upto(const float* A, int64_t lda, int a_div, const uint16_t* W, int64_t ldw, int64_t w_bs, const int32_t* w_idx,
                                    int n_idx, float* C, int64_t ldc, int Z, int N, int K, void* stream);
/* x[m] += mult * (sum_j w[m, j] y[r(m, j)] + sigmoid(sg[m * ldsg]) * shared[m]) with r(m, j) = slot_of ? slot_of[m * top + j] :
 * m * top + j; shared / sg may be NULL */
MN_API int mn_moe_combine_residual(float* x, int64_t ldx, const float* y, int64_t ldy, const int32_t* slot_of, const float* w, int top,
                                   const float* shared, int64_t lds, const float* sg, int64_t ldsg, float mult, int M, int n, void* stream);

typedef struct mn_pmix_layer {
  int32_t heads, kv_heads, dim, vdim;
  int32_t conv;                                    /* taps of the q / k / v filter, 0: none */
  int32_t rot_dims;                                /* 0: no rotation */
  int32_t unit_qk;                                 /* 1: q and k heads divided by their root mean square */
  int32_t window, pool;                            /* 0, 0: every earlier token */
  int32_t gru;                                     /* width of the recurrence */
  int32_t experts, top, ff, shared_ff;             /* experts 0: the layer has no feed-forward; shared_ff 0: no shared expert */
  float scale, rot_mag, left_scale, right_scale;
  const float* rot_freq;                           /* DEVICE fp32 [rot_dims / 2] */
  const uint16_t *norm1, *norm2;                   /* [width] */
  const uint16_t *canon1, *canon2;                 /* [width, taps] (model.taps 0: unused) */
  const uint16_t *w_in, *b_in;                     /* [q ; k ; v ; z ; x ; g] rows, bias (zero outside z and x) */
  const uint16_t *w_conv;                          /* [(heads + kv_heads) * dim + kv_heads * vdim, conv] */
  const uint16_t *w_out;                           /* [width, heads * vdim + gru] = [left o | right o] */
  const uint16_t *w_ff_in, *b_ff_in;               /* [shared gate ; shared up ; router ; shared gate logit ; zero rows up to a multiple of 8], bias (router's) */
  const uint16_t *w_shared_down;                   /* [width, shared_ff] */
  const uint16_t *w_gate_up;                       /* [experts, 2 ff, width] */
  const uint16_t *w_down;                          /* [experts, width, ff] */
} mn_pmix_layer;
typedef struct mn_pmix_model {
  int32_t width, n_layers, n_runs, taps, arith;    /* taps: of the sublayer-input filter, 0: none */
  float eps, mult;
  const mn_pmix_layer* layers;                     /* HOST array [n_layers] */
  const int32_t* run_layer;                        /* HOST [n_runs]: the layer of every run */
  const uint8_t* run_readd;                        /* HOST [n_runs]: 1 = the step's input rows are added to x before this run */
  const uint16_t* final_w;
} mn_pmix_model;
typedef struct mn_pmix_state {                     /* HOST arrays [n_runs] of device pointers, fp32 */
  float* const* k;                                 /* [n_seq, t_max, kv_heads * dim] */
  float* const* v;                                 /* [n_seq, t_max, kv_heads * vdim] */
  float* const* pk;                                /* [n_seq, n_pool_max, kv_heads * dim]  (pool 0: unused) */
  float* const* pv;
  float* const* canon;                             /* [2, n_seq, taps - 1, width]: mixer, feed-forward */
  float* const* conv;                              /* [n_seq, conv - 1, q + k + v channels] */
  float* const* gru;                               /* [n_seq, gru] */
  int32_t n_seq, t_max, n_pool_max;
} mn_pmix_state;
MN_API size_t mn_sizeof_pmix_layer(void);
MN_API size_t mn_sizeof_pmix_model(void);
MN_API size_t mn_sizeof_pmix_state(void);
/* One pass of the stack over M rows; rows, row arrays, out and trace as mn_seq_step (trace: fp32 [n_runs, M, width]).
 * blk_tab / n_blk: the rows cut into runs of <= mn_window_attn_block_rows() consecutive rows of one sequence (unused with
 * MN_SEQ_ROWS_DISTINCT); max_len >= every position + 1 (it sizes the attention's key splits).
 * flags: MN_SEQ_ROWS_DISTINCT = every row is alone in its sequence (a decode step): the residual add / norm / filter launches are
 * fused and the attention takes the rows one by one. */
MN_API size_t mn_pmix_workspace_bytes(const mn_pmix_model* m, int M);
MN_API int mn_pmix_step(const mn_pmix_model* m, const mn_pmix_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                        const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk, int max_len, int flags,
                        float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * 11. Hybrid-mixer sequence models (0.1.28): decoder stacks whose layers choose their mixer — a causal softmax attention with grouped
 *     key/value heads, per-head weighted RMS norm of queries and keys, a query temperature that grows with the position, and a learned
 *     sink per head in the softmax's denominator; or a decayed linear-attention recurrence ("lightning" attention: S = decay S + k v^T,
 *     o = S^T q on silu-activated projections, fp32 state per sequence, RMS norm over the joined heads times a sigmoid gate) — and
 *     run mixer and feed-forward in PARALLEL on one normed input: x += mixer(h) + ff(h), h = RMS(x) w.  The feed-forward is dense
 *     (squared relu) or a mixture of such experts whose router scores by softmax over all of its outputs, picks by score +
 *     correction, weighs by the picked scores over their sum, and counts its last `pass` outputs as "the input itself"; an optional
 *     shared expert is always on.  A contiguous range of layers may run several times with the same weights (each run owns its
 *     cache or state).  Rows are fp32, weights bf16 [out, in]; the residual stream, norms, temperature, scores, softmax, router,
 *     recurrence and its state are fp32 in both arithmetic modes (`arith` as in section 9 chooses the matrix products).
 * ------------------------------------------------------------------------------------------ */
/* Per row and head vector of qkv fp32 [M, (H + G) * dim + G * vdim]: q and k heads become x / sqrt(mean(x^2) + eps) * w (q_norm / k_norm
 * bf16 [dim], shared by the heads; NULL: no weight); q is further multiplied by q_scale * (1 + temp_coef * ln(floor((pos + 1) /
 * temp_every) + 1)) at position pos = row_slot[m] (temp_every <= 0: no temperature) and written to q_out [M, H * dim]; k and v are
 * appended to k_arena [n_seq, t_max, G * dim], v_arena [n_seq, t_max, G * vdim] at (row_seq[m], row_slot[m]).  dim <= 512. */
MN_API int mn_head_norm_temp_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* q_norm,
                                    const uint16_t* k_norm, float eps, float q_scale, float temp_coef, int temp_every,
                                    const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena,
                                    float* v_arena, int t_max, void* stream);
/* Decayed linear attention over each sequence's rows.  qkv fp32 [M, 2 H dim + H vdim] = [q ; k ; v] BEFORE their silu; per head h
 * S <- decay[h] S + k v^T, out[m, h vdim + c] = sum_i S[i, c] q[i]; state fp32 [n_seq, H, dim, vdim] (a row at slot 0 starts from
 * zero) is left at the sequence's last row.  Rows of one sequence are consecutive (row_back as in section 9); decay: device fp32 [H].
 * flags: MN_SEQ_ROWS_DISTINCT = every row is alone in its sequence (a decode step; row_back unused): a state column is then cut over
 * the threads of a workgroup, so that one row's state is read and written by many workgroups at once. */
MN_API int mn_lightning_rows(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                             const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, int flags, float* out, int64_t ldo,
                             void* stream);
/* The same as a chunked scan for steps of many rows (what mn_hyb_step runs above mn_lightning_chunk_rows() rows per step): chunks of
 * rows of one sequence (chunk_tab int32 [n_chunks, 2] = (first row, rows <= mn_lightning_chunk_rows()), in row order); pass 1: every
 * chunk's own sum of decayed k v^T; pass 2: the states at the chunks' starts, carried along each sequence; pass 3: every chunk's
 * outputs from its start state and its own keys.  workspace from mn_lightning_scan_workspace_bytes. */
MN_API int mn_lightning_chunk_rows(void);
MN_API size_t mn_lightning_scan_workspace_bytes(int n_chunks, int H, int dim, int vdim);
MN_API size_t mn_lightning_scan_lds_bytes(int dim, int vdim);   /* LDS a workgroup of the scan needs: the scan takes heads with at most 64 KiB */
/* The same with the output pass named: MN_LIGHTNING_SCAN_MFMA (what mn_lightning_rows_scan runs when its tiles fit 64 KiB of LDS) =
 * scores, carried-state and value products on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: fp32 operands and accumulation);
 * MN_LIGHTNING_SCAN_VALU = the fp32 FMA pass (the plain kernel the other is checked against). */
enum { MN_LIGHTNING_SCAN_MFMA = 0, MN_LIGHTNING_SCAN_VALU = 1 };
MN_API int mn_lightning_rows_scan_ex(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                                     const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* chunk_tab,
                                     int n_chunks, float* out, int64_t ldo, void* workspace, size_t workspace_bytes, int variant, void* stream);
MN_API int mn_lightning_rows_scan(const float* qkv, int64_t ldqkv, int M, int H, int dim, int vdim, const float* decay, float* state,
                                  const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* chunk_tab,
                                  int n_chunks, float* out, int64_t ldo, void* workspace, size_t workspace_bytes, void* stream);
/* y = x / sqrt(mean(x^2) + eps) * w * sigmoid(g); y16: optional bf16 copy */
MN_API int mn_rms_sigmoid_gate_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, const float* g, int64_t ldg, float* y,
                                    int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream);
/* y = max(x, 0)^2; y16: optional bf16 copy */
MN_API int mn_relu2_rows(const float* x, int64_t ldx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream);
/* Router: s = softmax(logits[m, 0 .. n)); the `top` largest of s + correction (device fp32 [n] or NULL; ties: the lower index); w = their
 * s over (the sum of their s + 1e-20).  Outputs at or past n_real name no expert ("pass the input through"): each is written as
 * index n_real.  idx int32 [M, top], w fp32 [M, top].  n <= 512.  relu_n > 0: the same launch also writes relu_y[m, c] =
 * max(relu_x[m, c], 0)^2 for c < relu_n (the shared expert's activation of decode rows reads the same stacked projection). */
MN_API int mn_router_softmax_topk_rows(const float* logits, int64_t ld, int M, int n, int n_real, int top, const float* correction,
                                       int32_t* idx, float* w, const float* relu_x, int64_t ldrx, float* relu_y, int64_t ldry, int relu_n,
                                       void* stream);
/* x[m] += add[m] + sum_j w[m, j] * (idx[m, j] < n_real ? y[r(m, j)] : h[m]) with r as in mn_moe_combine_residual; add may be NULL */
MN_API int mn_moe_combine_pass_residual(float* x, int64_t ldx, const float* y, int64_t ldy, const int32_t* slot_of, const int32_t* idx,
                                        const float* w, int top, int n_real, const float* h, int64_t ldh, const float* add, int64_t ldadd,
                                        int M, int n, void* stream);

enum { MN_HYB_ATTENTION = 0, MN_HYB_LIGHTNING = 1 };
enum { MN_HYB_FF_NONE = 0, MN_HYB_FF_DENSE = 1, MN_HYB_FF_MOE = 2 };
typedef struct mn_hyb_layer {
  int32_t kind;                                    /* MN_HYB_ATTENTION | MN_HYB_LIGHTNING */
  int32_t heads, kv_heads, dim, vdim;              /* lightning: kv_heads = heads */
  int32_t ff_kind;                                 /* MN_HYB_FF_* */
  int32_t ff;                                      /* dense: the feed-forward's width; moe: the shared expert's (0: none) */
  int32_t experts, pass, top, expert_ff;           /* moe: the router has experts + pass outputs, the last `pass` stand for the input itself */
  int32_t temp_every;                              /* attention: 0 = no query temperature */
  float scale, temp_coef;
  const float* sink;                               /* attention: DEVICE fp32 [heads] or NULL */
  const float* decay;                              /* lightning: DEVICE fp32 [heads] */
  const float* correction;                         /* moe: DEVICE fp32 [experts + pass] or NULL */
  const uint16_t *norm1;                           /* [width] */
  const uint16_t *q_norm, *k_norm;                 /* attention: [dim] */
  const uint16_t *mix_norm;                        /* lightning: [heads * vdim] */
  const uint16_t *w_in;                            /* rows [q ; k ; v ; (lightning: gate) ; up of the dense or shared expert ; router ; zero rows up to a multiple of 8] x width */
  const uint16_t *w_out;                           /* [width, heads * vdim + ff] = [mixer o | down of the dense or shared expert] */
  const uint16_t *w_up;                            /* moe: [experts, expert_ff, width] */
  const uint16_t *w_down;                          /* moe: [experts, width, expert_ff] */
} mn_hyb_layer;
typedef struct mn_hyb_model {
  int32_t width, n_layers, n_runs, arith;
  float eps;
  const mn_hyb_layer* layers;                      /* HOST array [n_layers] */
  const int32_t* run_layer;                        /* HOST [n_runs]: the layer of every run */
  const uint16_t* final_w;
} mn_hyb_model;
typedef struct mn_hyb_state {                      /* HOST arrays [n_runs] of device pointers, fp32 */
  float* const* k;                                 /* attention runs: [n_seq, t_max, kv_heads * dim] */
  float* const* v;                                 /* attention runs: [n_seq, t_max, kv_heads * vdim] */
  float* const* lin;                               /* lightning runs: [n_seq, heads, dim, vdim] */
  int32_t n_seq, t_max;
} mn_hyb_state;
MN_API size_t mn_sizeof_hyb_layer(void);
MN_API size_t mn_sizeof_hyb_model(void);
MN_API size_t mn_sizeof_hyb_state(void);
/* One pass of the stack over M rows; rows, row arrays, blk_tab / n_blk, max_len, flags, out and trace as mn_pmix_step (trace: fp32
 * [n_runs, M, width]).  chunk_tab / n_chunks: the rows cut into chunks of <= mn_lightning_chunk_rows() consecutive rows of one
 * sequence (NULL / 0: the recurrences walk their rows one by one). */
MN_API size_t mn_hyb_workspace_bytes(const mn_hyb_model* m, int M);
MN_API int mn_hyb_step(const mn_hyb_model* m, const mn_hyb_state* st, const float* x, int64_t ldx, int M, const int32_t* row_seq,
                       const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk, const int32_t* chunk_tab,
                       int n_chunks, int max_len, int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream);

/* The block attention of section 10 with a sink per head (or NULL), a soft cap of the scores (softcap > 0: every score s becomes
 * softcap * tanh(s / softcap) before the softmax; 0: none) and explicit row strides of the two arenas (ldk, ldv in floats; 0 = G * dim,
 * G * vdim): the value arena may be a view into the key arena — latent attention reads keys [latent ; rotated part] and values
 * [latent] from one arena with ldv = ldk.  A stride under heads of a multiple of 4 values must be a multiple of 4 itself. */
MN_API int mn_window_pool_attn_blocks_cap(const float* q, int64_t ldq, const float* k_arena, int64_t ldk, const float* v_arena, int64_t ldv,
                                          const float* pk, const float* pv, const float* sink, float softcap, const int32_t* row_seq,
                                          const int32_t* row_slot, const int32_t* blk_tab, int n_blk, int one_row, int H, int G, int dim,
                                          int vdim, int t_max, int n_pool_max, int window, int pool, float out_scale, float* out, int64_t ldo,
                                          uint16_t* out16, int64_t ldo16, int nsplit, void* workspace, size_t workspace_bytes, int variant,
                                          void* stream);

/* ------------------------------------------------------------------------------------------
 * 12. Post-norm mixed-mixer sequence models (0.1.29): decoder stacks whose sublayers read the residual stream as it is and whose
 *     RESULTS are RMS-normed before they are added: x += w1 rms(mixer(x)), x += w2 rms(ff(x)), and optionally a per-layer token
 *     input x += ws rms(P (gelu(G x) * e)), e a slice of a second embedding row of the token.  The mixer is chosen per layer:
 *     softmax attention (grouped heads, biases, RMS norm over the whole q and k projections, rotary pairs with optional
 *     long-context frequency scaling, soft-capped scores, sliding window, a sigmoid gate per head), latent attention (one normed
 *     latent and one rotated key part per token are cached; keys and values of every head are linear maps of the latent), or the
 *     gated delta rule (short causal filters and silu on q / k / v, unit-length q and k, a write strength and a decay per head
 *     and token, fp32 state per sequence).  The feed-forward is W_down (gelu(W_gate x) * W_up x), gelu in its tanh form.
 *     Rows are fp32, weights bf16 [out, in]; the residual stream, norms, angles, scores, softmax, gates, decays and the recurrent
 *     state are fp32 in both arithmetic modes (`arith` as in section 9 chooses the matrix products).
 * ------------------------------------------------------------------------------------------ */
/* Rotary frequencies base^(-2i / dims), i < dims / 2, rescaled by wavelength when factor > 0: a wavelength below original / high keeps
 * its frequency f, one above original / low gets f / factor, between them (1 - s) f / factor + s f with
 * s = (original / wavelength - low) / (high - low).  HOST output freq [dims / 2], computed in double. */
MN_API int mn_rotary_frequencies_scaled_host(int dims, double base, double factor, double low, double high, double original, float* freq);
/* x += y / sqrt(mean(y^2) + eps) * w; x16: optional bf16 copy of the new x */
MN_API int mn_rms_scale_add_rows(float* x, int64_t ldx, const float* y, int64_t ldy, const uint16_t* w, float eps, uint16_t* x16,
                                 int64_t ldx16, int M, int n, void* stream);
/* y[m, c] = gelu_tanh(a[m, c]) * b[m, c], or with b NULL times table[idx[m] * ldt + c] (bf16 table rows chosen per row; point
 * `table` at the first column of the slice).  y (fp32) and y16 (bf16) are both optional outputs. */
MN_API int mn_gelu_mul_rows(const float* a, int64_t lda, const float* b, int64_t ldb, const uint16_t* table, int64_t ldt,
                            const int32_t* idx, float* y, int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int n, void* stream);
/* Per row of qkv fp32 [M, H dim + G dim + G vdim]: q and k are divided by the root mean square of their WHOLE projection (all heads
 * at once) and multiplied by q_norm bf16 [H dim] / k_norm bf16 [G dim] (NULL: neither), then the first rot_dims values of every
 * head turn by position * freq[i] (freq device fp32 [rot_dims / 2]; interleaved 1: pairs (2i, 2i + 1), 0: pairs (i, i + rot_dims / 2));
 * q * q_scale goes to q_out [M, H dim], k and v are appended at (row_seq[m], row_slot[m]) of k_arena [n_seq, t_max, ldk] and
 * v_arena [n_seq, t_max, ldv]. */
MN_API int mn_proj_norm_rope_append(const float* qkv, int64_t ldqkv, int M, int H, int G, int dim, int vdim, const uint16_t* q_norm,
                                    const uint16_t* k_norm, float eps, int rot_dims, int interleaved, const float* freq, float q_scale,
                                    const int32_t* row_seq, const int32_t* row_slot, float* q_out, int64_t ldq, float* k_arena, int64_t ldk,
                                    float* v_arena, int64_t ldv, int t_max, void* stream);
/* Per row of qd fp32 [M, H (dim + rot) + rank + rot] = [queries head by head as (dim plain, rot rotated) ; down projection]:
 * arena[seq, slot, 0 .. rank) = RMS norm of the down projection's first rank values times c_norm; arena[seq, slot, rank .. rank + rot)
 * = its last rot values rotated; q_out[m, h (rank + rot) + rank + d] = q_scale * the rotated part of head h (the first `rank`
 * columns of every head are left for the caller's absorbed product).  Rotation as in mn_proj_norm_rope_append on the first
 * rot_dims <= rot values. */
MN_API int mn_latent_rope_append(const float* qd, int64_t ld, int M, int H, int dim, int rot, int rank, const uint16_t* c_norm, float eps,
                                 int rot_dims, int interleaved, const float* freq, float q_scale, const int32_t* row_seq,
                                 const int32_t* row_slot, float* q_out, int64_t ldq, float* arena, int64_t lda, int t_max, void* stream);
/* x[m, h vdim + c] *= sigmoid(g[m, h]); x16: optional bf16 copy */
MN_API int mn_head_sigmoid_gate_rows(float* x, int64_t ldx, const float* g, int64_t ldg, uint16_t* x16, int64_t ldx16, int M, int H,
                                     int vdim, void* stream);
/* Gated delta rule, preparation.  proj fp32 [M, ld]: raw channels [q: G dim ; k: G dim ; v: H vdim] from column 0, the write-strength
 * logits [H] from off_b and the decay logits [H] from off_a.  Every channel goes through its causal filter w_conv bf16 [channels, taps]
 * (last tap = the current row; earlier inputs from the rows before it in this call, then from state fp32 [n_seq, taps - 1, channels]
 * as mn_tap_filter_rows reads it) and silu; q and k heads become x / sqrt(sum(x^2) + unit_eps), q also times q_scale.  advance_state 0:
 * the state is read only and mn_tap_state_update moves it on afterwards; 1 (every row alone in its sequence, a decode step): the
 * launch moves it on by this row itself.  qkv fp32 [M, channels]; bd fp32 [M, 2 H] = [sigmoid(b) ; exp(-exp(a_log) softplus(a + dt_bias))]. */
MN_API int mn_delta_prep_rows(const float* proj, int64_t ld, int M, int H, int G, int dim, int vdim, int off_b, int off_a,
                              const uint16_t* w_conv, int taps, float* state, int advance_state, const float* a_log, const float* dt_bias,
                              float unit_eps, float q_scale, const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back,
                              float* qkv, int64_t ldo, float* bd, int64_t ldbd, void* stream);
/* Gated delta rule over each sequence's rows, per head h (q / k head h / (H / G)) with beta and g of the row:
 * S <- g S; u = beta (v - S^T k); S <- S + k u^T; out[m, h vdim + c] = (S^T q)[c].  state fp32 [n_seq, H, dim, vdim] (a row at slot 0
 * starts from zero) is left at the sequence's last row.  Rows of one sequence are consecutive (row_back as in section 9).
 * flags: MN_SEQ_ROWS_DISTINCT = every row is alone in its sequence (a decode step).  dim <= 512. */
MN_API int mn_gated_delta_rows(const float* qkv, int64_t ld, const float* bd, int64_t ldbd, int M, int H, int G, int dim, int vdim,
                               float* state, const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, int flags,
                               float* out, int64_t ldo, void* stream);
/* y[m, h vdim + c] = x / sqrt(mean over the head's vdim values of x^2 + eps) * w[c] * silu(g[m, h vdim + c]); y16: optional bf16 copy */
MN_API int mn_head_rms_silu_gate_rows(const float* x, int64_t ldx, const uint16_t* w, float eps, const float* g, int64_t ldg, float* y,
                                      int64_t ldy, uint16_t* y16, int64_t ldy16, int M, int H, int vdim, void* stream);

enum { MN_PN_ATTENTION = 0, MN_PN_LATENT = 1, MN_PN_DELTA = 2 };
typedef struct mn_pn_layer {
  int32_t kind;                                    /* MN_PN_* */
  int32_t heads, kv_heads, dim, vdim;              /* latent: kv_heads unused; dim = the plain part of a query / key head */
  int32_t rot, kv_rank;                            /* latent: rotated part of a head, latent size */
  int32_t rot_dims, rot_interleaved;               /* attention / latent: values of a head (of its rotated part) that turn; 0: none */
  int32_t window;                                  /* attention / latent: 0 = every earlier token */
  int32_t conv;                                    /* delta: taps of the q / k / v filters */
  int32_t ff;                                      /* 0: no feed-forward */
  int32_t side;                                    /* values of the per-layer token input, 0: none */
  int32_t has_gate;                                /* attention: 1 = a sigmoid gate per head follows v in the stack */
  float scale, softcap;                            /* softcap 0: none */
  float unit_eps;                                  /* delta: inside the root of the unit norms */
  const float* rot_freq;                           /* DEVICE fp32 [rot_dims / 2] */
  const float *a_log, *dt_bias;                    /* delta: DEVICE fp32 [heads] */
  const uint16_t *norm1, *norm2, *side_norm;       /* [width] */
  const uint16_t *w_in, *b_in;                     /* attention [q ; k ; v ; gate], latent [q ; down], delta [q ; k ; v ; b ; a ; g]; zero rows up to a multiple of 8; bias or NULL */
  const uint16_t *q_norm, *k_norm;                 /* attention: [heads dim], [kv_heads dim] or NULL; latent: k_norm = the latent's norm [kv_rank] */
  const uint16_t *w_conv;                          /* delta: [2 kv_heads dim + heads vdim, conv] */
  const uint16_t *mix_norm;                        /* delta: [vdim] */
  const uint16_t *w_ukT;                           /* latent: [heads, kv_rank, dim] */
  const uint16_t *w_uv;                            /* latent: [heads vdim, kv_rank] */
  const uint16_t *w_o, *b_o;                       /* [width, heads vdim], bias or NULL */
  const uint16_t *w_gate_up;                       /* [2 ff, width] = [gate ; up] */
  const uint16_t *w_down;                          /* [width, ff] */
  const uint16_t *w_side_gate;                     /* [side rounded up to a multiple of 8, width] */
  const uint16_t *w_side_proj;                     /* [width, side] */
  const uint16_t *side_table;                      /* the layer's first column of the token table */
} mn_pn_layer;
typedef struct mn_pn_model {
  int32_t width, n_layers, arith;
  float eps;
  int64_t side_ld;                                 /* row stride of the token table */
  const mn_pn_layer* layers;                       /* HOST array [n_layers] */
  const uint16_t* final_w;
} mn_pn_model;
typedef struct mn_pn_state {                       /* HOST arrays [n_layers] of device pointers, fp32 */
  float* const* k;                                 /* attention: [n_seq, t_max, kv_heads dim]; latent: [n_seq, t_max, ld_latent] */
  float* const* v;                                 /* attention: [n_seq, t_max, kv_heads vdim] */
  float* const* conv;                              /* delta: [n_seq, conv - 1, channels] */
  float* const* lin;                               /* delta: [n_seq, heads, dim, vdim] */
  int32_t n_seq, t_max;
} mn_pn_state;
MN_API size_t mn_sizeof_pn_layer(void);
MN_API size_t mn_sizeof_pn_model(void);
MN_API size_t mn_sizeof_pn_state(void);
/* Row stride of a latent arena: rank + rot rounded up to a multiple of 4 */
MN_API int mn_pn_latent_ld(int rank, int rot);
/* One pass of the stack over M rows; rows, row arrays, blk_tab / n_blk, max_len, flags, out and trace as mn_pmix_step (trace: fp32
 * [n_layers, M, width]); row_tok int32 [M]: the rows' token ids (read by layers with a token input). */
MN_API size_t mn_pn_workspace_bytes(const mn_pn_model* m, int M);
MN_API int mn_pn_step(const mn_pn_model* m, const mn_pn_state* st, const float* x, int64_t ldx, int M, const int32_t* row_tok,
                      const int32_t* row_seq, const int32_t* row_slot, const int32_t* row_back, const int32_t* blk_tab, int n_blk, int max_len,
                      int flags, float* out, float* trace, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MINGNATIVE_H */
