// seq_linear.h — product routing shared by the step functions of the sequence models (mingnative.h sections 9 and 10).
//   M <= 8 rows                      mn_skinny_gemm (weight streaming, fp32 FMA)
//   MN_SEQ_ARITH_BF16, 9 .. 64 rows  mn_skinny_gemm's weight-streaming MFMA route on bf16 hi/lo rows (fp32-class products)
//   MN_SEQ_ARITH_BF16, M > 64        mn_gemm_bf16 on the bf16 copy the producing kernel wrote (MFMA, fp32 accumulate)
//   MN_SEQ_ARITH_F32, or a K that is no multiple of 8 / an unaligned weight: mn_gemm_f32_batched (fp32 FMA tiles)
#pragma once
#include <string.h>

#include "common.h"

namespace {

inline size_t al(size_t n) { return (n + 255) & ~(size_t)255; }

inline bool mfma_ok(const uint16_t* W, int K) { return K >= 8 && (K % 8) == 0 && (((uintptr_t)W) & 15) == 0; }

// C fp32 [M, N] = A W^T + bias.  A16 (optional) = bf16 copy of A with row stride lda16; gws / gws_bytes: scratch of the weight-streaming
// MFMA route (mn_skinny_workspace_bytes).
inline int linear(int arith, int M, const float* A, int64_t lda, const uint16_t* A16, int64_t lda16, const uint16_t* W, int N, int K,
           const uint16_t* bias, float* C, int64_t ldc, void* gws, size_t gws_bytes, void* stream) {
  // <= 8 rows: weight streaming on fp32 FMA.  9 .. 64 rows (bf16 arithmetic): the weight-streaming MFMA route on hi/lo rows — every
  // weight byte once over all CUs, where the tiled GEMM would put a 32-row problem on N / 128 workgroups
  const bool stream_mfma = arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64 && gws && gws_bytes >= mn_skinny_workspace_bytes(M, N, K, MN_EPI_NONE);
  if ((M <= 8 || stream_mfma) && mfma_ok(W, K)) {
    mn_skinny_args a;
    memset(&a, 0, sizeof(a));
    a.x = A; a.ldx = lda; a.w = W; a.ldw = K; a.bias = bias; a.out = C; a.ldo = ldc;
    a.M = M; a.N = N; a.K = K;
    if (M > 8) { a.ws = gws; a.ws_bytes = gws_bytes; }
    return mn_skinny_gemm(&a, stream);
  }
  if (arith == MN_SEQ_ARITH_BF16 && A16 && mfma_ok(W, K) && (lda16 % 8) == 0 && (((uintptr_t)A16) & 15) == 0)
    return mn_gemm_bf16(A16, lda16, W, K, bias, C, ldc, M, N, K, MN_GEMM_F32, stream);
  return mn_gemm_f32_batched(A, lda, 0, W, K, 0, bias, C, ldc, 0, nullptr, 0, 0, nullptr, 0, 0, M, N, K, 1, 1.0f, stream);
}

// act fp32 [M, N] = gelu_tanh(A Wg^T) * (A Wu^T) with W = [Wg ; Wu] (2N rows) as the EPILOGUE of the weight-streaming product, for steps
// that take that route (<= 8 rows, or 9 .. 64 rows with scratch in the bf16 arithmetic).  *done says whether the step
// took it; if not, the caller runs the plain product and the activation launch.
inline int linear_geglu(int arith, int M, const float* A, int64_t lda, const uint16_t* W, int N, int K, float* act, int64_t ldact, void* gws,
                        size_t gws_bytes, void* stream, bool* done) {
  *done = false;
  const bool stream_mfma = arith == MN_SEQ_ARITH_BF16 && M > 8 && M <= 64 && gws && gws_bytes >= mn_skinny_workspace_bytes(M, N, K, MN_EPI_GEGLU_TANH);
  if (!((M <= 8 || stream_mfma) && mfma_ok(W, K))) return MN_OK;
  mn_skinny_args a;
  memset(&a, 0, sizeof(a));
  a.x = A; a.ldx = lda; a.w = W; a.ldw = K; a.out = act; a.ldo = ldact;
  a.M = M; a.N = N; a.K = K; a.epilogue = MN_EPI_GEGLU_TANH;
  if (M > 8) { a.ws = gws; a.ws_bytes = gws_bytes; }
  *done = true;
  return mn_skinny_gemm(&a, stream);
}

// the step's own copy of its input rows (a kernel, not a memcpy node: the step may be captured into a graph)
__global__ void copy_rows_kernel(const float* __restrict__ x, int64_t ldx, float* __restrict__ y, int n) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < n) y[(int64_t)blockIdx.y * n + c] = x[(int64_t)blockIdx.y * ldx + c];
}

}  // namespace
