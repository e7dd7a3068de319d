// Matrix products  C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias[N])  with every weight held
// [out, in], K contiguous for both operands.  Epilogues: bias, GELU (tanh or erf form),
// or accumulation into the 32-bit residual stream (x += A.W^T + bias).
//
// dn_gemm is the plain kernel: 32-bit multiply-adds in a fixed order over K, whatever M is,
// so a row's result does not depend on what else is in the batch.  It is the whole 32-bit
// path and takes bfloat16 operands too (converted exactly on load).
#include "common.h"

#define EPI_NONE 0
#define EPI_GELU_TANH 1
#define EPI_GELU_ERF 2

__device__ __forceinline__ float apply_epilogue(float v, int epi) {
  if (epi == EPI_GELU_TANH) {
    // crates/denno-engine/src/tensor.rs:1156-1161
    return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
  }
  if (epi == EPI_GELU_ERF) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
  return v;
}

namespace plain {
constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;

template <typename TI, typename TC>
__global__ __launch_bounds__(256) void gemm_kernel(const TI* __restrict__ A, int lda, const TI* __restrict__ W,
                                                    const float* __restrict__ bias, TC* __restrict__ C, int ldc,
                                                    float* __restrict__ resid, int ldr, int M, int N, int K,
                                                    int epi) {
  __shared__ float As[BK][BM + PAD];
  __shared__ float Ws[BK][BN + PAD];
  const int t = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lrow = t / 4, lk = (t % 4) * 4;   // loader: 64 rows x 4 groups of 4 k
  const int tx = t % 16, ty = t / 16;         // computer: 4x4 outputs
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      int m = m0 + lrow, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M && k < K) {
        const TI* p = A + static_cast<size_t>(m) * lda + k;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = to_float(p[i]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) As[lk + i][lrow] = v[i];
      int n = n0 + lrow;
      float w[4] = {0.f, 0.f, 0.f, 0.f};
      if (n < N && k < K) {
        const TI* p = W + static_cast<size_t>(n) * K + k;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = to_float(p[i]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) Ws[lk + i][lrow] = w[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      if (resid) {
        float* r = resid + static_cast<size_t>(m) * ldr + n;
        *r = *r + v;
      } else {
        C[static_cast<size_t>(m) * ldc + n] = from_float<TC>(apply_epilogue(v, epi));
      }
    }
  }
}
}  // namespace plain

extern "C" int dn_gemm(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid,
                       int ldr, int M, int N, int K, int in_dtype, int out_dtype, int epilogue,
                       hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 4 != 0 || lda < K) return DN_ERR_SHAPE;
  if (epilogue < EPI_NONE || epilogue > EPI_GELU_ERF) return DN_ERR_SHAPE;
  if (resid != nullptr && epilogue != EPI_NONE) return DN_ERR_SHAPE;
  dim3 grid((N + plain::BN - 1) / plain::BN, (M + plain::BM - 1) / plain::BM), block(256);
#define DN_LAUNCH(TI, TC)                                                                                     \
  hipLaunchKernelGGL((plain::gemm_kernel<TI, TC>), grid, block, 0, stream, static_cast<const TI*>(A), lda,    \
                     static_cast<const TI*>(W), bias, static_cast<TC*>(C), ldc, resid, ldr, M, N, K, epilogue)
  if (in_dtype == DN_F32 && out_dtype == DN_F32)
    DN_LAUNCH(float, float);
  else if (in_dtype == DN_F32 && out_dtype == DN_BF16)
    DN_LAUNCH(float, bf16_t);
  else if (in_dtype == DN_BF16 && out_dtype == DN_BF16)
    DN_LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == DN_BF16 && out_dtype == DN_F32)
    DN_LAUNCH(bf16_t, float);
  else
    return DN_ERR_DTYPE;
#undef DN_LAUNCH
  return dn_launch_status();
}
