// Matrix products  C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias[N])  with every weight held
// [out, in], K contiguous for both operands.  Epilogues: bias, GELU (tanh or erf form),
// or accumulation into the 32-bit residual stream (x += A.W^T + bias).
//
// Three kernels behind dn_gemm.  plain: 32-bit multiply-adds in a fixed order over K, whatever
// M is, so a row's result does not depend on what else is in the batch; it is the whole 32-bit
// path and takes bfloat16 operands too (converted exactly on load).  skinny: bfloat16, up to 64
// rows, MFMA, bound by reading W once (decode).  tiled: bfloat16, many rows, MFMA through LDS
// (prefill).
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


// ---------------------------------------------------------------------------------------
// Few rows (M <= 64), bfloat16: the decode step's products, bound by reading W once.
// A workgroup owns 16 output columns; its waves split K in steps of 32 (wave w takes steps
// w, w + WAVES, ...), each feeding v_mfma_f32_16x16x32_bf16 with 16 bytes of a W row per lane
// straight from memory (lane = column + 16 * (k / 8)) and the matching 16 bytes of up to four
// 16-row blocks of A.  The waves' sums meet in LDS and are added in wave order, so the result
// has one order of summation whatever M is.  No atomics.
// ---------------------------------------------------------------------------------------
namespace skinny {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
constexpr int UNROLL = 4;

template <int MB, int WAVES, typename TC>
__global__ __launch_bounds__(WAVES * 64) void gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                           const bf16_t* __restrict__ W,
                                                           const float* __restrict__ bias, TC* __restrict__ C,
                                                           int ldc, float* __restrict__ resid, int ldr, int M, int N,
                                                           int K, int epi) {
  __shared__ floatx4 red[WAVES][MB][64];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int col = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int n = min(n0 + col, N - 1);          // a tail tile reads the last row again; its result is not stored
  const bf16_t* wrow = W + static_cast<size_t>(n) * K + g * 8;
  const bf16_t* arow[MB];
  bool a_ok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    int row = mb * 16 + col;
    a_ok[mb] = row < M;
    arow[mb] = A + static_cast<size_t>(a_ok[mb] ? row : 0) * lda + g * 8;
  }
  floatx4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int ksteps = (K + 31) / 32;
  for (int ks0 = wave; ks0 < ksteps; ks0 += WAVES * UNROLL) {
    bf16x8 b[UNROLL], a[UNROLL][MB];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      int ks = ks0 + u * WAVES;
      bool ok = ks < ksteps && ks * 32 + g * 8 < K;
      b[u] = ok ? *reinterpret_cast<const bf16x8*>(wrow + ks * 32) : zero;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        a[u][mb] = (ok && a_ok[mb]) ? *reinterpret_cast<const bf16x8*>(arow[mb] + ks * 32) : zero;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][mb], b[u], acc[mb], 0, 0, 0);
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = acc[mb];
  __syncthreads();
  // acc[mb][r] of lane (col, g) is row mb*16 + g*4 + r, column n0 + col
  for (int o = threadIdx.x; o < MB * 64; o += WAVES * 64) {
    int mb = o / 64, ln = o % 64;
    floatx4 s = red[0][mb][ln];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) s += red[w][mb][ln];
    int nn = n0 + ln % 16;
    if (nn >= N) continue;
    float bv = bias ? bias[nn] : 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int m = mb * 16 + (ln / 16) * 4 + r;
      if (m >= M) continue;
      float v = s[r] + bv;
      if (resid) {
        float* x = resid + static_cast<size_t>(m) * ldr + nn;
        *x = *x + v;
      } else {
        C[static_cast<size_t>(m) * ldc + nn] = from_float<TC>(apply_epilogue(v, epi));
      }
    }
  }
}

template <int MB, int WAVES>
static void launch(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr,
                   int M, int N, int K, int out_dtype, int epi, hipStream_t stream) {
  dim3 grid((N + 15) / 16), block(WAVES * 64);
  if (out_dtype == DN_BF16)
    hipLaunchKernelGGL((gemm_kernel<MB, WAVES, bf16_t>), grid, block, 0, stream, static_cast<const bf16_t*>(A), lda,
                       static_cast<const bf16_t*>(W), bias, static_cast<bf16_t*>(C), ldc, resid, ldr, M, N, K, epi);
  else
    hipLaunchKernelGGL((gemm_kernel<MB, WAVES, float>), grid, block, 0, stream, static_cast<const bf16_t*>(A), lda,
                       static_cast<const bf16_t*>(W), bias, static_cast<float*>(C), ldc, resid, ldr, M, N, K, epi);
}

template <int WAVES>
static void launch_mb(int mb, const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid,
                      int ldr, int M, int N, int K, int out_dtype, int epi, hipStream_t stream) {
  switch (mb) {
    case 1: launch<1, WAVES>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, stream); break;
    case 2: launch<2, WAVES>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, stream); break;
    case 3: launch<3, WAVES>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, stream); break;
    default: launch<4, WAVES>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, stream); break;
  }
}

// operands must allow 16-byte loads: K and lda multiples of 8, bases aligned
static bool takes(const void* A, int lda, const void* W, int M, int K, int in_dtype) {
  return in_dtype == DN_BF16 && M <= 64 && K % 8 == 0 && lda % 8 == 0 &&
         reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
}
}  // namespace skinny

extern "C" int dn_gemm(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid,
                       int ldr, int M, int N, int K, int in_dtype, int out_dtype, int epilogue,
                       hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 4 != 0 || lda < K) return DN_ERR_SHAPE;
  if (epilogue < EPI_NONE || epilogue > EPI_GELU_ERF) return DN_ERR_SHAPE;
  if (resid != nullptr && epilogue != EPI_NONE) return DN_ERR_SHAPE;
  if (skinny::takes(A, lda, W, M, K, in_dtype)) {
    int mb = (M + 15) / 16;
    if (K >= 1024)
      skinny::launch_mb<8>(mb, A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epilogue, stream);
    else
      skinny::launch_mb<4>(mb, A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epilogue, stream);
    return dn_launch_status();
  }
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
