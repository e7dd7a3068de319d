#include "gemm_common.h"

// ---------------------------------------------------------------------------------------
// The plain product: 32-bit arithmetic for any dtype, one order of summation for every element
// whatever M is, so that logits do not depend on how a step was cut: K goes in segments of SEG; a
// segment's sum runs k ascending from zero, one fused multiply-add a step; the segments' sums are
// added in ascending order, starting from zero.  Two kernels keep to it.  Many rows (M > 64): 64 x 64
// tiles, a workgroup walks all of K.  Few rows: a tile of 8 to 64 rows x 64 columns, and where the
// column tiles alone do not fill the chip every segment is a workgroup of its own, which asks for its
// whole share of W (64 x 128: 32 KB) at once and leaves its sum in a workspace; a second kernel adds
// the segments' sums in order and ends with the epilogue.  (Few rows used to run in the many-rows
// kernel: a hundred workgroups, each walking all of K alone.)
// ---------------------------------------------------------------------------------------
namespace plain {
constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;
constexpr int SEG = 128;

template <typename TC>
__device__ __forceinline__ void finish(float v, int m, int n, const float* bias, TC* C, int ldc, float* resid, int ldr,
                                       int epi) {
  if (bias) v += bias[n];
  if (resid) {
    float* r = resid + static_cast<size_t>(m) * ldr + n;
    *r = *r + v;
  } else {
    C[static_cast<size_t>(m) * ldc + n] = from_float<TC>(apply_epilogue(v, epi));
  }
}

// WHOLE: K is a multiple of 4, so a thread's four elements along K are all inside or all outside
template <typename TI, typename TC, bool WHOLE>
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
  float acc[4][4], tot[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      int m = m0 + lrow, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M && k < K) {
        const TI* p = A + static_cast<size_t>(m) * lda + k;
        if (WHOLE || k + 4 <= K) {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = to_float(p[i]);
        } else {                                        // (K need be no multiple of 4: zeros beyond it)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (k + i < K) v[i] = to_float(p[i]);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) As[lk + i][lrow] = v[i];
      int n = n0 + lrow;
      float w[4] = {0.f, 0.f, 0.f, 0.f};
      if (n < N && k < K) {
        const TI* p = W + static_cast<size_t>(n) * K + k;
        if (WHOLE || k + 4 <= K) {
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = to_float(p[i]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (k + i < K) w[i] = to_float(p[i]);
        }
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
    if ((k0 + BK) % SEG == 0 || k0 + BK >= K) {     // a segment ends: its sum joins the others'
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
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
      finish<TC>(tot[i][j], m, n, bias, C, ldc, resid, ldr, epi);
    }
  }
}

// four consecutive elements in one load (the few-rows kernel is launched only where they are aligned)
__device__ __forceinline__ void load4(const float* p, float* v) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* v) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
}

// Few rows.  A workgroup: RM rows x 64 columns, the segments [seg0, seg0 + nseg) of K.  part == null:
// it owns all segments and ends with the epilogue; else it owns one (blockIdx.z) and writes its sum to
// part[seg][m][n].  A segment's share of W (64 rows x 128 k) and of A is asked for at once, 16 bytes a
// thread and load, eight threads to a row's 128 bytes, and goes through LDS in four slabs of 32.
template <typename TI, typename TC, int RM>
__global__ __launch_bounds__(256) void rows_kernel(const TI* __restrict__ A, int lda, const TI* __restrict__ W,
                                                    const float* __restrict__ bias, TC* __restrict__ C, int ldc,
                                                    float* __restrict__ resid, int ldr, int M, int N, int K, int epi,
                                                    float* __restrict__ part) {
  constexpr int SK = 32;                              // a slab
  constexpr int TN = RM >= 16 ? 4 : 2;                // columns per thread
  constexpr int TM = RM * BN / (256 * TN);            // rows per thread
  constexpr int CG = BN / TN;                         // threads along the columns
  static_assert(TM >= 1 && TM * TN * 256 == RM * BN, "tile");
  __shared__ float As[SK][RM + PAD];
  __shared__ float Ws[SK][BN + PAD];
  const int t = threadIdx.x;
  const int m0 = blockIdx.y * RM, n0 = blockIdx.x * BN;
  const int tx = t % CG, ty = t / CG;
  // loader: thread t takes 4 k at (t % 8) * 4 of row t / 8 (+ 32 for the second half of W's rows), in each slab
  const int lr = t / 8, lk = (t % 8) * 4;
  const int seg_first = part ? blockIdx.z : 0;
  const int seg_last = part ? blockIdx.z + 1 : (K + SEG - 1) / SEG;
  float tot[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) tot[i][j] = 0.f;

  for (int seg = seg_first; seg < seg_last; ++seg) {
    const int kseg = seg * SEG;
    // everything this segment needs, asked for at once
    float wv[SEG / SK][2][4];
    float av[SEG / SK][(RM + 31) / 32][4];
#pragma unroll
    for (int sl = 0; sl < SEG / SK; ++sl) {
      const int k = kseg + sl * SK + lk;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int n = n0 + lr + 32 * hf;
#pragma unroll
        for (int i = 0; i < 4; ++i) wv[sl][hf][i] = 0.f;
        if (n < N && k < K) load4(W + static_cast<size_t>(n) * K + k, wv[sl][hf]);
      }
#pragma unroll
      for (int hf = 0; hf < (RM + 31) / 32; ++hf) {
        const int r = lr + 32 * hf, m = m0 + r;
#pragma unroll
        for (int i = 0; i < 4; ++i) av[sl][hf][i] = 0.f;
        if (r < RM && m < M && k < K) load4(A + static_cast<size_t>(m) * lda + k, av[sl][hf]);
      }
    }
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;
#pragma unroll
    for (int sl = 0; sl < SEG / SK; ++sl) {
      __syncthreads();
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int i = 0; i < 4; ++i) Ws[lk + i][lr + 32 * hf] = wv[sl][hf][i];
#pragma unroll
      for (int hf = 0; hf < (RM + 31) / 32; ++hf)
        if (lr + 32 * hf < RM) {
#pragma unroll
          for (int i = 0; i < 4; ++i) As[lk + i][lr + 32 * hf] = av[sl][hf][i];
        }
      __syncthreads();
      if (kseg + sl * SK < K) {
#pragma unroll
        for (int k = 0; k < SK; ++k) {
          float a[TM], w[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) a[i] = As[k][ty * TM + i];
#pragma unroll
          for (int j = 0; j < TN; ++j) w[j] = Ws[k][tx * TN + j];
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) tot[i][j] += acc[i][j];
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n >= N) continue;
      if (part)
        part[(static_cast<size_t>(blockIdx.z) * M + m) * N + n] = tot[i][j];
      else
        finish<TC>(tot[i][j], m, n, bias, C, ldc, resid, ldr, epi);
    }
  }
}

// Where the key and value columns of a fused projection of few rows go besides C (slot_map == null: nowhere):
// as KVScatter says it, with pools of C's own type.
template <typename TC>
struct KVRows {
  const int32_t* slot_map;
  TC* k_pool;
  TC* v_pool;
  int q_width, kv_width, dh, page_size, Hkv;
};

// the segments' sums of each element, added in ascending order from zero, then the epilogue; the keys and values
// among the columns also go to their tokens' places in the cache, so that no kernel has to copy them there
template <typename TC>
__global__ __launch_bounds__(256) void join_kernel(const float* __restrict__ part, int nseg, const float* __restrict__ bias,
                                                    TC* __restrict__ C, int ldc, float* __restrict__ resid, int ldr,
                                                    int M, int N, int epi, KVRows<TC> kv) {
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (n >= N) return;
  float tot = 0.f;
  const float* p = part + static_cast<size_t>(m) * N + n;
  const size_t step = static_cast<size_t>(M) * N;
  int s = 0;
  for (; s + 8 <= nseg; s += 8) {       // eight loads at a time; the sum keeps its order
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = p[(s + i) * step];
#pragma unroll
    for (int i = 0; i < 8; ++i) tot += v[i];
  }
  for (; s < nseg; ++s) tot += p[s * step];
  finish<TC>(tot, m, n, bias, C, ldc, resid, ldr, epi);
  if (kv.slot_map != nullptr && n >= kv.q_width) {
    const int slot = kv.slot_map[m];
    if (slot < 0) return;
    int c = n - kv.q_width;
    const bool is_value = c >= kv.kv_width;
    if (is_value) c -= kv.kv_width;
    const int page = slot / kv.page_size, off = slot % kv.page_size;
    const int hh = c / kv.dh, d = c % kv.dh;
    const size_t base = (static_cast<size_t>(page) * kv.Hkv + hh) * kv.page_size * kv.dh;
    const TC x = from_float<TC>(apply_epilogue(bias ? tot + bias[n] : tot, epi));      // what finish stored in C
    if (is_value)
      kv.v_pool[base + static_cast<size_t>(d) * kv.page_size + off] = x;
    else
      kv.k_pool[base + static_cast<size_t>(off) * kv.dh + d] = x;
  }
}

constexpr int FEW_ROWS = 64;

// floats of workspace that a product of M rows needs (0: none)
long work_floats(int M, int N, int K) {
  if (M > FEW_ROWS) return 0;
  const int nseg = (K + SEG - 1) / SEG;
  const long tiles = (N + BN - 1) / BN;
  if (nseg < 2 || tiles >= 384) return 0;      // the column tiles alone fill the chip
  return static_cast<long>(nseg) * M * N;
}

// whether the few-rows kernel takes these operands (it loads four elements at a time: rows that do not start
// at multiples of that go the other way)
template <typename TI>
static bool few_rows_take(const void* A, int lda, const void* W, int M, int K) {
  const size_t quad = 4 * sizeof(TI);
  return M <= FEW_ROWS && reinterpret_cast<uintptr_t>(A) % quad == 0 && reinterpret_cast<uintptr_t>(W) % quad == 0 &&
         lda % 4 == 0 && K % 4 == 0;
}

// kv: a fused projection's cache write, done by the kernel that joins the segments (so only where there is one:
// few_rows_take and work_floats > 0)
template <typename TI, typename TC>
static int run(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr, int M,
               int N, int K, int epi, float* work, long have, hipStream_t stream, KVRows<TC> kv = KVRows<TC>{}) {
  const TI* a = static_cast<const TI*>(A);
  const TI* w = static_cast<const TI*>(W);
  TC* c = static_cast<TC*>(C);
  if (!few_rows_take<TI>(A, lda, W, M, K)) {
    if (kv.slot_map) return DN_ERR_SHAPE;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (K % 4 == 0)
      hipLaunchKernelGGL((gemm_kernel<TI, TC, true>), grid, dim3(256), 0, stream, a, lda, w, bias, c, ldc, resid, ldr, M, N,
                         K, epi);
    else
      hipLaunchKernelGGL((gemm_kernel<TI, TC, false>), grid, dim3(256), 0, stream, a, lda, w, bias, c, ldc, resid, ldr, M, N,
                         K, epi);
    return 0;
  }
  const long need = work_floats(M, N, K);
  if (need > 0 && (work == nullptr || have < need)) return DN_ERR_SHAPE;     // dn_gemm_work_floats says how much
  float* part = need > 0 ? work : nullptr;
  if (kv.slot_map && !part) return DN_ERR_SHAPE;
  const int nseg = (K + SEG - 1) / SEG;
  const int rm = M <= 8 ? 8 : M <= 16 ? 16 : M <= 32 ? 32 : 64;
  dim3 grid((N + BN - 1) / BN, (M + rm - 1) / rm, part ? nseg : 1);
#define DN_ROWS(RM)                                                                                                  \
  hipLaunchKernelGGL((rows_kernel<TI, TC, RM>), grid, dim3(256), 0, stream, a, lda, w, bias, c, ldc, resid, ldr, M, N, \
                     K, epi, part)
  if (rm == 8) DN_ROWS(8);
  else if (rm == 16) DN_ROWS(16);
  else if (rm == 32) DN_ROWS(32);
  else DN_ROWS(64);
#undef DN_ROWS
  if (part)
    hipLaunchKernelGGL((join_kernel<TC>), dim3((N + 255) / 256, M), dim3(256), 0, stream, part, nseg, bias, c, ldc, resid,
                       ldr, M, N, epi, kv);
  return 0;
}

// -- what the entry points call (one function per choice of types) ---------------------------------------
int few_rows_take_of(int dtype, const void* A, int lda, const void* W, int M, int K) {
  return dtype == DN_F32 ? few_rows_take<float>(A, lda, W, M, K) : dtype == DN_BF16 ? few_rows_take<bf16_t>(A, lda, W, M, K) : 0;
}

int run_of(int in_dtype, int out_dtype, const void* A, int lda, const void* W, const float* bias, void* C, int ldc,
           float* resid, int ldr, int M, int N, int K, int epilogue, float* work, long have, hipStream_t stream) {
#define DN_LAUNCH(TI, TC) return run<TI, TC>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epilogue, work, have, stream)
  if (in_dtype == DN_F32 && out_dtype == DN_F32) DN_LAUNCH(float, float);
  if (in_dtype == DN_F32 && out_dtype == DN_BF16) DN_LAUNCH(float, bf16_t);
  if (in_dtype == DN_BF16 && out_dtype == DN_BF16) DN_LAUNCH(bf16_t, bf16_t);
  if (in_dtype == DN_BF16 && out_dtype == DN_F32) DN_LAUNCH(bf16_t, float);
#undef DN_LAUNCH
  return DN_ERR_DTYPE;
}

// the fused projection of few rows: C and the pools have the operands' type
int run_qkv_of(int dtype, const void* A, int lda, const void* W, const float* bias, void* C, int ldc, int M, int N, int K,
               const int32_t* slot_map, void* k_pool, void* v_pool, int q_width, int Hkv, int dh, int page_size,
               float* work, long have, hipStream_t stream) {
  if (dtype == DN_F32) {
    KVRows<float> kv{slot_map, static_cast<float*>(k_pool), static_cast<float*>(v_pool), q_width, Hkv * dh, dh, page_size, Hkv};
    return run<float, float>(A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, EPI_NONE, work, have, stream, kv);
  }
  if (dtype == DN_BF16) {
    KVRows<bf16_t> kv{slot_map, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_width, Hkv * dh, dh, page_size,
                      Hkv};
    return run<bf16_t, bf16_t>(A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, EPI_NONE, work, have, stream, kv);
  }
  return DN_ERR_DTYPE;
}

// resid [M, N] += (part[0] + part[1] + ... in this order) + bias
void join_shares(const float* part, int shares, const float* bias, float* resid, int ldr, int M, int N, hipStream_t stream) {
  hipLaunchKernelGGL((join_kernel<float>), dim3((N + 255) / 256, M), dim3(256), 0, stream, part, shares, bias,
                     static_cast<float*>(nullptr), 0, resid, ldr, M, N, EPI_NONE, KVRows<float>{});
}
}  // namespace plain
