// Matrix products  C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias[N])  with every weight held
// [out, in], K contiguous for both operands.  Epilogues: bias, GELU (tanh or erf form),
// or accumulation into the 32-bit residual stream (x += A.W^T + bias).
//
// Four kernels behind dn_gemm.  plain: 32-bit multiply-adds in a fixed order over K, whatever
// M is, so a row's result does not depend on what else is in the batch; it is the whole 32-bit
// path and takes bfloat16 operands too (converted exactly on load).  skinny: bfloat16, up to 256
// rows, MFMA, waves split K, bound by reading W once (decode, and steps of a few short prompt
// portions).  direct: bfloat16, many rows, MFMA, slabs from memory straight into LDS, the tile
// chosen per product (prefill).  tiled: the same sizes through registers into swizzled LDS; it takes
// what direct refuses (K no multiple of 32, rows or a bias that do not allow 16-byte accesses).
//
// The MFMA kernels take W packed (dn_pack_matrix): blocks of 16 rows x 32 columns, block
// (n / 16, k / 32) at ((n / 16) * ceil(K / 32) + k / 32) * 512 elements, and inside a block the
// 8 elements k % 32 / 8 * 8 .. + 7 of row n % 16 at ((k % 32 / 8) * 16 + n % 16) * 8: the 16 bytes
// that lane (n % 16) + 16 * (k % 32 / 8) feeds to v_mfma_f32_16x16x32_bf16.  A wave then reads 1 KB
// in one piece per block; from rows of K elements the same load touches 16 cache lines per
// group of 16 lanes, and the rate of those lookups, not of bytes, bounds the kernel.  Rows and
// columns beyond N and K are zeros.
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

// The same for the MFMA kernels, whose results are rounded to bfloat16: the tanh form as
// v / (1 + 2^(-2 log2(e) u)) with the hardware's exponential and reciprocal (a dozen instructions
// where tanhf takes several dozen, which shows in the epilogue of a product with many columns).
__device__ __forceinline__ float apply_epilogue_fast(float v, int epi) {
  if (epi == EPI_GELU_TANH) {
    const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-2.8853900817779268f * u));
  }
  if (epi == EPI_GELU_ERF) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
  return v;
}

// Where a fused projection's key and value columns go besides C: columns q_width .. of row m are
// the keys, then the values, of the token whose slot is slot_map[m] (page * page_size + offset,
// < 0: none).  Pools as in the cache: keys [page, Hkv, page_size, dh], values [page, Hkv, dh, page_size].
struct KVScatter {
  const int32_t* slot_map;
  bf16_t* k_pool;
  bf16_t* v_pool;
  int q_width, kv_width, dh, page_size, Hkv;
  int c_cols;     // columns of C that are stored: all of them, or q_width (nobody reads keys and values from C)
  int page_shift; // log2(page_size) where that is a power of two, else -1 (kv_scatter_for sets it)
};

static int page_shift_of(int page_size) {
  int s = 0;
  while ((1 << s) < page_size) ++s;
  return (1 << s) == page_size ? s : -1;
}

// a slot's page and offset: a shift and a mask where the page size allows it (a division by a number known
// only at run time is some forty instructions, and the kernels' epilogues do two per token or per value)
__device__ __forceinline__ void page_and_offset(const KVScatter& kv, int slot, int& page, int& off) {
  if (kv.page_shift >= 0) {
    page = slot >> kv.page_shift;
    off = slot & (kv.page_size - 1);
  } else {
    page = slot / kv.page_size;
    off = slot % kv.page_size;
  }
}


// The same for four columns nn .. nn + 3 (nn a multiple of 4, so they are one head's): a key's
// four dims are 8 bytes side by side.
__device__ __forceinline__ void scatter_kv4(const KVScatter& kv, int m, int nn, const bf16_t* cv) {
  if (nn < kv.q_width) return;
  int c = nn - kv.q_width;
  const bool is_value = c >= kv.kv_width;
  if (is_value) c -= kv.kv_width;
  const int slot = kv.slot_map[m];
  if (slot < 0) return;
  int page, off;
  page_and_offset(kv, slot, page, off);
  const int hh = c / kv.dh, d = c % kv.dh;
  const size_t base = (static_cast<size_t>(page) * kv.Hkv + hh) * kv.page_size * kv.dh;
  if (is_value) {
#pragma unroll
    for (int e = 0; e < 4; ++e) kv.v_pool[base + static_cast<size_t>(d + e) * kv.page_size + off] = cv[e];
  } else {
    *reinterpret_cast<uint2*>(kv.k_pool + base + static_cast<size_t>(off) * kv.dh + d) =
        *reinterpret_cast<const uint2*>(cv);
  }
}

// slot: the row's entry of the slot map (a kernel that ends with this asks for it when it starts)
__device__ __forceinline__ void scatter_kv_at(const KVScatter& kv, int slot, int nn, bf16_t cv) {
  if (nn < kv.q_width) return;
  int c = nn - kv.q_width;
  const bool is_value = c >= kv.kv_width;
  if (is_value) c -= kv.kv_width;
  if (slot < 0) return;
  int page, off;
  page_and_offset(kv, slot, page, off);
  const int hh = c / kv.dh, d = c % kv.dh;
  const size_t base = (static_cast<size_t>(page) * kv.Hkv + hh) * kv.page_size * kv.dh;
  if (is_value)
    kv.v_pool[base + static_cast<size_t>(d) * kv.page_size + off] = cv;
  else
    kv.k_pool[base + static_cast<size_t>(off) * kv.dh + d] = cv;
}

__device__ __forceinline__ void scatter_kv(const KVScatter& kv, int m, int nn, bf16_t cv) {
  scatter_kv_at(kv, kv.slot_map[m], nn, cv);
}

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
static long work_floats(int M, int N, int K) {
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
}  // namespace plain


// ---------------------------------------------------------------------------------------
// Few rows (M <= 256), bfloat16: the decode step's products, bound by reading W once.
// A workgroup owns 16, 32 or 64 output columns; its waves split K in steps of 32 (wave w takes
// steps w, w + WAVES, ...), each feeding v_mfma_f32_16x16x32_bf16 with one packed block of W per
// 16 columns straight from memory (16 bytes per lane) and the matching 16 bytes of up to four
// 16-row blocks of A (lane = row + 16 * (k / 8)).  The waves' sums meet in LDS and are added in
// wave order, so the result has one order of summation whatever M is.  No atomics.
// ---------------------------------------------------------------------------------------
#define PACKED_W 1
#define PACKED_A 2
#define PACKED_C 4

namespace skinny {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

// The norm that stands between two such products of few rows runs inside them (NORM_OUT in the product before
// it, NORM_IN in the one after), so that it is no kernel of its own: a LayerNorm of a few rows is
// all launch and latency and no work.  With y = (x - mean) / sqrt(var + eps) * gamma + beta
// (crates/denno-engine/src/tensor.rs:1101-1112),
//     y . W^T + b = ((x * gamma) . W^T - mean * c1) / sqrt(var + eps) + c2,
//     c1[n] = sum_k gamma[k] W[n,k],  c2[n] = sum_k beta[k] W[n,k] + b[n]      (made once per weight),
// so the product itself runs on rows that are not normalised, and the norm is two numbers per row in
// the epilogue.  NORM_OUT: a product that adds into the residual stream also stores the updated rows
// times gamma (the next norm's), rounded to bfloat16, and, for each row, the mean and the sum of
// squared distances from it of its 16 columns.  NORM_IN: A is such a copy; each wave joins two rows'
// N / 16 pairs (means are averaged; the squares add up with 16 times the squared distance of each
// block's mean from the row's: exact, and as stable as two passes over the row) while the operands
// travel, and wave 0 applies them at the end.  The rows are rounded to bfloat16 before the mean is
// taken off, not after: right where a row's mean is not large beside its spread.
struct NormIO {
  const float* stats_in;     // NORM_IN: [M][blocks_in][2]
  int blocks_in;             // K / 16
  const float* c1;           // NORM_IN: [N]  (c2 comes as the bias)
  float eps;
  int no_mean;               // NORM_IN: the norm takes no mean off (x / sqrt(mean(x^2) + eps) * gamma): the row's mean counts as 0
  const float* gamma_out;    // NORM_OUT: [N] the next norm's weight
  bf16_t* copy_out;          // NORM_OUT: [M, ldcopy] the updated rows times gamma_out in bfloat16
  int ldcopy;
  float* stats_out;          // NORM_OUT: [M][N / 16][2]
};
#define NORM_NONE 0
#define NORM_IN 1
#define NORM_OUT 2


// MB row blocks and NB column blocks of 16 per workgroup; U steps of K in flight per wave.
template <int MB, int NB, int WAVES, int U, typename TC, bool KV, int NORM = NORM_NONE>
__global__ __launch_bounds__(WAVES * 64) void gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                           const bf16_t* __restrict__ W,
                                                           const float* __restrict__ bias, TC* __restrict__ C,
                                                           int ldc, float* __restrict__ resid, int ldr, int M, int N,
                                                           int K, int epi, int packed, KVScatter kv, NormIO nio) {
  constexpr int BLOCKS = MB * NB;                          // 16 x 16 blocks of C in this workgroup
  constexpr int PASSES = (BLOCKS + WAVES - 1) / WAVES;     // wave w finishes blocks w, w + WAVES, ...
  __shared__ floatx4 red[WAVES][BLOCKS][64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;   // (a scalar: what follows from it is the scalar unit's work)
  const int col = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * (16 * NB);
  const int row0 = blockIdx.y * (MB * 16);     // the rows may be shared out among workgroups too (blockIdx.y)
  const int ksteps = (K + 31) / 32, nblocks = (N + 15) / 16;
  const bf16_t* wblk[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    // a block beyond N reads the last one again; its result is not stored
    const int blk = min(blockIdx.x * NB + nb, nblocks - 1);
    wblk[nb] = W + (static_cast<size_t>(blk) * ksteps * 64 + lane) * 8;
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // what the epilogue will read (bias, the residual stream) is asked for first of all
  float epi_bias[PASSES];
  float epi_x[PASSES][4];
  int epi_slot[KV ? PASSES : 1][4];
  float epi_norm[NORM != NORM_NONE ? PASSES : 1];          // NORM_IN: c1 of the lane's column; NORM_OUT: the next norm's gamma
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int blk = wave + p * WAVES;
    epi_bias[p] = 0.f;
    if constexpr (NORM != NORM_NONE) {
      const int nn = min(n0 + (blk < BLOCKS ? blk % NB : 0) * 16 + col, N - 1);
      epi_norm[p] = NORM == NORM_IN ? nio.c1[nn] : nio.gamma_out[nn];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) epi_x[p][r] = 0.f;
    if constexpr (KV) {
#pragma unroll
      for (int r = 0; r < 4; ++r) epi_slot[p][r] = -1;
    }
    if (blk < BLOCKS) {
      const int mb = blk / NB, nb = blk % NB;
      const int nn = min(n0 + nb * 16 + col, N - 1);
      if (bias) epi_bias[p] = bias[nn];
      if constexpr (KV) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = row0 + mb * 16 + g * 4 + r;
          epi_slot[p][r] = m < M ? kv.slot_map[m] : -1;
        }
      }
      if (resid) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = min(row0 + mb * 16 + g * 4 + r, M - 1);
          epi_x[p][r] = resid[static_cast<size_t>(m) * ldr + nn];
        }
      }
    }
  }
  // NORM_IN: wave w joins the statistics of rows w, w + WAVES, ...: their pairs are asked for now, before
  // the operands (up to SP * 64 blocks of 16 columns a row)
  constexpr int SP = 2, SR = MB * 16 / WAVES;
  __shared__ float rowstat[NORM == NORM_IN ? MB * 16 : 1][2];
  float2 st[NORM == NORM_IN ? SR : 1][SP];
  if constexpr (NORM == NORM_IN) {
#pragma unroll
    for (int t = 0; t < SR; ++t) {
      const int row = min(row0 + wave + t * WAVES, M - 1);
#pragma unroll
      for (int i = 0; i < SP; ++i)
        st[t][i] = *reinterpret_cast<const float2*>(nio.stats_in + (static_cast<size_t>(row) * nio.blocks_in + min(lane + 64 * i, nio.blocks_in - 1)) * 2);
    }
  }
  // Loads are never conditional and nothing uses a loaded value before all loads of a round are
  // issued (a predicated load, or a use in between, makes each load wait for the one before it).
  // A step beyond K reads W's first block instead (finite numbers) and meets a zeroed piece of A.
  // The first round of W is on its way while the rest of the prologue works.
  bf16x8 b[U][NB];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int ks = 2 * (wave + (u / 2) * WAVES) + u % 2;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      b[u][nb] = *reinterpret_cast<const bf16x8*>(ks < ksteps ? wblk[nb] + ks * 512 : W + lane * 8);
  }

  // A in rows, or packed like W (PACKED_A): then a wave reads 1 KB in one piece per block
  const bf16_t* arow[MB];
  const bf16_t* asafe[MB];
  bool a_ok[MB];
  const int astep = (packed & PACKED_A) ? 512 : 32;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    int row = row0 + mb * 16 + col;
    a_ok[mb] = row < M;
    // (a block of rows beyond M, where MB is more than the rows need, reads the last one again: packed
    // rows end with the block that holds row M - 1)
    arow[mb] = (packed & PACKED_A) ? A + (static_cast<size_t>(min(static_cast<int>(blockIdx.y) * MB + mb, (M + 15) / 16 - 1)) * ksteps * 64 + lane) * 8
                                   : A + static_cast<size_t>(a_ok[mb] ? row : 0) * lda + g * 8;
    // where a step's piece lies beyond K the load goes to an address that is surely inside A instead: the start
    // of the row (with K < 32 the row's piece g itself may lie beyond the row, and the last row's beyond A)
    asafe[mb] = (packed & PACKED_A) ? arow[mb] : A + static_cast<size_t>(a_ok[mb] ? row : 0) * lda;
  }
  // NORM_IN: the rows' means and 1 / sqrt(var + eps), joined while the first round of operands travels (a
  // wave does it in its first turn of the loop below, which every wave has: K >= 1024); the finishing
  // waves meet them behind the barrier further down
  auto join_stats = [&]() {
    const float blocks = static_cast<float>(nio.blocks_in);
#pragma unroll
    for (int t = 0; t < SR; ++t) {
      const int row = wave + t * WAVES;
      float sm = 0.f;
#pragma unroll
      for (int i = 0; i < SP; ++i)
        if (lane + 64 * i < nio.blocks_in) sm += st[t][i].x;
      const float mean = nio.no_mean ? 0.f : wave_sum(sm) / blocks;      // (without it the squares are taken about 0)
      float sq = 0.f;
#pragma unroll
      for (int i = 0; i < SP; ++i)
        if (lane + 64 * i < nio.blocks_in) {
          const float d = st[t][i].x - mean;
          sq += st[t][i].y + 16.f * d * d;
        }
      const float var = wave_sum(sq) / (16.f * blocks);
      if (lane == 0) {
        rowstat[row][0] = row0 + row < M ? mean : 0.f;
        rowstat[row][1] = row0 + row < M ? 1.0f / sqrtf(var + nio.eps) : 0.f;
      }
    }
  };
  floatx4 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the steps go to the waves in pairs: wave w takes steps 2w, 2w + 1, 2 (w + WAVES), ... (the same
  // shares as in gemm16_kernel, so that both sum in the same order)
  for (int p0 = wave; 2 * p0 < ksteps; p0 += WAVES * (U / 2)) {
    bf16x8 a[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = 2 * (p0 + (u / 2) * WAVES) + u % 2;
      const bool ok = ks < ksteps && ks * 32 + g * 8 < K;
      if (p0 != wave) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          b[u][nb] = *reinterpret_cast<const bf16x8*>(ks < ksteps ? wblk[nb] + ks * 512 : W + lane * 8);
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        a[u][mb] = *reinterpret_cast<const bf16x8*>(ok ? arow[mb] + ks * astep : asafe[mb]);
    }
    if constexpr (NORM == NORM_IN) {
      if (p0 == wave) join_stats();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = 2 * (p0 + (u / 2) * WAVES) + u % 2;
      const bool ok = ks < ksteps && ks * 32 + g * 8 < K;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        if (!(ok && a_ok[mb])) a[u][mb] = zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][mb], b[u][nb], acc[mb][nb], 0, 0, 0);
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) red[wave][mb * NB + nb][lane] = acc[mb][nb];
  __syncthreads();
  // acc[mb][nb][r] of lane (col, g) is row mb*16 + g*4 + r, column n0 + nb*16 + col
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int blk = wave + p * WAVES;
    if (blk >= BLOCKS) break;
    const int mb = blk / NB, nb = blk % NB;
    const int nn = n0 + nb * 16 + col;
    floatx4 s = red[0][blk][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) s += red[w][blk][lane];
    if constexpr (NORM == NORM_OUT) {
      // a row's 16 columns of this block lie in the 16 lanes of a row of lanes (N is a multiple of 16)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float x = epi_x[p][r] + (s[r] + epi_bias[p]);
        const float mean = group_reduce<16>(x, SumOp()) * (1.0f / 16.0f);
        const float d = x - mean;
        const float sq = group_reduce<16>(d * d, SumOp());
        const int m = row0 + mb * 16 + g * 4 + r;
        if (col == 0 && m < M)
          *reinterpret_cast<float2*>(nio.stats_out + (static_cast<size_t>(m) * nblocks + blockIdx.x * NB + nb) * 2) = float2{mean, sq};
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int m = row0 + mb * 16 + g * 4 + r;
      if (m >= M || nn >= N) continue;
      float v = s[r] + epi_bias[p];
      if constexpr (NORM == NORM_IN) v = (s[r] - rowstat[m - row0][0] * epi_norm[p]) * rowstat[m - row0][1] + epi_bias[p];
      if (resid) {
        resid[static_cast<size_t>(m) * ldr + nn] = epi_x[p][r] + v;
        if constexpr (NORM == NORM_OUT)
          nio.copy_out[nio.ldcopy > 0 ? static_cast<size_t>(m) * nio.ldcopy + nn : packed_index(m, nn, N / 32)] =
              from_float<bf16_t>((epi_x[p][r] + v) * epi_norm[p]);
      } else {
        TC cv = from_float<TC>(apply_epilogue_fast(v, epi));
        if (!KV || nn < kv.c_cols)
          C[(packed & PACKED_C) ? packed_index(m, nn, N / 32) : static_cast<size_t>(m) * ldc + nn] = cv;
        if constexpr (KV) scatter_kv_at(kv, epi_slot[p][r], nn, cv);
      }
    }
  }
}

// Up to 16 rows of A in rows.  In the operands' layout 16 lanes are 16 rows, and a load of A from
// memory touches as many cache lines (four times as many lookups as the packed W costs, and they
// were what this product of 8 rows waited for).  Here a wave takes the steps of K in pairs
// (wave w: steps 2w, 2w + 1, then 2 (w + WAVES), ...), so that a row's share of a pair is one cache
// line of 128 bytes; it loads A eight lanes to a row, turns each pair round through a piece of LDS
// of its own (no barrier: a wave's LDS operations keep their order) and reads the operands from
// there, two pairs at a time through two such pieces, so that the way into LDS and out of it is
// waited for once per two pairs.  16 columns per workgroup, sums joined through LDS in wave order, as in gemm_kernel.
template <int WAVES, typename TC, bool KV, int NORM, bool TWO>
__global__ __launch_bounds__(WAVES * 64) void gemm16_kernel(const bf16_t* __restrict__ A, int lda,
                                                             const bf16_t* __restrict__ W,
                                                             const float* __restrict__ bias, TC* __restrict__ C,
                                                             int ldc, float* __restrict__ resid, int ldr, int M,
                                                             int N, int K, int epi, KVScatter kv, NormIO nio) {
  typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
  constexpr int U = 4;                                     // pairs of steps in flight per wave
  constexpr int ROW = 9 * 8;                               // elements per row of a wave's piece: 8 chunks and one of padding
  __shared__ floatx4 red[WAVES][64];
  constexpr int PIECES = 2;                                // pairs turned round at a time
  static_assert(U % PIECES == 0, "pairs in flight come in whole groups");
  __shared__ __attribute__((aligned(16))) bf16_t turn[WAVES][PIECES][16 * ROW];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int col = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int ksteps = (K + 31) / 32, npairs = (ksteps + 1) / 2, nblocks = (N + 15) / 16;
  const bf16_t* wblk = W + (static_cast<size_t>(min(static_cast<int>(blockIdx.x), nblocks - 1)) * ksteps * 64 + lane) * 8;
  // (TWO: rows 8 .. 15 need a second load per pair)
  // NORM_IN: the rows' pairs of statistics are asked for before the operands (loads come back in the
  // order asked): wave w joins rows w, w + WAVES, ...; a lane holds up to SP pairs of a row
  constexpr int SP = 4, SR = 16 / WAVES;
  __shared__ float rowstat[16][2];
  // what the epilogue will read is asked for first of all (wave 0 finishes the block)
  float epi_bias = 0.f;
  float epi_x[4] = {0.f, 0.f, 0.f, 0.f};
  int epi_slot[4] = {-1, -1, -1, -1};
  if (wave == 0) {
    const int nn = min(n0 + col, N - 1);
    if (bias) epi_bias = bias[nn];
    if constexpr (KV) {
#pragma unroll
      for (int r = 0; r < 4; ++r) epi_slot[r] = g * 4 + r < M ? kv.slot_map[g * 4 + r] : -1;
    }
    if (resid) {
#pragma unroll
      for (int r = 0; r < 4; ++r) epi_x[r] = resid[static_cast<size_t>(min(g * 4 + r, M - 1)) * ldr + nn];
    }
  }
  // (after the epilogue's loads and before the operands': they are back before the operands are)
  float2 st[SR][SP];
  float epi_c1 = 0.f, epi_gamma = 1.f;
  if constexpr (NORM == NORM_IN) {
#pragma unroll
    for (int t = 0; t < SR; ++t) {
      const int row = min(wave + t * WAVES, M - 1);
#pragma unroll
      for (int i = 0; i < SP; ++i)
        st[t][i] = *reinterpret_cast<const float2*>(nio.stats_in + (static_cast<size_t>(row) * nio.blocks_in + min(lane + 64 * i, nio.blocks_in - 1)) * 2);
    }
    epi_c1 = nio.c1[min(n0 + col, N - 1)];
  }
  if constexpr (NORM == NORM_OUT) epi_gamma = nio.gamma_out[min(n0 + col, N - 1)];
  // never a conditional load; a step beyond K reads W's first block and meets zeros of A
  const int lrow = lane / 8, lch = lane % 8;               // as loader: row and 16-byte chunk of the pair's 128 bytes
  const bf16_t* a0 = A + static_cast<size_t>(min(lrow, M - 1)) * lda + lch * 8;
  const bf16_t* a1 = A + static_cast<size_t>(min(lrow + 8, M - 1)) * lda + lch * 8;
  // a chunk beyond K is not loaded; its load goes to the start of the row instead, which is surely inside A (a0
  // itself is not where K < 64: chunk lch of a row of 32 elements lies in the next row, the last row's beyond A)
  const bf16_t* asafe = A + static_cast<size_t>(min(lrow, M - 1)) * lda;
  bf16_t* mine = turn[wave][0];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  // a round: U pairs of steps per wave, all its loads issued at once (asking for the next round
  // before this one is used, into a second set of registers, was slower)
  auto ask = [&](int p0, bf16x8 (*b)[2], u32x4 (*al)[2]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * WAVES, ks = 2 * p;
      b[u][0] = *reinterpret_cast<const bf16x8*>(ks < ksteps ? wblk + ks * 512 : W + lane * 8);
      b[u][1] = *reinterpret_cast<const bf16x8*>(ks + 1 < ksteps ? wblk + (ks + 1) * 512 : W + lane * 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * WAVES;
      const bool ok = p * 64 + lch * 8 < K;
      al[u][0] = *reinterpret_cast<const u32x4*>(ok ? a0 + p * 64 : asafe);
      if constexpr (TWO) al[u][1] = *reinterpret_cast<const u32x4*>(ok ? a1 + p * 64 : asafe);
    }
  };
  auto use = [&](int p0, const bf16x8 (*b)[2], const u32x4 (*al)[2]) {
#pragma unroll
    for (int u0 = 0; u0 < U; u0 += PIECES) {
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const int p = p0 + (u0 + i) * WAVES;
        const bool ok = p < npairs && p * 64 + lch * 8 < K;
        bf16_t* piece = mine + i * 16 * ROW;
        *reinterpret_cast<u32x4*>(piece + lrow * ROW + lch * 8) = ok ? al[u0 + i][0] : zero4;
        if constexpr (TWO) *reinterpret_cast<u32x4*>(piece + (lrow + 8) * ROW + lch * 8) = ok ? al[u0 + i][1] : zero4;
      }
      // as operand: lane (row col, chunk g) of each of a pair's two steps
      bf16x8 f[PIECES][2];
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const bf16_t* piece = mine + i * 16 * ROW;
        f[i][0] = *reinterpret_cast<const bf16x8*>(piece + col * ROW + g * 8);
        f[i][1] = *reinterpret_cast<const bf16x8*>(piece + col * ROW + (4 + g) * 8);
      }
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[i][0], b[u0 + i][0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[i][1], b[u0 + i][1], acc, 0, 0, 0);
      }
    }
  };
  bf16x8 b0[U][2];
  u32x4 al0[U][2];
  // NORM_IN: the first round is asked for by every wave, with or without steps of its own (so that the
  // wait for the statistics, which were asked for before, counts these loads exactly and depends on
  // no branch), and the rows' statistics are joined while it travels
  if (NORM == NORM_IN || wave < npairs) ask(wave, b0, al0);
  if constexpr (NORM == NORM_IN) {
    // the rows' means and 1 / sqrt(var + eps) for wave 0, which meets them behind the barrier further down
    const float blocks = static_cast<float>(nio.blocks_in);
#pragma unroll
    for (int t = 0; t < SR; ++t) {
      const int row = wave + t * WAVES;
      float sm = 0.f;
#pragma unroll
      for (int i = 0; i < SP; ++i)
        if (lane + 64 * i < nio.blocks_in) sm += st[t][i].x;
      const float mean = nio.no_mean ? 0.f : wave_sum(sm) / blocks;      // (without it the squares are taken about 0)
      float sq = 0.f;
#pragma unroll
      for (int i = 0; i < SP; ++i)
        if (lane + 64 * i < nio.blocks_in) {
          const float d = st[t][i].x - mean;
          sq += st[t][i].y + 16.f * d * d;
        }
      const float var = wave_sum(sq) / (16.f * blocks);
      if (lane == 0) {
        rowstat[row][0] = row < M ? mean : 0.f;
        rowstat[row][1] = row < M ? 1.0f / sqrtf(var + nio.eps) : 0.f;
      }
    }
  }
  for (int p0 = wave; p0 < npairs; p0 += WAVES * U) {
    if (p0 != wave) ask(p0, b0, al0);
    use(p0, b0, al0);
  }
  red[wave][lane] = acc;
  __syncthreads();
  // acc[r] of lane (col, g) is row g*4 + r, column n0 + col
  if (wave == 0) {
    const int nn = n0 + col;
    floatx4 sm = red[0][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sm += red[w][lane];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = g * 4 + r;
      if (m >= M || nn >= N) continue;
      float v = sm[r] + epi_bias;
      if constexpr (NORM == NORM_IN) v = (sm[r] - rowstat[m][0] * epi_c1) * rowstat[m][1] + epi_bias;
      if (resid) {
        resid[static_cast<size_t>(m) * ldr + nn] = epi_x[r] + v;
        if constexpr (NORM == NORM_OUT)
          nio.copy_out[static_cast<size_t>(m) * nio.ldcopy + nn] = from_float<bf16_t>((epi_x[r] + v) * epi_gamma);
      } else {
        const TC cv = from_float<TC>(apply_epilogue_fast(v, epi));
        if (!KV || nn < kv.c_cols) C[static_cast<size_t>(m) * ldc + nn] = cv;
        if constexpr (KV) scatter_kv_at(kv, epi_slot[r], nn, cv);
      }
    }
    if constexpr (NORM == NORM_OUT) {
      // a row's 16 columns of this block lie in the 16 lanes of a row of lanes (N is a multiple of 16)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float x = epi_x[r] + (sm[r] + epi_bias);
        const float mean = group_reduce<16>(x, SumOp()) * (1.0f / 16.0f);
        const float d = x - mean;
        const float sq = group_reduce<16>(d * d, SumOp());
        const int m = g * 4 + r;
        if (col == 0 && m < M)
          *reinterpret_cast<float2*>(nio.stats_out + (static_cast<size_t>(m) * nblocks + blockIdx.x) * 2) = float2{mean, sq};
      }
    }
  }
}

struct Call {
  const void* A; int lda; const void* W; const float* bias; void* C; int ldc; float* resid; int ldr;
  int M, N, K, out_dtype, epi, packed;
  const KVScatter* kv;
};

template <int MB, int NB, int WAVES, int U, typename TC, bool KV>
static void launch_one(const Call& c, hipStream_t stream) {
  // (MB row blocks per workgroup: where the rows need more, the second grid dimension shares them out)
  dim3 grid((c.N + 16 * NB - 1) / (16 * NB), ((c.M + 15) / 16 + MB - 1) / MB), block(WAVES * 64);
  KVScatter kv = c.kv ? *c.kv : KVScatter{};
  hipLaunchKernelGGL((gemm_kernel<MB, NB, WAVES, U, TC, KV>), grid, block, 0, stream,
                     static_cast<const bf16_t*>(c.A), c.lda, static_cast<const bf16_t*>(c.W), c.bias,
                     static_cast<TC*>(c.C), c.ldc, c.resid, c.ldr, c.M, c.N, c.K, c.epi, c.packed, kv, NormIO{});
}

// the same with the norm before the product (NORM_IN: bfloat16 out) or after it (NORM_OUT: into the
// residual stream), for 17 to 64 rows
template <int MB, int NB, int WAVES, int U>
static void launch_norm(const Call& c, const NormIO& nio, int norm, hipStream_t stream) {
  dim3 grid((c.N + 16 * NB - 1) / (16 * NB), ((c.M + 15) / 16 + MB - 1) / MB), block(WAVES * 64);
  KVScatter kv = c.kv ? *c.kv : KVScatter{};
#define DN_LN(TC, KV, NORM)                                                                                        \
  hipLaunchKernelGGL((gemm_kernel<MB, NB, WAVES, U, TC, KV, NORM>), grid, block, 0, stream,                       \
                     static_cast<const bf16_t*>(c.A), c.lda, static_cast<const bf16_t*>(c.W), c.bias,             \
                     static_cast<TC*>(c.C), c.ldc, c.resid, c.ldr, c.M, c.N, c.K, c.epi, c.packed, kv, nio)
  if (norm == NORM_OUT)
    DN_LN(float, false, NORM_OUT);
  else if (c.kv)
    DN_LN(bf16_t, true, NORM_IN);
  else
    DN_LN(bf16_t, false, NORM_IN);
#undef DN_LN
}

// 17 to 64 rows with a norm inside: the shapes that launch_mb picks for these rows (8 waves: K >= 1024)
static void launch_mb_norm(const Call& c, const NormIO& nio, int norm, hipStream_t stream) {
  const int mb = (c.M + 15) / 16;
  if (c.N >= 2560) {
    switch (mb) {
      // (four steps in flight a wave: with six, the norm's sums beside them no longer fit the registers, and the
      // product that also scatters keys and values took 24 us where it takes 13)
      case 2: return launch_norm<2, 2, 8, 4>(c, nio, norm, stream);
      case 3: return launch_norm<3, 2, 8, 4>(c, nio, norm, stream);
      default: return launch_norm<4, 2, 8, 4>(c, nio, norm, stream);
    }
  }
  // (few columns: the rows in two halves, so that there are workgroups for all CUs)
  return launch_norm<2, 1, 8, 8>(c, nio, norm, stream);
}

template <int MB, int NB, int WAVES, int U>
static void launch(const Call& c, hipStream_t stream) {
  if (c.kv) return launch_one<MB, NB, WAVES, U, bf16_t, true>(c, stream);
  if (c.out_dtype == DN_BF16) return launch_one<MB, NB, WAVES, U, bf16_t, false>(c, stream);
  return launch_one<MB, NB, WAVES, U, float, false>(c, stream);
}

template <int WAVES, typename TC, bool KV>
static void launch16_one(const Call& c, hipStream_t stream) {
  KVScatter kv = c.kv ? *c.kv : KVScatter{};
  if (c.M > 8)
    hipLaunchKernelGGL((gemm16_kernel<WAVES, TC, KV, NORM_NONE, true>), dim3((c.N + 15) / 16), dim3(WAVES * 64), 0, stream,
                       static_cast<const bf16_t*>(c.A), c.lda, static_cast<const bf16_t*>(c.W), c.bias,
                       static_cast<TC*>(c.C), c.ldc, c.resid, c.ldr, c.M, c.N, c.K, c.epi, kv, NormIO{});
  else
    hipLaunchKernelGGL((gemm16_kernel<WAVES, TC, KV, NORM_NONE, false>), dim3((c.N + 15) / 16), dim3(WAVES * 64), 0, stream,
                       static_cast<const bf16_t*>(c.A), c.lda, static_cast<const bf16_t*>(c.W), c.bias,
                       static_cast<TC*>(c.C), c.ldc, c.resid, c.ldr, c.M, c.N, c.K, c.epi, kv, NormIO{});
}

// the same with the norm before the product (NORM_IN: bfloat16 out) or after it (NORM_OUT: into the residual stream)
template <int WAVES>
static void launch16_norm(const Call& c, const NormIO& nio, int norm, hipStream_t stream) {
  KVScatter kv = c.kv ? *c.kv : KVScatter{};
  const dim3 grid((c.N + 15) / 16), block(WAVES * 64);
#define DN_L16_ROWS(TC, KV, NORM, TWO)                                                                                   \
  hipLaunchKernelGGL((gemm16_kernel<WAVES, TC, KV, NORM, TWO>), grid, block, 0, stream, static_cast<const bf16_t*>(c.A), \
                     c.lda, static_cast<const bf16_t*>(c.W), c.bias, static_cast<TC*>(c.C), c.ldc, c.resid, c.ldr,       \
                     c.M, c.N, c.K, c.epi, kv, nio)
#define DN_L16(TC, KV, NORM)                 \
  do {                                       \
    if (c.M > 8)                             \
      DN_L16_ROWS(TC, KV, NORM, true);       \
    else                                     \
      DN_L16_ROWS(TC, KV, NORM, false);      \
  } while (0)
  if (norm == NORM_OUT)
    DN_L16(float, false, NORM_OUT);
  else if (c.kv)
    DN_L16(bf16_t, true, NORM_IN);
  else
    DN_L16(bf16_t, false, NORM_IN);
#undef DN_L16
#undef DN_L16_ROWS
}

template <int WAVES>
static void launch16(const Call& c, hipStream_t stream) {
  if (c.kv) return launch16_one<WAVES, bf16_t, true>(c, stream);
  if (c.out_dtype == DN_BF16) return launch16_one<WAVES, bf16_t, false>(c, stream);
  return launch16_one<WAVES, float, false>(c, stream);
}

// With more than 16 rows every workgroup reads all of A (16 cache lines per load and 16 lanes,
// as A lies in rows), so wider workgroups read less in total, as long as enough of them remain
// to keep the memory system busy: 2 column blocks per workgroup from 2,560 columns on (with 2,304 columns
// that way was the slower), 4 from 32,768 on, else 1.
template <int WAVES>
static void launch_mb(const Call& c, hipStream_t stream) {
  const int mb = (c.M + 15) / 16;
  // 65 to 256 rows of a product with few columns and a short K (an output projection): four row blocks and two
  // column blocks per workgroup, the rows shared out among workgroups (at 1,600 x 1,600: 6.7 us at 128 rows and 8.0
  // at 256, where sixteen row blocks x one column block took 7.7 and 12.6: every workgroup read all rows)
  if (mb > 4 && c.N < 2048 && c.K < 4096) return launch<4, 2, WAVES, 4>(c, stream);
  if (mb == 1 && !(c.packed & (PACKED_A | PACKED_C)) && c.M > 1) return launch16<WAVES>(c, stream);
  if (mb == 1) return launch<1, 1, WAVES, 8>(c, stream);
  if (mb > 4) {
    // 65 to 256 rows: 16 columns per workgroup, the waves' sums for all row blocks through LDS
    // (the tiled kernel has too few tiles to fill the chip at so few rows, and walks a long K in
    // as many steps whatever M is)
    if (mb <= 6) return launch<6, 1, WAVES, 2>(c, stream);
    if (mb <= 8) return launch<8, 1, WAVES, 2>(c, stream);
    if (mb <= 12) return launch<12, 1, WAVES, 2>(c, stream);
    return launch<16, 1, WAVES, 2>(c, stream);
  }
  if (c.N >= 32768) {
    switch (mb) {
      case 2: return launch<2, 4, WAVES, 4>(c, stream);
      case 3: return launch<3, 4, WAVES, 4>(c, stream);
      default: return launch<4, 4, WAVES, 4>(c, stream);
    }
  }
  if (c.N >= 2560) {
    // (six steps in flight a wave: with K = 1,600 a wave's seven steps are one round and a step, where four in
    // flight made two rounds: 4,800 and 6,400 columns at 64 rows 10.3 -> 9.6 and 10.0 -> 9.1 us)
    switch (mb) {
      case 2: return launch<2, 2, WAVES, 6>(c, stream);
      case 3: return launch<3, 2, WAVES, 6>(c, stream);
      default: return launch<4, 2, WAVES, 6>(c, stream);
    }
  }
  // (few columns: the rows in two halves, so that there are workgroups for all CUs)
  return launch<2, 1, WAVES, 8>(c, stream);
}

static void run(const Call& c, hipStream_t stream) {
  if (c.K >= 1024)
    launch_mb<8>(c, stream);
  else
    launch_mb<4>(c, stream);
}

// A must allow 16-byte loads: in rows with K and lda multiples of 8 and the base aligned, or packed
// (K a multiple of 32 then: nothing zeroes a packed block's columns beyond K); W is packed
static bool takes(const void* A, int lda, const void* W, int M, int K, int packed) {
  if (M > 256 || reinterpret_cast<uintptr_t>(A) % 16 != 0 || reinterpret_cast<uintptr_t>(W) % 16 != 0) return false;
  return (packed & PACKED_A) ? K % 32 == 0 : (K % 8 == 0 && lda % 8 == 0);
}
}  // namespace skinny


// ---------------------------------------------------------------------------------------
// Many rows, bfloat16: the prefill's products, bound by the matrix cores.
// A workgroup of WM x 2 waves makes a tile of C; each wave makes 2 x 2 tiles of
// v_mfma_f32_32x32x16_bf16, a 64 x 64 share (4 x 2 tiles per wave were measured slower: their
// registers leave room for one wave per SIMD only, and nothing then hides the latency of LDS).
// Two waves per SIMD are asked for.  K advances BK (64 or 32) at a time through two sets of slabs in LDS: while the
// matrix cores work on one set, the next slabs travel from memory to registers and then into
// the other set; one barrier per step.  In LDS a row is BK/8 chunks of 16 bytes, chunk c stored
// at c ^ swz(row), so that the rows a lane group reads fall on different banks.
// Workgroup ids are remapped so that tiles which share a slab of W run on the same XCD (each
// XCD has its own L2; ids go round the 8 XCDs).
// ---------------------------------------------------------------------------------------
namespace tiled {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
constexpr int XCDS = 8;

template <typename TC, int WM, int TM, int TN, int BK, bool KV>
__global__ __launch_bounds__(WM * 128) __attribute__((amdgpu_waves_per_eu(2))) void gemm_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    TC* __restrict__ C, int ldc, float* __restrict__ resid, int ldr, int M, int N, int K, int epi, int tiles_m,
    int tiles_n, KVScatter kv) {
  constexpr int THREADS = WM * 128;                       // WM x 2 waves
  constexpr int BM = WM * 32 * TM, BN = 64 * TN;
  constexpr int CH = BK / 8;                              // 16-byte chunks in a row of a slab
  constexpr int KS = BK / 32;                             // packed blocks of W along K in a slab
  const int ksteps = (K + 31) / 32, nblocks = (N + 15) / 16;
  constexpr int UA = BM * CH / THREADS, UW = BN * CH / THREADS;   // chunks per thread and slab
  // a row's chunk c lies at c ^ swz(row): 16 consecutive rows then cover all 16 bank groups
  auto swz = [](int row) { return (row / (16 / CH)) % CH; };
  extern __shared__ u32x4 lds[];                          // [2][(BM + BN) * CH]
  // logical tile: consecutive ids on one XCD walk down a column of tiles (same slab of W)
  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if (total % XCDS == 0) pid = (pid % XCDS) * (total / XCDS) + pid / XCDS;   // a permutation if 8 divides total
  const int tm = pid % tiles_m, tn = pid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;
  const int t = threadIdx.x, wave = t / 64, lane = t % 64;
  const int wm = (wave / 2) * (BM / WM), wn = (wave % 2) * (BN / 2);
  const int r32 = lane % 32, g = lane / 32;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 pa[UA], pw[UW];
  // never a conditional load, and no use between loads: an address outside is replaced by one
  // inside; what lies outside of A is zeroed afterwards, what lies outside of W meets those zeros
  // or is not stored
  auto fetch = [&](int kt) {
#pragma unroll
    for (int u = 0; u < UA; ++u) {
      const int c = t + u * THREADS, row = c / CH, ch = c % CH;
      const int k = kt * BK + ch * 8, m = m0 + row;
      const bool ok = k < K && m < M;
      pa[u] = *reinterpret_cast<const u32x4*>(A + static_cast<size_t>(ok ? m : 0) * lda + (ok ? k : 0));
    }
    // W is packed: 64 consecutive threads take one block of 16 rows x 32 columns, 1 KB in one piece
#pragma unroll
    for (int u = 0; u < UW; ++u) {
      const int c = t + u * THREADS, blk = c / 64, in = c % 64;
      const int ks = kt * KS + blk % KS, nblk = n0 / 16 + blk / KS;
      const bool ok = ks < ksteps && nblk < nblocks;
      pw[u] = *reinterpret_cast<const u32x4*>(W + (ok ? (static_cast<size_t>(nblk) * ksteps + ks) * 512 + in * 8 : 0));
    }
  };
  auto stash = [&](int kt, u32x4* As, u32x4* Ws) {
#pragma unroll
    for (int u = 0; u < UA; ++u) {
      const int c = t + u * THREADS, row = c / CH, ch = c % CH;
      const bool ok = kt * BK + ch * 8 < K && m0 + row < M;
      As[row * CH + (ch ^ swz(row))] = ok ? pa[u] : zero;
    }
    // 16 consecutive lanes write the same chunk of 16 consecutive rows: no two on one bank
#pragma unroll
    for (int u = 0; u < UW; ++u) {
      const int c = t + u * THREADS, blk = c / 64, in = c % 64;
      const int row = (blk / KS) * 16 + in % 16, ch = (blk % KS) * 4 + in / 16;
      Ws[row * CH + (ch ^ swz(row))] = pw[u];
    }
  };
  const int ktiles = (K + BK - 1) / BK;
  constexpr int SET = (BM + BN) * CH;
  fetch(0);
  stash(0, lds, lds + BM * CH);
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const u32x4* As = lds + (kt & 1) * SET;
    const u32x4* Ws = As + BM * CH;
    if (kt + 1 < ktiles) fetch(kt + 1);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[TM], wf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm + i * 32 + r32;
        af[i] = __builtin_bit_cast(bf16x8, As[row * CH + ((kk * 2 + g) ^ swz(row))]);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn + j * 32 + r32;
        wf[j] = __builtin_bit_cast(bf16x8, Ws[row * CH + ((kk * 2 + g) ^ swz(row))]);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ktiles) {
      u32x4* An = lds + ((kt + 1) & 1) * SET;
      stash(kt + 1, An, An + BM * CH);
    }
    __syncthreads();     // the next set is written and this one has been read by every wave
  }
  // acc[i][j][r]: row m0 + wm + 32 i + 8 (r / 4) + 4 g + r % 4, column n0 + wn + 32 j + lane % 32:
  // a lane holds one column, so stores straight from the accumulators would be 2 or 4 bytes at a
  // stride of a row.  Each wave turns its 32 x 32 blocks round through a piece of LDS of its own
  // (the slabs are done with: the loop ended at a barrier) and stores 16 bytes per lane along rows.
  // Rows that do not allow that (a width or leading dimension that is no multiple of 4) take the
  // element-wise path.
  const bool vec = N % 4 == 0 && (resid ? ldr % 4 == 0 && reinterpret_cast<uintptr_t>(resid) % 16 == 0
                                        : ldc % 4 == 0 && reinterpret_cast<uintptr_t>(C) % 16 == 0);
  if (vec) {
    constexpr int RS = 40;                               // floats per row of the piece: no bank shared by the two halves
    float* piece = reinterpret_cast<float*>(lds) + wave * (32 * RS);
    const int prow = lane / 8, pcol = (lane % 8) * 4;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int nb = n0 + wn + j * 32;
      const float bv = (bias && nb + r32 < N) ? bias[nb + r32] : 0.f;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float v = acc[i][j][r] + bv;
          piece[(8 * (r / 4) + 4 * g + (r % 4)) * RS + r32] = resid ? v : apply_epilogue_fast(v, epi);
        }
        if constexpr (KV) {
          // A block of value columns: a value's place in its page is [dim][offset], so four rows
          // (tokens) whose slots follow one another from an offset that is a multiple of 4 are 8
          // bytes side by side for one dim.  Lane = column, and the block is read down its columns.
          if (nb >= kv.q_width + kv.kv_width && nb >= kv.c_cols) {
            const int cc = nb + r32 - kv.q_width - kv.kv_width, hh = cc / kv.dh, d = cc % kv.dh;
#pragma unroll
            for (int it = 0; it < 4; ++it) {
              const int lr = it * 8 + g * 4, m = m0 + wm + i * 32 + lr;
              alignas(8) bf16_t cv[4];
              int slot[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                cv[e] = from_float<bf16_t>(piece[(lr + e) * RS + r32]);
                slot[e] = m + e < M ? kv.slot_map[m + e] : -1;
              }
              if (nb + r32 >= N) continue;
              const bool run = kv.page_size % 4 == 0 && slot[0] >= 0 && slot[0] % 4 == 0 && slot[1] == slot[0] + 1 && slot[2] == slot[0] + 2 &&
                               slot[3] == slot[0] + 3;
              if (run) {
                int page, off;
                page_and_offset(kv, slot[0], page, off);
                *reinterpret_cast<uint2*>(kv.v_pool + ((static_cast<size_t>(page) * kv.Hkv + hh) * kv.dh + d) * kv.page_size +
                                          off) = *reinterpret_cast<const uint2*>(cv);
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  if (slot[e] < 0) continue;
                  int page, off;
                  page_and_offset(kv, slot[e], page, off);
                  kv.v_pool[((static_cast<size_t>(page) * kv.Hkv + hh) * kv.dh + d) * kv.page_size + off] = cv[e];
                }
              }
            }
            continue;
          }
        }
        const int n = nb + pcol;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int lr = it * 8 + prow, m = m0 + wm + i * 32 + lr;
          const floatx4 v = *reinterpret_cast<const floatx4*>(piece + lr * RS + pcol);
          if (m >= M || n >= N) continue;
          if (resid) {
            floatx4* x = reinterpret_cast<floatx4*>(resid + static_cast<size_t>(m) * ldr + n);
            *x = *x + v;
          } else if constexpr (sizeof(TC) == 4) {
            *reinterpret_cast<floatx4*>(C + static_cast<size_t>(m) * ldc + n) = v;
          } else {
            alignas(8) bf16_t cv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) cv[e] = from_float<bf16_t>(v[e]);
            if (!KV || n < kv.c_cols)
              *reinterpret_cast<uint2*>(C + static_cast<size_t>(m) * ldc + n) = *reinterpret_cast<const uint2*>(cv);
            if constexpr (KV) scatter_kv4(kv, m, n, cv);
          }
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn + j * 32 + r32;
    if (n >= N) continue;
    const float bv = bias ? bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + 8 * (r / 4) + 4 * g + (r % 4);
        if (m >= M) continue;
        float v = acc[i][j][r] + bv;
        if (resid) {
          float* x = resid + static_cast<size_t>(m) * ldr + n;
          *x = *x + v;
        } else {
          const TC cv = from_float<TC>(apply_epilogue_fast(v, epi));
          if (!KV || n < kv.c_cols) C[static_cast<size_t>(m) * ldc + n] = cv;
          if constexpr (KV) scatter_kv(kv, m, n, cv);
        }
      }
  }
}

static bool takes(const void* A, int lda, const void* W, int K) {
  return K % 8 == 0 && lda % 8 == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(W) % 16 == 0;
}

template <typename TC, int WM, int TM, int TN, int BK, bool KV>
static int launch(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr,
                  int M, int N, int K, int epi, const KVScatter* kv, hipStream_t stream) {
  constexpr int BM = WM * 32 * TM, BN = 64 * TN;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t lds = 2 * static_cast<size_t>(BM + BN) * (BK / 8) * 16;
  static bool raised = false;      // more than 64 KB of LDS has to be asked for once per kernel
  if (lds > 65536 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<TC, WM, TM, TN, BK, KV>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
    raised = true;
  }
  hipLaunchKernelGGL((gemm_kernel<TC, WM, TM, TN, BK, KV>), dim3(tiles_m * tiles_n), dim3(WM * 128), lds, stream,
                     static_cast<const bf16_t*>(A), lda, static_cast<const bf16_t*>(W), bias, static_cast<TC*>(C), ldc,
                     resid, ldr, M, N, K, epi, tiles_m, tiles_n, kv ? *kv : KVScatter{});
  return 0;
}

template <int WM, int BK, int TM = 2>
static int launch_bk(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr,
                     int M, int N, int K, int out_dtype, int epi, const KVScatter* kv, hipStream_t stream) {
  if (kv) return launch<bf16_t, WM, TM, 2, BK, true>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epi, kv, stream);
  if (out_dtype == DN_BF16)
    return launch<bf16_t, WM, TM, 2, BK, false>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epi, nullptr, stream);
  return launch<float, WM, TM, 2, BK, false>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epi, nullptr, stream);
}

static int run(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr, int M,
               int N, int K, int out_dtype, int epi, const KVScatter* kv, hipStream_t stream) {
  // Where 128 x 128 tiles would be many (two or more per CU), a workgroup of 8 waves takes 256 x 128
  // with slabs of 32 along K: each slab of W serves twice the rows.  Else 4 waves, 128 x 128, slabs
  // of 64 (half the barriers).
  const long tiles = static_cast<long>((M + 127) / 128) * ((N + 127) / 128);
  if (tiles >= 512) return launch_bk<4, 32>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, kv, stream);
  // Fewer tiles than CUs: 64 x 128 tiles (each wave 32 x 64) make twice as many workgroups.
  if (tiles < 256 && M > 64)
    return launch_bk<2, 64, 1>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, kv, stream);
  return launch_bk<2, 64>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epi, kv, stream);
}
}  // namespace tiled

// ---------------------------------------------------------------------------------------
// Many rows, bfloat16, slabs carried from memory straight into LDS (global_load_lds_dwordx4: 16
// bytes per lane, lane l's at the wave's LDS address + 16 l, no register and no LDS store between).
// A slab of 32 along K is a list of 1 KB blocks in the packed layout, 16 rows x 32 columns each:
// a block of W is 1 KB of memory as it lies and is read back at 16 l by lane l; a block of A is
// made by the load itself, in an order of its own: the vector cache looks a load's lines up per 16
// lanes, so 16 lanes take 64 bytes from each of four rows (four lines) and not 16 bytes from each of
// sixteen (with a lane per row the lookups, 52 per load on average, kept the cache busy for three
// quarters of the kernel's time), and the four 16-byte pieces of a row are exchanged by the row's
// number so that the operand read (lane l wants row l % 16, piece l / 16) meets every bank once.  STAGES slabs are in flight (vmcnt counts a wave's
// own loads; one barrier per slab publishes them and frees the slab read before).
//
// The MFMA takes W as its first operand and A as its second: a lane then holds four consecutive
// columns of one row of C, which it stores as 8 bytes (bfloat16) or adds as 16 (the 32-bit
// residual) without a turn through LDS; for the fused QKV product they are one key's or one
// value's four dims.
//
// What bounds these products here is the traffic from L2 into the CUs and the rounding of tiles to
// 256 CUs, not the matrix cores: measured per tile and slab, time = 2.26e-7 us x BM x BN (matrix
// cores at nine tenths of their peak) + 3.07e-5 us x (BM + BN) (loads), the two adding up rather
// than overlapping, + 1.9e-4 us x BM x BN for the stores at the end.  So the tile is chosen per
// product from a list, by that model: the largest that still fills the chip in whole rounds
// (a tile count just above a multiple of 256 costs a whole further round).
// ---------------------------------------------------------------------------------------
namespace direct {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
constexpr int XCDS = 8, CUS = 256, LDS_PER_CU = 160 * 1024;

// not a template: the host pass must not see the builtin inside one
__device__ __forceinline__ void load_to_lds(const void* src, void* dst) {
  __builtin_amdgcn_global_load_lds(src, dst, 16, 0, 0);
}

// element `which` (0..3, the lane's own choice) of the vector that lane E of this lane's quad holds
template <int E>
__device__ __forceinline__ float quad_pick(const floatx4& v, int which) {
  const float b0 = dpp_move<0x55 * E>(v[0]), b1 = dpp_move<0x55 * E>(v[1]), b2 = dpp_move<0x55 * E>(v[2]),
              b3 = dpp_move<0x55 * E>(v[3]);
  return which == 0 ? b0 : which == 1 ? b1 : which == 2 ? b2 : b3;
}

// four values rounded to bfloat16, as the 8 bytes of one store (built in registers: an array that
// is read back through a pointer of another type can end up in scratch memory)
__device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
  return uint2{static_cast<uint32_t>(from_float<bf16_t>(a).bits) | static_cast<uint32_t>(from_float<bf16_t>(b).bits) << 16,
               static_cast<uint32_t>(from_float<bf16_t>(c).bits) | static_cast<uint32_t>(from_float<bf16_t>(d).bits) << 16};
}

template <int N>
__device__ __forceinline__ void wait_loads() {      // until at most N of this wave's loads are in flight
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// WM x WN waves, each TM x TN blocks of 16 x 16: the tile is 16 WM TM rows x 16 WN TN columns
template <typename TC, int WM, int WN, int TM, int TN, int STAGES, bool KV, int KB = 1>
__global__ __launch_bounds__(WM * WN * 64) void gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                           const bf16_t* __restrict__ W, const float* __restrict__ bias,
                                                           TC* __restrict__ C, int ldc, float* __restrict__ resid, int ldr,
                                                           int M, int N, int K, int epi, int packed, int tiles_m,
                                                           int tiles_n, KVScatter kv, float* __restrict__ part,
                                                           int split_slabs) {
  constexpr int NW = WM * WN;
  constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
  constexpr int AB = BM / 16, WB = BN / 16;              // 1 KB blocks per slab of 32 along K
  constexpr int PER = (AB + WB) * KB;                    // blocks per stage: KB slabs travel and are multiplied together
  constexpr int SLAB = PER * 64;                         // a stage, in u32x4
  constexpr int HI = (PER + NW - 1) / NW, REM = PER % NW;   // waves below REM load HI blocks, the others HI - 1
  static_assert((STAGES - 2) * HI < 64, "vmcnt has six bits");
  extern __shared__ u32x4 lds[];
  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if (total % XCDS == 0) pid = (pid % XCDS) * (total / XCDS) + pid / XCDS;   // an XCD walks down a column of tiles
  const int tm = pid % tiles_m, tn = pid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;
  const int lane = threadIdx.x % 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int wmb = (wave / WN) * TM, wnb = (wave % WN) * TN;     // in blocks
  // part: K is shared out among the workgroups of blockIdx.y, split_slabs slabs each; a workgroup leaves
  // its sums in part[blockIdx.y][m][n] and a second kernel adds them in order and ends with the epilogue
  // (stages of KB slabs: the host launches KB > 1 only where K is a multiple of 32 KB; split_slabs counts stages)
  const int kall = K / 32, nblocks = (N + 15) / 16;
  const int first = part ? blockIdx.y * split_slabs : 0;
  const int ksteps = part ? min(split_slabs, kall / KB - first) : kall / KB;
  // where the 16 bytes of row lane % 16, columns 8 (lane / 16) .. of a block of A lie in its 1 KB
  // (see the loads below): any 8 and any 16 consecutive lanes read all banks once
  // (a packed A is in the operand's order already: lane l reads at 16 l)
  const int aslot = (packed & PACKED_A) ? lane : 16 * (lane % 4) + 4 * ((lane % 16) / 4) + ((lane / 16) ^ (lane % 4));

  floatx4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // where this lane's share of each of the wave's blocks starts; a row beyond M or a block of
  // columns beyond N is replaced by the last inside (its results are not stored)
  const bf16_t* src[HI];
  int step[HI];
#pragma unroll
  for (int u = 0; u < HI; ++u) {
    const int q = min(wave + u * NW, PER - 1);
    const int b = q % (AB + WB), kb = q / (AB + WB);      // block b of the stage's slab kb
    if (b < AB) {
      // 16 lanes in a row take 64 bytes from each of four rows (g, g + 4, g + 8, g + 12 of the block):
      // four cache lines, where a lane per row would touch sixteen
      const int g = lane / 16, h = (lane % 16) / 4, piece = (lane % 4) ^ g;
      if (packed & PACKED_A) {      // a block of packed rows is 1 KB as it lies, like a block of W
        src[u] = A + static_cast<size_t>(min(m0 / 16 + b, (M + 15) / 16 - 1)) * kall * 512 + lane * 8;
        step[u] = 512;
      } else {
        src[u] = A + static_cast<size_t>(min(m0 + b * 16 + 4 * h + g, M - 1)) * lda + piece * 8;
        step[u] = 32;
      }
    } else {
      src[u] = W + static_cast<size_t>(min(n0 / 16 + b - AB, nblocks - 1)) * kall * 512 + lane * 8;
      step[u] = 512;
    }
    src[u] += (static_cast<size_t>(first) * KB + kb) * step[u];
    step[u] *= KB;
  }
  auto issue = [&](int kt) {
    u32x4* slab = lds + (kt % STAGES) * SLAB;
#pragma unroll
    for (int u = 0; u < HI; ++u) {
      const int q = wave + u * NW;
      if (u < HI - 1 || REM == 0 || wave < REM) load_to_lds(src[u] + static_cast<size_t>(kt) * step[u], slab + q * 64);
    }
  };
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < ksteps) issue(s);
  for (int kt = 0; kt < ksteps; ++kt) {
    // slab kt of this wave has landed when only the loads of the STAGES - 2 slabs after it are out
    if (kt + STAGES - 2 < ksteps) {
      if (REM == 0 || wave < REM)
        wait_loads<(STAGES - 2) * HI>();
      else
        wait_loads<(STAGES - 2) * (HI - 1)>();
    } else {
      wait_loads<0>();
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();      // every wave's share of slab kt is there, and slab kt - 1 has been read
    if (kt + STAGES - 1 < ksteps) issue(kt + STAGES - 1);
    const u32x4* slab = lds + (kt % STAGES) * SLAB;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const u32x4* sl = slab + kb * (AB + WB) * 64;
      bf16x8 af[TM], wf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = __builtin_bit_cast(bf16x8, sl[(wmb + i) * 64 + aslot]);
#pragma unroll
      for (int j = 0; j < TN; ++j) wf[j] = __builtin_bit_cast(bf16x8, sl[(AB + wnb + j) * 64 + lane]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
    }
  }
  // acc[i][j][r]: row m0 + 16 (wmb + i) + lane % 16, column n0 + 16 (wnb + j) + 4 (lane / 16) + r
  //
  // Where the fused projection's keys and values go is worked out once per row, outside the loop over
  // the column blocks (a slot's page and offset are divisions by numbers known only at run time; done
  // per block and lane they cost more than the product's own epilogue).  Keys: the lane's row.  Values:
  // in its page a value lies as [dim][offset], so four tokens whose slots follow one another from a
  // multiple of 4 are 8 bytes side by side for one dim: the four lanes of a quad, which hold four
  // tokens x four dims, exchange them (a 4 x 4 turn), and each stores four tokens of one dim.
  int kpage[KV ? TM : 1], koff[KV ? TM : 1], vpage[KV ? TM : 1], voff[KV ? TM : 1];
  int vslot[KV ? TM : 1][4];      // the quad's four tokens' slots, for values that do not lie side by side (decoded tokens)
  if constexpr (KV) {
#pragma clang loop unroll(full)
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + (wmb + i) * 16 + lane % 16, mq = m - lane % 4;
      const int slot = m < M ? kv.slot_map[m] : -1;
      page_and_offset(kv, max(slot, 0), kpage[i], koff[i]);
      if (slot < 0) kpage[i] = -1, koff[i] = 0;
      int sq[4];
#pragma clang loop unroll(full)
      for (int e = 0; e < 4; ++e) sq[e] = mq + e < M ? kv.slot_map[mq + e] : -1;
      const bool run = kv.page_size % 4 == 0 && sq[0] >= 0 && sq[0] % 4 == 0 && sq[1] == sq[0] + 1 && sq[2] == sq[0] + 2 &&
                       sq[3] == sq[0] + 3;
      page_and_offset(kv, max(sq[0], 0), vpage[i], voff[i]);
      if (!run) vpage[i] = -1, voff[i] = 0;
#pragma clang loop unroll(full)
      for (int e = 0; e < 4; ++e) vslot[i][e] = sq[e];
    }
  }
  if (part) {
#pragma clang loop unroll(full)
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + (wnb + j) * 16 + (lane / 16) * 4;
      if (n >= N) continue;
#pragma clang loop unroll(full)
      for (int i = 0; i < TM; ++i) {
        const int m = m0 + (wmb + i) * 16 + lane % 16;
        if (m < M) *reinterpret_cast<floatx4*>(part + (static_cast<size_t>(blockIdx.y) * M + m) * N + n) = acc[i][j];
      }
    }
    return;
  }
  // every load of the epilogue before its first store: a wait for a load is a wait for the stores
  // issued before it as well (one counter), and a load per column block made the blocks take turns
  floatx4 bvs[TN];
#pragma clang loop unroll(full)
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + (wnb + j) * 16 + (lane / 16) * 4;
    bvs[j] = bias && n < N ? *reinterpret_cast<const floatx4*>(bias + n) : floatx4{0.f, 0.f, 0.f, 0.f};
  }
#pragma clang loop unroll(full)
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + (wnb + j) * 16 + (lane / 16) * 4;
    if (n >= N) continue;
    const floatx4 bv = bvs[j];
    // the block's place among the keys or the values: head hh, dims d .. d + 3 (a block of 16 columns is
    // all queries, all keys or all values, and of one head: the widths are multiples of 16)
    bool is_key = false, is_value = false;
    int hh = 0, d = 0;
    if constexpr (KV) {
      is_key = n >= kv.q_width && n < kv.q_width + kv.kv_width;
      is_value = n >= kv.q_width + kv.kv_width;
      const int c = n - kv.q_width - (is_value ? kv.kv_width : 0);
      hh = c / kv.dh, d = c % kv.dh;
    }
#pragma clang loop unroll(full)
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + (wmb + i) * 16 + lane % 16;
      if (m >= M) continue;
      const floatx4 v = acc[i][j] + bv;
      if (resid) {
        floatx4* x = reinterpret_cast<floatx4*>(resid + static_cast<size_t>(m) * ldr + n);
        *x = *x + v;
      } else if constexpr (sizeof(TC) == 4) {
        floatx4 o;
#pragma clang loop unroll(full)
        for (int r = 0; r < 4; ++r) o[r] = apply_epilogue_fast(v[r], epi);
        *reinterpret_cast<floatx4*>(C + static_cast<size_t>(m) * ldc + n) = o;
      } else {
        const uint2 cv = pack4(apply_epilogue_fast(v[0], epi), apply_epilogue_fast(v[1], epi), apply_epilogue_fast(v[2], epi),
                               apply_epilogue_fast(v[3], epi));
        // (in packed rows, four columns from a multiple of 4 are 8 bytes side by side too)
        if (!KV || n < kv.c_cols)
          *reinterpret_cast<uint2*>(C + ((packed & PACKED_C) ? packed_index(m, n, N / 32) : static_cast<size_t>(m) * ldc + n)) = cv;
        if constexpr (KV) {
          if (is_key && kpage[i] >= 0)
            *reinterpret_cast<uint2*>(kv.k_pool + ((static_cast<size_t>(kpage[i]) * kv.Hkv + hh) * kv.page_size + koff[i]) * kv.dh +
                                      d) = cv;
        }
      }
    }
    if constexpr (KV) {
      if (is_value) {
        const int q = lane % 4;       // this lane's dim of the four after the turn
#pragma clang loop unroll(full)
        for (int i = 0; i < TM; ++i) {
          const int mq = m0 + (wmb + i) * 16 + (lane % 16) / 4 * 4;      // the quad's first token
          const floatx4 v = acc[i][j] + bv;
          // token mq + e, dim d + q: lane e of the quad holds it in v[q]
          const float t0 = quad_pick<0>(v, q), t1 = quad_pick<1>(v, q), t2 = quad_pick<2>(v, q), t3 = quad_pick<3>(v, q);
          if (vpage[i] >= 0) {
            *reinterpret_cast<uint2*>(kv.v_pool + ((static_cast<size_t>(vpage[i]) * kv.Hkv + hh) * kv.dh + d + q) * kv.page_size +
                                      voff[i]) = pack4(t0, t1, t2, t3);
          } else {
#pragma clang loop unroll(full)
            for (int e = 0; e < 4; ++e) {
              const int slot = vslot[i][e];
              if (slot < 0) continue;
              int page, off;
              page_and_offset(kv, slot, page, off);
              kv.v_pool[((static_cast<size_t>(page) * kv.Hkv + hh) * kv.dh + d + q) * kv.page_size + off] =
                  from_float<bf16_t>(e == 0 ? t0 : e == 1 ? t1 : e == 2 ? t2 : t3);
            }
          }
        }
      }
    }
  }
}

// everything 16 bytes at a time: slabs of 32 along K, rows of A and C (or the residual) and the bias
static bool takes(const void* A, int lda, const void* W, const float* bias, const void* C, int ldc, const float* resid,
                  int ldr, int N, int K, int out_dtype, int packed) {
  auto aligned = [](const void* p, int a) { return reinterpret_cast<uintptr_t>(p) % a == 0; };
  if (K % 32 != 0 || N % 4 != 0 || !aligned(A, 16) || !aligned(W, 16) || !aligned(bias, 16)) return false;
  if (!(packed & PACKED_A) && lda % 8 != 0) return false;
  if (resid) return ldr % 4 == 0 && aligned(resid, 16);
  if (packed & PACKED_C) return N % 32 == 0 && out_dtype == DN_BF16 && aligned(C, 8);
  return ldc % 4 == 0 && aligned(C, out_dtype == DN_F32 ? 16 : 8);
}

struct Args {
  const void* A; int lda; const void* W; const float* bias; void* C; int ldc; float* resid; int ldr;
  int M, N, K, out_dtype, epi, packed; const KVScatter* kv;
  float* part = nullptr; int splits = 1;       // part: K in `splits` shares, their sums in part[share][m][n]
};

template <typename TC, int WM, int WN, int TM, int TN, int STAGES, bool KV, int KB = 1>
static int launch(const Args& a, hipStream_t stream) {
  constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  constexpr size_t lds = static_cast<size_t>(STAGES) * KB * (BM + BN) / 16 * 1024;
  if (a.K % (32 * KB) != 0) return DN_ERR_SHAPE;
  static bool raised = false;      // more than 64 KB of LDS has to be asked for once per kernel
  if (lds > 65536 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<TC, WM, WN, TM, TN, STAGES, KV, KB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
    raised = true;
  }
  const int split_slabs = (a.K / (32 * KB) + a.splits - 1) / a.splits;
  hipLaunchKernelGGL((gemm_kernel<TC, WM, WN, TM, TN, STAGES, KV, KB>), dim3(tiles_m * tiles_n, a.part ? a.splits : 1),
                     dim3(WM * WN * 64), lds, stream, static_cast<const bf16_t*>(a.A), a.lda,
                     static_cast<const bf16_t*>(a.W), a.bias, static_cast<TC*>(a.C), a.ldc, a.resid, a.ldr, a.M, a.N, a.K,
                     a.epi, a.packed, tiles_m, tiles_n, a.kv ? *a.kv : KVScatter{}, a.part, split_slabs);
  return 0;
}

template <int WM, int WN, int TM, int TN, int STAGES, int KB = 1>
static int launch_as(const Args& a, hipStream_t stream) {
  if (a.kv) return launch<bf16_t, WM, WN, TM, TN, STAGES, true, KB>(a, stream);
  if (a.out_dtype == DN_BF16 && !a.resid) return launch<bf16_t, WM, WN, TM, TN, STAGES, false, KB>(a, stream);
  return launch<float, WM, WN, TM, TN, STAGES, false, KB>(a, stream);
}

// The tiles on offer: rows x columns, slabs in flight.  256 rows: 8 waves as 4 x 2, one workgroup
// per CU; the small ones leave room for several workgroups per CU.  64 x 64 and 32 x 64 (4 waves) are
// for products with few rows and a long K, whose larger tiles would leave most CUs idle.
struct Shape { int bm, bn, stages; };
constexpr Shape SHAPES[] = {{64, 128, 4}, {128, 128, 4}, {256, 128, 4}, {256, 160, 4}, {256, 192, 4},
                            {256, 224, 4}, {256, 256, 4}, {256, 320, 3}, {64, 64, 4}, {32, 64, 4}, {64, 64, 4}};
constexpr int PICKED = 10;        // the shapes that `pick` chooses among
constexpr int MID = 10;           // 64 x 64 with two slabs a stage: `mid_rows`

static double model_us(const Shape& s, int M, int N, int K) {
  const double tiles = static_cast<double>((M + s.bm - 1) / s.bm) * ((N + s.bn - 1) / s.bn);
  const size_t lds = static_cast<size_t>(s.stages) * (s.bm + s.bn) / 16 * 1024;
  // two workgroups that share a CU hide some of each other's waits (measured: 1.5 to 1.8 times one's time for two rounds)
  const double whole = static_cast<double>((static_cast<long>(tiles) + CUS - 1) / CUS);
  const double rounds = 2 * lds <= LDS_PER_CU && whole > 1 ? 0.9 * whole : whole;
  const double area = static_cast<double>(s.bm) * s.bn;
  return rounds * (K * (2.26e-7 * area + 3.07e-5 * (s.bm + s.bn)) + 1.9e-4 * area);
}

static int pick(int M, int N, int K) {
  int best = 0;
  double best_us = 1e30;
  for (int i = 0; i < PICKED; ++i) {
    const double us = model_us(SHAPES[i], M, N, K);
    if (us < best_us) best_us = us, best = i;
  }
  return best;
}

// 65 to 512 rows.  A tile's walk along K costs a wave some dozens of instructions a slab beside its four matrix
// instructions, and with one or two waves a SIMD nothing hides them: tiles of 64 x 64 take two slabs a stage
// (SHAPES[MID]), which halves that and fills the chip from 65 rows on where the product is wide.  Measured on the
// four products of a layer 1,600 wide (rows and weights that no cache holds; us, before -> now):
//   128 rows: 4,800 columns 18.7 -> 15.7, 6,400 columns 15.3 -> 12.3, 1,600 columns from K = 6,400 19.4 -> 15.2
//   256 rows: 25.6 -> 23.2, 19.3 -> 18.0, 25.6 -> 21.4;  512 rows, 1,600 columns: K = 1,600 12.6 -> 10.7, K = 6,400 38.7 -> 35.4
// -> whether this kernel takes the product with SHAPES[MID] (else `pick` chooses, or the few-rows kernel runs)
static bool mid_rows(int M, int N, int K) {
  if (M <= 64 || M > 512 || K % 64 != 0) return false;
  if (N < 2048) return K >= 4096 || M > 256;      // (few columns and a short K up to 256 rows: the few-rows kernel)
  return M <= 256;
}

// Up to 256 rows the few-rows kernel takes the product too (both read and write packed rows): it stays ahead,
// or level, where the product has few columns and a short K; everywhere else from 65 rows on this kernel is
// the faster (`mid_rows`), and beyond 256 rows it is the only one.
static bool beats_few_rows(int M, int N, int K) {
  return mid_rows(M, N, K) || (M > 104 && N >= 4096) || (M > 208 && N >= 2048);
}

// A long K beside few columns and few rows: the tiles are few and each walks all of K, a slab at a time,
// so K is shared out among several workgroups per tile (whole, such a product takes the same time whatever
// its rows up to 256, and a quarter of K less than a third of it).  The number of shares, 0 for none.  With
// fewer than 2,048 columns: 4 up to 128 rows, 2 up to 256, none beyond (1,600 columns, K = 6,400: 15.2, 21.4
// and 35.4 us at 128, 256 and 512 rows; with 8, 4 and 4 shares of smaller tiles 19.4, 25.6, 38.7).  From 2,048 columns: 8
// where the tiles of 32 x 64 are at most 96, else 4.
static int shares_of_k(int M, int N, int K, int packed, bool kv) {
  if (kv || (packed & PACKED_C) || M <= 64 || M > 512 || N >= 4096 || K < 4096) return 0;
  if (N < 2048 && K % 64 == 0) return M <= 128 ? 4 : M <= 256 ? 2 : 0;
  return ((M + 31) / 32) * ((N + 63) / 64) <= 96 ? 8 : 4;
}

// A product into the residual stream whose sum a norm's kernel adds (dn_gemm_deferred): the shares of K that it
// is cut into, 0 if it is not worth it.  Few columns and 65 to 256 rows: the tiles are too few to fill the chip,
// and with the shares' sums left for the next kernel to add nothing has to join them here (1,600 x 1,600 at 128
// and 256 rows: 4.8 and 6.2 us where the whole product takes 6.7 and 8.0; K = 6,400: the kernel that adds the
// shares, 4.5 us, falls away).
static int deferred_shares(int M, int N, int K) {
  if (M <= 64 || M > 256 || N >= 2048 || K % 64 != 0) return 0;
  if (K >= 4096) return M <= 128 ? 4 : 2;
  return K / 64 >= 8 ? 2 : 0;
}

static int run(const Args& a, hipStream_t stream) {
  if (mid_rows(a.M, a.N, a.K) || (a.part && a.N < 2048 && a.K % 64 == 0)) return launch_as<2, 2, 2, 2, 4, 2>(a, stream);
  switch (pick(a.M, a.N, a.part ? a.K / a.splits : a.K)) {
    case 0: return launch_as<2, 2, 2, 4, 4>(a, stream);
    case 1: return launch_as<4, 2, 2, 4, 4>(a, stream);
    case 2: return launch_as<4, 2, 4, 4, 4>(a, stream);
    case 3: return launch_as<4, 2, 4, 5, 4>(a, stream);
    case 4: return launch_as<4, 2, 4, 6, 4>(a, stream);
    case 5: return launch_as<4, 2, 4, 7, 4>(a, stream);
    case 6: return launch_as<4, 2, 4, 8, 4>(a, stream);
    case 7: return launch_as<4, 2, 4, 10, 3>(a, stream);
    case 8: return launch_as<2, 2, 2, 2, 4>(a, stream);
    default: return launch_as<2, 2, 1, 2, 4>(a, stream);
  }
}
}  // namespace direct

// the tile that a product of these sizes gets from the kernel above: rows * 1000 + columns
extern "C" int dn_gemm_tile(int M, int N, int K) {
  const direct::Shape& s = direct::SHAPES[direct::mid_rows(M, N, K) ? direct::MID : direct::pick(M, N, K)];
  return s.bm * 1000 + s.bn;
}

// packed: bit flags.  W in rows of K elements (the plain kernel, any dtype), or packed bfloat16
// (PACKED_W 1: the MFMA kernels, which need A in bfloat16 and loadable 16 bytes at a time).  With
// at most 256 rows A may be packed too (PACKED_A 2; lda is not read) and so may a bfloat16 C
// (PACKED_C 4; N a multiple of 32; ldc is not read).
extern "C" int dn_gemm(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid,
                       int ldr, int M, int N, int K, int in_dtype, int out_dtype, int epilogue, int packed,
                       float* work, long work_floats, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (lda < K && !(packed & PACKED_A))) return DN_ERR_SHAPE;
  if ((packed & PACKED_W) && K % 8 != 0) return DN_ERR_SHAPE;      // (the plain kernels take any K)
  if (epilogue < EPI_NONE || epilogue > EPI_GELU_ERF) return DN_ERR_SHAPE;
  if (resid != nullptr && epilogue != EPI_NONE) return DN_ERR_SHAPE;
  if ((packed & (PACKED_A | PACKED_C)) && (!(packed & PACKED_W) || M > 256)) return DN_ERR_SHAPE;
  if ((packed & PACKED_C) && (resid != nullptr || out_dtype != DN_BF16 || N % 32 != 0)) return DN_ERR_SHAPE;
  if (packed & PACKED_W) {
    if (in_dtype != DN_BF16) return DN_ERR_DTYPE;
    const bool few = skinny::takes(A, lda, W, M, K, packed);
    const bool many = direct::takes(A, lda, W, bias, C, ldc, resid, ldr, N, K, out_dtype, packed);
    // (products that add into the residual stream only: the others keep one order of summation whether
    // their result goes to rows or to packed rows)
    const int shares = many && resid ? direct::shares_of_k(M, N, K, packed, false) : 0;
    if (shares > 0 && work != nullptr && work_floats >= static_cast<long>(shares) * M * N) {
      direct::Args a{A, lda, W, nullptr, nullptr, 0, nullptr, 0, M, N, K, DN_F32, EPI_NONE, packed & ~PACKED_C, nullptr};
      a.part = work, a.splits = shares;
      int rc = direct::run(a, stream);
      if (rc != 0) return rc;
      hipLaunchKernelGGL((plain::join_kernel<float>), dim3((N + 255) / 256, M), dim3(256), 0, stream, work, shares, bias,
                         static_cast<float*>(nullptr), 0, resid, ldr, M, N, EPI_NONE, plain::KVRows<float>{});
      return dn_launch_status();
    }
    if (many && (!few || direct::beats_few_rows(M, N, K))) {
      int rc = direct::run(direct::Args{A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epilogue, packed, nullptr}, stream);
      return rc != 0 ? rc : dn_launch_status();
    }
    if (few) {
      skinny::Call c{A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epilogue, packed, nullptr};
      skinny::run(c, stream);
      return dn_launch_status();
    }
    if (packed & (PACKED_A | PACKED_C)) return DN_ERR_SHAPE;
    if (!tiled::takes(A, lda, W, K)) return DN_ERR_SHAPE;
    int rc = tiled::run(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, out_dtype, epilogue, nullptr, stream);
    return rc != 0 ? rc : dn_launch_status();
  }
  int rc;
#define DN_LAUNCH(TI, TC) \
  rc = plain::run<TI, TC>(A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epilogue, work, work_floats, stream)
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
  return rc != 0 ? rc : dn_launch_status();
}

// The fused projection of few rows in the plain kernels (32-bit, or bfloat16 weights in rows): C [M, N] = A . W^T +
// bias, and the key columns (q_width ..) and the value columns behind them also go to the slots slot_map[m] of the
// pools (keys [page, Hkv, page_size, dh], values [page, Hkv, dh, page_size], of C's type), written by the kernel
// that adds the segments' sums.  Only where the product has that kernel: dn_gemm_plain_qkv_takes.
extern "C" int dn_gemm_plain_qkv_takes(const void* A, int lda, const void* W, int M, int N, int K, int dtype) {
  if (plain::work_floats(M, N, K) <= 0) return 0;
  return dtype == DN_F32 ? plain::few_rows_take<float>(A, lda, W, M, K)
                         : dtype == DN_BF16 ? plain::few_rows_take<bf16_t>(A, lda, W, M, K) : 0;
}

extern "C" int dn_gemm_plain_qkv(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, int M,
                                 int N, int K, int dtype, const int32_t* slot_map, void* k_pool, void* v_pool,
                                 int q_width, int Hkv, int dh, int page_size, float* work, long work_floats,
                                 hipStream_t stream) {
  if (M <= 0) return 0;
  if (N < 1 || K < 1 || lda < K || ldc < N || !slot_map || !k_pool || !v_pool || Hkv < 1 || dh < 1 || page_size < 1 ||
      q_width < 0 || q_width + 2 * Hkv * dh != N)
    return DN_ERR_SHAPE;
  int rc;
  if (dtype == DN_F32) {
    plain::KVRows<float> kv{slot_map, static_cast<float*>(k_pool), static_cast<float*>(v_pool), q_width, Hkv * dh, dh,
                            page_size, Hkv};
    rc = plain::run<float, float>(A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, EPI_NONE, work, work_floats, stream, kv);
  } else if (dtype == DN_BF16) {
    plain::KVRows<bf16_t> kv{slot_map, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_width, Hkv * dh,
                             dh, page_size, Hkv};
    rc = plain::run<bf16_t, bf16_t>(A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, EPI_NONE, work, work_floats, stream, kv);
  } else {
    return DN_ERR_DTYPE;
  }
  return rc != 0 ? rc : dn_launch_status();
}

// floats of workspace that dn_gemm wants for these sizes (`work`; 0: none): the plain product of few rows
// leaves the sums of K's segments there, and the MFMA product of a long K beside few rows and columns that
// adds into the residual stream the sums of K's shares (without the workspace it runs in the kernels that
// need none; packed: the flags of a product that has a residual)
extern "C" long dn_gemm_work_floats(int M, int N, int K, int packed) {
  if (packed & PACKED_W) return static_cast<long>(direct::shares_of_k(M, N, K, packed, false)) * M * N;
  return plain::work_floats(M, N, K);
}

// A product whose sum somebody else adds into the residual stream: part[share][m][n] (32-bit) = the share's part of
// A . W^T, for dn_gemm_deferred_shares(M, N, K) shares of K; no bias, no epilogue.  dn_layernorm_join (the norm
// that reads the stream next) or dn_join adds them, in order.  A bfloat16 in rows or packed, W packed.
extern "C" int dn_gemm_deferred_shares(int M, int N, int K) { return direct::deferred_shares(M, N, K); }

extern "C" int dn_gemm_deferred(const void* A, int lda, const void* W, int M, int N, int K, int packed, float* part,
                                long part_floats, hipStream_t stream) {
  const int shares = direct::deferred_shares(M, N, K);
  if (shares < 1 || !part || part_floats < static_cast<long>(shares) * M * N) return DN_ERR_SHAPE;
  if (!(packed & PACKED_W) || (packed & PACKED_C) || ((packed & PACKED_A) && M > 256)) return DN_ERR_SHAPE;
  if (!direct::takes(A, lda, W, nullptr, nullptr, 0, part, N, N, K, DN_F32, packed)) return DN_ERR_SHAPE;
  direct::Args a{A, lda, W, nullptr, nullptr, 0, nullptr, 0, M, N, K, DN_F32, EPI_NONE, packed, nullptr};
  a.part = part, a.splits = shares;
  const int rc = direct::run(a, stream);
  return rc != 0 ? rc : dn_launch_status();
}

// resid [M, N] += (part[0] + part[1] + ...) + bias: the shares' sums of a deferred product, where no norm adds them
extern "C" int dn_join(const float* part, int shares, const float* bias, float* resid, int ldr, int M, int N,
                       hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!part || !resid || shares < 1 || ldr < N) return DN_ERR_SHAPE;
  hipLaunchKernelGGL((plain::join_kernel<float>), dim3((N + 255) / 256, M), dim3(256), 0, stream, part, shares, bias,
                     static_cast<float*>(nullptr), 0, resid, ldr, M, N, EPI_NONE, plain::KVRows<float>{});
  return dn_launch_status();
}

// A product of few rows that adds into the residual stream and leaves what the norm after it needs:
// resid [M, N] += A . W^T + bias; copy = the updated rows times gamma [N] (that norm's weight) in
// bfloat16, in rows of ldcopy elements or (ldcopy == 0, N a multiple of 32) as packed rows; stats
// [M][N / 16][2] = mean and sum of squared distances from it of each row's blocks of 16 columns.
// A [M, K] bfloat16 in rows or (lda == 0) packed, W packed, N a multiple of 16.  Up to 16 rows (A in
// rows), or 17 to 64 rows with K >= 1024.
extern "C" int dn_gemm_norm_out(const void* A, int lda, const void* W, const float* bias, float* resid, int ldr, int M,
                                int N, int K, const float* gamma, void* copy, int ldcopy, float* stats,
                                hipStream_t stream) {
  if (M < 1 || M > 64 || N < 16 || N % 16 != 0 || K < 8 || ldr < N || !resid || !copy || !stats || !gamma) return DN_ERR_SHAPE;
  if ((lda != 0 && lda < K) || (ldcopy != 0 && ldcopy < N) || (ldcopy == 0 && N % 32 != 0)) return DN_ERR_SHAPE;
  if (M <= 16 ? lda == 0 : K < 1024) return DN_ERR_SHAPE;
  const int packed = PACKED_W | (lda == 0 ? PACKED_A : 0);
  if (!skinny::takes(A, lda, W, M, K, packed)) return DN_ERR_SHAPE;
  skinny::Call c{A, lda, W, bias, nullptr, 0, resid, ldr, M, N, K, DN_F32, EPI_NONE, packed, nullptr};
  skinny::NormIO nio{nullptr, 0, nullptr, 0.f, 0, gamma, static_cast<bf16_t*>(copy), ldcopy, stats};
  if (M > 16)
    skinny::launch_mb_norm(c, nio, NORM_OUT, stream);
  else if (K >= 1024)
    skinny::launch16_norm<8>(c, nio, NORM_OUT, stream);
  else
    skinny::launch16_norm<4>(c, nio, NORM_OUT, stream);
  return dn_launch_status();
}

// The product after such a norm: C [M, N] bfloat16 = act(LayerNorm(x) . W^T + b), where A is the
// copy of x times gamma [M, K] (in rows, or lda == 0: packed rows) and stats [M][K / 16][2] what
// dn_gemm_norm_out left, c1[n] = sum_k gamma[k] W[n,k] and c2[n] = sum_k beta[k] W[n,k] + b[n].
// no_mean: the norm is x / sqrt(mean(x^2) + eps) * gamma (no mean taken off, no beta: c1 is not used).
// Up to 16 rows (A in rows, K a multiple of 16 up to 4,096), or 17 to 64 rows (K from 1,024 to 2,048).
// With slot_map, the key and value columns go to their pages as in dn_gemm_qkv; without, ldc == 0 asks
// for C in packed rows (17 rows and more, N a multiple of 32).
extern "C" int dn_gemm_norm_in(const void* A, int lda, const float* stats, const float* c1, const float* c2,
                               float eps, const void* W, void* C, int ldc, int M, int N, int K,
                               int epilogue, const int32_t* slot_map, void* k_pool, void* v_pool, int q_width,
                               int Hkv, int dh, int page_size, int c_cols, int no_mean, hipStream_t stream) {
  if (M < 1 || M > 64 || N < 1 || K < 16 || K % 16 != 0 || K > 4096 || (lda != 0 && lda < K) || !stats || !c1 || !c2 || !C)
    return DN_ERR_SHAPE;
  if (M <= 16 ? lda == 0 : (K < 1024 || K > 2048)) return DN_ERR_SHAPE;
  if (epilogue < EPI_NONE || epilogue > EPI_GELU_ERF) return DN_ERR_SHAPE;
  const int packed = PACKED_W | (lda == 0 ? PACKED_A : 0);
  if (!skinny::takes(A, lda, W, M, K, packed) || reinterpret_cast<uintptr_t>(stats) % 8 != 0) return DN_ERR_SHAPE;
  KVScatter kv{};
  if (slot_map) {
    if (q_width < 0 || q_width + 2 * Hkv * dh != N || page_size < 1 || !k_pool || !v_pool || epilogue != EPI_NONE)
      return DN_ERR_SHAPE;
    if ((c_cols != N && c_cols != q_width) || ldc < c_cols) return DN_ERR_SHAPE;
    kv = KVScatter{slot_map, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_width, Hkv * dh, dh,
                   page_size, Hkv, c_cols, page_shift_of(page_size)};
  } else if (ldc == 0 ? (M <= 16 || N % 32 != 0) : ldc < N) {      // ldc == 0: C in packed rows (17 rows and more)
    return DN_ERR_SHAPE;
  }
  skinny::Call c{A, lda, W, c2, C, ldc, nullptr, 0, M, N, K, DN_BF16, epilogue, packed | (ldc == 0 ? PACKED_C : 0),
                 slot_map ? &kv : nullptr};
  skinny::NormIO nio{stats, K / 16, c1, eps, no_mean ? 1 : 0, nullptr, nullptr, 0, nullptr};
  if (M > 16)
    skinny::launch_mb_norm(c, nio, NORM_IN, stream);
  else if (K >= 1024)
    skinny::launch16_norm<8>(c, nio, NORM_IN, stream);
  else
    skinny::launch16_norm<4>(c, nio, NORM_IN, stream);
  return dn_launch_status();
}

// The fused projection q | k | v with packed W: C = A . W^T + bias as dn_gemm computes it, and the
// key and value columns also go to their pages (see KVScatter), from the epilogue of the few-rows
// or of the tiled kernel.  a_packed: A is packed (at most 256 rows).  c_cols: N, or q_width: C then
// is [M, q_width] and gets the query columns only.
extern "C" int dn_gemm_qkv(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, int M, int N,
                           int K, const int32_t* slot_map, void* k_pool, void* v_pool, int q_width, int Hkv, int dh,
                           int page_size, int a_packed, int c_cols, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  const int packed = PACKED_W | (a_packed ? PACKED_A : 0);
  if (K <= 0 || (lda < K && !a_packed)) return DN_ERR_SHAPE;
  const bool few = skinny::takes(A, lda, W, M, K, packed);
  const bool many = direct::takes(A, lda, W, bias, C, ldc, nullptr, 0, N, K, DN_BF16, packed);
  if (!few && !many && (a_packed || !tiled::takes(A, lda, W, K))) return DN_ERR_SHAPE;
  if (q_width < 0 || q_width + 2 * Hkv * dh != N || page_size < 1 || dh % 4 != 0) return DN_ERR_SHAPE;
  if ((c_cols != N && c_cols != q_width) || ldc < c_cols) return DN_ERR_SHAPE;
  KVScatter kv{slot_map, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_width, Hkv * dh, dh,
               page_size, Hkv, c_cols, page_shift_of(page_size)};
  if (many && (!few || direct::beats_few_rows(M, N, K))) {
    int rc = direct::run(direct::Args{A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, DN_BF16, EPI_NONE, packed, &kv}, stream);
    return rc != 0 ? rc : dn_launch_status();
  }
  if (few) {
    skinny::Call c{A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, DN_BF16, EPI_NONE, packed, &kv};
    skinny::run(c, stream);
    return dn_launch_status();
  }
  int rc = tiled::run(A, lda, W, bias, C, ldc, nullptr, 0, M, N, K, DN_BF16, EPI_NONE, &kv, stream);
  return rc != 0 ? rc : dn_launch_status();
}

// dst (packed, (ceil(N/16) * ceil(K/32) * 512 elements) from src [N, K] in rows.
__global__ void pack_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, int N, int K, int ksteps,
                            long chunks) {
  const long c = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;     // one 16-byte chunk each
  if (c >= chunks) return;
  const int in = c % 64;
  const long blk = c / 64;
  const int ks = blk % ksteps, nblk = blk / ksteps;
  const int n = nblk * 16 + in % 16, k = ks * 32 + (in / 16) * 8;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    bf16_t v;
    v.bits = 0;
    if (n < N && k + j < K) v = src[static_cast<size_t>(n) * K + k + j];
    dst[c * 8 + j] = v;
  }
}

extern "C" int dn_pack_matrix(const void* src, void* dst, int N, int K, hipStream_t stream) {
  if (N <= 0 || K <= 0) return DN_ERR_SHAPE;
  const int ksteps = (K + 31) / 32;
  const long chunks = static_cast<long>((N + 15) / 16) * ksteps * 64;
  hipLaunchKernelGGL(pack_kernel, dim3((chunks + 255) / 256), dim3(256), 0, stream,
                     static_cast<const bf16_t*>(src), static_cast<bf16_t*>(dst), N, K, ksteps, chunks);
  return dn_launch_status();
}
