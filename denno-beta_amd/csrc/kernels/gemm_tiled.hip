#include "gemm_common.h"

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

bool takes(const void* A, int lda, const void* W, int K) {
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

int run(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr, int M,
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
