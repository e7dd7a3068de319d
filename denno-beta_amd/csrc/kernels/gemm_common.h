// What the product kernels share: the epilogues, where a fused projection's keys and values go, the flags of the
// packed layouts, and what each kernel family (one source file each: gemm_plain.hip, gemm_skinny.hip,
// gemm_tiled.hip, gemm_direct.hip) offers to the entry points in gemm.hip.  The families are compiled side by
// side and linked into one library.
#pragma once
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

static inline int page_shift_of(int page_size) {
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

// flags of dn_gemm's `packed`: W, A or C in the packed layout (see gemm.hip)
#define PACKED_W 1
#define PACKED_A 2
#define PACKED_C 4

// a norm inside a few-rows product: before it (NORM_IN) or after it (NORM_OUT); see gemm_skinny.hip
#define NORM_NONE 0
#define NORM_IN 1
#define NORM_OUT 2

namespace plain {
long work_floats(int M, int N, int K);
int few_rows_take_of(int dtype, const void* A, int lda, const void* W, int M, int K);
int run_of(int in_dtype, int out_dtype, const void* A, int lda, const void* W, const float* bias, void* C, int ldc,
           float* resid, int ldr, int M, int N, int K, int epilogue, float* work, long have, hipStream_t stream);
int run_qkv_of(int dtype, const void* A, int lda, const void* W, const float* bias, void* C, int ldc, int M, int N, int K,
               const int32_t* slot_map, void* k_pool, void* v_pool, int q_width, int Hkv, int dh, int page_size,
               float* work, long have, hipStream_t stream);
void join_shares(const float* part, int shares, const float* bias, float* resid, int ldr, int M, int N, hipStream_t stream);
}  // namespace plain

namespace skinny {
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

struct Call {
  const void* A; int lda; const void* W; const float* bias; void* C; int ldc; float* resid; int ldr;
  int M, N, K, out_dtype, epi, packed;
  const KVScatter* kv;
};
bool takes(const void* A, int lda, const void* W, int M, int K, int packed);
void run(const Call& c, hipStream_t stream);
void launch_mb_norm(const Call& c, const NormIO& nio, int norm, hipStream_t stream);
void launch16_norm_of(int waves, const Call& c, const NormIO& nio, int norm, hipStream_t stream);
}  // namespace skinny

namespace tiled {
bool takes(const void* A, int lda, const void* W, int K);
int run(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, float* resid, int ldr, int M,
        int N, int K, int out_dtype, int epi, const KVScatter* kv, hipStream_t stream);
}  // namespace tiled

namespace direct {
struct Args {
  const void* A; int lda; const void* W; const float* bias; void* C; int ldc; float* resid; int ldr;
  int M, N, K, out_dtype, epi, packed; const KVScatter* kv;
  float* part = nullptr; int splits = 1;       // part: K in `splits` shares, their sums in part[share][m][n]
};
struct Shape { int bm, bn, stages; };
bool takes(const void* A, int lda, const void* W, const float* bias, const void* C, int ldc, const float* resid,
           int ldr, int N, int K, int out_dtype, int packed);
int pick(int M, int N, int K, bool kv = false);
bool mid_rows(int M, int N, int K);
bool beats_few_rows(int M, int N, int K);
int shares_of_k(int M, int N, int K, int packed, bool kv);
int deferred_shares(int M, int N, int K);
int run(const Args& a, hipStream_t stream);
int tile_of(int M, int N, int K, bool kv = false);
}  // namespace direct
