// Matrix products  C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias[N])  with every weight held
// [out, in], K contiguous for both operands.  Epilogues: bias, GELU (tanh or erf form),
// or accumulation into the 32-bit residual stream (x += A.W^T + bias).
//
// Four kernel families behind dn_gemm, a source file each (gemm_plain.hip, gemm_skinny.hip, gemm_direct.hip,
// gemm_tiled.hip; this file holds the entry points and gemm_common.h what they share).  plain: 32-bit multiply-adds in a fixed order over K, whatever
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
#include "gemm_common.h"

// the tile that a product of these sizes gets from the kernel above: rows * 1000 + columns
extern "C" int dn_gemm_tile(int M, int N, int K) { return direct::tile_of(M, N, K); }
// the same for a fused projection that writes the cache (some tiles are not on offer to it)
extern "C" int dn_gemm_tile_qkv(int M, int N, int K) { return direct::tile_of(M, N, K, true); }

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
      plain::join_shares(work, shares, bias, resid, ldr, M, N, stream);
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
  if ((in_dtype != DN_F32 && in_dtype != DN_BF16) || (out_dtype != DN_F32 && out_dtype != DN_BF16)) return DN_ERR_DTYPE;
  const int rc = plain::run_of(in_dtype, out_dtype, A, lda, W, bias, C, ldc, resid, ldr, M, N, K, epilogue, work,
                               work_floats, stream);
  return rc != 0 ? rc : dn_launch_status();
}

// The fused projection of few rows in the plain kernels (32-bit, or bfloat16 weights in rows): C [M, N] = A . W^T +
// bias, and the key columns (q_width ..) and the value columns behind them also go to the slots slot_map[m] of the
// pools (keys [page, Hkv, page_size, dh], values [page, Hkv, dh, page_size], of C's type), written by the kernel
// that adds the segments' sums.  Only where the product has that kernel: dn_gemm_plain_qkv_takes.
extern "C" int dn_gemm_plain_qkv_takes(const void* A, int lda, const void* W, int M, int N, int K, int dtype) {
  if (plain::work_floats(M, N, K) <= 0) return 0;
  return plain::few_rows_take_of(dtype, A, lda, W, M, K);
}

extern "C" int dn_gemm_plain_qkv(const void* A, int lda, const void* W, const float* bias, void* C, int ldc, int M,
                                 int N, int K, int dtype, const int32_t* slot_map, void* k_pool, void* v_pool,
                                 int q_width, int Hkv, int dh, int page_size, float* work, long work_floats,
                                 hipStream_t stream) {
  if (M <= 0) return 0;
  if (N < 1 || K < 1 || lda < K || ldc < N || !slot_map || !k_pool || !v_pool || Hkv < 1 || dh < 1 || page_size < 1 ||
      q_width < 0 || q_width + 2 * Hkv * dh != N)
    return DN_ERR_SHAPE;
  if (dtype != DN_F32 && dtype != DN_BF16) return DN_ERR_DTYPE;
  const int rc = plain::run_qkv_of(dtype, A, lda, W, bias, C, ldc, M, N, K, slot_map, k_pool, v_pool, q_width, Hkv, dh,
                                   page_size, work, work_floats, stream);
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
  plain::join_shares(part, shares, bias, resid, ldr, M, N, stream);
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
  else
    skinny::launch16_norm_of(K >= 1024 ? 8 : 4, c, nio, NORM_OUT, stream);
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
  else
    skinny::launch16_norm_of(K >= 1024 ? 8 : 4, c, nio, NORM_IN, stream);
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
