// Embedding, LayerNorm, cache write, casts: the memory-bound, row-wise kernels.
// The residual stream is 32-bit in both precisions; LayerNorm's statistics and affine are
// 32-bit; only what feeds a matrix product is rounded to bfloat16.
#include "common.h"

// ---------------------------------------------------------------------------------------
// x[t,:] = wte[token_t,:] * token_scale + wpe[pos_t,:]   (crates/denno-engine/src/model/gpt2.rs:142-150,
// where the scale is 1), as the first two entries of a list of tables that are added up.
// ---------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t words4;
// element i of the 16 bytes w as a table of TW holds them
template <typename TW>
__device__ __forceinline__ float element(const words4& w, int i);
template <>
__device__ __forceinline__ float element<float>(const words4& w, int i) { return __uint_as_float(w[i]); }
template <>
__device__ __forceinline__ float element<bf16_t>(const words4& w, int i) {
  return __uint_as_float(i % 2 == 0 ? w[i / 2] << 16 : w[i / 2] & 0xffff0000u);
}

// x[t,:] = sum over the listed tables, in the list's order, of table_i[index_i[t],:] * scale_i: the token table
// and the position table for this architecture; an architecture with a further table (a second one over the
// tokens, one over another per-row integer) lists it behind them.
constexpr int EMBED_TABLES_MAX = 4;
struct EmbedTables {
  const void* table[EMBED_TABLES_MAX];
  const int32_t* index[EMBED_TABLES_MAX];
  int rows[EMBED_TABLES_MAX];
  float scale[EMBED_TABLES_MAX];
  int n;
};

template <typename TW>
__global__ void embed_kernel(EmbedTables tb, float* __restrict__ x, int T, int E, int wide) {
  int t = blockIdx.x;
  if (t >= T) return;
  int id[EMBED_TABLES_MAX];
  bool ok = true;
#pragma unroll
  for (int i = 0; i < EMBED_TABLES_MAX; ++i) {
    id[i] = i < tb.n ? tb.index[i][t] : 0;
    ok = ok && (i >= tb.n || (id[i] >= 0 && id[i] < tb.rows[i]));
  }
  const float nan = __uint_as_float(0x7fc00000u);   // an id outside a table: NaN, never a neighbour's row
  if (wide) {
    // 16 bytes of each table per thread and step (E a multiple of that many elements, the tables aligned):
    // a row of 1,600 is one step, all its loads on their way at once
    constexpr int VEC = 16 / sizeof(TW);
    for (int e = threadIdx.x * VEC; e < E; e += blockDim.x * VEC) {
      float v[VEC];
      if (ok) {
        words4 w[EMBED_TABLES_MAX];
#pragma unroll
        for (int i = 0; i < EMBED_TABLES_MAX; ++i)
          if (i < tb.n) w[i] = *reinterpret_cast<const words4*>(static_cast<const TW*>(tb.table[i]) + static_cast<size_t>(id[i]) * E + e);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          v[k] = element<TW>(w[0], k);
          if (tb.scale[0] != 1.0f) v[k] *= tb.scale[0];
        }
#pragma unroll
        for (int i = 1; i < EMBED_TABLES_MAX; ++i)
          if (i < tb.n) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
              float a = element<TW>(w[i], k);
              if (tb.scale[i] != 1.0f) a *= tb.scale[i];
              v[k] += a;
            }
          }
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) v[k] = nan;
      }
      float* dst = x + static_cast<size_t>(t) * E + e;
#pragma unroll
      for (int k = 0; k < VEC; k += 4) *reinterpret_cast<float4*>(dst + k) = float4{v[k], v[k + 1], v[k + 2], v[k + 3]};
    }
    return;
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    float v = nan;
    if (ok) {
      v = to_float(static_cast<const TW*>(tb.table[0])[static_cast<size_t>(id[0]) * E + e]);
      if (tb.scale[0] != 1.0f) v *= tb.scale[0];
      for (int i = 1; i < tb.n; ++i) {
        float a = to_float(static_cast<const TW*>(tb.table[i])[static_cast<size_t>(id[i]) * E + e]);
        if (tb.scale[i] != 1.0f) a *= tb.scale[i];
        v += a;
      }
    }
    x[static_cast<size_t>(t) * E + e] = v;
  }
}

// tables, indices, rows, scales: n <= 4 entries each (host arrays); every table [rows_i, E] of table_dtype
extern "C" int dn_embed_sum(const void* const* tables, const int32_t* const* indices, const int* rows,
                            const float* scales, int n, float* x, int T, int E, int table_dtype,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (n < 1 || n > EMBED_TABLES_MAX || E < 1) return DN_ERR_SHAPE;
  EmbedTables tb{};
  tb.n = n;
  const int vec = table_dtype == DN_F32 ? 4 : 8;
  int wide = E % vec == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
  for (int i = 0; i < n; ++i) {
    if (!tables[i] || !indices[i] || rows[i] < 1) return DN_ERR_SHAPE;
    tb.table[i] = tables[i], tb.index[i] = indices[i], tb.rows[i] = rows[i], tb.scale[i] = scales[i];
    wide = wide && reinterpret_cast<uintptr_t>(tables[i]) % 16 == 0;
  }
  dim3 grid(T), block(256);
  if (table_dtype == DN_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, tb, x, T, E, wide);
  else if (table_dtype == DN_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, tb, x, T, E, wide);
  else
    return DN_ERR_DTYPE;
  return dn_launch_status();
}

// the token table and, unless it is null, the position table
extern "C" int dn_embed(const int32_t* tokens, const int32_t* positions, const void* wte, const void* wpe,
                        float* x, int T, int E, int vocab, int n_pos, int table_dtype, float token_scale,
                        hipStream_t stream) {
  const void* tables[2] = {wte, wpe};
  const int32_t* indices[2] = {tokens, positions};
  const int rows[2] = {vocab, n_pos};
  const float scales[2] = {token_scale, 1.0f};
  return dn_embed_sum(tables, indices, rows, scales, wpe ? 2 : 1, x, T, E, table_dtype, stream);
}

// ---------------------------------------------------------------------------------------
// LayerNorm of selected rows: mean, biased variance of (x - mean), then affine
// (crates/denno-engine/src/tensor.rs:1101-1112).  One wave per row; the row is read three
// times (it stays in cache), so any width works.  rows == null: row r of the output is
// row r of x.
// ---------------------------------------------------------------------------------------
template <typename TO>
__global__ void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                 const float* __restrict__ beta, TO* __restrict__ out,
                                 const int32_t* __restrict__ rows, int R, int E, float eps, int packed) {
  int wave = threadIdx.x / DN_WAVE, lane = threadIdx.x % DN_WAVE;
  int r = blockIdx.x * (blockDim.x / DN_WAVE) + wave;
  if (r >= R) return;
  int src = rows ? rows[r] : r;
  const float* xr = x + static_cast<size_t>(src) * E;
  float s = 0.f;
  for (int e = lane; e < E; e += DN_WAVE) s += xr[e];
  float mean = wave_sum(s) / static_cast<float>(E);
  float v = 0.f;
  for (int e = lane; e < E; e += DN_WAVE) {
    float d = xr[e] - mean;
    v += d * d;
  }
  float inv = 1.0f / sqrtf(wave_sum(v) / static_cast<float>(E) + eps);
  for (int e = lane; e < E; e += DN_WAVE) {
    float y = (xr[e] - mean) * inv * gamma[e];
    if (beta) y += beta[e];
    out[packed ? packed_index(r, e, E / 32) : static_cast<size_t>(r) * E + e] = from_float<TO>(y);
  }
}

// The same with one workgroup per row and the row held in registers (one read of x): the
// kernel for every width up to 256 * 32.  Sums meet in a fixed order: lanes by butterfly, the
// four waves one after the other.
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / DN_WAVE, lane = threadIdx.x % DN_WAVE;
  __syncthreads();   // scratch may still be read from the call before
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
}

// What a product left for this norm to add into the rows before it norms them (JOIN): the sums of its shares
// of K, part[share][row][e] (`stride` floats from one share to the next), and its bias.  The rows become
// x + ((part[0] + part[1] + ...) + bias), shares in ascending order from zero, as the kernel that only adds
// them makes it (gemm.hip, plain::join_kernel), and are stored back before they are normed.
struct PendingSum {
  const float* part;
  const float* bias;
  long long stride;
  int shares;
};

template <typename TO, int VPT, bool JOIN = false>
__global__ __launch_bounds__(256) void layernorm_row_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ gamma,
                                                             const float* __restrict__ beta, TO* __restrict__ out,
                                                             const int32_t* __restrict__ rows, int E, float eps,
                                                             int packed, PendingSum pend, float* __restrict__ x_out) {
  __shared__ float scratch[4];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const float* xr = x + static_cast<size_t>(src) * E;
  // loads are never conditional (a predicated load waits for the one before it)
  float v[VPT], gm[VPT], bt[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int e = min(static_cast<int>(threadIdx.x) + i * 256, E - 1);
    v[i] = xr[e];
    gm[i] = gamma[e];
    bt[i] = beta ? beta[e] : 0.f;
  }
  if constexpr (JOIN) {
    const float* pr = pend.part + static_cast<size_t>(src) * E;
    float tot[VPT], pb[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      tot[i] = 0.f;
      pb[i] = pend.bias ? pend.bias[min(static_cast<int>(threadIdx.x) + i * 256, E - 1)] : 0.f;
    }
    for (int sh = 0; sh < pend.shares; ++sh) {
      float p[VPT];
#pragma unroll
      for (int i = 0; i < VPT; ++i) p[i] = pr[sh * pend.stride + min(static_cast<int>(threadIdx.x) + i * 256, E - 1)];
#pragma unroll
      for (int i = 0; i < VPT; ++i) tot[i] += p[i];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = threadIdx.x + i * 256;
      v[i] = v[i] + (pend.bias ? tot[i] + pb[i] : tot[i]);
      if (e < E) x_out[static_cast<size_t>(src) * E + e] = v[i];
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (static_cast<int>(threadIdx.x) + i * 256 >= E) v[i] = 0.f;
    s += v[i];
  }
  const float mean = block_sum_256(s, scratch) / static_cast<float>(E);
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int e = threadIdx.x + i * 256;
    float d = e < E ? v[i] - mean : 0.f;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum_256(q, scratch) / static_cast<float>(E) + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int e = threadIdx.x + i * 256;
    if (e < E) {
      float y = (v[i] - mean) * inv * gm[i];
      if (beta) y += bt[i];
      out[packed ? packed_index(r, e, E / 32) : static_cast<size_t>(r) * E + e] = from_float<TO>(y);
    }
  }
}

template <typename TO>
static void launch_layernorm(const float* x, const float* gamma, const float* beta, TO* out, const int32_t* rows,
                             int R, int E, float eps, int packed, hipStream_t stream) {
  const PendingSum none{};
  if (E <= 512)
    hipLaunchKernelGGL((layernorm_row_kernel<TO, 2>), dim3(R), dim3(256), 0, stream, x, gamma, beta, out, rows, E, eps, packed, none, nullptr);
  else if (E <= 2048)
    hipLaunchKernelGGL((layernorm_row_kernel<TO, 8>), dim3(R), dim3(256), 0, stream, x, gamma, beta, out, rows, E, eps, packed, none, nullptr);
  else if (E <= 8192)
    hipLaunchKernelGGL((layernorm_row_kernel<TO, 32>), dim3(R), dim3(256), 0, stream, x, gamma, beta, out, rows, E,
                       eps, packed, none, nullptr);
  else {
    const int waves = 4;
    hipLaunchKernelGGL(layernorm_kernel<TO>, dim3((R + waves - 1) / waves), dim3(waves * DN_WAVE), 0, stream, x, gamma,
                       beta, out, rows, R, E, eps, packed);
  }
}

// LayerNorm of all R rows of x [R, E] after what a product left for them has been added (see PendingSum): x is
// updated in place, out gets the normed rows.  E up to 8,192.
extern "C" int dn_layernorm_join(float* x, const float* part, int shares, long long share_stride, const float* bias,
                                 const float* gamma, const float* beta, void* out, int R, int E, float eps,
                                 int out_dtype, int packed, hipStream_t stream) {
  if (R <= 0) return 0;
  if (!part || shares < 1 || share_stride < static_cast<long long>(R) * E || E > 8192) return DN_ERR_SHAPE;
  if (packed && (out_dtype != DN_BF16 || E % 32 != 0)) return DN_ERR_SHAPE;
  const PendingSum pend{part, bias, share_stride, shares};
#define DN_LNJ(TO, VPT)                                                                                              \
  hipLaunchKernelGGL((layernorm_row_kernel<TO, VPT, true>), dim3(R), dim3(256), 0, stream, x, gamma, beta,            \
                     static_cast<TO*>(out), static_cast<const int32_t*>(nullptr), E, eps, packed, pend, x)
#define DN_LNJ_E(TO)        \
  do {                      \
    if (E <= 512)           \
      DN_LNJ(TO, 2);        \
    else if (E <= 2048)     \
      DN_LNJ(TO, 8);        \
    else                    \
      DN_LNJ(TO, 32);       \
  } while (0)
  if (out_dtype == DN_F32)
    DN_LNJ_E(float);
  else if (out_dtype == DN_BF16)
    DN_LNJ_E(bf16_t);
  else
    return DN_ERR_DTYPE;
#undef DN_LNJ_E
#undef DN_LNJ
  return dn_launch_status();
}

// packed: out is a packed matrix of ceil(R / 16) * 16 rows (bfloat16, E a multiple of 32)
extern "C" int dn_layernorm(const float* x, const float* gamma, const float* beta, void* out, const int32_t* rows,
                            int R, int E, float eps, int out_dtype, int packed, hipStream_t stream) {
  if (R <= 0) return 0;
  if (packed && (out_dtype != DN_BF16 || E % 32 != 0)) return DN_ERR_SHAPE;
  if (out_dtype == DN_F32)
    launch_layernorm<float>(x, gamma, beta, static_cast<float*>(out), rows, R, E, eps, 0, stream);
  else if (out_dtype == DN_BF16)
    launch_layernorm<bf16_t>(x, gamma, beta, static_cast<bf16_t*>(out), rows, R, E, eps, packed, stream);
  else
    return DN_ERR_DTYPE;
  return dn_launch_status();
}

// ---------------------------------------------------------------------------------------
// Keys and values of this step's tokens go to their pages before attention reads them
// (crates/denno-engine/src/model/gpt2.rs:159-167).  src is [T, ld]; keys are columns
// k_col .. k_col + Hkv*dh, values v_col .. ; slot_map[t] = page * page_size + offset, or < 0
// for a row that is padding.  The key pool is [n_pages, Hkv, page_size, dh]; the value pool is
// [n_pages, Hkv, dh, page_size] (a page's values transposed), which is how attention's second
// product reads them: for one dim, the keys of a page side by side.
// ---------------------------------------------------------------------------------------
template <typename TS>
__global__ void kv_write_kernel(const TS* __restrict__ src, int ld, int k_col, int v_col,
                                const int32_t* __restrict__ slot_map, TS* __restrict__ k_pool,
                                TS* __restrict__ v_pool, int T, int Hkv, int dh, int page_size) {
  int t = blockIdx.x;
  if (t >= T) return;
  int slot = slot_map[t];
  if (slot < 0) return;
  int page = slot / page_size, off = slot % page_size;
  int width = Hkv * dh;
  const TS* row = src + static_cast<size_t>(t) * ld;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    int h = c / dh, d = c % dh;
    size_t base = (static_cast<size_t>(page) * Hkv + h) * page_size * dh;
    k_pool[base + static_cast<size_t>(off) * dh + d] = row[k_col + c];
    v_pool[base + static_cast<size_t>(d) * page_size + off] = row[v_col + c];
  }
}

extern "C" int dn_kv_write(const void* src, int ld, int k_col, int v_col, const int32_t* slot_map, void* k_pool,
                           void* v_pool, int T, int Hkv, int dh, int page_size, int dtype, hipStream_t stream) {
  if (T <= 0) return 0;
  dim3 grid(T), block(256);
  if (dtype == DN_F32)
    hipLaunchKernelGGL(kv_write_kernel<float>, grid, block, 0, stream, static_cast<const float*>(src), ld, k_col,
                       v_col, slot_map, static_cast<float*>(k_pool), static_cast<float*>(v_pool), T, Hkv, dh,
                       page_size);
  else if (dtype == DN_BF16)
    hipLaunchKernelGGL(kv_write_kernel<bf16_t>, grid, block, 0, stream, static_cast<const bf16_t*>(src), ld,
                       k_col, v_col, slot_map, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), T, Hkv,
                       dh, page_size);
  else
    return DN_ERR_DTYPE;
  return dn_launch_status();
}

// ---------------------------------------------------------------------------------------
// Element-wise conversion between the two precisions (rows of a matrix product whose
// weight is held in the other precision).
// ---------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (; i < n; i += stride) out[i] = from_float<TO>(to_float(in[i]));
}

extern "C" int dn_cast(const void* in, void* out, long long n, int in_dtype, int out_dtype, hipStream_t stream) {
  if (n <= 0) return 0;
  size_t blocks = (static_cast<size_t>(n) + 255) / 256;
  dim3 grid(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)), block(256);
  if (in_dtype == DN_BF16 && out_dtype == DN_F32)
    hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream, static_cast<const bf16_t*>(in),
                       static_cast<float*>(out), static_cast<size_t>(n));
  else if (in_dtype == DN_F32 && out_dtype == DN_BF16)
    hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream, static_cast<const float*>(in),
                       static_cast<bf16_t*>(out), static_cast<size_t>(n));
  else
    return DN_ERR_DTYPE;
  return dn_launch_status();
}

// ---------------------------------------------------------------------------------------
// What a head may do to its logits, in place: l = l * scale, then, if cap > 0, l = cap * tanh(l / cap).
// ---------------------------------------------------------------------------------------
__global__ void logits_post_kernel(float* __restrict__ logits, int ld, int V, float scale, float cap) {
  float* row = logits + static_cast<size_t>(blockIdx.y) * ld;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < V; i += gridDim.x * blockDim.x) {
    float l = row[i] * scale;
    if (cap > 0.f) l = cap * tanhf(l / cap);
    row[i] = l;
  }
}

extern "C" int dn_logits_post(float* logits, int ld, int R, int V, float scale, float cap, hipStream_t stream) {
  if (R <= 0 || V <= 0) return 0;
  if (ld < V || R > 65535) return DN_ERR_SHAPE;
  hipLaunchKernelGGL(logits_post_kernel, dim3((V + 1023) / 1024 > 64 ? 64 : (V + 1023) / 1024, R), dim3(256), 0, stream,
                     logits, ld, V, scale, cap);
  return dn_launch_status();
}
