// Causal attention over the paged cache, for a mixed batch: portions of prompts beside
// single decoded tokens (crates/denno-engine/src/model/gpt2.rs:170-202 for one request).
//
// The batch's query rows are cut into tiles of up to 16 consecutive rows of one request;
// a tile table (request, first row, rows, first position) tells each workgroup its work.
// The row at position p of a request reads keys max(0, p - window + 1) .. p (window 0: all)
// through that request's block table.  Key tiles start at absolute multiples of the tile
// length and the softmax is the running ("online") one in 32-bit, so a row's result does not
// depend on where its portion was cut or on what else is in the batch.
//
// A pool is [n_pages, Hkv, page_size, dh]; query head h reads key head h / (H / Hkv).
#include "common.h"

#include <math.h>

namespace plain {
constexpr int BQ = 16;
constexpr int THREADS = 256;

template <typename T>
__global__ __launch_bounds__(THREADS) void attention_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows, const int32_t* __restrict__ tile_pos0, int H, int Hkv, int dh,
    int page_size, int BK, float scale, int window) {
  extern __shared__ float smem[];
  float* Qs = smem;                    // [BQ][dh]
  float* Ks = Qs + BQ * dh;            // [BK][dh + 1]
  float* Vs = Ks + BK * (dh + 1);      // [BK][dh]
  float* Ps = Vs + BK * dh;            // [BQ][BK]

  const int tile = blockIdx.x, h = blockIdx.y;
  const int seq = tile_seq[tile];
  if (seq < 0) return;   // padding of a fixed-size launch
  const int row0 = tile_row0[tile], nrows = tile_nrows[tile], pos0 = tile_pos0[tile];
  const int hk = h / (H / Hkv);
  const int32_t* bt = block_tables + static_cast<size_t>(seq) * max_blocks;
  const int t = threadIdx.x, qi = t / 16, g = t % 16;
  const float NEG_INF = -INFINITY;

  for (int e = t; e < BQ * dh; e += THREADS) {
    int r = e / dh, d = e % dh;
    Qs[e] = r < nrows ? to_float(q[static_cast<size_t>(row0 + r) * ldq + h * dh + d]) : 0.f;
  }
  const bool row_ok = qi < nrows;
  const int my_pos = pos0 + qi;
  const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
  const int last_pos = pos0 + nrows - 1;
  const int first_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int nd = dh / 16, nc = BK / 16;

  float m = NEG_INF, l = 0.f;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;

  for (int kt = (first_lo / BK) * BK; kt <= last_pos; kt += BK) {
    __syncthreads();
    for (int e = t; e < BK * dh; e += THREADS) {
      int j = e / dh, d = e % dh;
      int key = kt + j;
      float kv = 0.f, vv = 0.f;
      if (key <= last_pos) {
        int page = bt[key / page_size];
        if (page >= 0) {
          size_t src = ((static_cast<size_t>(page) * Hkv + hk) * page_size + key % page_size) * dh + d;
          kv = to_float(k_pool[src]);
          vv = to_float(v_pool[src]);
        }
      }
      Ks[j * (dh + 1) + d] = kv;
      Vs[j * dh + d] = vv;
    }
    __syncthreads();

    float s[4];
    float tmax = NEG_INF;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s[c] = NEG_INF;
      if (c < nc) {
        int j = g + 16 * c;
        int key = kt + j;
        float dot = 0.f;
        const float* qr = Qs + qi * dh;
        const float* kr = Ks + j * (dh + 1);
        for (int d = 0; d < dh; ++d) dot = fmaf(qr[d], kr[d], dot);
        bool ok = row_ok && key >= my_lo && key <= my_pos;
        s[c] = ok ? dot * scale : NEG_INF;
        tmax = fmaxf(tmax, s[c]);
      }
    }
#pragma unroll
    for (int mask = 8; mask >= 1; mask >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, mask, DN_WAVE));

    float alpha = 1.f, psum = 0.f;
    if (tmax > NEG_INF) {
      float m_new = fmaxf(m, tmax);
      alpha = m > NEG_INF ? expf(m - m_new) : 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (c < nc) {
          float p = s[c] > NEG_INF ? expf(s[c] - m_new) : 0.f;
          Ps[qi * BK + g + 16 * c] = p;
          psum += p;
        }
      }
      m = m_new;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (c < nc) Ps[qi * BK + g + 16 * c] = 0.f;
    }
#pragma unroll
    for (int mask = 8; mask >= 1; mask >>= 1) psum += __shfl_xor(psum, mask, DN_WAVE);
    l = l * alpha + psum;
    __syncthreads();

#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (i < nd) {
        int d = g + 16 * i;
        float a = acc[i] * alpha;
        const float* pr = Ps + qi * BK;
        for (int j = 0; j < BK; ++j) a = fmaf(pr[j], Vs[j * dh + d], a);
        acc[i] = a;
      }
    }
  }
  if (row_ok) {
    float inv = 1.0f / l;
    T* o = out + static_cast<size_t>(row0 + qi) * ldo + h * dh;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i < nd) o[g + 16 * i] = from_float<T>(acc[i] * inv);
  }
}
}  // namespace plain

extern "C" int dn_attention(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                            const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                            const int32_t* tile_row0, const int32_t* tile_nrows, const int32_t* tile_pos0,
                            int n_tiles, int H, int Hkv, int dh, int page_size, float scale, int window, int dtype,
                            hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (dh < 16 || dh > 256 || dh % 16 != 0 || Hkv < 1 || H % Hkv != 0 || page_size < 1 || max_blocks < 1)
    return DN_ERR_SHAPE;
  int BK = dh <= 64 ? 64 : (dh <= 128 ? 32 : 16);
  size_t lds = sizeof(float) * (static_cast<size_t>(plain::BQ) * dh + static_cast<size_t>(BK) * (dh + 1) +
                                static_cast<size_t>(BK) * dh + static_cast<size_t>(plain::BQ) * BK);
  dim3 grid(n_tiles, H), block(plain::THREADS);
  if (dtype == DN_F32)
    hipLaunchKernelGGL(plain::attention_kernel<float>, grid, block, lds, stream, static_cast<const float*>(q), ldq,
                       static_cast<float*>(out), ldo, static_cast<const float*>(k_pool),
                       static_cast<const float*>(v_pool), block_tables, max_blocks, tile_seq, tile_row0, tile_nrows,
                       tile_pos0, H, Hkv, dh, page_size, BK, scale, window);
  else if (dtype == DN_BF16)
    hipLaunchKernelGGL(plain::attention_kernel<bf16_t>, grid, block, lds, stream, static_cast<const bf16_t*>(q),
                       ldq, static_cast<bf16_t*>(out), ldo, static_cast<const bf16_t*>(k_pool),
                       static_cast<const bf16_t*>(v_pool), block_tables, max_blocks, tile_seq, tile_row0,
                       tile_nrows, tile_pos0, H, Hkv, dh, page_size, BK, scale, window);
  else
    return DN_ERR_DTYPE;
  return dn_launch_status();
}
