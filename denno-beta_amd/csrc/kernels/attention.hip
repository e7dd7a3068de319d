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
// The key pool is [n_pages, Hkv, page_size, dh], the value pool [n_pages, Hkv, dh, page_size];
// query head h reads key head h / (H / Hkv).
#include "common.h"
#include "attention.h"

#include <math.h>

#include <mutex>

namespace plain {
constexpr int BQ = 16;
constexpr int THREADS = 256;

// One order of summation for every row, whichever kernel runs it and however its step was cut.  Keys
// go in tiles of BK that start at absolute multiples of BK.  A tile alone gives, for a row, its largest
// score m_T, the sum l_T of exp(score - m_T) and the values weighted with those, a_T; tiles are joined
// in ascending order: the first as it is, a later one by
//     m' = max(m, m_T),  l' = l exp(m - m') + l_T exp(m_T - m'),  a' = a exp(m - m') + a_T exp(m_T - m').
// Inside a tile 16 threads share a row: thread g has the keys g, g + 16, ... (each score summed over
// the dims in ascending order) and the dims g, g + 16, ... (each summed over the tile's keys in
// ascending order); the 16 partial sums of l_T meet in the order of group_reduce<16>.

// q . k over the dims in ascending order, one fused multiply-add a dim (16 dims' operands are read at a
// time, so that the reads do not wait for one another; the sums keep their order)
__device__ __forceinline__ float key_dot(const float* qr, const float* kr, int dh) {
  float dot = 0.f;
  for (int d0 = 0; d0 < dh; d0 += 16) {
    float a[16], b[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = qr[d0 + i], b[i] = kr[d0 + i];
#pragma unroll
    for (int i = 0; i < 16; ++i) dot = fmaf(a[i], b[i], dot);
  }
  return dot;
}

// sum over the tile's keys, in ascending order, of p[j] times one dim of the values (vs: that dim of key 0)
__device__ __forceinline__ float dim_sum(const float* ps, const float* vs, int dh, int BK) {
  float a = 0.f;
  for (int j0 = 0; j0 < BK; j0 += 16) {
    float p[16], v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) p[i] = ps[j0 + i], v[i] = vs[(j0 + i) * (dh + 1)];
#pragma unroll
    for (int i = 0; i < 16; ++i) a = fmaf(p[i], v[i], a);
  }
  return a;
}

// the scores of one row against the tile in Ks: p[j] to Ps (this row's BK entries), -> m_T, l_T
__device__ __forceinline__ void tile_scores(const float* qr, const float* Ks, float* ps, int g, int nc, int dh, int kt,
                                            int lo, int pos, bool row_ok, float scale, float& m_t, float& l_t) {
  const float NEG_INF = -INFINITY;
  float s[4];
  float tmax = NEG_INF;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    s[c] = NEG_INF;
    if (c < nc) {
      const int j = g + 16 * c;
      const int key = kt + j;
      const float dot = key_dot(qr, Ks + j * (dh + 1), dh);
      const bool ok = row_ok && key >= lo && key <= pos;
      s[c] = ok ? dot * scale : NEG_INF;
      tmax = fmaxf(tmax, s[c]);
    }
  }
  tmax = group_reduce<16>(tmax, MaxOp());
  float psum = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    if (c < nc) {
      const float p = s[c] > NEG_INF ? expf(s[c] - tmax) : 0.f;     // (a tile without a key: zeros)
      ps[g + 16 * c] = p;
      psum += p;
    }
  }
  m_t = tmax;
  l_t = group_reduce<16>(psum, SumOp());
}

// a_T[i] for the dims g + 16 i, from the row's p in ps and the tile's values in Vs
__device__ __forceinline__ void tile_values(const float* ps, const float* Vs, int g, int nd, int dh, int BK,
                                            float* a_t) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    a_t[i] = 0.f;
    if (i < nd) {
      a_t[i] = dim_sum(ps, Vs + g + 16 * i, dh, BK);
    }
  }
}

// joins a tile (m_t > -inf) to what the tiles before it gave
__device__ __forceinline__ void join_tile(float& m, float& l, float* acc, float m_t, float l_t, const float* a_t,
                                          int nd) {
  if (!(m > -INFINITY)) {
    m = m_t;
    l = l_t;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i < nd) acc[i] = a_t[i];
    return;
  }
  const float m_new = fmaxf(m, m_t);
  const float alpha = expf(m - m_new), beta = expf(m_t - m_new);
  l = fmaf(l_t, beta, l * alpha);
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i < nd) acc[i] = fmaf(a_t[i], beta, acc[i] * alpha);
  m = m_new;
}

// the tile of BK keys from kt of one request and key head into LDS, a key's dims and values ld floats apart
// (keys beyond last_pos and pages given back: zeros).  Where each key's dims and each key's values start in the pools is worked out
// first (Kb, Vb: BK entries each, -1 without a page), so that the loads of the keys and values
// themselves wait for nothing, go out many at a time and need no division (BK is a power of two;
// a thread's place in a key's dims moves on by carrying).  Every thread of the workgroup calls it; it
// ends with a barrier.
template <typename T>
__device__ __forceinline__ void load_tile(float* Ks, float* Vs, long long* Kb, long long* Vb, const T* k_pool,
                                          const T* v_pool, const int32_t* bt, int kt, int last_pos, int BK, int dh,
                                          int page_size, int Hkv, int hk, int ld) {
  for (int j = threadIdx.x; j < BK; j += THREADS) {
    const int key = kt + j;
    const int page = key <= last_pos ? bt[key / page_size] : -1;
    const int off = key % page_size;
    const long long head = static_cast<long long>(max(page, 0)) * Hkv + hk;
    Kb[j] = page >= 0 ? (head * page_size + off) * dh : -1;
    Vb[j] = page >= 0 ? head * dh * page_size + off : -1;
  }
  __syncthreads();
  // BK * dh is at most 4,096 (tile_keys): 16 elements of the keys and 16 of the values per thread, all asked
  // for before the first is put into LDS
  constexpr int PER = 4096 / THREADS;
  const int n = BK * dh;
  float kv[PER], vv[PER];
  const int shift = 31 - __clz(BK);
  {
    int j = threadIdx.x / dh, d = threadIdx.x % dh;      // keys: consecutive threads along a key's dims
    const int dj = THREADS / dh, dd = THREADS % dh;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = threadIdx.x + i * THREADS;
      kv[i] = vv[i] = 0.f;
      if (e < n) {
        const long long at = Kb[j];
        if (at >= 0) kv[i] = to_float(k_pool[at + d]);
        // values: consecutive threads along the keys of a dim (a page holds a dim's values side by side)
        const long long av = Vb[e & (BK - 1)];
        if (av >= 0) vv[i] = to_float(v_pool[av + static_cast<long long>(e >> shift) * page_size]);
      }
      j += dj, d += dd;
      if (d >= dh) d -= dh, j += 1;
    }
  }
  {
    int j = threadIdx.x / dh, d = threadIdx.x % dh;
    const int dj = THREADS / dh, dd = THREADS % dh;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = threadIdx.x + i * THREADS;
      if (e < n) {
        Ks[j * ld + d] = kv[i];
        Vs[(e & (BK - 1)) * ld + (e >> shift)] = vv[i];
      }
      j += dj, d += dd;
      if (d >= dh) d -= dh, j += 1;
    }
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(THREADS) void attention_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows, const int32_t* __restrict__ tile_pos0, int H, int Hkv, int dh,
    int page_size, int BK, float scale, int window) {
  // A head size that is no multiple of 16 lies in LDS padded to the next one (dhp): the dims beyond dh are
  // zeros in the queries and the keys, add nothing to a score (a fused multiply-add of zeros leaves a sum as
  // it is), and are not stored; the real dims keep their order of summation.
  const int dhp = (dh + 15) / 16 * 16;
  extern __shared__ float smem[];
  float* Qs = smem;                    // [BQ][dhp]
  float* Ks = Qs + BQ * dhp;           // [BK][dhp + 1]
  float* Vs = Ks + BK * (dhp + 1);     // [BK][dhp + 1]
  float* Ps = Vs + BK * (dhp + 1);     // [BQ][BK]
  long long* Kb = reinterpret_cast<long long*>(Ps + BQ * BK);   // [BK], [BK]
  long long* Vb = Kb + BK;

  const int tile = blockIdx.x, h = blockIdx.y;
  const int seq = tile_seq[tile];
  if (seq < 0) return;   // padding of a fixed-size launch
  const int row0 = tile_row0[tile], nrows = tile_nrows[tile], pos0 = tile_pos0[tile];
  const int hk = h / (H / Hkv);
  const int32_t* bt = block_tables + static_cast<size_t>(seq) * max_blocks;
  const int t = threadIdx.x, qi = t / 16, g = t % 16;
  const float NEG_INF = -INFINITY;

  for (int e = t; e < BQ * dhp; e += THREADS) {
    int r = e / dhp, d = e % dhp;
    Qs[e] = r < nrows && d < dh ? to_float(q[static_cast<size_t>(row0 + r) * ldq + h * dh + d]) : 0.f;
  }
  if (dhp != dh) {      // (load_tile writes the real dims only)
    const int pad = dhp - dh;
    for (int e = t; e < BK * pad; e += THREADS) Ks[(e / pad) * (dhp + 1) + dh + e % pad] = Vs[(e / pad) * (dhp + 1) + dh + e % pad] = 0.f;
  }
  const bool row_ok = qi < nrows;
  const int my_pos = pos0 + qi;
  const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
  const int last_pos = pos0 + nrows - 1;
  const int first_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int nd = dhp / 16, nc = BK / 16;

  float m = NEG_INF, l = 0.f;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;

  for (int kt = (first_lo / BK) * BK; kt <= last_pos; kt += BK) {
    __syncthreads();
    load_tile(Ks, Vs, Kb, Vb, k_pool, v_pool, bt, kt, last_pos, BK, dh, page_size, Hkv, hk, dhp + 1);
    float m_t, l_t, a_t[16];
    tile_scores(Qs + qi * dhp, Ks, Ps + qi * BK, g, nc, dhp, kt, my_lo, my_pos, row_ok, scale, m_t, l_t);
    __syncthreads();
    if (m_t > NEG_INF) {                // the same for the 16 threads of a row
      tile_values(Ps + qi * BK, Vs, g, nd, dhp, BK, a_t);
      join_tile(m, l, acc, m_t, l_t, a_t, nd);
    }
  }
  if (row_ok) {
    float inv = 1.0f / l;
    T* o = out + static_cast<size_t>(row0 + qi) * ldo + h * dh;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i < nd && g + 16 * i < dh) o[g + 16 * i] = from_float<T>(acc[i] * inv);
  }
}

// A step of single rows (request s = tile s = row s): every tile of keys is a workgroup of its own, so
// that a context of a thousand keys is sixteen workgroups side by side and not sixteen steps of one.  It
// leaves (m_T, l_T, a_T) in part[((tile * H + h) * n_key_tiles + key tile) * (dh + 2)]; m_T = -inf: the
// tile holds no key of this row.  row_join_kernel joins them in ascending order.
template <typename T>
__global__ __launch_bounds__(THREADS) void row_tiles_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tile_seq,
    const int32_t* __restrict__ tile_pos0, float* __restrict__ part, int n_key_tiles, int H, int Hkv, int dh,
    int page_size, int BK, float scale, int window) {
  extern __shared__ float smem[];
  float* Qs = smem;                    // [dh]
  float* Ks = Qs + dh;                 // [BK][dh + 1]
  float* Vs = Ks + BK * (dh + 1);      // [BK][dh + 1]
  float* Ps = Vs + BK * (dh + 1);      // [BK]
  long long* Kb = reinterpret_cast<long long*>(Ps + BK);   // [BK], [BK]
  long long* Vb = Kb + BK;
  const int ktile = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
  const int seq = tile_seq[tile];
  if (seq < 0) return;
  const int pos = tile_pos0[tile];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int kt = ktile * BK;
  const int t = threadIdx.x, g = t % 16;
  float* mine = part + ((static_cast<size_t>(tile) * H + h) * n_key_tiles + ktile) * (dh + 2);
  if (kt > pos || kt + BK <= lo) {
    if (t == 0) mine[0] = -INFINITY;
    return;
  }
  const int hk = h / (H / Hkv);
  const int32_t* bt = block_tables + static_cast<size_t>(seq) * max_blocks;
  for (int d = t; d < dh; d += THREADS) Qs[d] = to_float(q[static_cast<size_t>(tile) * ldq + h * dh + d]);
  load_tile(Ks, Vs, Kb, Vb, k_pool, v_pool, bt, kt, pos, BK, dh, page_size, Hkv, hk, dh + 1);
  // One row.  The same sums in the same order as 16 threads of the kernel above make them, spread wider:
  // a thread per key for the scores, 16 threads for the sum of p as there, a thread per dim for the values.
  const float NEG_INF = -INFINITY;
  __shared__ float ml[2];
  if (t < 64) {
    float s = NEG_INF;
    if (t < BK) {
      const int key = kt + t;
      const float dot = key_dot(Qs, Ks + t * (dh + 1), dh);
      s = (key >= lo && key <= pos) ? dot * scale : NEG_INF;
    }
    const float tmax = wave_max(s);
    if (t < BK) Ps[t] = s > NEG_INF ? expf(s - tmax) : 0.f;
    // (the lanes of one wave: what they wrote to Ps is there for their reads)
    float psum = 0.f;
    if (t < 16)
      for (int c = 0; c < BK / 16; ++c) psum += Ps[t + 16 * c];
    psum = group_reduce<16>(psum, SumOp());
    if (t == 0) {
      ml[0] = tmax;
      ml[1] = psum;
      mine[0] = tmax;
      mine[1] = psum;
    }
  }
  __syncthreads();
  if (!(ml[0] > NEG_INF)) return;
  for (int d = t; d < dh; d += THREADS) mine[2 + d] = dim_sum(Ps, Vs + d, dh, BK);
}

// four consecutive elements in one load
__device__ __forceinline__ void load4(const float* p, float* v) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* v) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
}

// row_tiles_kernel for heads of 64 and pages that hold a multiple of 4 keys: the same sums in the same
// order, a workgroup being one wave.  Four keys from a multiple of 4 lie in one page, so a page is looked
// up once per four keys, by the wave and not by the lane.  The keys come 16 lanes to a key's 64 dims,
// 16 bytes each, are laid down in LDS as they came (keys 68 floats apart: no bank shared by the 16-byte
// stores or reads) and are read back a lane per key; the values come a lane per dim, four keys' values
// of that dim in one load (a page holds a dim's values side by side), and stay in registers.  All loads
// are asked for before the first is used, and none depends on another's result but for the page table's.
template <typename T>
__global__ __launch_bounds__(64) void row_tile64_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tile_seq,
    const int32_t* __restrict__ tile_pos0, float* __restrict__ part, int n_key_tiles, int H, int Hkv, int page_size,
    float scale, int window) {
  constexpr int DH = 64, BK = 64, LD = DH + 4, QUADS = BK / 4;
  __shared__ __attribute__((aligned(16))) float Ks[BK * LD];
  __shared__ __attribute__((aligned(16))) float Qs[DH];
  __shared__ __attribute__((aligned(16))) float Ps[BK];
  const int ktile = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
  const int seq = tile_seq[tile];
  if (seq < 0) return;
  const int pos = tile_pos0[tile];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int kt = ktile * BK;
  const int lane = threadIdx.x;
  float* mine = part + ((static_cast<size_t>(tile) * H + h) * n_key_tiles + ktile) * (DH + 2);
  if (kt > pos || kt + BK <= lo) {
    if (lane == 0) mine[0] = -INFINITY;
    return;
  }
  const int hk = h / (H / Hkv);
  const int32_t* bt = block_tables + static_cast<size_t>(seq) * max_blocks;
  // the page of each four keys (-1: beyond the row's position, or given back)
  int page[QUADS];
#pragma unroll
  for (int i = 0; i < QUADS; ++i) page[i] = kt + 4 * i <= pos ? bt[(kt + 4 * i) / page_size] : -1;
  const float qd = to_float(q[static_cast<size_t>(tile) * ldq + h * DH + lane]);
  const int r = lane / 16, c = lane % 16;
  float kv[QUADS][4], vv[QUADS][4];
#pragma unroll
  for (int i = 0; i < QUADS; ++i) {
    const size_t head = static_cast<size_t>(max(page[i], 0)) * Hkv + hk;
    const int off = (kt + 4 * i) % page_size;
    load4(k_pool + (head * page_size + off + r) * DH + 4 * c, kv[i]);
    load4(v_pool + (head * DH + lane) * page_size + off, vv[i]);
  }
  Qs[lane] = qd;
  // keys beyond the row's position and pages given back: zeros, as in load_tile
#pragma unroll
  for (int i = 0; i < QUADS; ++i) {
    const bool k_in = page[i] >= 0 && kt + 4 * i + r <= pos;
    *reinterpret_cast<float4*>(&Ks[(4 * i + r) * LD + 4 * c]) =
        k_in ? float4{kv[i][0], kv[i][1], kv[i][2], kv[i][3]} : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (!(page[i] >= 0 && kt + 4 * i + e <= pos)) vv[i][e] = 0.f;
  }
  __syncthreads();
  const float NEG_INF = -INFINITY;
  // a lane per key: the score over the dims in ascending order, as key_dot sums it
  float dot = 0.f;
#pragma unroll
  for (int d4 = 0; d4 < DH / 4; ++d4) {
    const float4 a = *reinterpret_cast<const float4*>(&Qs[4 * d4]);
    const float4 b = *reinterpret_cast<const float4*>(&Ks[lane * LD + 4 * d4]);
    dot = fmaf(a.x, b.x, dot);
    dot = fmaf(a.y, b.y, dot);
    dot = fmaf(a.z, b.z, dot);
    dot = fmaf(a.w, b.w, dot);
  }
  const int key = kt + lane;
  const float sc = (key >= lo && key <= pos) ? dot * scale : NEG_INF;
  const float tmax = wave_max(sc);
  Ps[lane] = sc > NEG_INF ? expf(sc - tmax) : 0.f;
  __syncthreads();
  // the sum of p as 16 threads of a row make it in the kernels above
  float psum = 0.f;
  if (lane < 16)
    for (int cc = 0; cc < BK / 16; ++cc) psum += Ps[lane + 16 * cc];
  psum = group_reduce<16>(psum, SumOp());
  if (lane == 0) {
    mine[0] = tmax;
    mine[1] = psum;
  }
  if (!(tmax > NEG_INF)) return;
  // a lane per dim: the tile's keys in ascending order, as dim_sum sums them
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < QUADS; ++i) {
    const float4 p4 = *reinterpret_cast<const float4*>(&Ps[4 * i]);
    a = fmaf(p4.x, vv[i][0], a);
    a = fmaf(p4.y, vv[i][1], a);
    a = fmaf(p4.z, vv[i][2], a);
    a = fmaf(p4.w, vv[i][3], a);
  }
  mine[2 + lane] = a;
}

template <typename T>
__global__ void row_join_kernel(const float* __restrict__ part, T* __restrict__ out, int ldo,
                                const int32_t* __restrict__ tile_seq, int n_key_tiles, int H, int dh) {
  const int tile = blockIdx.x, h = blockIdx.y;
  if (tile_seq[tile] < 0) return;
  const int g = threadIdx.x;           // 16 threads, the dims g + 16 i each, as in the kernels above
  const int nd = dh / 16;
  const float* base = part + (static_cast<size_t>(tile) * H + h) * n_key_tiles * (dh + 2);
  float m = -INFINITY, l = 0.f;
  float acc[16], a_t[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  // four tiles' results are asked for at a time (a tile without a key left only its first number: the rest
  // of its entry is read and not used); they are joined one after the other, in order
  for (int kt0 = 0; kt0 < n_key_tiles; kt0 += 4) {
    float m_t[4], l_t[4], a4[4][16];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float* p = base + static_cast<size_t>(min(kt0 + u, n_key_tiles - 1)) * (dh + 2);
      m_t[u] = p[0];
      l_t[u] = p[1];
#pragma unroll
      for (int i = 0; i < 16; ++i) a4[u][i] = i < nd ? p[2 + g + 16 * i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (kt0 + u >= n_key_tiles || !(m_t[u] > -INFINITY)) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) a_t[i] = a4[u][i];
      join_tile(m, l, acc, m_t[u], l_t[u], a_t, nd);
    }
  }
  const float inv = 1.0f / l;
  T* o = out + static_cast<size_t>(tile) * ldo + h * dh;
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i < nd) o[g + 16 * i] = from_float<T>(acc[i] * inv);
}

// keys in a tile: a power of two, and at most 4,096 / dh (load_tile)
static int tile_keys(int dh) { return dh <= 64 ? 64 : (dh <= 128 ? 32 : 16); }
}  // namespace plain

extern "C" int dn_attention(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                            const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                            const int32_t* tile_row0, const int32_t* tile_nrows, const int32_t* tile_pos0,
                            int n_tiles, int H, int Hkv, int dh, int page_size, float scale, int window, int dtype,
                            hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  // (any head size up to 256: one that is no multiple of 16 is padded to the next inside the kernel)
  if (dh < 1 || dh > 256 || Hkv < 1 || H % Hkv != 0 || page_size < 1 || max_blocks < 1) return DN_ERR_SHAPE;
  const int dhp = (dh + 15) / 16 * 16;
  int BK = plain::tile_keys(dhp);
  size_t lds = sizeof(float) * (static_cast<size_t>(plain::BQ) * dhp + 2 * static_cast<size_t>(BK) * (dhp + 1) +
                                static_cast<size_t>(plain::BQ) * BK + 4 * BK);
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

// A step of single rows with the plain kernels, every tile of keys a workgroup of its own: the same bits as
// dn_attention gives (one order of summation).  max_context: the longest context of the step; part:
// n_tiles * H * ceil(max_context / tile) * (dh + 2) floats, the tile being dn_attention_rows_tile(dh) keys.
extern "C" int dn_attention_rows_tile(int dh) { return plain::tile_keys(dh); }

extern "C" int dn_attention_rows(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                                 const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                                 const int32_t* tile_pos0, int n_tiles, float* part, int max_context, int H, int Hkv,
                                 int dh, int page_size, float scale, int window, int dtype, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (dh < 16 || dh > 256 || dh % 16 != 0 || Hkv < 1 || H % Hkv != 0 || page_size < 1 || max_blocks < 1 ||
      max_context < 1 || !part || n_tiles > 65535 || H > 65535)
    return DN_ERR_SHAPE;
  const int BK = plain::tile_keys(dh);
  const int n_key_tiles = (max_context + BK - 1) / BK;
  const size_t lds = sizeof(float) * (static_cast<size_t>(dh) + 2 * static_cast<size_t>(BK) * (dh + 1) + 5 * BK);
  dim3 grid(n_key_tiles, H, n_tiles), block(plain::THREADS);
  const bool wave_tiles = dh == 64 && page_size % 4 == 0 && reinterpret_cast<uintptr_t>(k_pool) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(v_pool) % 16 == 0;
#define DN_ROWS(T)                                                                                                   \
  if (wave_tiles)                                                                                                    \
    hipLaunchKernelGGL(plain::row_tile64_kernel<T>, grid, dim3(64), 0, stream, static_cast<const T*>(q), ldq,        \
                       static_cast<const T*>(k_pool), static_cast<const T*>(v_pool), block_tables, max_blocks,       \
                       tile_seq, tile_pos0, part, n_key_tiles, H, Hkv, page_size, scale, window);                    \
  else                                                                                                               \
    hipLaunchKernelGGL(plain::row_tiles_kernel<T>, grid, block, lds, stream, static_cast<const T*>(q), ldq,          \
                       static_cast<const T*>(k_pool), static_cast<const T*>(v_pool), block_tables, max_blocks,       \
                       tile_seq, tile_pos0, part, n_key_tiles, H, Hkv, dh, page_size, BK, scale, window);            \
  hipLaunchKernelGGL(plain::row_join_kernel<T>, dim3(n_tiles, H), dim3(16), 0, stream, part, static_cast<T*>(out), ldo, \
                     tile_seq, n_key_tiles, H, dh)
  if (dtype == DN_F32) {
    DN_ROWS(float);
  } else if (dtype == DN_BF16) {
    DN_ROWS(bf16_t);
  } else {
    return DN_ERR_DTYPE;
  }
#undef DN_ROWS
  return dn_launch_status();
}

// =======================================================================================
// bfloat16 kernels.  Both need page_size % 16 == 0 (a run of 16 keys lies in one page).
// =======================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

__device__ __forceinline__ __bf16 to_bf16(float f) { return static_cast<__bf16>(f); }

// eight values rounded to bfloat16, two per conversion (v_cvt_pk_bf16_f32 takes a pair)
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
__device__ __forceinline__ bf16x8 to_bf16x8(const float* v) {
  typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{v[2 * i], v[2 * i + 1]}, bf16x2));
  return __builtin_bit_cast(bf16x8, w);
}

// ---------------------------------------------------------------------------------------
// flash: portions of prompts.  A workgroup takes up to 128 consecutive rows of one request
// and one head.  It has GROUPS x 4 waves: wave w owns the 32 rows 32 (w % 4), and the groups
// share out the keys, tile of 32 by tile (group w / 4 takes tiles w / 4, w / 4 + GROUPS, ...):
// what a wave does for one tile is a chain of dependent steps (scores, maximum, exponentials,
// sum, values) of some thousand cycles whatever else runs, so a row's time is the number of
// tiles its wave walks; two groups halve it, and join their running maxima, sums and weighted
// values through LDS at the end, in group order.  With one group a wave takes two tiles per step
// (up to a head size of 96: the tiles of two steps must fit 64 KB of LDS), under one maximum, one
// sum and one rescaling.
// A tile's keys and values come from the pages once per workgroup, 16 bytes per thread along
// rows (two cache lines per 16 lanes), and lie in LDS for the four waves that need them, two
// steps deep: the tiles of the step after the next are on their way to registers while this
// step's are multiplied.
//   S^T[key, q] = K . Q^T : lane (key = lane % 32, half g = lane / 32) gives 8 dims of a key.
//   The result leaves each lane with 16 keys of ONE query (its column), so the running
//   softmax is lane-local but for one exchange between the halves.
//   O^T[d, q] += V^T . P^T : the lane's 16 probabilities are, eight by eight, exactly the
//   B operand of two MFMAs whose k slots are the keys 16a + 4g + {0..3, 8..11}; the A
//   operand reads those keys of dim d from the transposed values, 8 bytes at a time.
// Two waves per SIMD at least are asked for: with room for one wave only, the compiler keeps the
// MFMA results in accumulation registers and copies all of them to and fro around every rescaling.
// ---------------------------------------------------------------------------------------
namespace flash {
constexpr int ROWS = 128;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;

// POW2: the page size is a power of two (page_size = 1 << page_shift), so that a key's page and its place in
// the page are a shift and a mask: a tile's keys need four such pairs a step, and a division by a number
// known only at run time is some twenty-five vector instructions.
template <int DH16, int GROUPS, int TPS, bool POW2>     // head size / 16; groups of 4 waves; tiles a wave takes per step
__global__ __launch_bounds__(256 * GROUPS) __attribute__((amdgpu_waves_per_eu(DH16 > 12 && GROUPS == 1 ? 1 : 2))) void kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows, const int32_t* __restrict__ tile_pos0, int H, int Hkv, int page_size,
    int page_shift, float scale, int window) {
  constexpr int DH = DH16 * 16;
  constexpr int DB = (DH + 31) / 32;
  auto page_index = [&](int key) { return POW2 ? key >> page_shift : key / page_size; };
  auto page_offset = [&](int key) { return POW2 ? key & (page_size - 1) : key % page_size; };
  constexpr int CH = DH / 8;                 // 16-byte chunks in a key
  constexpr int KROW = (CH + 1) * 8;         // a key's row in LDS, one chunk of padding: 16 rows, 16 bank groups
  constexpr int VROW = 40;                   // a dim's row of 32 keys in LDS, 16 bytes of padding
  constexpr int KCH = 32 * CH, VCH = DH * 4; // chunks of a tile of keys, of values
  constexpr int KU = (KCH + 255) / 256, VU = (VCH + 255) / 256;
  constexpr int KSZ = 32 * KROW, TSZ = KSZ + DH * VROW;     // elements of a tile's keys, of a whole tile
  constexpr int STEP = 32 * GROUPS * TPS;    // keys per step
  constexpr int JOIN = 2 + 16 * DB;          // floats a lane hands over at the end
  constexpr int BYTES_TILES = 2 * GROUPS * TPS * TSZ * 2, BYTES_JOIN = GROUPS > 1 ? 4 * 64 * JOIN * 4 : 0;
  __shared__ __attribute__((aligned(16))) unsigned char smem[BYTES_TILES > BYTES_JOIN ? BYTES_TILES : BYTES_JOIN];
  bf16_t* const tiles_lds = reinterpret_cast<bf16_t*>(smem);      // [2 steps][GROUPS][TPS][keys | values]
  // workgroups start in the order of the tile table, all heads of a tile together: the table lists
  // the tiles with the longest contexts first, so the longest work is not what starts last
  const int h = blockIdx.x, tile = blockIdx.y;
  const int seq = tile_seq[tile];
  if (seq < 0) return;                       // the whole workgroup
  const int row0 = tile_row0[tile], nrows = tile_nrows[tile], pos0 = tile_pos0[tile];
  // (the wave's number through readfirstlane: what follows from it, the wave's rows and keys, which tiles it
  // carries and whether a tile touches an edge, is then worked out once per wave by the scalar unit, and its
  // page numbers come by scalar loads)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int grp = wave / 4;                  // which tiles this wave multiplies
  const int t = threadIdx.x % 256, ti = wave / 4;   // this thread carries chunk t of the step's tiles ti TPS ..
  const int wrow0 = (wave % 4) * 32;
  const bool has_rows = wrow0 < nrows;       // a wave without rows still carries tiles into LDS
  const int qcol = lane % 32, g = lane / 32;
  const int hk = h / (H / Hkv);
  const int32_t* bt = block_tables + static_cast<size_t>(seq) * max_blocks;
  const bool row_ok = wrow0 + qcol < nrows;
  const int my_row = min(wrow0 + qcol, nrows - 1);
  const int my_pos = pos0 + my_row;
  const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
  const int lo_w = window > 0 ? max(0, pos0 + wrow0 - window + 1) : 0;      // this wave's keys
  const int hi_w = pos0 + min(wrow0 + 31, nrows - 1);
  const int lo_g = window > 0 ? max(0, pos0 - window + 1) : 0;              // the workgroup's
  const int hi_g = pos0 + nrows - 1;
  const float NEG_INF = -INFINITY;
  const float scale2 = scale * 1.44269504088896340736f;    // log2(e)
  const u32x4 zero4 = {0u, 0u, 0u, 0u};

  bf16x8 qf[DH16];
  {
    const bf16_t* qr = q + static_cast<size_t>(row0 + my_row) * ldq + h * DH + g * 8;
#pragma unroll
    for (int c = 0; c < DH16; ++c) qf[c] = *reinterpret_cast<const bf16x8*>(qr + c * 16);
  }
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m = NEG_INF, l = 0.f;

  // A tile of 32 keys lies in two pages (or in one, if pages are longer): pg[0] for keys
  // kt .. kt+15, pg[1] for kt+16 .. kt+31; -1 beyond the rows' last key.
  struct Pages { int a, b; };
  auto pages_of = [&](int kt_) {
    return Pages{kt_ <= hi_g ? bt[page_index(kt_)] : -1, kt_ + 16 <= hi_g ? bt[page_index(kt_ + 16)] : -1};
  };
  // Thread t's share of its tile: chunk t (+ 256 u) of the keys, counted along a key's dims and
  // then from key to key, and of the values, counted along a dim's 16 keys of a page, then from
  // dim to dim, then the second run of 16.  Never a conditional load: what has no page reads the
  // pool's start and is stored as zeros.
  u32x4 kregs[TPS][KU], vregs[TPS][VU];
  auto fetch = [&](int kt_, const Pages pg, u32x4* kreg, u32x4* vreg) {
    const int off0 = page_offset(kt_), off1 = page_offset(kt_ + 16);
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int idx = min(t + 256 * u, KCH - 1), key = idx / CH, ch = idx % CH;
      const int page = key < 16 ? pg.a : pg.b;
      const int off = (key < 16 ? off0 : off1) + key % 16;
      kreg[u] = *reinterpret_cast<const u32x4*>(
          k_pool + (page >= 0 ? ((static_cast<size_t>(page) * Hkv + hk) * page_size + off) * DH : 0) + ch * 8);
    }
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int idx = min(t + 256 * u, VCH - 1), a0 = idx / (DH * 2), d = (idx % (DH * 2)) / 2, half = idx % 2;
      const int page = a0 ? pg.b : pg.a;
      vreg[u] = *reinterpret_cast<const u32x4*>(
          v_pool + (page >= 0 ? ((static_cast<size_t>(page) * Hkv + hk) * DH + d) * page_size + (a0 ? off1 : off0) : 0) +
          half * 8);
    }
  };
  auto stash = [&](const Pages pg, bf16_t* dst, const u32x4* kreg, const u32x4* vreg) {
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int idx = t + 256 * u, key = idx / CH, ch = idx % CH;
      if (idx < KCH)
        *reinterpret_cast<u32x4*>(dst + key * KROW + ch * 8) = (key < 16 ? pg.a : pg.b) >= 0 ? kreg[u] : zero4;
    }
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int idx = t + 256 * u, a0 = idx / (DH * 2), d = (idx % (DH * 2)) / 2, half = idx % 2;
      if (idx < VCH)
        *reinterpret_cast<u32x4*>(dst + KSZ + d * VROW + a0 * 16 + half * 8) = (a0 ? pg.b : pg.a) >= 0 ? vreg[u] : zero4;
    }
  };

  // Step kt first puts the tiles of step kt + STEP (asked for during the step before) from
  // registers into the half of LDS that the step before read (every wave has left it: the
  // barrier), then asks for the tiles of step kt + 2 STEP, then multiplies.
  const int kt0 = (lo_g / STEP) * STEP;
  const int mine = 32 * TPS * ti;            // this thread carries the tiles at kt + mine + 32 c
  Pages pg_now[TPS], pg_reg[TPS], pg_far[TPS];    // pages of the tiles in registers and of those to ask for next
#pragma clang loop unroll(full)
  for (int c = 0; c < TPS; ++c) {
    pg_now[c] = pages_of(kt0 + mine + 32 * c);
    fetch(kt0 + mine + 32 * c, pg_now[c], kregs[c], vregs[c]);
    pg_reg[c] = pages_of(kt0 + STEP + mine + 32 * c);
  }
#pragma clang loop unroll(full)
  for (int c = 0; c < TPS; ++c) {
    stash(pg_now[c], tiles_lds + (ti * TPS + c) * TSZ, kregs[c], vregs[c]);
    fetch(kt0 + STEP + mine + 32 * c, pg_reg[c], kregs[c], vregs[c]);
    pg_far[c] = pages_of(kt0 + 2 * STEP + mine + 32 * c);
  }
  __syncthreads();
  int buf = 0;
  for (int kt = kt0; kt <= hi_g; kt += STEP, buf ^= 1) {
#pragma clang loop unroll(full)
    for (int c = 0; c < TPS; ++c) {
      if (kt + STEP <= hi_g) stash(pg_reg[c], tiles_lds + (((buf ^ 1) * GROUPS + ti) * TPS + c) * TSZ, kregs[c], vregs[c]);
      if (kt + 2 * STEP <= hi_g) fetch(kt + 2 * STEP + mine + 32 * c, pg_far[c], kregs[c], vregs[c]);
      pg_reg[c] = pg_far[c];
      pg_far[c] = pages_of(kt + 3 * STEP + mine + 32 * c);
    }

    // this wave's tiles of the step: kw0 + 32 c.  They share one maximum, one sum and one rescaling:
    // the chain of dependent steps (scores, maximum, exponentials, sum, values) is as long for two
    // tiles as for one, and it is that chain, not the work, which a wave's time is made of
    const int kw0 = kt + 32 * TPS * grp;
    bool act[TPS], any = false;
#pragma unroll
    for (int c = 0; c < TPS; ++c) {
      act[c] = has_rows && kw0 + 32 * c <= hi_w && kw0 + 32 * c + 31 >= lo_w;     // the same for the whole wave
      any = any || act[c];
    }
    if (any) {
      const bf16_t* Tb = tiles_lds + (buf * GROUPS + grp) * TPS * TSZ;
      // (the first product of a tile starts from a constant zero: no registers to clear)
      const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      floatx16 s[TPS];
#pragma unroll
      for (int c = 0; c < TPS; ++c) {
        if (!act[c]) {
#pragma unroll
          for (int i = 0; i < 16; ++i) s[c][i] = NEG_INF;
          continue;
        }
        const bf16_t* Kb = Tb + c * TSZ;
#pragma unroll
        for (int cc = 0; cc < DH16; ++cc) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(Kb + qcol * KROW + (2 * cc + g) * 8);
          s[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[cc], cc == 0 ? zero16 : s[c], 0, 0, 0);
        }
      }
      // s[c][i]: key kw + 8*(i/4) + 4*g + i%4, query = this lane's column.  The running maximum is kept
      // times scale * log2(e) (the scale is positive: the largest score is the largest product), so that
      // each probability is one multiply-add and one v_exp_f32 on the product as the MFMA left it.  Only a
      // tile that touches the causal edge (or the window's) of one of the wave's rows needs the mask; the
      // others skip it, the same for the whole wave.
      float tmax = NEG_INF;
#pragma unroll
      for (int c = 0; c < TPS; ++c) {
        const int kw = kw0 + 32 * c;
        const bool edge = kw + 31 > pos0 + wrow0 || (window > 0 && kw < hi_w - window + 1);
        if (!act[c]) continue;
        if (edge) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int key = kw + 8 * (i / 4) + 4 * g + (i % 4);
            bool ok = key >= my_lo && key <= my_pos;
            s[c][i] = ok ? s[c][i] : NEG_INF;
            tmax = fmaxf(tmax, s[c][i]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[c][i]);
        }
      }
      tmax = fmaxf(tmax, other_half(tmax)) * scale2;      // (-inf stays -inf)
      float p[TPS][16];
      float psum = 0.f, alpha = 1.f;
      if (tmax > NEG_INF) {
        float m_new = fmaxf(m, tmax);
        alpha = __builtin_amdgcn_exp2f(m - m_new);      // m = -inf at first: 2^-inf = 0
#pragma unroll
        for (int c = 0; c < TPS; ++c)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            p[c][i] = __builtin_amdgcn_exp2f(fmaf(s[c][i], scale2, -m_new));  // a masked score is -inf: 0
            psum += p[c][i];
          }
        m = m_new;
      } else {
#pragma unroll
        for (int c = 0; c < TPS; ++c)
#pragma unroll
          for (int i = 0; i < 16; ++i) p[c][i] = 0.f;
      }
      psum += other_half(psum);
      l = l * alpha + psum;
      bf16x8 pb[TPS][2];
#pragma unroll
      for (int c = 0; c < TPS; ++c)
#pragma unroll
        for (int a0 = 0; a0 < 2; ++a0) pb[c][a0] = to_bf16x8(&p[c][8 * a0]);
      // alpha belongs to the lane's query, and so do all of the lane's accumulators; once the running
      // maxima have settled it is 1 for the whole wave, tile after tile
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
      }
      // values: as A operand the lane's row is a dim, its 8 k slots the keys 16 a0 + 4 g + {0..3, 8..11}
#pragma unroll
      for (int c = 0; c < TPS; ++c) {
        if (!act[c]) continue;
        const bf16_t* Vb = Tb + c * TSZ + KSZ;
#pragma unroll
        for (int a0 = 0; a0 < 2; ++a0) {
          if (kw0 + 32 * c + 16 * a0 > hi_w) continue;       // the same for every lane of the wave: all its probabilities are 0
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const bf16_t* vr = Vb + min(32 * db + qcol, DH - 1) * VROW + 16 * a0 + 4 * g;
            const bf16x4 vlo = *reinterpret_cast<const bf16x4*>(vr), vhi = *reinterpret_cast<const bf16x4*>(vr + 8);
            bf16x8 vf = bf16x8{vlo[0], vlo[1], vlo[2], vlo[3], vhi[0], vhi[1], vhi[2], vhi[3]};
            if (32 * db + qcol >= DH) vf = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
            o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[c][a0], o[db], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();      // the other half of LDS is written and this one has been read by every wave
  }
  if constexpr (GROUPS > 1) {
    // the second group hands its maxima, sums and weighted values to the first, lane to lane (both
    // hold the same queries in the same lanes); the tiles in LDS are done with
    float* join = reinterpret_cast<float*>(smem) + ((wave % 4) * 64 + lane) * JOIN;
    if (grp == 1) {
      join[0] = m;
      join[1] = l;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) join[2 + 16 * db + i] = o[db][i];
    }
    __syncthreads();
    if (grp == 1) return;
    const float m1 = join[0], l1 = join[1];
    const float m_new = fmaxf(m, m1);
    const float f0 = m > NEG_INF ? __builtin_amdgcn_exp2f(m - m_new) : 0.f;
    const float f1 = m1 > NEG_INF ? __builtin_amdgcn_exp2f(m1 - m_new) : 0.f;
    l = l * f0 + l1 * f1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] = o[db][i] * f0 + join[2 + 16 * db + i] * f1;
  }
  if (has_rows && row_ok) {
    const float inv = 1.0f / l;
    // rows, or packed rows (ldo == 0): four dims from a multiple of 4 are 8 bytes side by side in both
    const int orow_i = row0 + my_row;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d0 = 32 * db + 8 * a + 4 * g;
        if (d0 < DH) {
          bf16x4 w = {to_bf16(o[db][4 * a] * inv), to_bf16(o[db][4 * a + 1] * inv), to_bf16(o[db][4 * a + 2] * inv),
                      to_bf16(o[db][4 * a + 3] * inv)};
          bf16_t* dst = ldo > 0 ? out + static_cast<size_t>(orow_i) * ldo + h * DH + d0
                                : out + packed_index(orow_i, h * DH + d0, H * DH / 32);
          *reinterpret_cast<bf16x4*>(dst) = w;
        }
      }
  }
}
}  // namespace flash

extern "C" int dn_attention_flash(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                                  const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                                  const int32_t* tile_row0, const int32_t* tile_nrows, const int32_t* tile_pos0,
                                  int n_tiles, int H, int Hkv, int dh, int page_size, float scale, int window,
                                  hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  // ldo == 0: out is a packed matrix of H * dh columns (a multiple of 32); the kernel takes the largest score
  // for the largest product of a query and a key, so the scale is positive
  if (!(scale > 0.f)) return DN_ERR_SHAPE;
  if (Hkv < 1 || H % Hkv != 0 || page_size % 16 != 0 || max_blocks < 1 || ldq % 8 != 0 || ldo % 4 != 0 || ldo < 0 ||
      (ldo == 0 && (H * dh) % 32 != 0) || reinterpret_cast<uintptr_t>(q) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(out) % 8 != 0)
    return DN_ERR_SHAPE;
  // Two groups of waves up to a head size of 64: a wave's chain of dependent steps per tile bounds a
  // workgroup's time, and two groups halve the tiles a wave walks (the faster, or level, at every grid
  // size measured).  Beyond, one group: with heads of 96 and 128 two were the slower wherever the
  // workgroups outnumber the CUs.
  if (n_tiles > 65535) return DN_ERR_SHAPE;      // the grid's second dimension
  dim3 grid(H, n_tiles);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const bool pow2 = (1 << page_shift) == page_size;
#define DN_FLASH_P(D, G, T, P)                                                                                        \
  hipLaunchKernelGGL((flash::kernel<D, G, T, P>), grid, dim3(256 * G), 0, stream, static_cast<const bf16_t*>(q), ldq, \
                     static_cast<bf16_t*>(out), ldo, static_cast<const bf16_t*>(k_pool),                             \
                     static_cast<const bf16_t*>(v_pool), block_tables, max_blocks, tile_seq, tile_row0, tile_nrows,   \
                     tile_pos0, H, Hkv, page_size, page_shift, scale, window)
#define DN_FLASH_G(D, G, T)    \
  if (pow2)                    \
    DN_FLASH_P(D, G, T, true); \
  else                         \
    DN_FLASH_P(D, G, T, false)
#define DN_FLASH2(D) DN_FLASH_G(D, 2, 1)                      /* two groups of waves, a tile each */
#define DN_FLASH1(D) DN_FLASH_G(D, 1, (D <= 6 ? 2 : 1))       /* one group, two tiles a step where registers allow */
  switch (dh) {
    case 16: DN_FLASH2(1); break;
    case 32: DN_FLASH2(2); break;
    case 48: DN_FLASH2(3); break;
    case 64: DN_FLASH2(4); break;
    case 80: DN_FLASH1(5); break;
    case 96: DN_FLASH1(6); break;
    case 112: DN_FLASH1(7); break;
    case 128: DN_FLASH1(8); break;
    case 144: DN_FLASH1(9); break;
    case 160: DN_FLASH1(10); break;
    case 176: DN_FLASH1(11); break;
    case 192: DN_FLASH1(12); break;
    case 208: DN_FLASH1(13); break;
    case 224: DN_FLASH1(14); break;
    case 240: DN_FLASH1(15); break;
    case 256: DN_FLASH1(16); break;
    default: return DN_ERR_SHAPE;
  }
#undef DN_FLASH1
#undef DN_FLASH2
#undef DN_FLASH_G
#undef DN_FLASH_P
  return dn_launch_status();
}

// ---------------------------------------------------------------------------------------
// decode: one row per request, request s being tile s and row s of the step (tile_seq[s] < 0:
// padding; tile_pos0[s]: its position).  A workgroup has 4, 8 or 16 waves, 64 keys each at a time
// (its chunk: 256, 512 or 1024 keys), chosen so that a short context is one chunk: every load of
// a wave is then issued at once, behind one lookup of its pages.  The context is cut into
// n_splits runs of `chunks` chunks; a workgroup walks its run chunk by chunk (each wave with a
// running maximum, sum and weighted values, joined through LDS at the end) and, if there is
// more than one split, a second kernel joins the splits' results in split order
// (crates/denno-engine/kernels/kernels_elem.cu:577-603 has this two-kernel shape).
// Scores: dh/8 lanes share a key, 16 bytes each, so one load instruction reads whole keys side
// by side; all loads of 64 keys are issued before the first is used.  Values: lane = dim,
// 16 keys (32 bytes) of a transposed page at a time.  Nothing but registers and lane
// exchanges inside the loop.
// ---------------------------------------------------------------------------------------
namespace decode {
// POW2: page_size = 1 << page_shift; a key's page and its place in the page are then a shift and a mask (a lane
// works out a dozen such pairs per 64 keys before it can ask for the keys and values: as divisions by a number
// known only at run time they were some six hundred instructions in front of the loads)
// A key's 16-byte pieces lie on LPK lanes side by side, LPK the power of two that holds them: with a head size
// that is no power of two (48, 80, 96, ...) the lanes beyond the key's last piece hold zeros.
constexpr int lanes_per_key(int dh) { return dh <= 16 ? 2 : dh <= 32 ? 4 : dh <= 64 ? 8 : dh <= 128 ? 16 : 32; }

template <int DH, int WAVES, bool POW2>   // head size (a multiple of 16 up to 256); waves per workgroup
__global__ __launch_bounds__(WAVES * 64) void partial_kernel(const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out,
                                                       int ldo, const bf16_t* __restrict__ k_pool,
                                                       const bf16_t* __restrict__ v_pool,
                                                       const int32_t* __restrict__ block_tables, int max_blocks,
                                                       const int32_t* __restrict__ tile_seq,
                                                       const int32_t* __restrict__ tile_row0,
                                                       const int32_t* __restrict__ tile_pos0,
                                                       float* __restrict__ part, int n_splits, int chunks, int H,
                                                       int Hkv, int page_size, int page_shift, float scale,
                                                       int window) {
  static_assert(DH % 16 == 0 && DH >= 16 && DH <= 256, "head size");
  constexpr int LPK = lanes_per_key(DH);
  constexpr int PIECES = DH / 8;         // 16-byte pieces of a key: the lanes sub < PIECES of its LPK
  auto page_index = [&](int key) { return POW2 ? key >> page_shift : key / page_size; };
  auto page_offset = [&](int key) { return POW2 ? key & (page_size - 1) : key % page_size; };
  constexpr int KPI = 64 / LPK;          // keys per load instruction
  constexpr int DPL = (DH + 63) / 64;    // dims per lane in the second product
  constexpr int GROUP = LPK < 8 ? LPK : 8;   // load instructions issued together
  constexpr int CHUNK = WAVES * 64;          // keys that the workgroup's waves take at a time
  __shared__ float wm[WAVES], wl[WAVES];
  __shared__ float wacc[WAVES][DH];
  // In a step of single rows request s brings row s and is tile s: the block table and the query
  // are addressed by the workgroup's index, so their loads do not wait for the tile table's.
  const int split = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
  const int row = tile;
  const int32_t* bt = block_tables + static_cast<size_t>(tile) * max_blocks;
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);   // (a scalar)
  const int sub = lane % LPK, grp = lane / LPK;
  const bool holds = PIECES == LPK || sub < PIECES;     // (a lane without a piece: zeros, which add nothing to a score)
  bf16x8 qv = {};
  if (holds) qv = *reinterpret_cast<const bf16x8*>(q + static_cast<size_t>(row) * ldq + h * DH + sub * 8);
  if (tile_seq[tile] < 0) return;
  const int pos = tile_pos0[tile];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int key0 = split * chunks * CHUNK;
  const float NEG_INF = -INFINITY;
  float* mypart = part + ((static_cast<size_t>(tile) * H + h) * n_splits + split) * (DH + 2);
  if (key0 > pos || key0 + chunks * CHUNK <= lo) {
    if (n_splits > 1 && threadIdx.x == 0) {
      mypart[0] = NEG_INF;     // the join skips it
      mypart[1] = 0.f;
    }
    return;
  }
  const int hk = h / (H / Hkv);
  float qr[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) qr[i] = static_cast<float>(qv[i]) * scale;
  float m_run = NEG_INF, l_run = 0.f;
  float acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) acc[i] = 0.f;

  for (int c = 0; c < chunks; ++c) {
    const int kbase = key0 + c * CHUNK + wave * 64;
    if (kbase > pos || kbase + 64 <= lo) continue;     // the same for the whole wave; no barrier in this loop
    // values: lane = dim; 16 keys of one page at a time.  They are asked for first, before the keys
    // (whose use would otherwise stand between them and memory): keys and values then make one trip
    bf16x8 v0[4][DPL], v1[4][DPL];
    bool live[4];
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      const int kb = kbase + blk * 16;
      live[blk] = kb <= pos && kb + 16 > lo;
      const int kk = live[blk] ? kb : (pos / 16) * 16;
      const int page = bt[page_index(kk)];
      live[blk] = live[blk] && page >= 0;
      const bf16_t* vb = v_pool + (static_cast<size_t>(max(page, 0)) * Hkv + hk) * DH * page_size + page_offset(kk);
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int d = min(lane + 64 * i, DH - 1);
        v0[blk][i] = *reinterpret_cast<const bf16x8*>(vb + static_cast<size_t>(d) * page_size);
        v1[blk][i] = *reinterpret_cast<const bf16x8*>(vb + static_cast<size_t>(d) * page_size + 8);
      }
    }
    // scores: lane (key group grp, part sub of the key); after the sum over the key's lanes every
    // lane of group grp holds, in sc[it], the score of key kbase + it * KPI + grp
    float sc[LPK];
#pragma unroll
    for (int it0 = 0; it0 < LPK; it0 += GROUP) {
      bf16x8 kv[GROUP];
#pragma unroll
      for (int u = 0; u < GROUP; ++u) {
        const int key = kbase + (it0 + u) * KPI + grp;
        const int kk = (key >= lo && key <= pos) ? key : pos;     // a key that surely has a page
        const int page = bt[page_index(kk)];
        kv[u] = bf16x8{};
        if (holds)
          kv[u] = *reinterpret_cast<const bf16x8*>(
              k_pool + ((static_cast<size_t>(page) * Hkv + hk) * page_size + page_offset(kk)) * DH + sub * 8);
      }
#pragma unroll
      for (int u = 0; u < GROUP; ++u) {
        const int key = kbase + (it0 + u) * KPI + grp;
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) dot = fmaf(qr[i], static_cast<float>(kv[u][i]), dot);
        dot = group_reduce<LPK>(dot, SumOp());
        sc[it0 + u] = (key >= lo && key <= pos) ? dot : NEG_INF;
      }
    }
    float m_c = NEG_INF;
#pragma unroll
    for (int it = 0; it < LPK; ++it) m_c = fmaxf(m_c, sc[it]);
    m_c = wave_max(m_c);
    if (!(m_c > NEG_INF)) continue;
    const float m_new = fmaxf(m_run, m_c);
    const float alpha = m_run > NEG_INF ? __expf(m_run - m_new) : 0.f;
    float p[LPK];
    float psum = 0.f;
#pragma unroll
    for (int it = 0; it < LPK; ++it) {
      p[it] = sc[it] > NEG_INF ? __expf(sc[it] - m_new) : 0.f;
      psum += p[it];
    }
    // each key is held by LPK lanes: its first lane counts it
    l_run = l_run * alpha + wave_sum(sub == 0 ? psum : 0.f);
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[i] *= alpha;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      if (!live[blk]) continue;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int key = blk * 16 + j;      // key = it * KPI + grp: held by lane grp * LPK in p[it]
        const float pj = lane_value(p[key / KPI], (key % KPI) * LPK);
#pragma unroll
        for (int i = 0; i < DPL; ++i)
          acc[i] = fmaf(pj, static_cast<float>(j < 8 ? v0[blk][i][j] : v1[blk][i][j - 8]), acc[i]);
      }
    }
  }
  if (lane == 0) {
    wm[wave] = m_run;
    wl[wave] = l_run;
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i)
    if (lane + 64 * i < DH) wacc[wave][lane + 64 * i] = acc[i];
  __syncthreads();
  for (int d = threadIdx.x; d < DH; d += WAVES * 64) {
    float M = wm[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) M = fmaxf(M, wm[w]);
    float L = 0.f, A = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      if (wm[w] > NEG_INF) {
        float f = __expf(wm[w] - M);
        L += wl[w] * f;
        A += wacc[w][d] * f;
      }
    }
    if (n_splits == 1) {
      out[ldo > 0 ? static_cast<size_t>(row) * ldo + h * DH + d : packed_index(row, h * DH + d, H * DH / 32)] =
          from_float<bf16_t>(A / L);
    } else {
      mypart[2 + d] = A;
      if (d == 0) {
        mypart[0] = M;
        mypart[1] = L;
      }
    }
  }
}

__global__ void join_kernel(const float* __restrict__ part, bf16_t* __restrict__ out, int ldo,
                            const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_row0, int n_splits,
                            int H, int DH) {
  const int tile = blockIdx.x, h = blockIdx.y;
  if (tile_seq[tile] < 0) return;
  const float* base = part + (static_cast<size_t>(tile) * H + h) * n_splits * (DH + 2);
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, base[static_cast<size_t>(s) * (DH + 2)]);
  for (int d = threadIdx.x; d < DH; d += blockDim.x) {
    float L = 0.f, A = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float* ps = base + static_cast<size_t>(s) * (DH + 2);
      if (ps[0] > -INFINITY) {
        float f = __expf(ps[0] - M);
        L += ps[1] * f;
        A += ps[2 + d] * f;
      }
    }
    out[ldo > 0 ? static_cast<size_t>(tile) * ldo + h * DH + d : packed_index(tile, h * DH + d, H * DH / 32)] =
        from_float<bf16_t>(A / L);
  }
}
}  // namespace decode

// part: 32-bit workspace of n_tiles * H * n_splits * (dh + 2) floats (unused when n_splits == 1);
// waves: 4, 8 or 16 per workgroup (16 up to a head size of 64, 8 up to 128); the splits cover
// n_splits * chunks * waves * 64 keys, which must reach the longest context.
// ldo == 0: out is a packed matrix of H * dh columns (a multiple of 32)
extern "C" int dn_attention_decode(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                                   const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                                   const int32_t* tile_row0, const int32_t* tile_pos0, int n_tiles, float* part,
                                   int n_splits, int chunks, int waves, int H, int Hkv, int dh, int page_size,
                                   float scale, int window, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (Hkv < 1 || H % Hkv != 0 || page_size % 16 != 0 || max_blocks < 1 || n_splits < 1 || chunks < 1 ||
      ldq % 8 != 0 || ldo < 0 || (ldo == 0 && (H * dh) % 32 != 0) || reinterpret_cast<uintptr_t>(q) % 16 != 0 || reinterpret_cast<uintptr_t>(k_pool) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(v_pool) % 16 != 0)
    return DN_ERR_SHAPE;
  if (waves != 4 && !(waves == 8 && dh <= 128) && !(waves == 16 && dh <= 64)) return DN_ERR_SHAPE;
  dim3 grid(n_splits, H, n_tiles), block(waves * 64);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const bool pow2 = (1 << page_shift) == page_size;
#define DN_DECODE_P(L, W, P)                                                                                          \
  hipLaunchKernelGGL((decode::partial_kernel<L, W, P>), grid, block, 0, stream, static_cast<const bf16_t*>(q), ldq,   \
                     static_cast<bf16_t*>(out), ldo, static_cast<const bf16_t*>(k_pool),                              \
                     static_cast<const bf16_t*>(v_pool), block_tables, max_blocks, tile_seq, tile_row0, tile_pos0,    \
                     part, n_splits, chunks, H, Hkv, page_size, page_shift, scale, window)
#define DN_DECODE_W(L, W)    \
  do {                       \
    if (pow2)                \
      DN_DECODE_P(L, W, true);  \
    else                     \
      DN_DECODE_P(L, W, false); \
  } while (0)
#define DN_DECODE(D)                  \
  if (waves == 16) {                  \
    if constexpr (D <= 64) DN_DECODE_W(D, 16); \
  } else if (waves == 8) {            \
    if constexpr (D <= 128) DN_DECODE_W(D, 8);  \
  } else                              \
    DN_DECODE_W(D, 4)
  switch (dh) {
    case 16: DN_DECODE(16); break;
    case 32: DN_DECODE(32); break;
    case 48: DN_DECODE(48); break;
    case 64: DN_DECODE(64); break;
    case 80: DN_DECODE(80); break;
    case 96: DN_DECODE(96); break;
    case 112: DN_DECODE(112); break;
    case 128: DN_DECODE(128); break;
    case 144: DN_DECODE(144); break;
    case 160: DN_DECODE(160); break;
    case 176: DN_DECODE(176); break;
    case 192: DN_DECODE(192); break;
    case 208: DN_DECODE(208); break;
    case 224: DN_DECODE(224); break;
    case 240: DN_DECODE(240); break;
    case 256: DN_DECODE(256); break;
    default: return DN_ERR_SHAPE;
  }
#undef DN_DECODE
#undef DN_DECODE_W
#undef DN_DECODE_P
  if (n_splits > 1)
    hipLaunchKernelGGL(decode::join_kernel, dim3(n_tiles, H), dim3(64), 0, stream, part, static_cast<bf16_t*>(out),
                       ldo, tile_seq, tile_row0, n_splits, H, dh);
  return dn_launch_status();
}

// ---------------------------------------------------------------------------------------
// The split decode kernels with the library's own memory for the split results: for callers that
// cannot allocate (attention.h).  `scratch` below is a host-side stand-in in host code, not a device
// address; the address on each GPU comes from hipGetSymbolAddress, once per GPU, and is what the
// kernels get.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[DN_DECODE_STATIC_SCRATCH_FLOATS];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_lock;
float* scratch_on_device[MAX_DEVICES];   // zero-initialised: not looked up yet

// the address of `scratch` on the current GPU; 0 and *err set if it cannot be had
float* scratch_here(int* err) {
  int dev = -1;
  hipError_t rc = hipGetDevice(&dev);
  if (rc != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *err = rc != hipSuccess ? static_cast<int>(rc) : DN_ERR_SHAPE;
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (scratch_on_device[dev] == nullptr) {
    void* p = nullptr;
    rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess || p == nullptr) {
      *err = rc != hipSuccess ? static_cast<int>(rc) : DN_ERR_SCRATCH;
      return nullptr;
    }
    scratch_on_device[dev] = static_cast<float*>(p);
  }
  return scratch_on_device[dev];
}
}  // namespace

extern "C" int dn_attention_decode_static(const void* q, int ldq, void* out, int ldo, const void* k_pool,
                                          const void* v_pool, const int32_t* block_tables, int max_blocks,
                                          const int32_t* tile_seq, const int32_t* tile_row0,
                                          const int32_t* tile_pos0, int n_tiles, int n_splits, int chunks, int waves,
                                          int H, int Hkv, int dh, int page_size, float scale, int window,
                                          hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (n_splits < 1 || H < 1 || dh < 1) return DN_ERR_SHAPE;
  float* part = nullptr;
  if (n_splits > 1) {
    const long long need = static_cast<long long>(n_tiles) * H * n_splits * (dh + 2);
    if (need > DN_DECODE_STATIC_SCRATCH_FLOATS) return DN_ERR_SCRATCH;
    int err = 0;
    part = scratch_here(&err);
    if (part == nullptr) return err;
  }
  return dn_attention_decode(q, ldq, out, ldo, k_pool, v_pool, block_tables, max_blocks, tile_seq, tile_row0, tile_pos0,
                             n_tiles, part, n_splits, chunks, waves, H, Hkv, dh, page_size, scale, window, stream);
}
