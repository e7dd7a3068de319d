// Sampling from rows of 32-bit logits, after the reference's sampler
// (crates/denno-engine/src/sampler.rs): greedy is the first maximum with NaN ignored
// (:301-331, 350-367); with a temperature, z = logit/T, e_i = exp(z_i - max z), and the
// token is the first i whose running sum of e reaches u * sum(e), walking i upwards
// (:440-463); the last index if rounding leaves none.  The uniform number u comes from the
// request's own generator on the host, so a request's tokens do not depend on the batch.
//
// The penalties before sampling (sampler.rs:42-58, 99-118, 150-172, order :164-179) are one
// kernel over each row's context.  No reduction here uses atomics.
#include "common.h"

#include <math.h>

namespace sampling {
constexpr int THREADS = 1024;
constexpr int WAVES = THREADS / DN_WAVE;

struct Best {
  float v;
  int i;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  // the larger value; of equal values the lower index.  NaN never compares greater.
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ Best block_best(Best x, Best* scratch) {
#pragma unroll
  for (int m = DN_WAVE / 2; m >= 1; m >>= 1) {
    Best o{__shfl_xor(x.v, m, DN_WAVE), __shfl_xor(x.i, m, DN_WAVE)};   // once per row: the slow exchange will do
    x = better(x, o);
  }
  int wave = threadIdx.x / DN_WAVE, lane = threadIdx.x % DN_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = x;
  __syncthreads();
  Best r = scratch[0];
  for (int w = 1; w < WAVES; ++w) r = better(r, scratch[w]);
  return r;
}

__device__ float block_max(float x, float* scratch) {
  x = wave_max(x);
  int wave = threadIdx.x / DN_WAVE, lane = threadIdx.x % DN_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = x;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < WAVES; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

__global__ __launch_bounds__(THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int V,
                                                          const float* __restrict__ temperature,
                                                          const float* __restrict__ uniform,
                                                          int32_t* __restrict__ out) {
  __shared__ Best best_scratch[WAVES];
  __shared__ float f_scratch[WAVES];
  const int r = blockIdx.x, t = threadIdx.x;
  const float* row = logits + static_cast<size_t>(r) * ld;
  const float T = temperature[r];

  if (!(T > 0.f)) {
    // (eight loads asked for at a time: one after the other they were most of the kernel's time)
    Best b{-INFINITY, 0x7fffffff};
    for (int i0 = t; i0 < V; i0 += 8 * THREADS) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = row[min(i0 + j * THREADS, V - 1)];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (i0 + j * THREADS < V && v[j] > b.v) b = Best{v[j], i0 + j * THREADS};
    }
    b = block_best(b, best_scratch);
    if (t == 0) out[r] = b.i == 0x7fffffff ? 0 : b.i;
    return;
  }

  // The walk goes upwards through the vocabulary: the token is the first whose running sum of exp(z - max)
  // reaches uniform x total.  The sums are made block by block (a block: BLK consecutive tokens, BLK a multiple
  // of 64 such that there are at most MAXB blocks), a wave per block, 64 consecutive tokens per load; the first
  // wave then finds the block in which the running sum reaches the target (each lane a run of consecutive
  // blocks, a scan over the lanes, the lane whose run it is walks it), and walks that block 64 tokens at a time
  // (a scan over the lanes again).  Every sum is taken in the order of the tokens.
  constexpr int MAXB = 4096;
  __shared__ float block_sum[MAXB];
  const int wave = t / DN_WAVE, lane = t % DN_WAVE;
  const int per64 = (V + 64 * MAXB - 1) / (64 * MAXB);      // loads of 64 tokens per block
  const int BLK = 64 * per64;
  const int NB = (V + BLK - 1) / BLK;
  const float inv_T = 1.0f / T;
  float mx = -INFINITY;
  for (int i0 = t; i0 < V; i0 += 8 * THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = row[min(i0 + j * THREADS, V - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float z = v[j] * inv_T;
      if (i0 + j * THREADS < V && z > mx) mx = z;
    }
  }
  mx = block_max(mx, f_scratch);
  // (a multiplication by 1 / T and the hardware's exponential: one workgroup has a row's whole vocabulary to get
  // through, and a division and a full-precision exp per token were most of its time)
  auto weight = [&](int i) { return i < V ? __expf(fmaf(row[i], inv_T, -mx)) : 0.f; };
  // an inclusive scan over the wave's lanes, in lane order
  auto scan = [&](float x) {
#pragma unroll
    for (int d = 1; d < DN_WAVE; d <<= 1) {
      const float o = __shfl_up(x, d, DN_WAVE);
      if (lane >= d) x += o;
    }
    return x;
  };
  for (int b0 = wave; b0 < NB; b0 += 4 * WAVES) {
    float e[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int blk = b0 + u * WAVES;
      e[u] = 0.f;
      if (blk < NB)
        for (int k = 0; k < per64; ++k) e[u] += weight(blk * BLK + k * 64 + lane);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int blk = b0 + u * WAVES;
      const float sum = wave_sum(e[u]);      // (one fixed order, whatever the batch)
      if (blk < NB && lane == 0) block_sum[blk] = sum;
    }
  }
  __syncthreads();
  if (wave == 0) {
    const int per = (NB + DN_WAVE - 1) / DN_WAVE;      // consecutive blocks per lane
    float mine = 0.f;
    for (int j = 0; j < per; ++j) {
      const int blk = lane * per + j;
      if (blk < NB) mine += block_sum[blk];
    }
    const float incl = scan(mine);
    const float total = __shfl(incl, DN_WAVE - 1, DN_WAVE);
    const float target = uniform[r] * total;
    const unsigned long long reached = __ballot(incl >= target && lane * per < NB);
    int found = -1;
    float base = 0.f;
    if (reached != 0ull) {
      const int first = __ffsll(static_cast<long long>(reached)) - 1;
      const float before = __shfl_up(incl, 1, DN_WAVE);      // the sum of the lanes before (lane 0: nothing)
      if (lane == first) {
        float run = lane == 0 ? 0.f : before;
        for (int j = 0; j < per; ++j) {
          const int blk = lane * per + j;
          if (blk >= NB) break;
          // (the run's last block, if rounding lets this walk end short of what the scan said)
          found = blk;
          base = run;
          const float next = run + block_sum[blk];
          if (next >= target) break;
          run = next;
        }
      }
    }
    // the wave goes on alone: what lane `first` found comes to the others through the exchange below
    const int src = reached != 0ull ? __ffsll(static_cast<long long>(reached)) - 1 : 0;
    found = __shfl(found, src, DN_WAVE);
    base = __shfl(base, src, DN_WAVE);
    if (found < 0) {
      if (lane == 0) out[r] = V - 1;
      return;
    }
    float run = base;
    int pick = min(V, (found + 1) * BLK) - 1;      // the block's last token, if rounding lets the walk run out
    for (int k = 0; k < per64; ++k) {
      const int i = found * BLK + k * 64 + lane;
      const float x = weight(i);
      const float cum = run + scan(x);
      const unsigned long long hit = __ballot(cum >= target && i < V);
      if (hit != 0ull) {
        pick = found * BLK + k * 64 + __ffsll(static_cast<long long>(hit)) - 1;
        break;
      }
      run = __shfl(cum, DN_WAVE - 1, DN_WAVE);
    }
    if (lane == 0) out[r] = pick;
  }
}

constexpr int HELD = 8192;      // tokens of a context that the penalties keep in the workgroup's memory (32 KB)

// One workgroup per row.  Row r's context (prompt + generated) is ctx[ctx_begin[r] .. + ctx_len[r]): the
// contexts one after the other, or each in its request's row of a table of token histories that lives on the
// device.  Each distinct token is handled by the thread that holds its first occurrence, so no two threads
// write one logit in a phase.
__global__ __launch_bounds__(THREADS) void penalties_kernel(float* __restrict__ logits, int ld, int V,
                                                             const int32_t* __restrict__ ctx,
                                                             const int32_t* __restrict__ ctx_begin,
                                                             const int32_t* __restrict__ ctx_len,
                                                             const float* __restrict__ repetition,
                                                             const float* __restrict__ frequency,
                                                             const float* __restrict__ presence,
                                                             const int32_t* __restrict__ ngram) {
  const int r = blockIdx.x;
  float* row = logits + static_cast<size_t>(r) * ld;
  const int32_t* c = ctx + ctx_begin[r];
  const int n = ctx_len[r];
  const float rep = repetition[r], fq = frequency[r], pr = presence[r];
  const int ng = ngram[r];
  const bool counts = rep != 1.0f || fq != 0.f || pr != 0.f;
  if (!counts && !(ng > 1 && n >= ng)) return;      // (the same for the whole workgroup)
  // Every thread compares its token with the whole context: a context of up to HELD tokens is brought into the
  // workgroup's memory once, where all lanes of a wave read one word at a time; a longer one is read where it is.
  __shared__ int32_t held[HELD];
  auto run = [&](const int32_t* __restrict__ s) {
    if (counts) {
      for (int i = threadIdx.x; i < n; i += THREADS) {
        const int tok = s[i];
        if (tok < 0 || tok >= V) continue;
        bool earlier = false;
#pragma unroll 8
        for (int j = 0; j < i; ++j) earlier |= s[j] == tok;
        if (earlier) continue;
        int count = 0;
#pragma unroll 8
        for (int j = i; j < n; ++j) count += s[j] == tok ? 1 : 0;
        float l = row[tok];
        if (rep != 1.0f) l = l > 0.f ? l / rep : l * rep;
        float sub = 0.f;
        if (fq != 0.f) sub += fq * static_cast<float>(count);
        if (pr != 0.f) sub += pr;
        if (sub != 0.f) l -= sub;
        row[tok] = l;
      }
    }
    __syncthreads();
    if (ng > 1 && n >= ng) {
      const int32_t* prefix = s + n - (ng - 1);
      for (int i = threadIdx.x; i <= n - ng; i += THREADS) {
        bool same = true;
        for (int k = 0; k < ng - 1 && same; ++k) same = s[i + k] == prefix[k];
        if (same) {
          int f = s[i + ng - 1];
          if (f >= 0 && f < V) row[f] = -INFINITY;
        }
      }
    }
  };
  if (n <= HELD) {
    for (int i = threadIdx.x; i < n; i += THREADS) held[i] = c[i];
    __syncthreads();
    run(held);
  } else {
    run(c);
  }
}

// The sampled tokens of the listed rows into their requests' histories: history[begin[j] + len[j]] =
// tokens[rows[j]] (a history's next place), so that the next step's penalties find them without the host.
__global__ void history_append_kernel(int32_t* __restrict__ history, const int32_t* __restrict__ begin,
                                      const int32_t* __restrict__ len, const int32_t* __restrict__ rows,
                                      const int32_t* __restrict__ tokens, int n) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j < n) history[begin[j] + len[j]] = tokens[rows[j]];
}

// ---------------------------------------------------------------------------------------
// top-k / top-p (sampler.rs:372-435, 487-514): the m largest of z = logit/T (ties: the lower
// index first) in descending order, e_i = exp(z_i - z_0); with top-p the list is cut where
// the running sum of e_i / sum(e) reaches p; then the walk with u * sum(kept e) in that order.
// m = min(k, 2048, V); with top-p alone m = min(2048, V), the reference's subset, and as there
// (sampler.rs:387-435) a row whose cut does not fall before the last of the 2048 is not
// decided here: its place in `undecided` is set and sample_full_kernel below takes it.
// ---------------------------------------------------------------------------------------
constexpr int CAND = 2048;

__device__ __forceinline__ uint32_t order_key(float z) {
  if (z != z) return 0u;   // NaN sorts last
  uint32_t u = __float_as_uint(z);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

__global__ __launch_bounds__(THREADS) void sample_top_kernel(const float* __restrict__ logits, int ld, int V,
                                                              const int32_t* __restrict__ rows,
                                                              const float* __restrict__ temperature,
                                                              const float* __restrict__ uniform,
                                                              const int32_t* __restrict__ top_k,
                                                              const float* __restrict__ top_p,
                                                              int32_t* __restrict__ out,
                                                              int32_t* __restrict__ undecided,
                                                              uint32_t* __restrict__ work) {
  __shared__ uint32_t cand_key[CAND];
  __shared__ int32_t cand_idx[CAND];
  __shared__ __attribute__((aligned(16))) float cand_e[CAND];
  __shared__ __attribute__((aligned(16))) float cand_q[CAND];
  __shared__ float total_s;
  // the 256 bins in eight copies, a lane's by its number, 257 apart (so that the copies lie in different
  // banks): in the first pass nearly every key goes to one of two or three bins, and additions to one address
  // wait for each other
  constexpr int COPIES = 8, HSTRIDE = 257;
  __shared__ int hist_copy[COPIES * HSTRIDE];
  __shared__ int hist[256];
  constexpr int EQ_LIST = 2048;
  __shared__ int eq_idx[EQ_LIST];
  __shared__ int cnt_eq[THREADS];
  __shared__ uint32_t sel_prefix;
  __shared__ int sel_remaining, n_gt, n_eq;
  const int t = threadIdx.x;
  const int r = rows[blockIdx.x];
  const float* row = logits + static_cast<size_t>(r) * ld;
  const float T = temperature[r];
  int k = top_k[blockIdx.x];
  const int m = min(min(k > 0 ? k : CAND, CAND), V);

  // 0. every key once (one division per token), into `keys`; a thread writes the keys that it reads in the
  // passes below, eight loads asked for at a time (one workgroup has a row's whole vocabulary to get through on
  // one CU, several times: it counts instructions)
  uint32_t* keys = work + static_cast<size_t>(blockIdx.x) * V;
  for (int i0 = t; i0 < V; i0 += 8 * THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = row[min(i0 + j * THREADS, V - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (i0 + j * THREADS < V) keys[i0 + j * THREADS] = order_key(v[j] / T);
  }
  // 1. the m-th largest key, by four passes over 8 bits each
  if (t == 0) {
    sel_prefix = 0u;
    sel_remaining = m;
    n_gt = 0;
    n_eq = 0;
  }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int i = t; i < COPIES * HSTRIDE; i += THREADS) hist_copy[i] = 0;
    __syncthreads();
    const uint32_t prefix = sel_prefix;
    const uint32_t mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    for (int i0 = t; i0 < V; i0 += 8 * THREADS) {
      uint32_t key[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) key[j] = keys[min(i0 + j * THREADS, V - 1)];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (i0 + j * THREADS < V && (key[j] & mask) == prefix)
          atomicAdd(&hist_copy[(t % COPIES) * HSTRIDE + ((key[j] >> shift) & 0xff)], 1);
    }
    __syncthreads();
    if (t < 256) {
      int n = 0;
#pragma unroll
      for (int c = 0; c < COPIES; ++c) n += hist_copy[c * HSTRIDE + t];
      hist[t] = n;
    }
    __syncthreads();
    if (t < DN_WAVE) {
      // the bin in which the count from the top reaches what remains: lane l holds bins 255 - 4 l .. 252 - 4 l,
      // a scan over the lanes counts from the top, and the first lane that reaches the mark looks among its four
      const int remaining = sel_remaining;
      int own[4], mine = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        own[q] = hist[255 - 4 * t - q];
        mine += own[q];
      }
      int incl = mine;
#pragma unroll
      for (int d = 1; d < DN_WAVE; d <<= 1) {
        const int o = __shfl_up(incl, d, DN_WAVE);
        if (t >= d) incl += o;
      }
      const unsigned long long reached = __ballot(incl >= remaining);
      // (the whole row counts at least `remaining` keys in this pass, so the last lane reaches the mark)
      const int first = reached != 0ull ? __ffsll(static_cast<long long>(reached)) - 1 : DN_WAVE - 1;
      if (t == first) {
        int left = remaining - (incl - mine), b = 255 - 4 * t;
#pragma unroll
        for (int q = 0; q < 3; ++q) {
          if (own[q] >= left) break;
          left -= own[q];
          b -= 1;
        }
        sel_prefix = prefix | (static_cast<uint32_t>(b) << shift);
        sel_remaining = left;
      }
    }
    __syncthreads();
  }
  const uint32_t thr = sel_prefix;
  const int quota = sel_remaining;       // how many keys equal to thr belong to the m
  const int greater = m - quota;         // and how many keys are greater
  // 2. the candidates: every key above thr, in any place (the sort below puts them in order), and of the keys
  // equal to thr the `quota` with the lowest indices: these are listed first and ranked among themselves
  for (int i = t; i < CAND; i += THREADS) {
    cand_key[i] = 0u;
    cand_idx[i] = 0x7fffffff;
  }
  __syncthreads();
  for (int i0 = t; i0 < V; i0 += 8 * THREADS) {
    uint32_t key[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) key[j] = keys[min(i0 + j * THREADS, V - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j * THREADS;
      if (i >= V) continue;
      if (key[j] > thr) {
        const int at = atomicAdd(&n_gt, 1);
        cand_key[at] = key[j];
        cand_idx[at] = i;
      } else if (key[j] == thr) {
        const int at = atomicAdd(&n_eq, 1);
        if (at < EQ_LIST) eq_idx[at] = i;
      }
    }
  }
  __syncthreads();
  const int equals = n_eq;
  if (equals <= EQ_LIST) {
    for (int j = t; j < equals; j += THREADS) {
      const int mine = eq_idx[j];
      int rank = 0;
      for (int o = 0; o < equals; ++o) rank += eq_idx[o] < mine;
      if (rank < quota) {
        cand_key[greater + rank] = thr;
        cand_idx[greater + rank] = mine;
      }
    }
  } else {
    // more equal keys than the list holds (a row of nearly equal logits): in the order of their indices, a
    // thread a stretch of the row, one thread the stretches' counts
    __syncthreads();      // (every thread's keys are in memory)
    const int seg = (V + THREADS - 1) / THREADS;
    const int lo = min(V, t * seg), hi = min(V, lo + seg);
    int mine = 0;
    for (int i = lo; i < hi; ++i) mine += keys[i] == thr;
    cnt_eq[t] = mine;
    __syncthreads();
    if (t == 0) {
      int before = 0;
      for (int i = 0; i < THREADS; ++i) {
        const int e = cnt_eq[i];
        cnt_eq[i] = before;
        before += e;
      }
    }
    __syncthreads();
    int rank = cnt_eq[t];
    for (int i = lo; i < hi && rank < quota; ++i) {
      if (keys[i] == thr) {
        cand_key[greater + rank] = thr;
        cand_idx[greater + rank] = i;
        rank += 1;
      }
    }
  }
  __syncthreads();
  // 3. bitonic sort: key descending, equal keys by ascending index; of the first n_sort places (the others
  // hold nothing)
  int n_sort = 2;
  while (n_sort < m) n_sort <<= 1;
  for (int size = 2; size <= n_sort; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = t; i < n_sort / 2; i += THREADS) {
        int a = 2 * i - (i & (stride - 1));
        int b = a + stride;
        bool descending = (a & size) == 0;
        uint32_t ka = cand_key[a], kb = cand_key[b];
        int ia = cand_idx[a], ib = cand_idx[b];
        bool a_first = ka > kb || (ka == kb && ia < ib);
        if (a_first != descending) {
          cand_key[a] = kb;
          cand_key[b] = ka;
          cand_idx[a] = ib;
          cand_idx[b] = ia;
        }
      }
      __syncthreads();
    }
  }
  // 4. softmax numerators, cut, walk: every sum in the list's order, one addition after the other as the
  // reference makes them, by one thread.  It reads sixteen numbers at a time (four 16-byte reads, asked for
  // together) and looks only after every sixteen additions whether the running sum has reached its mark (it
  // never goes back: the numbers are not negative), then finds the place among those sixteen: a thread that
  // fetched each number by itself and tested after each spent a hundred cycles per number, two thousand times
  // a sum.
  const float z0 = key_value(cand_key[0]);
  for (int i = t; i < m; i += THREADS) cand_e[i] = expf(key_value(cand_key[i]) - z0);
  __syncthreads();
  const float p = top_p[blockIdx.x];
  // x[i0 .. i0 + 15], those from n on as zeros (adding 0 changes nothing)
  auto sixteen = [](const float* x, int i0, int n, float* v) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 f = *reinterpret_cast<const float4*>(x + i0 + 4 * q);
      v[4 * q] = f.x, v[4 * q + 1] = f.y, v[4 * q + 2] = f.z, v[4 * q + 3] = f.w;
    }
    if (i0 + 16 > n) {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (i0 + j >= n) v[j] = 0.f;
    }
  };
  auto sum_of = [&](int n) {
    float total = 0.f;
    for (int i0 = 0; i0 < n; i0 += 16) {
      float v[16];
      sixteen(cand_e, i0, n, v);
#pragma unroll
      for (int j = 0; j < 16; ++j) total += v[j];
    }
    return total;
  };
  if (p < 1.0f) {
    if (t == 0) total_s = sum_of(m);
    __syncthreads();
    const float total = total_s;
    for (int i = t; i < m; i += THREADS) cand_q[i] = cand_e[i] / total;      // (each share by the same division)
    __syncthreads();
  }
  if (t == 0) {
    int keep = m;
    if (p < 1.0f) {
      float cum = 0.f;
      for (int i0 = 0; i0 < m; i0 += 16) {
        float v[16];
        sixteen(cand_q, i0, m, v);
        const float before = cum;
#pragma unroll
        for (int j = 0; j < 16; ++j) cum += v[j];
        if (cum >= p) {
          float again = before;
          for (int j = 0; j < 16; ++j) {
            again += v[j];
            if (again >= p) {
              keep = i0 + j + 1;
              break;
            }
          }
          break;
        }
      }
    }
    // top-p alone over a vocabulary larger than the subset: a cut that is not reached before the
    // subset's last member needs the tail (sampler.rs:425-433)
    undecided[blockIdx.x] = (k <= 0 && V > CAND && keep == m) ? 1 : 0;
    float u = uniform[r] * sum_of(keep);
    int place = keep - 1;
    for (int i0 = 0; i0 < keep; i0 += 16) {
      float v[16];
      sixteen(cand_e, i0, keep, v);
      const float before = u;
#pragma unroll
      for (int j = 0; j < 16; ++j) u -= v[j];
      if (u <= 0.f) {
        float again = before;
        for (int j = 0; j < 16; ++j) {
          again -= v[j];
          if (again <= 0.f) {
            place = min(i0 + j, keep - 1);
            break;
          }
        }
        break;
      }
    }
    out[r] = cand_idx[place];
  }
}

// ---------------------------------------------------------------------------------------
// top-p over the whole vocabulary (sampler.rs:466-476, 487-514): every z = logit/T in descending
// order (ties: the lower index first), e_i = exp(z_i - z_0), the list cut where the running sum of
// e_i / sum(e) reaches p, then the walk with u * sum(kept e).  One workgroup per listed row sorts
// the row in `work` (per row: n_pad keys, n_pad indices, n_pad numerators; n_pad the power of
// two from V up).  Sums run in the list's order by segments: a thread adds its own stretch, one
// thread adds the stretches' sums, so the result does not depend on timing.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(THREADS) void sample_full_kernel(const float* __restrict__ logits, int ld, int V,
                                                               int n_pad, const int32_t* __restrict__ rows,
                                                               const float* __restrict__ temperature,
                                                               const float* __restrict__ uniform,
                                                               const float* __restrict__ top_p,
                                                               const int32_t* __restrict__ only,
                                                               uint32_t* __restrict__ work,
                                                               int32_t* __restrict__ out) {
  __shared__ float seg_sum[THREADS];
  __shared__ float seg_base[THREADS];
  __shared__ float total_s;
  __shared__ int first_s;
  // only: a flag per listed row (none: all are meant); a row whose flag is 0 is left as it is, so that the
  // caller can launch this behind sample_top_kernel without reading what that left undecided
  if (only != nullptr && only[blockIdx.x] == 0) return;
  const int t = threadIdx.x;
  const int r = rows[blockIdx.x];
  const float* row = logits + static_cast<size_t>(r) * ld;
  const float T = temperature[r];
  uint32_t* key = work + static_cast<size_t>(blockIdx.x) * 3 * n_pad;
  int32_t* idx = reinterpret_cast<int32_t*>(key + n_pad);
  float* e = reinterpret_cast<float*>(key + 2 * static_cast<size_t>(n_pad));
  for (int i = t; i < n_pad; i += THREADS) {
    key[i] = i < V ? order_key(row[i] / T) : 0u;
    idx[i] = i < V ? i : 0x7fffffff;
  }
  __syncthreads();
  for (int size = 2; size <= n_pad; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = t; i < n_pad / 2; i += THREADS) {
        int a = 2 * i - (i & (stride - 1));
        int b = a + stride;
        bool descending = (a & size) == 0;
        uint32_t ka = key[a], kb = key[b];
        int ia = idx[a], ib = idx[b];
        bool a_first = ka > kb || (ka == kb && ia < ib);
        if (a_first != descending) {
          key[a] = kb;
          key[b] = ka;
          idx[a] = ib;
          idx[b] = ia;
        }
      }
      __syncthreads();
    }
  }
  // a value that is NaN has key 0 like the padding but a real index, which sorts before the padding's:
  // the first V places hold the row
  const float z0 = key_value(key[0]);
  const int seg = (V + THREADS - 1) / THREADS;
  const int lo = min(V, t * seg), hi = min(V, lo + seg);
  float s = 0.f;
  for (int i = lo; i < hi; ++i) {
    float v = key[i] != 0u ? expf(key_value(key[i]) - z0) : 0.f;     // key 0: NaN, which nothing can pick
    e[i] = v;
    s += v;
  }
  seg_sum[t] = s;
  if (t == 0) first_s = V;
  __syncthreads();
  if (t == 0) {
    float run = 0.f;
    for (int k = 0; k < THREADS; ++k) {
      seg_base[k] = run;
      run += seg_sum[k];
    }
    total_s = run;
  }
  __syncthreads();
  const float p = top_p[blockIdx.x];
  int keep = V;
  if (p < 1.0f) {
    const float total = total_s;
    float cum = seg_base[t] / total;
    // (the reference adds e_i / total term by term; here a stretch starts from its base / total)
    for (int i = lo; i < hi; ++i) {
      cum += e[i] / total;
      if (cum >= p) {
        atomicMin(&first_s, i);
        break;
      }
    }
    __syncthreads();
    keep = min(V, first_s + 1);
    __syncthreads();
  }
  // the kept list's sum, then the walk
  s = 0.f;
  for (int i = lo; i < min(hi, keep); ++i) s += e[i];
  seg_sum[t] = s;
  if (t == 0) first_s = keep;
  __syncthreads();
  if (t == 0) {
    float run = 0.f;
    for (int k = 0; k < THREADS; ++k) {
      seg_base[k] = run;
      run += seg_sum[k];
    }
    total_s = run;
  }
  __syncthreads();
  {
    float u = uniform[r] * total_s - seg_base[t];
    for (int i = lo; i < min(hi, keep); ++i) {
      u -= e[i];
      if (u <= 0.f) {
        atomicMin(&first_s, i);
        break;
      }
    }
  }
  __syncthreads();
  if (t == 0) out[r] = idx[min(first_s, keep - 1)];
}
}  // namespace sampling

extern "C" int dn_sample(const float* logits, int ld, int R, int V, const float* temperature, const float* uniform,
                         int32_t* out, hipStream_t stream) {
  if (R <= 0) return 0;
  if (V < 1 || ld < V) return DN_ERR_SHAPE;
  hipLaunchKernelGGL(sampling::sample_kernel, dim3(R), dim3(sampling::THREADS), 0, stream, logits, ld, V,
                     temperature, uniform, out);
  return dn_launch_status();
}

extern "C" int dn_penalties(float* logits, int ld, int R, int V, const int32_t* ctx, const int32_t* ctx_begin,
                            const int32_t* ctx_len, const float* repetition, const float* frequency,
                            const float* presence, const int32_t* ngram, hipStream_t stream) {
  if (R <= 0) return 0;
  if (V < 1 || ld < V) return DN_ERR_SHAPE;
  hipLaunchKernelGGL(sampling::penalties_kernel, dim3(R), dim3(sampling::THREADS), 0, stream, logits, ld, V, ctx,
                     ctx_begin, ctx_len, repetition, frequency, presence, ngram);
  return dn_launch_status();
}

// (the host has checked that every begin[j] + len[j] lies inside the history and every rows[j] inside tokens)
extern "C" int dn_history_append(int32_t* history, const int32_t* begin, const int32_t* len, const int32_t* rows,
                                 const int32_t* tokens, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(sampling::history_append_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, history, begin,
                     len, rows, tokens, n);
  return dn_launch_status();
}

extern "C" int dn_sample_top(const float* logits, int ld, int n_rows, int V, const int32_t* rows,
                             const float* temperature, const float* uniform, const int32_t* top_k,
                             const float* top_p, int32_t* out, int32_t* undecided, void* work,
                             hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V < 1 || ld < V || work == nullptr) return DN_ERR_SHAPE;      // work: V 32-bit words per listed row
  hipLaunchKernelGGL(sampling::sample_top_kernel, dim3(n_rows), dim3(sampling::THREADS), 0, stream, logits, ld, V,
                     rows, temperature, uniform, top_k, top_p, out, undecided, static_cast<uint32_t*>(work));
  return dn_launch_status();
}

// work: 3 * n_pad 32-bit words per listed row, n_pad the power of two from V up
extern "C" int dn_sample_full(const float* logits, int ld, int n_rows, int V, int n_pad, const int32_t* rows,
                              const float* temperature, const float* uniform, const float* top_p,
                              const int32_t* only, void* work, int32_t* out, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V < 1 || ld < V || n_pad < V || n_pad < 2 || (n_pad & (n_pad - 1)) != 0) return DN_ERR_SHAPE;
  hipLaunchKernelGGL(sampling::sample_full_kernel, dim3(n_rows), dim3(sampling::THREADS), 0, stream, logits, ld, V,
                     n_pad, rows, temperature, uniform, top_p, only, static_cast<uint32_t*>(work), out);
  return dn_launch_status();
}
