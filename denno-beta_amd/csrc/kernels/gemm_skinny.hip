#include "gemm_common.h"

// ---------------------------------------------------------------------------------------
// Few rows (M <= 256), bfloat16: the decode step's products, bound by reading W once.
// A workgroup owns 16, 32 or 64 output columns; its waves split K in steps of 32 (wave w takes
// steps w, w + WAVES, ...), each feeding v_mfma_f32_16x16x32_bf16 with one packed block of W per
// 16 columns straight from memory (16 bytes per lane) and the matching 16 bytes of up to four
// 16-row blocks of A (lane = row + 16 * (k / 8)).  The waves' sums meet in LDS and are added in
// wave order, so the result has one order of summation whatever M is.  No atomics.
// ---------------------------------------------------------------------------------------

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
void launch_mb_norm(const Call& c, const NormIO& nio, int norm, hipStream_t stream) {
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

void run(const Call& c, hipStream_t stream) {
  if (c.K >= 1024)
    launch_mb<8>(c, stream);
  else
    launch_mb<4>(c, stream);
}

// A must allow 16-byte loads: in rows with K and lda multiples of 8 and the base aligned, or packed
// (K a multiple of 32 then: nothing zeroes a packed block's columns beyond K); W is packed
bool takes(const void* A, int lda, const void* W, int M, int K, int packed) {
  if (M > 256 || reinterpret_cast<uintptr_t>(A) % 16 != 0 || reinterpret_cast<uintptr_t>(W) % 16 != 0) return false;
  return (packed & PACKED_A) ? K % 32 == 0 : (K % 8 == 0 && lda % 8 == 0);
}

// up to 16 rows with a norm inside, by the number of waves a workgroup (8: K >= 1024, else 4)
void launch16_norm_of(int waves, const Call& c, const NormIO& nio, int norm, hipStream_t stream) {
  if (waves == 8)
    launch16_norm<8>(c, nio, norm, stream);
  else
    launch16_norm<4>(c, nio, norm, stream);
}
}  // namespace skinny
