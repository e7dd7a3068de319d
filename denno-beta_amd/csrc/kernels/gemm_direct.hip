#include "gemm_common.h"

// ---------------------------------------------------------------------------------------
// Many rows, bfloat16, slabs carried from memory straight into LDS (global_load_lds_dwordx4: 16
// bytes per lane, lane l's at the wave's LDS address + 16 l, no register and no LDS store between).
// A slab of 32 along K is a list of 1 KB blocks in the packed layout, 16 rows x 32 columns each:
// a block of W is 1 KB of memory as it lies and is read back at 16 l by lane l; a block of A is
// made by the load itself, in an order of its own: the vector cache looks a load's lines up per 16
// lanes, so 16 lanes take 64 bytes from each of four rows (four lines) and not 16 bytes from each of
// sixteen (with a lane per row the lookups, 52 per load on average, kept the cache busy for three
// quarters of the kernel's time), and the four 16-byte pieces of a row are exchanged by the row's
// number so that the operand read (lane l wants row l % 16, piece l / 16) meets every bank once.  STAGES
// stages of KB slabs are in flight (vmcnt counts a wave's own loads; one barrier per stage publishes them and
// frees the stage read before).
//
// The MFMA takes W as its first operand and A as its second: a lane then holds four consecutive
// columns of one row of C, which it stores as 8 bytes (bfloat16) or adds as 16 (the 32-bit
// residual) without a turn through LDS; for the fused QKV product they are one key's or one
// value's four dims.
//
// What bounds these products here is not the matrix cores (busy 30 % of the time with eight waves a workgroup)
// but a wave's chain of loads, waits and barriers, and the rounding of tiles to 256 CUs.  Measured per tile and
// slab with eight waves: time = 2.26e-7 us x BM x BN (matrix cores at nine tenths of their peak) + 3.07e-5 us x
// (BM + BN) (loads), the two adding up rather than overlapping, + 1.9e-4 us x BM x BN for the stores at the end.
// The tile is chosen per product from a list, by that model: the largest that still fills the chip in whole
// rounds (a tile count just above a multiple of 256 costs a whole further round); and the waves of a workgroup
// are as many as give every SIMD four (see `run`), so that one of them can issue while the others wait.
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
bool takes(const void* A, int lda, const void* W, const float* bias, const void* C, int ldc, const float* resid,
                  int ldr, int N, int K, int out_dtype, int packed) {
  auto aligned = [](const void* p, int a) { return reinterpret_cast<uintptr_t>(p) % a == 0; };
  if (K % 32 != 0 || N % 4 != 0 || !aligned(A, 16) || !aligned(W, 16) || !aligned(bias, 16)) return false;
  if (!(packed & PACKED_A) && lda % 8 != 0) return false;
  if (resid) return ldr % 4 == 0 && aligned(resid, 16);
  if (packed & PACKED_C) return N % 32 == 0 && out_dtype == DN_BF16 && aligned(C, 8);
  return ldc % 4 == 0 && aligned(C, out_dtype == DN_F32 ? 16 : 8);
}


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

// (for tiles that never write the cache: the variant with the cache write is not built)
template <int WM, int WN, int TM, int TN, int STAGES, int KB = 1>
static int launch_without_kv(const Args& a, hipStream_t stream) {
  if (a.out_dtype == DN_BF16 && !a.resid) return launch<bf16_t, WM, WN, TM, TN, STAGES, false, KB>(a, stream);
  return launch<float, WM, WN, TM, TN, STAGES, false, KB>(a, stream);
}

// The tiles that `pick` chooses among: rows x columns, and the slabs in flight that its model counts LDS with.
// 128 and 256 rows: one workgroup per CU; the small ones (four waves) leave room for several workgroups per CU and
// are for products with few rows and a long K, whose larger tiles would leave most CUs idle.  (Tiles of 256 x 320
// were on the list while the others ran with eight waves a workgroup; no product chooses them now.)
constexpr Shape SHAPES[] = {{64, 128, 4}, {128, 128, 4}, {256, 128, 4}, {256, 160, 4}, {256, 192, 4},
                            {256, 224, 4}, {256, 256, 4}, {64, 64, 4}, {32, 64, 4}};
constexpr int PICKED = 9;

static double model_us(const Shape& s, int M, int N, int K) {
  const double tiles = static_cast<double>((M + s.bm - 1) / s.bm) * ((N + s.bn - 1) / s.bn);
  const size_t lds = static_cast<size_t>(s.stages) * (s.bm + s.bn) / 16 * 1024;
  // two workgroups that share a CU hide some of each other's waits (measured: 1.5 to 1.8 times one's time for two rounds)
  const double whole = static_cast<double>((static_cast<long>(tiles) + CUS - 1) / CUS);
  const double rounds = 2 * lds <= LDS_PER_CU && whole > 1 ? 0.9 * whole : whole;
  const double area = static_cast<double>(s.bm) * s.bn;
  return rounds * (K * (2.26e-7 * area + 3.07e-5 * (s.bm + s.bn)) + 1.9e-4 * area);
}

int pick(int M, int N, int K, bool kv) {
  int best = 0;
  double best_us = 1e30;
  for (int i = 0; i < PICKED; ++i) {
    double us = model_us(SHAPES[i], M, N, K);
    // (the model is of eight waves a workgroup; the tiles that run with sixteen, see `run`, take about three
    // quarters of its time, which moves the choice at 4,096 rows and more: the fused projection of 8,192 rows
    // 185 -> 165 us)
    if (i >= 1 && i <= 6 && !(kv && i >= 5)) us *= 0.75;
    if (us < best_us) best_us = us, best = i;
  }
  return best;
}

// 65 to 512 rows.  A tile's walk along K costs a wave some dozens of instructions a slab beside its four matrix
// instructions, and with one or two waves a SIMD nothing hides them: tiles of 64 x 64 take two slabs a stage
// which halves that and fills the chip from 65 rows on where the product is wide.  Measured on the
// four products of a layer 1,600 wide (rows and weights that no cache holds; us, before -> now):
//   128 rows: 4,800 columns 18.7 -> 15.7, 6,400 columns 15.3 -> 12.3, 1,600 columns from K = 6,400 19.4 -> 15.2
//   256 rows: 25.6 -> 23.2, 19.3 -> 18.0, 25.6 -> 21.4;  512 rows, 1,600 columns: K = 1,600 12.6 -> 10.7, K = 6,400 38.7 -> 35.4
// -> whether this kernel takes the product with those tiles (else `pick` chooses, or the few-rows kernel runs)
bool mid_rows(int M, int N, int K) {
  if (M <= 64 || M > 512 || K % 64 != 0) return false;
  if (N < 2048) return K >= 4096 || M > 256;      // (few columns and a short K up to 256 rows: the few-rows kernel)
  return M <= 256;
}

// Up to 256 rows the few-rows kernel takes the product too (both read and write packed rows): it stays ahead,
// or level, where the product has few columns and a short K; everywhere else from 65 rows on this kernel is
// the faster (`mid_rows`), and beyond 256 rows it is the only one.
bool beats_few_rows(int M, int N, int K) {
  return mid_rows(M, N, K) || (M > 104 && N >= 4096) || (M > 208 && N >= 2048);
}

// A long K beside few columns and few rows: the tiles are few and each walks all of K, a slab at a time,
// so K is shared out among several workgroups per tile (whole, such a product takes the same time whatever
// its rows up to 256, and a quarter of K less than a third of it).  The number of shares, 0 for none.  With
// fewer than 2,048 columns: 4 up to 128 rows, 2 up to 256, none beyond (1,600 columns, K = 6,400: 15.2, 21.4
// and 35.4 us at 128, 256 and 512 rows; with 8, 4 and 4 shares of smaller tiles 19.4, 25.6, 38.7).  From 2,048 columns: 8
// where the tiles of 32 x 64 are at most 96, else 4.
int shares_of_k(int M, int N, int K, int packed, bool kv) {
  if (kv || (packed & PACKED_C) || M <= 64 || M > 512 || N >= 4096 || K < 4096) return 0;
  if (N < 2048 && K % 64 == 0) return M <= 128 ? 4 : M <= 256 ? 2 : 0;
  return ((M + 31) / 32) * ((N + 63) / 64) <= 96 ? 8 : 4;
}

// A product into the residual stream whose sum a norm's kernel adds (dn_gemm_deferred): the shares of K that it
// is cut into, 0 if it is not worth it.  Few columns and 65 to 256 rows: the tiles are too few to fill the chip,
// and with the shares' sums left for the next kernel to add nothing has to join them here (1,600 x 1,600 at 128
// and 256 rows: 4.8 and 6.2 us where the whole product takes 6.7 and 8.0; K = 6,400: the kernel that adds the
// shares, 4.5 us, falls away).
int deferred_shares(int M, int N, int K) {
  if (M <= 64 || M > 256 || N >= 2048 || K % 64 != 0) return 0;
  if (K >= 4096) return M <= 128 ? 4 : 2;
  return K / 64 >= 8 ? 2 : 0;
}

static bool wide_mid(int M, int N) { return N >= 2048 && M <= 256; }
static long tiles_of(int M, int N, int bm, int bn) { return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn); }
static long mid_tiles_64(int M, int N) { return tiles_of(M, N, 64, 64); }

int run(const Args& a, hipStream_t stream) {
  if (mid_rows(a.M, a.N, a.K) || (a.part && a.N < 2048 && a.K % 64 == 0)) {
    // Wide products: sixteen waves a workgroup, four a SIMD, each with one 16 x 16 block of a 64 x 64 tile (a wave
    // of such a product waits on a counter for more than half of its life, and with one wave a SIMD nothing else
    // runs meanwhile: 16.0 -> 13.9 and 12.8 -> 11.3 us for 4,800 and 6,400 columns at 128 rows); where those tiles
    // are more than the chip has CUs, tiles of 128 x 64 with two blocks a wave (at 256 rows 23.3 -> 20.2 and
    // 18.1 -> 15.2 us).  The narrow ones, whose K is shared out, take neither way faster: four waves as before.
    if (wide_mid(a.M, a.N) && !a.part)
      return mid_tiles_64(a.M, a.N) <= CUS ? launch_as<4, 4, 1, 1, 4, 2>(a, stream) : launch_as<4, 4, 2, 1, 4, 2>(a, stream);
    return launch_as<2, 2, 2, 2, 4, 2>(a, stream);
  }
  // Tiles of 128 and 256 rows: sixteen waves a workgroup, four a SIMD, as 8 x 2 (a wave: 32 rows x a half of the
  // tile's columns) or 4 x 4, where eight waves as 4 x 2 with twice the rows each left the SIMDs waiting (a wave
  // waits on a counter for more than half of its life and the matrix cores were busy 30 % of the time).  At 2,048
  // rows of the XL layer: 56.1 -> 41.0, 25.2 -> 21.3, 57.1 -> 46.6 and 71.8 -> 56.9 us.  Two slabs a stage where K
  // allows it; a long K wants more stages in flight than a short one (with two, the MLP projection of 4,096 rows
  // took 145 us for 125), and LDS decides how many fit.  The cache write's epilogue needs registers that sixteen
  // waves do not leave beside seven column blocks and more a wave: those keep eight waves.
  const bool sixteen = !a.part, two = a.K % 64 == 0, short_k = a.K < 4096;
  switch (pick(a.M, a.N, a.part ? a.K / a.splits : a.K, a.kv != nullptr)) {
    case 0:      // (the small tiles with sixteen waves too, where one round of them covers the product: several
                 // workgroups of four waves share a CU, one of sixteen has it alone)
      if (sixteen && two && tiles_of(a.M, a.N, 64, 128) <= CUS) return launch_as<4, 4, 1, 2, 4, 2>(a, stream);
      return launch_as<2, 2, 2, 4, 4>(a, stream);
    case 1: return sixteen && two ? launch_as<4, 4, 2, 2, 3, 2>(a, stream) : launch_as<4, 2, 2, 4, 4>(a, stream);
    case 2: return sixteen && two ? launch_as<8, 2, 2, 4, 3, 2>(a, stream) : launch_as<4, 2, 4, 4, 4>(a, stream);
    case 3: return sixteen && two ? launch_as<8, 2, 2, 5, 3, 2>(a, stream) : launch_as<4, 2, 4, 5, 4>(a, stream);
    case 4:
      if (!sixteen) return launch_as<4, 2, 4, 6, 4>(a, stream);
      return two && short_k ? launch_as<8, 2, 2, 6, 2, 2>(a, stream) : launch_as<8, 2, 2, 6, 3>(a, stream);
    case 5:
      if (a.kv || !sixteen) return launch_as<4, 2, 4, 7, 4>(a, stream);
      return two && short_k ? launch_without_kv<8, 2, 2, 7, 2, 2>(a, stream) : launch_without_kv<8, 2, 2, 7, 5>(a, stream);
    case 6:
      if (a.kv || !sixteen) return launch_as<4, 2, 4, 8, 4>(a, stream);
      return two && short_k ? launch_without_kv<8, 2, 2, 8, 2, 2>(a, stream) : launch_without_kv<8, 2, 2, 8, 3>(a, stream);
    case 7:
      if (sixteen && two && tiles_of(a.M, a.N, 64, 64) <= CUS) return launch_as<4, 4, 1, 1, 4, 2>(a, stream);
      return launch_as<2, 2, 2, 2, 4>(a, stream);
    default: return launch_as<2, 2, 1, 2, 4>(a, stream);
  }
}

// the tile that a product of these sizes gets: rows * 1000 + columns
int tile_of(int M, int N, int K, bool kv) {
  if (mid_rows(M, N, K)) return wide_mid(M, N) && mid_tiles_64(M, N) > CUS ? 128064 : 64064;
  const Shape& s = SHAPES[pick(M, N, K, kv)];
  return s.bm * 1000 + s.bn;
}
}  // namespace direct
