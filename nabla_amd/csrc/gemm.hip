// GEMM for gfx950: C[b] = alpha * A[b] @ B[b] (+bias) (act) (+residual).
//
// bf16 path (fp32 accumulate): v_mfma_f32_32x32x16_bf16.  A workgroup of four
// waves (2 x 2; 128 x 128 tile) or eight (2 x 4; 256 x 256 tile) owns a BM x BN tile of C;
// K advances in steps of 64 through two LDS buffers.  Both operands sit in LDS as [row][64 k] with 128-byte rows whose
// eight 16-byte chunks are XOR-swizzled by (row % 8) ^ (row / 8 % 8), which makes
// the 16-byte fragment reads of the MFMA (32 consecutive rows, one chunk) and
// both kinds of tile writes below conflict-free without padding.
//   * an operand that is contiguous along K is copied 16 bytes at a time;
//   * an operand that is contiguous along its row index (the transposed operand
//     of the two backward products, and B of the forward product) is read as
//     8 x 8 blocks and transposed in registers before it is written, so the
//     swap_axes of the backward GEMMs never touches memory.
// fp32 path: v_mfma_f32_32x32x2f32 with a 128 x 128 x 16 tile, operands kept
// k-major in LDS.
#include "nbk_common.h"

#include <utility>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// 16-byte register / LDS unit.  A native vector (an SSA value), not the uint4 struct:
// arrays of structs that are filled by loads and drained by stores are turned into
// memcpy through a stack slot, which puts the staging registers in scratch.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Compile-time loop: accumulator tiles must be indexed with constants or they
// leave the register file.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Part i of `total` items dealt as evenly as possible into `parts` consecutive shares.
constexpr int share(int total, int parts, int i) {
  return total * (i + 1) / parts - total * i / parts;
}

struct GemmArgs {
  const void* A; const void* B; void* C; const void* bias; const void* residual;
  int64_t M, N, K;
  int64_t a_rs, a_cs, b_rs, b_cs, ldc;
  int64_t a_bs, b_bs, c_bs;
  int64_t batch_inner, a_bs2, b_bs2, c_bs2;  // batch_inner >= 1
  int32_t dtype_c, act;
  float alpha;
  int32_t tiles_m, tiles_n;
  int32_t a_vec, b_vec;  // 16-byte accesses are legal for this operand
};

__device__ __forceinline__ float gemm_act(float v, int act) {
  if (act == NBK_ACT_RELU) return fmaxf(v, 0.f);
  if (act == NBK_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
  return v;
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Re-number them so that every XCD works on one contiguous run of tiles, then
// walk that run in groups of 8 tile-rows per tile-column: workgroups that share
// an L2 also share the A and B panels they read.
__device__ __forceinline__ void gemm_tile_coords(int bid, int tiles_m, int tiles_n, int& tm,
                                                 int& tn) {
  {
    const int n = tiles_m * tiles_n;
    const int xcd = bid & 7, local = bid >> 3;
    const int per = n >> 3, rem = n & 7;
    bid = xcd < rem ? xcd * (per + 1) + local : rem * (per + 1) + (xcd - rem) * per + local;
  }
  const int group = 8;
  const int per_group = group * tiles_n;
  const int g = bid / per_group;
  const int first_m = g * group;
  const int gsize = min(group, tiles_m - first_m);
  const int r = bid - g * per_group;
  tm = first_m + r % gsize;
  tn = r / gsize;
}

// ---------------------------------------------------------------------------- bf16
__device__ __forceinline__ int swz(int row, int chunk) {
  return row * 8 + (chunk ^ (row & 7) ^ ((row >> 3) & 7));
}

// 16-byte guarded load of 8 consecutive bf16 along the unit-stride axis.
__device__ __forceinline__ u32x4 ld8_bf16(const uint16_t* p, int64_t valid, bool vec) {
  u32x4 r = {0u, 0u, 0u, 0u};
  if (valid >= 8 && vec) return *(const u32x4*)p;
  if (valid <= 0) return r;
  uint16_t t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = i < valid ? p[i] : (uint16_t)0;
  r.x = t[0] | ((uint32_t)t[1] << 16);
  r.y = t[2] | ((uint32_t)t[3] << 16);
  r.z = t[4] | ((uint32_t)t[5] << 16);
  r.w = t[6] | ((uint32_t)t[7] << 16);
  return r;
}

// FAST loaders assume 16-byte-aligned operands, K % 64 == 0 and, for an operand
// that is contiguous along its rows, a row count that is a multiple of 8; then
// every access is one unconditional 16-byte load and the K loop has no branches.
// Rows past the edge are clamped to the last valid row (their products are never
// stored).  Everything else goes through the guarded element-wise path (FAST=false),
// which is kept out of the hot kernels because its code size alone would push
// the main loop out of the instruction cache.
template <int ROWS, bool KC, bool FAST, int NT>
struct TileLoader {
  // NT lanes (256 or 512) share the tile.
  // KC : operand contiguous along K    -> ROWS*8 chunk tasks, ROWS*8/NT per lane.
  // !KC: operand contiguous along rows -> every lane transposes a KPT(k) x 8(rows) block:
  //      one 8x8 block per lane for 256 rows on 256 lanes, half a block (4 k-values) when
  //      there are twice as many lanes as blocks, so that all lanes take part and the K loop
  //      has no divergent branch.
  static constexpr int KPT = 8 * ROWS / NT;
  static constexpr int NREG = KC ? ROWS * 8 / NT : KPT;
  static_assert((ROWS == 256 || ROWS == 128) && (KPT == 8 || KPT == 4), "tile rows / lanes");
  u32x4 reg[NREG];

  __device__ __forceinline__ void load(const uint16_t* base, int64_t rs, int64_t cs, int64_t row0,
                                       int64_t rows_total, int64_t k0, int64_t K, bool vec) {
    const int tid = threadIdx.x;
    if (KC) {
#pragma unroll
      for (int s = 0; s < NREG; ++s) {
        const int t = tid + s * NT;
        const int row = t >> 3, c = t & 7;
        const int64_t gr = row0 + row, gk = k0 + c * 8;
        if (FAST) {
          const int64_t r = gr < rows_total ? gr : rows_total - 1;
          reg[s] = *(const u32x4*)(base + r * rs + gk);
        } else {
          if (gr < rows_total) reg[s] = ld8_bf16(base + gr * rs + gk, K - gk, vec);
          else reg[s] = (u32x4){0u, 0u, 0u, 0u};
        }
      }
    } else {
      constexpr int NC = ROWS / 8;
      const int nc = tid % NC, kq = tid / NC;  // kq: which KPT-row slice of the 64 k
      const int64_t gr = row0 + nc * 8;
#pragma unroll
      for (int r = 0; r < KPT; ++r) {
        const int64_t gk = k0 + kq * KPT + r;
        if (FAST) {
          const int64_t rr = gr < rows_total ? gr : rows_total - 8;
          reg[r] = *(const u32x4*)(base + gk * cs + rr);
        } else {
          if (gk < K) reg[r] = ld8_bf16(base + gk * cs + gr, rows_total - gr, vec);
          else reg[r] = (u32x4){0u, 0u, 0u, 0u};
        }
      }
    }
  }

  // The tile goes to LDS in NPIECE independent pieces so that the K loop can place
  // them between its matrix instructions.
  static constexpr int NPIECE = KC ? NREG : 8;
  template <int P>
  __device__ __forceinline__ void store_piece(u32x4* lds) {
    const int tid = threadIdx.x;
    if (KC) {
      const int t = tid + P * NT;
      lds[swz(t >> 3, t & 7)] = reg[P];
    } else {
      constexpr int NC = ROWS / 8;
      const int nc = tid % NC, kq = tid / NC;
      // row P of the transpose of 16-bit elements: the lane's k-values of column P
      constexpr uint32_t sel = (P & 1) ? 0x07060302u : 0x05040100u;
      if (KPT == 8) {
        u32x4 o;
        o.x = __builtin_amdgcn_perm(reg[1][P >> 1], reg[0][P >> 1], sel);
        o.y = __builtin_amdgcn_perm(reg[3][P >> 1], reg[2][P >> 1], sel);
        o.z = __builtin_amdgcn_perm(reg[5 % NREG][P >> 1], reg[4 % NREG][P >> 1], sel);
        o.w = __builtin_amdgcn_perm(reg[7 % NREG][P >> 1], reg[6 % NREG][P >> 1], sel);
        lds[swz(nc * 8 + P, kq)] = o;
      } else {
        uint2 o;
        o.x = __builtin_amdgcn_perm(reg[1][P >> 1], reg[0][P >> 1], sel);
        o.y = __builtin_amdgcn_perm(reg[3][P >> 1], reg[2][P >> 1], sel);
        uint2* dst = (uint2*)(lds + swz(nc * 8 + P, kq >> 1)) + (kq & 1);
        *dst = o;
      }
    }
  }
  __device__ __forceinline__ void store(u32x4* lds) {
    static_for<NPIECE>([&](auto pc) { store_piece<decltype(pc)::value>(lds); });
  }
};

extern __shared__ __align__(16) u32x4 gemm_lds[];

// NW waves: 4 as 2 x 2, or 8 as 2 x 4 (two waves per SIMD, each with half the accumulators:
// they cover each other's waits at the price of 1.5 x the LDS fragment traffic).
template <int BM, int BN, bool A_KC, bool B_KC, bool FAST, bool EPI, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_kernel(const GemmArgs g) {
  constexpr int NT = NW * 64, WGN = NW / 2;
  constexpr int WM = BM / 2, WN = BN / WGN;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int TILE_CHUNKS = (BM + BN) * 8;
  int tm_i, tn_i;
  gemm_tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tm_i, tn_i);
  const int64_t m0 = (int64_t)tm_i * BM, n0 = (int64_t)tn_i * BN;
  const int64_t bo = (int64_t)blockIdx.y / g.batch_inner, bi = (int64_t)blockIdx.y % g.batch_inner;
  const uint16_t* A = (const uint16_t*)g.A + bo * g.a_bs + bi * g.a_bs2;
  const uint16_t* B = (const uint16_t*)g.B + bo * g.b_bs + bi * g.b_bs2;
  const int64_t c_off = bo * g.c_bs + bi * g.c_bs2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / WGN) * WM, wn = (wave % WGN) * WN;
  const int li = lane & 31, kg = lane >> 5;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (f32x16)(0.f);

  TileLoader<BM, A_KC, FAST, NT> la;
  TileLoader<BN, B_KC, FAST, NT> lb;
  const int64_t nk = (g.K + 63) / 64;
  // A is rows = m; for the loader a K-contiguous operand has (rs = row stride, k unit),
  // a row-contiguous one has (cs = k stride, row unit).
  la.load(A, g.a_rs, g.a_cs, m0, g.M, 0, g.K, g.a_vec);
  lb.load(B, g.b_cs, g.b_rs, n0, g.N, 0, g.K, g.b_vec);
  la.store(gemm_lds);
  lb.store(gemm_lds + BM * 8);
  __syncthreads();

  // Fragment addresses.  swz(row, ks * 2 + kg) = (row * 8 | t) ^ (ks * 2) with
  // t = kg ^ (row % 8) ^ (row / 8 % 8): only a constant XOR moves with ks.
  int a_addr[TM], b_addr[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = wm + i * 32 + li;
    a_addr[i] = row * 8 + (kg ^ (row & 7) ^ ((row >> 3) & 7));
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = wn + j * 32 + li;
    b_addr[j] = BM * 8 + row * 8 + (kg ^ (row & 7) ^ ((row >> 3) & 7));
  }

  // Software pipeline.  A SIMD holds one or two waves of the tile, so little hides a
  // stall but the wave's own instruction stream; every load is therefore issued one
  // stage before its use and sits between matrix instructions:
  //   * fragments of k-step ks + 1 are read from LDS while the MFMAs of ks run
  //     (two fragment sets, frag[0] / frag[1]);
  //   * the tile of iteration kt + 1, fetched from global memory during iteration
  //     kt - 1, is written to the other LDS buffer during k-step 2;
  //   * the global loads of tile kt + 2 are issued behind those writes;
  //   * the workgroup barrier falls in the middle of k-step 3, whose remaining
  //     MFMAs cover the first fragment reads of the next tile.
  bf16x8 fa[2][TM], fb[2][TN];
  constexpr int NFRAG = TM + TN, NMFMA = TM * TN;
  // read fragment r (A tiles first, then B) of k-step ks from `tile` into set SET
  auto read_frag = [&](auto set, auto r, const u32x4* tile, int ks) {
    // order of use by the MFMAs (row-major over the wave's tiles): A0, every B, A1, A2 ...
    constexpr int SET = decltype(set)::value, R0 = decltype(r)::value;
    constexpr int R = R0 == 0 ? 0 : (R0 <= TN ? TM + R0 - 1 : R0 - TN);
    // The XOR is recomputed at every read: hoisted out of the K loop, the 4 x (TM + TN)
    // x 2 variants of these addresses would spill the accumulating kernel.
    int sel = ks * 2;
    asm volatile("" : "+s"(sel));
    if constexpr (R < TM) {
      const u32x4 u = tile[a_addr[R] ^ sel];
      fa[SET][R] = *(const bf16x8*)&u;
    } else {
      const u32x4 u = tile[b_addr[R - TM] ^ sel];
      fb[SET][R - TM] = *(const bf16x8*)&u;
    }
  };
  auto mfma = [&](auto set, auto q) {
    constexpr int SET = decltype(set)::value, Q = decltype(q)::value;
    constexpr int i = Q / TN, j = Q % TN;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[SET][i], fb[SET][j], acc[i][j], 0, 0, 0);
  };
  // k-step on fragment set SET while set 1 - SET is filled for k-step `ks_next` of `tile`
  auto stage = [&](auto set, const u32x4* tile, int ks_next) {
    constexpr int SET = decltype(set)::value;
    static_for<NFRAG>([&](auto r) {
      read_frag(std::integral_constant<int, 1 - SET>{}, r, tile, ks_next);
    });
    static_for<NMFMA>([&](auto q) { mfma(set, q); });
    // interleave: one fragment read, then its share of the MFMAs
    static_for<NFRAG>([&](auto r) {
      constexpr int n = share(NMFMA, NFRAG, decltype(r)::value);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
      if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x008, n, 0);  // MFMAs
    });
    __builtin_amdgcn_sched_barrier(0);  // later stages' work (and its waits) stays behind
  };

  static_for<NFRAG>([&](auto r) { read_frag(std::integral_constant<int, 0>{}, r, gemm_lds, 0); });
  {
    const int64_t k1 = nk > 1 ? 64 : 0;  // a single-tile problem re-reads tile 0 (never stored)
    la.load(A, g.a_rs, g.a_cs, m0, g.M, k1, g.K, g.a_vec);
    lb.load(B, g.b_cs, g.b_rs, n0, g.N, k1, g.K, g.b_vec);
  }
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  for (int64_t kt = 0; kt + 1 < nk; ++kt) {
    const u32x4* cur = gemm_lds + (kt & 1) * TILE_CHUNKS;
    u32x4* nxt = gemm_lds + ((kt + 1) & 1) * TILE_CHUNKS;
    stage(S0{}, cur, 1);
    stage(S1{}, cur, 2);
    // k-step 2, with tile kt + 1 going from registers to LDS
    // (LDS reads and writes keep their program order, so they alternate in the source)
    {
      using LA = TileLoader<BM, A_KC, FAST, NT>;
      using LB = TileLoader<BN, B_KC, FAST, NT>;
      constexpr int NPA = LA::NPIECE, NP = LA::NPIECE + LB::NPIECE;
      constexpr int PER = (NP + NFRAG - 1) / NFRAG;
      static_for<NFRAG>([&](auto r) {
        read_frag(S1{}, r, cur, 3);
        static_for<PER>([&](auto e) {
          constexpr int P = decltype(r)::value * PER + decltype(e)::value;
          if constexpr (P < NPA) la.template store_piece<P>(nxt);
          else if constexpr (P < NP) lb.template store_piece<P - NPA>(nxt + BM * 8);
        });
      });
      static_for<NMFMA>([&](auto q) { mfma(S0{}, q); });
      static_for<NFRAG>([&](auto r) {
        constexpr int n = share(NMFMA, NFRAG, decltype(r)::value);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
        if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x200, PER, 0);  // DS writes
        if constexpr (n > 1) __builtin_amdgcn_sched_group_barrier(0x008, n - 1, 0);  // MFMA
      });
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 3: fetch tile kt + 2 (the last iteration re-fetches tile nk - 1, unused),
    // half of the MFMAs, barrier, first fragments of the next tile, the other half
    {
      const int64_t k2 = (kt + 2 < nk ? kt + 2 : nk - 1) * 64;
      la.load(A, g.a_rs, g.a_cs, m0, g.M, k2, g.K, g.a_vec);
      lb.load(B, g.b_cs, g.b_rs, n0, g.N, k2, g.K, g.b_vec);
    }
    static_for<NMFMA / 2>([&](auto q) { mfma(S1{}, q); });
    {
      constexpr int NL = TileLoader<BM, A_KC, FAST, NT>::NREG + TileLoader<BN, B_KC, FAST, NT>::NREG;
      static_for<NMFMA / 2>([&](auto q) {
        constexpr int n = share(NL, NMFMA / 2, decltype(q)::value);
        if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x020, n, 0);  // VMEM reads
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      });
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    __builtin_amdgcn_sched_barrier(0);
    static_for<NFRAG>([&](auto r) { read_frag(S0{}, r, nxt, 0); });
    static_for<NMFMA / 2>([&](auto q) {
      mfma(S1{}, std::integral_constant<int, decltype(q)::value + NMFMA / 2>{});
    });
    static_for<NFRAG>([&](auto r) {
      constexpr int n = share(NMFMA / 2, NFRAG, decltype(r)::value);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x008, n, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    // last tile: nothing left to stage
    const u32x4* cur = gemm_lds + ((nk - 1) & 1) * TILE_CHUNKS;
    stage(S0{}, cur, 1);
    stage(S1{}, cur, 2);
    stage(S0{}, cur, 3);
    static_for<NMFMA>([&](auto q) { mfma(S1{}, q); });
  }
  __syncthreads();  // the epilogue reuses the tile buffers as per-wave slabs

  // Epilogue.  D[i][j] of a 32x32 MFMA tile lives in lane (j, (i / 4) % 2),
  // register (i / 8) * 4 + i % 4.  Each wave passes its accumulators through a
  // private LDS slab, 32 rows at a time, so that C is written as whole
  // 16-byte (bf16) / 32-byte (fp32) pieces of a row: 8 columns per lane.
  // The plain form (no bias / activation / residual) is a separate
  // instantiation: the fused form carries erf() bodies, and an epilogue that does
  // not fit the instruction cache costs more than the whole K loop of a short GEMM.
  constexpr int SLAB_LD = WN + 4;  // floats per slab row (padding spreads the two row groups)
  float* slab = (float*)gemm_lds + wave * (32 * SLAB_LD);
  const bool out_f32 = g.dtype_c == NBK_F32;
  constexpr int LANES_PER_ROW = WN / 8;        // each lane writes 8 consecutive columns
  constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
  const int sub_r = lane / LANES_PER_ROW, sub_c = (lane % LANES_PER_ROW) * 8;
  const int64_t col = n0 + wn + sub_c;
  const bool vec_store = FAST && (col + 8 <= g.N) && ((g.ldc & 7) == 0) && ((g.c_bs & 7) == 0) &&
                         ((g.c_bs2 & 7) == 0);
  float bias_v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bias_v[e] = 0.f;
  if (EPI && g.bias) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (col + e < g.N) bias_v[e] = nbk_load_as_f32(g.bias, col + e, g.dtype_c);
  }
  static_for<TM>([&](auto ti) {
    constexpr int i = decltype(ti)::value;
    static_for<TN>([&](auto tj) {
      constexpr int j = decltype(tj)::value;
      const f32x16 a = acc[i][j];
#pragma unroll
      for (int r = 0; r < 16; ++r)
        slab[((r >> 2) * 8 + kg * 4 + (r & 3)) * SLAB_LD + j * 32 + li] = a[r];
    });
    // the slab is private to the wave: no workgroup barrier, only LDS ordering
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
#pragma unroll 1
    for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
      const int lr = pass * ROWS_PER_PASS + sub_r;
      const int64_t row = m0 + wm + i * 32 + lr;
      float v[8];
      const float4 p0 = *(const float4*)&slab[lr * SLAB_LD + sub_c];
      const float4 p1 = *(const float4*)&slab[lr * SLAB_LD + sub_c + 4];
      v[0] = p0.x; v[1] = p0.y; v[2] = p0.z; v[3] = p0.w;
      v[4] = p1.x; v[5] = p1.y; v[6] = p1.z; v[7] = p1.w;
      if (row < g.M && col < g.N) {
        const int64_t idx = c_off + row * g.ldc + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= g.alpha;
        if (EPI) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float x = gemm_act(v[e] + bias_v[e], g.act);
            if (g.residual && col + e < g.N) x += nbk_load_as_f32(g.residual, idx + e, g.dtype_c);
            v[e] = x;
          }
        }
        if (vec_store && !out_f32) {
          uint4 o;
          o.x = (uint32_t)nbk_f32_to_bf16(v[0]) | ((uint32_t)nbk_f32_to_bf16(v[1]) << 16);
          o.y = (uint32_t)nbk_f32_to_bf16(v[2]) | ((uint32_t)nbk_f32_to_bf16(v[3]) << 16);
          o.z = (uint32_t)nbk_f32_to_bf16(v[4]) | ((uint32_t)nbk_f32_to_bf16(v[5]) << 16);
          o.w = (uint32_t)nbk_f32_to_bf16(v[6]) | ((uint32_t)nbk_f32_to_bf16(v[7]) << 16);
          *(uint4*)((uint16_t*)g.C + idx) = o;
        } else if (vec_store && out_f32) {
          float4* dst = (float4*)((float*)g.C + idx);
          dst[0] = make_float4(v[0], v[1], v[2], v[3]);
          dst[1] = make_float4(v[4], v[5], v[6], v[7]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < g.N) {
              if (out_f32) ((float*)g.C)[idx + e] = v[e];
              else ((uint16_t*)g.C)[idx + e] = nbk_f32_to_bf16(v[e]);
            }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // slab reads done before the next tile row overwrites it
  });
}

// ---------------------------------------------------------------------------- fp32
// 128 x 128 x 16 tile, LDS k-major ([k][rows], rows padded by 4 floats).
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmArgs g) {
  constexpr int BM = 128, BN = 128, BK = 16, LD = 128 + 4;
  __shared__ float As[2][BK][LD];
  __shared__ float Bs[2][BK][LD];
  int tm_i, tn_i;
  gemm_tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tm_i, tn_i);
  const int64_t m0 = (int64_t)tm_i * BM, n0 = (int64_t)tn_i * BN;
  const int64_t bo = (int64_t)blockIdx.y / g.batch_inner, bi = (int64_t)blockIdx.y % g.batch_inner;
  const float* A = (const float*)g.A + bo * g.a_bs + bi * g.a_bs2;
  const float* B = (const float*)g.B + bo * g.b_bs + bi * g.b_bs2;
  const int64_t c_off = bo * g.c_bs + bi * g.c_bs2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int li = lane & 31, kg = lane >> 5;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (f32x16)(0.f);

  // each lane stages 8 floats of A and 8 of B per k-tile (128*16 / 256)
  float ra[8], rb[8];
  auto load_tile = [&](const float* P, int64_t rs, int64_t cs, int64_t row0, int64_t rows_total,
                       int64_t k0, bool kc, bool vec, float* r) {
    if (kc) {
      // unit stride along k: lane -> (row = tid/2, 8 consecutive k)
      const int row = tid >> 1, kk = (tid & 1) * 8;
      const int64_t gr = row0 + row;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int64_t gk = k0 + kk + e;
        r[e] = (gr < rows_total && gk < g.K) ? P[gr * rs + gk] : 0.f;
      }
    } else {
      // unit stride along rows: lane -> (k = tid/16, 8 consecutive rows)
      const int kk = tid >> 4, rr = (tid & 15) * 8;
      const int64_t gk = k0 + kk;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int64_t gr = row0 + rr + e;
        r[e] = (gr < rows_total && gk < g.K) ? P[gk * cs + gr] : 0.f;
      }
    }
  };
  auto store_tile = [&](float (*S)[LD], bool kc, const float* r) {
    if (kc) {
      const int row = tid >> 1, kk = (tid & 1) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) S[kk + e][row] = r[e];
    } else {
      const int kk = tid >> 4, rr = (tid & 15) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) S[kk][rr + e] = r[e];
    }
  };

  const int64_t nk = (g.K + BK - 1) / BK;
  load_tile(A, g.a_rs, g.a_cs, m0, g.M, 0, A_KC, g.a_vec, ra);
  load_tile(B, g.b_cs, g.b_rs, n0, g.N, 0, B_KC, g.b_vec, rb);
  store_tile(As[0], A_KC, ra);
  store_tile(Bs[0], B_KC, rb);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      load_tile(A, g.a_rs, g.a_cs, m0, g.M, (kt + 1) * BK, A_KC, g.a_vec, ra);
      load_tile(B, g.b_cs, g.b_rs, n0, g.N, (kt + 1) * BK, B_KC, g.b_vec, rb);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      const int k = ks * 2 + kg;
      float fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = As[cur][k][wm + i * 32 + li];
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = Bs[cur][k][wn + j * 32 + li];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      store_tile(As[cur ^ 1], A_KC, ra);
      store_tile(Bs[cur ^ 1], B_KC, rb);
    }
    __syncthreads();
  }
  float* C = (float*)g.C;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = n0 + wn + j * 32 + li;
      if (col >= g.N) continue;
      float bv = g.bias ? ((const float*)g.bias)[col] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm + i * 32 + (r >> 2) * 8 + kg * 4 + (r & 3);
        if (row >= g.M) continue;
        float v = gemm_act(acc[i][j][r] * g.alpha + bv, g.act);
        const int64_t idx = c_off + row * g.ldc + col;
        if (g.residual) v += ((const float*)g.residual)[idx];
        C[idx] = v;
      }
    }
}

// --------------------------------------------------------------- fp32, small problems
// A product with only a handful of 128 x 128 tiles (the layers of a small MLP, a
// classifier head) leaves most of the GPU idle and is bound by the latency of one
// workgroup's K loop.  Here a workgroup owns a 32 x 32 tile of C, its four waves
// split K between them (wave w takes k-steps w, w + 4, ...), operands go from global
// memory straight to the MFMA registers in chunks of 8 k-steps that are all in
// flight together while the previous chunk is multiplied, and the four partial
// tiles meet in LDS.
// Lane l of a v_mfma_f32_32x32x2f32 supplies A[row l % 32][k = l / 32] and
// B[k = l / 32][col l % 32]; which two k values share an instruction is free as
// long as A and B agree, so the lane with half h = l / 32 owns k = kb + 4h .. 4h + 3
// of every 8-wide step and issues four instructions per step.
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(const GemmArgs g) {
  constexpr int U = 8;  // k-steps (of 8) per chunk
  __shared__ float part[4][32][33];
  const int tn_i = blockIdx.x % g.tiles_n, tm_i = blockIdx.x / g.tiles_n;
  const int64_t m0 = (int64_t)tm_i * 32, n0 = (int64_t)tn_i * 32;
  const int64_t bo = (int64_t)blockIdx.y / g.batch_inner, bi = (int64_t)blockIdx.y % g.batch_inner;
  const float* A = (const float*)g.A + bo * g.a_bs + bi * g.a_bs2;
  const float* B = (const float*)g.B + bo * g.b_bs + bi * g.b_bs2;
  const int64_t c_off = bo * g.c_bs + bi * g.c_bs2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 31, h = lane >> 5;
  const int64_t m = m0 + li, n = n0 + li;
  const bool m_ok = m < g.M, n_ok = n < g.N;
  const float* a_base = A_KC ? A + (m_ok ? m : 0) * g.a_rs : A + (m_ok ? m : 0);
  const float* b_base = B_KC ? B + (n_ok ? n : 0) * g.b_cs : B + (n_ok ? n : 0);
  const int64_t K = g.K;
  // k-steps of this wave: s = wave + 4 * i, covering k in [8 s, 8 s + 8)
  const int64_t n_steps = (K + 7) / 8;
  const int64_t my_steps = n_steps > wave ? (n_steps - wave + 3) / 4 : 0;

  auto fetch = [&](int64_t i, float* a, float* b) {
    const int64_t kb = (wave + 4 * i) * 8 + 4 * h;
    const bool in = i < my_steps;
    if (A_KC) {
      if (in && m_ok && g.a_vec && kb + 3 < K) {
        const float4 v = *(const float4*)(a_base + kb);
        a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = (in && m_ok && kb + j < K) ? a_base[kb + j] : 0.f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) a[j] = (in && m_ok && kb + j < K) ? a_base[(kb + j) * g.a_cs] : 0.f;
    }
    if (B_KC) {
      if (in && n_ok && g.b_vec && kb + 3 < K) {
        const float4 v = *(const float4*)(b_base + kb);
        b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = (in && n_ok && kb + j < K) ? b_base[kb + j] : 0.f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = (in && n_ok && kb + j < K) ? b_base[(kb + j) * g.b_rs] : 0.f;
    }
  };

  f32x16 acc = (f32x16)(0.f);
  float ca[U][4], cb[U][4], na[U][4], nb[U][4];
#pragma unroll
  for (int u = 0; u < U; ++u) fetch(u, ca[u], cb[u]);
  for (int64_t c0 = 0; c0 < my_steps; c0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) fetch(c0 + U + u, na[u], nb[u]);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[u][j], cb[u][j], acc, 0, 0, 0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) { ca[u][j] = na[u][j]; cb[u][j] = nb[u][j]; }
  }
  // D register r of lane (col li, half h) is row (r / 4) * 8 + h * 4 + r % 4
#pragma unroll
  for (int r = 0; r < 16; ++r) part[wave][(r >> 2) * 8 + h * 4 + (r & 3)][li] = acc[r];
  __syncthreads();
  float* C = (float*)g.C;
  for (int e = threadIdx.x; e < 32 * 32; e += 256) {
    const int r = e >> 5, c = e & 31;
    const int64_t row = m0 + r, col = n0 + c;
    if (row >= g.M || col >= g.N) continue;
    float v = (part[0][r][c] + part[1][r][c]) + (part[2][r][c] + part[3][r][c]);
    v = gemm_act(v * g.alpha + (g.bias ? ((const float*)g.bias)[col] : 0.f), g.act);
    const int64_t idx = c_off + row * g.ldc + col;
    if (g.residual) v += ((const float*)g.residual)[idx];
    C[idx] = v;
  }
}

// ------------------------------------------------------------------------- dispatch
template <int BM, int BN, bool FAST, int NW = 4>
static int launch_bf16(const GemmArgs& a, bool akc, bool bkc, int64_t batch, hipStream_t st) {
  GemmArgs g = a;
  g.tiles_m = (int)((a.M + BM - 1) / BM);
  g.tiles_n = (int)((a.N + BN - 1) / BN);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
  const size_t pipe = 2 * (size_t)(BM + BN) * 8 * sizeof(uint4);
  const size_t slabs = NW * 32 * (size_t)(BN / (NW / 2) + 4) * sizeof(float);
  const size_t lds = pipe > slabs ? pipe : slabs;
  const bool epi = a.bias != nullptr || a.residual != nullptr || a.act != NBK_ACT_NONE;
#define NBK_LAUNCH_BF16(AK, BK_)                                                              \
  do {                                                                                        \
    if (epi) NBK_LAUNCH_BF16_E(AK, BK_, true);                                                \
    else NBK_LAUNCH_BF16_E(AK, BK_, false);                                                   \
  } while (0)
#define NBK_LAUNCH_BF16_E(AK, BK_, EP)                                                        \
  do {                                                                                        \
    auto kern = gemm_bf16_kernel<BM, BN, AK, BK_, FAST, EP, NW>;                              \
    static bool attr_set = false; /* idempotent, so a race only repeats the call */          \
    if (!attr_set) {                                                                          \
      NBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                  (int)lds));                                                 \
      attr_set = true;                                                                        \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, st, g);                                \
  } while (0)
  if (akc && bkc) NBK_LAUNCH_BF16(true, true);
  else if (akc && !bkc) NBK_LAUNCH_BF16(true, false);
  else if (!akc && bkc) NBK_LAUNCH_BF16(false, true);
  else NBK_LAUNCH_BF16(false, false);
#undef NBK_LAUNCH_BF16
#undef NBK_LAUNCH_BF16_E
  return nbk_check_launch("gemm_bf16_kernel");
}

extern "C" int nbk_gemm(const nbk_gemm_desc* d, void* stream) {
  NBK_REQUIRE(d != nullptr, "gemm: null descriptor");
  NBK_REQUIRE(d->A && d->B && d->C, "gemm: null operand pointer");
  NBK_REQUIRE(d->M > 0 && d->N > 0 && d->K > 0, "gemm: empty problem %lld x %lld x %lld",
              (long long)d->M, (long long)d->N, (long long)d->K);
  NBK_REQUIRE(d->batch >= 1 && d->batch <= 65535, "gemm: batch %lld out of range",
              (long long)d->batch);
  NBK_REQUIRE(d->dtype_ab == NBK_F32 || d->dtype_ab == NBK_BF16, "gemm: operand dtype %d",
              d->dtype_ab);
  NBK_REQUIRE(d->dtype_c == NBK_F32 || d->dtype_c == NBK_BF16, "gemm: result dtype %d",
              d->dtype_c);
  NBK_REQUIRE(d->dtype_ab == NBK_BF16 || d->dtype_c == NBK_F32,
              "gemm: fp32 operands need an fp32 result");
  NBK_REQUIRE(d->a_rs == 1 || d->a_cs == 1, "gemm: A needs a unit stride (rs=%lld, cs=%lld)",
              (long long)d->a_rs, (long long)d->a_cs);
  NBK_REQUIRE(d->b_rs == 1 || d->b_cs == 1, "gemm: B needs a unit stride (rs=%lld, cs=%lld)",
              (long long)d->b_rs, (long long)d->b_cs);
  NBK_REQUIRE(d->ldc >= d->N, "gemm: ldc %lld < N %lld", (long long)d->ldc, (long long)d->N);
  NBK_REQUIRE(d->batch_reduce == 0, "gemm: batch_reduce is folded into K by the caller");
  hipStream_t st = (hipStream_t)stream;
  GemmArgs a;
  a.A = d->A; a.B = d->B; a.C = d->C; a.bias = d->bias; a.residual = d->residual;
  a.M = d->M; a.N = d->N; a.K = d->K;
  a.a_rs = d->a_rs; a.a_cs = d->a_cs; a.b_rs = d->b_rs; a.b_cs = d->b_cs; a.ldc = d->ldc;
  a.a_bs = d->a_bs; a.b_bs = d->b_bs; a.c_bs = d->c_bs;
  a.batch_inner = d->batch_inner > 1 ? d->batch_inner : 1;
  NBK_REQUIRE(d->batch % a.batch_inner == 0, "gemm: batch %lld is not a multiple of batch_inner %lld",
              (long long)d->batch, (long long)a.batch_inner);
  a.a_bs2 = a.batch_inner > 1 ? d->a_bs2 : 0;
  a.b_bs2 = a.batch_inner > 1 ? d->b_bs2 : 0;
  a.c_bs2 = a.batch_inner > 1 ? d->c_bs2 : 0;
  a.dtype_c = d->dtype_c; a.act = d->act; a.alpha = d->alpha;
  // K-contiguous when the stride along k is 1 (ties: a single row / column counts as K-contiguous)
  const bool akc = d->a_cs == 1;
  const bool bkc = d->b_rs == 1;
  const int esz = d->dtype_ab == NBK_F32 ? 4 : 2;
  auto vec_ok = [&](const void* p, int64_t other_stride, int64_t bs, int64_t bs2) {
    const int64_t q = 16 / esz;
    return ((uintptr_t)p % 16 == 0) && (other_stride % q == 0) && (bs % q == 0) && (bs2 % q == 0);
  };
  a.a_vec = vec_ok(d->A, akc ? d->a_rs : d->a_cs, d->a_bs, a.a_bs2);
  a.b_vec = vec_ok(d->B, bkc ? d->b_cs : d->b_rs, d->b_bs, a.b_bs2);
  if (d->dtype_ab == NBK_BF16) {
    const bool fast = a.a_vec && a.b_vec && (d->K % 64 == 0) && (akc || d->M % 8 == 0) &&
                      (bkc || d->N % 8 == 0) && d->M >= 8 && d->N >= 8;
    if (!fast) return launch_bf16<128, 128, false>(a, akc, bkc, d->batch, st);
    // 256 x 256 tiles run at about twice the rate of 128 x 128 ones per CU, one workgroup
    // per CU at a time: take them when the rounds of workgroups they need are at least
    // 60 % full (256 tiles on 256 CUs is the ideal case, 128 or 300 tiles are not).
    const int64_t big_tiles = ((d->M + 255) / 256) * ((d->N + 255) / 256) * d->batch;
    const int64_t cus = nbk_num_cus();
    const int64_t rounds = (big_tiles + cus - 1) / cus;
    // (a K loop of one or two iterations is all prologue and epilogue: there two co-resident
    // 128 x 128 workgroups per CU overlap better than one 256 x 256)
    // (eight waves on the big tile: 8-16 % faster than four on every shape measured)
    if (big_tiles * 10 >= rounds * cus * 6 && d->M >= 256 && d->N >= 256 && d->K > 128)
      return launch_bf16<256, 256, true, 8>(a, akc, bkc, d->batch, st);
    // (a 256 x 128 tile was measured and is no faster than 128 x 128 on mid-sized problems:
    // with one workgroup per CU a short K loop is bound by load latency, and two co-resident
    // 128 x 128 workgroups hide it better)
    return launch_bf16<128, 128, true>(a, akc, bkc, d->batch, st);
  }
  a.tiles_m = (int)((d->M + 127) / 128);
  a.tiles_n = (int)((d->N + 127) / 128);
  if ((int64_t)a.tiles_m * a.tiles_n * d->batch <= 32) {
    // too few big tiles to occupy the GPU: 32 x 32 tiles with K split inside the workgroup
    a.tiles_m = (int)((d->M + 31) / 32);
    a.tiles_n = (int)((d->N + 31) / 32);
    dim3 sgrid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)d->batch);
    if (akc && bkc) hipLaunchKernelGGL((gemm_f32_small_kernel<true, true>), sgrid, dim3(256), 0, st, a);
    else if (akc) hipLaunchKernelGGL((gemm_f32_small_kernel<true, false>), sgrid, dim3(256), 0, st, a);
    else if (bkc) hipLaunchKernelGGL((gemm_f32_small_kernel<false, true>), sgrid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_f32_small_kernel<false, false>), sgrid, dim3(256), 0, st, a);
    return nbk_check_launch("gemm_f32_small_kernel");
  }
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)d->batch);
  if (akc && bkc) hipLaunchKernelGGL((gemm_f32_kernel<true, true>), grid, dim3(256), 0, st, a);
  else if (akc) hipLaunchKernelGGL((gemm_f32_kernel<true, false>), grid, dim3(256), 0, st, a);
  else if (bkc) hipLaunchKernelGGL((gemm_f32_kernel<false, true>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((gemm_f32_kernel<false, false>), grid, dim3(256), 0, st, a);
  return nbk_check_launch("gemm_f32_kernel");
}
