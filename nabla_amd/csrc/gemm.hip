// GEMM for gfx950: C[b] = alpha * A[b] @ B[b] (+bias) (act) (+residual).
//
// bf16 path (fp32 accumulate): v_mfma_f32_32x32x16_bf16.  A workgroup of four waves (2 x 2;
// 128 x 128 tile) or eight (2 x 4; 256 x 256 tile) owns a BM x BN tile of C; K advances in
// steps of 64 through two LDS buffers.
//   * an operand that is contiguous along K sits in LDS as [row][64 k], 128-byte rows whose
//     eight 16-byte chunks are XOR-swizzled, so that the 16-byte fragment reads of the MFMA
//     (32 consecutive rows, one chunk) are conflict-free without padding;
//   * an operand that is contiguous along its row index (the transposed operand of the two
//     backward products, and B of the forward product) sits in LDS k-major, [64 k][rows], and
//     its MFMA fragments come out through the transposing read (ds_read_b64_tr_b16): the
//     swap_axes of the backward GEMMs never touches memory or the vector ALU.
// Two kernels share this layout idea: gemm_bf16_dl_kernel (aligned operands, K % 64 == 0) copies
// global memory straight into LDS (global_load_lds_dwordx4); gemm_bf16_kernel takes every other
// shape through guarded element-wise loads and registers.
// fp32 path: v_mfma_f32_32x32x2f32 with a 128 x 128 x 16 tile, operands kept
// k-major in LDS.
#include "nbk_common.h"

#include <utility>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
  int32_t res_mul;  // the residual multiplies instead of adding
  float alpha;
  int32_t tiles_m, tiles_n;
  int32_t a_vec, b_vec;  // 16-byte accesses are legal for this operand
  void* C2;              // second result (derivative of the activation), or null
  const float* b_scales; // NF4-coded B only: one scale per `b_block` consecutive codes
  int32_t b_block;
  int32_t c_stream;      // C is larger than the last-level cache: store it with the non-temporal hint
  void* colsum;          // null, or [batch][N] in C's dtype: the column sums of B over K
  // More operand pairs whose products join the accumulator: C = A B + sum_i A_i B_i, all
  // oriented like A and B.  Direct-to-LDS kernels only.
  //   shallow pairs (n_shallow <= 2; K <= 64 each, own strides): one K tile each, the first tiles
  //   of the launch;
  //   deep pairs (n_deep <= 2; K % 64 == 0, the strides of A and B): their K tiles follow those
  //   of A and B.
  struct Shallow { const void* A; const void* B; int64_t K, a_rs, a_cs, b_rs, b_cs; } shallow[2];
  struct Deep { const void* A; const void* B; int64_t K; } deep[2];
  int32_t n_shallow, n_deep;
};

__device__ __forceinline__ float gemm_act(float v, int act) {
  if (act == NBK_ACT_RELU) return fmaxf(v, 0.f);
  if (act == NBK_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
  return v;
}

// Activation and its derivative at the same point (the second result of a launch).  LOWP: the
// results are stored as 16-bit floats, so hardware exp and a 1.5e-7 erf do.
template <bool LOWP>
__device__ __forceinline__ void gemm_act_pair(float x, int act, float& y, float& dy) {
  if (act == NBK_ACT_RELU) {
    y = fmaxf(x, 0.f);
    dy = x > 0.f ? 1.f : 0.f;
  } else if (act == NBK_ACT_GELU) {
    const float z = x * 0.70710678118654752440f;
    const float e = LOWP ? __expf(-z * z) : expf(-z * z);
    const float cdf = 0.5f * (1.f + (LOWP ? nbk_fast_erf_with(z, e) : erff(z)));
    y = x * cdf;
    dy = cdf + x * 0.39894228040143267794f * e;
  } else {
    y = x;
    dy = 1.f;
  }
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

// ---- NF4-coded B operand --------------------------------------------------------------------
// The sixteen levels (nabla/nn/finetune/qlora.py:18-38), copied to LDS by the kernels that
// dequantise: a lane looks up eight different entries per load.
__device__ const float nbk_nf4_levels[16] = {-1.0f,    -0.6962f, -0.5251f, -0.3949f, -0.2844f, -0.1848f,
                                             -0.0911f, 0.0f,     0.0796f,  0.1609f,  0.2461f,  0.3379f,
                                             0.4407f,  0.5626f,  0.7230f,  1.0f};
// Eight consecutive weights from their codes: level[code] * scale of the block the codes lie
// in (`flat` is the index of the first code in the flattened weight, a multiple of 8, and the
// block length is a multiple of 8, so the eight share a block); entries from `valid` on are 0.
__device__ __forceinline__ void nf4_load8(const uint8_t* codes, const float* scales, int block,
                                          const float* table, int64_t flat, int64_t valid, float* out) {
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = 0.f;
  if (valid <= 0) return;
  const float s = scales[flat / block];
  uint64_t raw = 0;
  if (valid >= 8) {
    raw = *(const uint64_t*)(codes + flat);
  } else {
    for (int e = 0; e < valid; ++e) raw |= (uint64_t)codes[flat + e] << (8 * e);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (e < valid) out[e] = table[(raw >> (8 * e)) & 15] * s;
}

// ------------------------------------------------------- bf16, guarded register-staged loads
// The general form: any alignment, any K, ragged edges.  Every access is guarded element by
// element; it is kept out of the hot kernel because its code size alone would push the main
// loop out of the instruction cache.
// LDS geometry of one operand tile, in 16-byte chunks.  K-contiguous: [row][8 chunks],
// swizzled.  Row-contiguous: [64 k][ROWS / 8 + 4 chunks]; the pitch is 64 bytes past a
// multiple of 256, so the eight 32-byte row segments that half a wave touches in one
// transposing read (4 k-rows x 2 groups of 16 rows) fall on eight different bank groups.
template <int ROWS, bool KC>
struct TileGeom {
  static constexpr int PITCH = ROWS / 8 + 4;
  static constexpr int CHUNKS = KC ? ROWS * 8 : 64 * PITCH;
};

template <int ROWS, bool KC, int NT>
struct TileLoader {
  // NT lanes (256 or 512) share the tile: ROWS * 8 chunk tasks, ROWS * 8 / NT per lane.
  // KC : operand contiguous along K    -> task t is chunk t % 8 of row t / 8.
  // !KC: operand contiguous along rows -> task t is rows 8 * (t % (ROWS / 8)) .. + 8 of
  //      k-row t / (ROWS / 8): consecutive lanes read consecutive 16 bytes of one k-row.
  static constexpr int NREG = ROWS * 8 / NT;
  static constexpr int NC = ROWS / 8;
  static constexpr int PITCH = TileGeom<ROWS, KC>::PITCH;
  static_assert(ROWS == 256 || ROWS == 128, "tile rows");
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
        if (gr < rows_total) reg[s] = ld8_bf16(base + gr * rs + gk, K - gk, vec);
        else reg[s] = (u32x4){0u, 0u, 0u, 0u};
      }
    } else {
#pragma unroll
      for (int s = 0; s < NREG; ++s) {
        const int t = tid + s * NT;
        const int k = t / NC, c = t % NC;
        const int64_t gr = row0 + c * 8, gk = k0 + k;
        if (gk < K) reg[s] = ld8_bf16(base + gk * cs + gr, rows_total - gr, vec);
        else reg[s] = (u32x4){0u, 0u, 0u, 0u};
      }
    }
  }

  // The same tile from NF4 codes: `codes` addressed like `base` above, dequantised in registers
  // and rounded to bf16 once.
  __device__ __forceinline__ void load_nf4(const uint8_t* codes, const float* scales, int block,
                                           const float* table, int64_t rs, int64_t cs, int64_t row0,
                                           int64_t rows_total, int64_t k0, int64_t K) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int s = 0; s < NREG; ++s) {
      const int t = tid + s * NT;
      float w[8];
      if (KC) {
        const int row = t >> 3, c = t & 7;
        const int64_t gr = row0 + row, gk = k0 + c * 8;
        nf4_load8(codes, scales, block, table, gr * rs + gk, gr < rows_total ? K - gk : 0, w);
      } else {
        const int k = t / NC, c = t % NC;
        const int64_t gr = row0 + c * 8, gk = k0 + k;
        nf4_load8(codes, scales, block, table, gk * cs + gr, gk < K ? rows_total - gr : 0, w);
      }
      u32x4 r;
      r.x = (uint32_t)nbk_f32_to_bf16(w[0]) | ((uint32_t)nbk_f32_to_bf16(w[1]) << 16);
      r.y = (uint32_t)nbk_f32_to_bf16(w[2]) | ((uint32_t)nbk_f32_to_bf16(w[3]) << 16);
      r.z = (uint32_t)nbk_f32_to_bf16(w[4]) | ((uint32_t)nbk_f32_to_bf16(w[5]) << 16);
      r.w = (uint32_t)nbk_f32_to_bf16(w[6]) | ((uint32_t)nbk_f32_to_bf16(w[7]) << 16);
      reg[s] = r;
    }
  }

  // The tile goes to LDS in NPIECE independent pieces so that the K loop can place
  // them between its matrix instructions.
  static constexpr int NPIECE = NREG;
  template <int P>
  __device__ __forceinline__ void store_piece(u32x4* lds) {
    const int t = threadIdx.x + P * NT;
    if (KC) lds[swz(t >> 3, t & 7)] = reg[P];
    else lds[(t / NC) * PITCH + t % NC] = reg[P];
  }
  __device__ __forceinline__ void store(u32x4* lds) {
    static_for<NPIECE>([&](auto pc) { store_piece<decltype(pc)::value>(lds); });
  }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// Transposing LDS read: the 16 lanes of a group hand in 16 addresses of 4 consecutive
// 16-bit values, In[p][e]; lane i of the group receives In[4 j + i / 4][i % 4], j = 0..3.
// With lane p pointing at (k-row p / 4, rows 4 * (p % 4) .. + 4) of a k-major tile, lane i
// ends up with 4 consecutive k of row i: half an MFMA operand fragment.
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
}

// The same read as inline assembly, for kernels that fill LDS with global_load_lds: the
// compiler puts a wait for every such copy in flight in front of the intrinsic form (it cannot
// tell that the two never touch the same buffer between two barriers).  It knows nothing about
// the result being asynchronous either: lds_wait_for() has to stand between these reads and
// the first use of their results.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ bf16x8 lds_read_tr_pair(uint32_t addr, int off_lo, int off_hi) {
  s16x4 lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "n"(off_lo) : "memory");
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(off_hi) : "memory");
  const s16x8 u = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return *(const bf16x8*)&u;
}
__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t addr) {
  u32x4 u;
  asm volatile("ds_read_b128 %0, %1" : "=v"(u) : "v"(addr) : "memory");
  return *(const bf16x8*)&u;
}
template <int N>
__device__ __forceinline__ void lds_wait_for(bf16x8 (&f)[N]) {
  static_assert(N == 2 || N == 4 || N == 8, "fragments per set");
  if constexpr (N == 2)
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1])::"memory");
  else if constexpr (N == 4)
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3])::"memory");
  else
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]),
                   "+v"(f[7])::"memory");
}

extern __shared__ __align__(16) u32x4 gemm_lds[];

// Epilogue shared by the bf16 kernels (the caller has passed a workgroup barrier: the tile
// buffers are free).
// EPI: 0 plain, 1 bias only (as lean as the plain form), 2 bias / activation / residual (the
// residual requested for the whole wave tile up front), 3 bias and an added residual read pass by
// pass (for kernels whose occupancy hides that latency and must not lose it to registers), 4 bias
// and an added bf16 residual that the caller requested before its product (`pre`: the 16-byte
// piece of every pass of every band, in this function's lane layout -- gemm_residual_prefetch).
// Each wave passes its accumulators through a private LDS slab, a band of 32 rows of its tile
// at a time (`scatter(band, slab)` writes the band's accumulators there, row-major with a
// pitch of WN + 4 floats), so that C is written as whole 16-byte (bf16) / 32-byte (fp32)
// pieces of a row: 8 columns per lane.  The plain form (no bias / activation / residual)
// is a separate instantiation: the fused form carries erf() bodies, and an epilogue that does
// not fit the instruction cache costs more than the whole K loop of a short GEMM.
// The residual pieces this lane adds in an EPI 4 epilogue, requested up front (rows and columns
// past the edge read a valid address and are never used).  The caller has checked that C is
// bf16 and that residual, ldc and N allow 16-byte pieces.
template <int TM, int WN>
__device__ __forceinline__ void gemm_residual_prefetch(const GemmArgs& g, int64_t m0, int64_t n0, int wm,
                                                       int wn, int lane, uint4 (&pre)[TM * (WN / 16)]) {
  constexpr int LANES_PER_ROW = WN / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW, NP = 32 / ROWS_PER_PASS;
  const int sub_r = lane / LANES_PER_ROW, sub_c = (lane % LANES_PER_ROW) * 8;
  int64_t col = n0 + wn + sub_c;
  col = col + 8 <= g.N ? col : 0;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int pass = 0; pass < NP; ++pass) {
      int64_t row = m0 + wm + i * 32 + pass * ROWS_PER_PASS + sub_r;
      row = row < g.M ? row : g.M - 1;
      pre[i * NP + pass] = *(const uint4*)((const uint16_t*)g.residual + row * g.ldc + col);
    }
}

template <int TM, int WN, bool FAST, int EPI, typename Scatter>
__device__ __forceinline__ void gemm_epilogue_bands(Scatter&& scatter, const GemmArgs& g, int64_t m0,
                                                    int64_t n0, int wm, int wn, int64_t c_off, int wave,
                                                    int lane, const uint4* pre = nullptr) {
  constexpr int SLAB_LD = WN + 4;  // floats per slab row (padding spreads the row groups)
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
  if (EPI != 0 && g.bias) {
    if (!out_f32 && col + 8 <= g.N && (((uintptr_t)g.bias + 2 * (uintptr_t)col) & 15) == 0) {
      const uint4 bu = *(const uint4*)((const uint16_t*)g.bias + col);  // eight 16-bit values at once
      bias_v[0] = __uint_as_float(bu.x << 16); bias_v[1] = __uint_as_float(bu.x & 0xffff0000u);
      bias_v[2] = __uint_as_float(bu.y << 16); bias_v[3] = __uint_as_float(bu.y & 0xffff0000u);
      bias_v[4] = __uint_as_float(bu.z << 16); bias_v[5] = __uint_as_float(bu.z & 0xffff0000u);
      bias_v[6] = __uint_as_float(bu.w << 16); bias_v[7] = __uint_as_float(bu.w & 0xffff0000u);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (col + e < g.N) bias_v[e] = nbk_load_as_f32(g.bias, col + e, g.dtype_c);
    }
  }
  constexpr int NP = 32 / ROWS_PER_PASS;
  const bool res_vec = EPI == 2 && g.residual && vec_store && !out_f32;
  // the residual of the whole wave tile is requested before the first slab round trip, so that
  // its latency is paid once and not pass by pass (the K loop's registers are free by now)
  uint4 rpre[EPI == 2 ? TM : 1][NP];
  if constexpr (EPI == 2) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int pass = 0; pass < NP; ++pass) {
        const int64_t row = m0 + wm + i * 32 + pass * ROWS_PER_PASS + sub_r;
        rpre[i][pass] = make_uint4(0u, 0u, 0u, 0u);
        if (res_vec && row < g.M)
          rpre[i][pass] = *(const uint4*)((const uint16_t*)g.residual + c_off + row * g.ldc + col);
      }
  }
  static_for<TM>([&](auto ti) {
    constexpr int i = decltype(ti)::value;
    scatter(ti, slab);
    // the slab is private to the wave: no workgroup barrier, only LDS ordering
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    auto one_pass = [&](int pass, const uint4 u) {
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
        if (EPI == 1 || EPI == 3 || EPI == 4) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += bias_v[e];
        }
        if (EPI == 4) {
          v[0] += __uint_as_float(u.x << 16); v[1] += __uint_as_float(u.x & 0xffff0000u);
          v[2] += __uint_as_float(u.y << 16); v[3] += __uint_as_float(u.y & 0xffff0000u);
          v[4] += __uint_as_float(u.z << 16); v[5] += __uint_as_float(u.z & 0xffff0000u);
          v[6] += __uint_as_float(u.w << 16); v[7] += __uint_as_float(u.w & 0xffff0000u);
        }
        if (EPI == 3 && g.residual) {
          if (vec_store && !out_f32) {
            const uint4 ru = *(const uint4*)((const uint16_t*)g.residual + idx);
            v[0] += __uint_as_float(ru.x << 16); v[1] += __uint_as_float(ru.x & 0xffff0000u);
            v[2] += __uint_as_float(ru.y << 16); v[3] += __uint_as_float(ru.y & 0xffff0000u);
            v[4] += __uint_as_float(ru.z << 16); v[5] += __uint_as_float(ru.z & 0xffff0000u);
            v[6] += __uint_as_float(ru.w << 16); v[7] += __uint_as_float(ru.w & 0xffff0000u);
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (col + e < g.N) v[e] += nbk_load_as_f32(g.residual, idx + e, g.dtype_c);
          }
        }
        if (EPI == 2) {
          float res[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) res[e] = 0.f;
          if (res_vec) {
            res[0] = __uint_as_float(u.x << 16); res[1] = __uint_as_float(u.x & 0xffff0000u);
            res[2] = __uint_as_float(u.y << 16); res[3] = __uint_as_float(u.y & 0xffff0000u);
            res[4] = __uint_as_float(u.z << 16); res[5] = __uint_as_float(u.z & 0xffff0000u);
            res[6] = __uint_as_float(u.w << 16); res[7] = __uint_as_float(u.w & 0xffff0000u);
          } else if (g.residual) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (col + e < g.N) res[e] = nbk_load_as_f32(g.residual, idx + e, g.dtype_c);
          }
          if (g.C2) {
            // two results: the activation goes to C below, its derivative to C2 here
            float d2[8];
            if (out_f32) {
#pragma unroll
              for (int e = 0; e < 8; ++e) gemm_act_pair<false>(v[e] + bias_v[e], g.act, v[e], d2[e]);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e) gemm_act_pair<true>(v[e] + bias_v[e], g.act, v[e], d2[e]);
            }
            if (vec_store && !out_f32) {
              uint4 o;
              o.x = (uint32_t)nbk_f32_to_bf16(d2[0]) | ((uint32_t)nbk_f32_to_bf16(d2[1]) << 16);
              o.y = (uint32_t)nbk_f32_to_bf16(d2[2]) | ((uint32_t)nbk_f32_to_bf16(d2[3]) << 16);
              o.z = (uint32_t)nbk_f32_to_bf16(d2[4]) | ((uint32_t)nbk_f32_to_bf16(d2[5]) << 16);
              o.w = (uint32_t)nbk_f32_to_bf16(d2[6]) | ((uint32_t)nbk_f32_to_bf16(d2[7]) << 16);
              *(uint4*)((uint16_t*)g.C2 + idx) = o;
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (col + e < g.N) {
                  if (out_f32) ((float*)g.C2)[idx + e] = d2[e];
                  else ((uint16_t*)g.C2)[idx + e] = nbk_f32_to_bf16(d2[e]);
                }
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float x = gemm_act(v[e] + bias_v[e], g.act);
              v[e] = !g.residual ? x : (g.res_mul ? x * res[e] : x + res[e]);
            }
          }
        }
        if (vec_store && !out_f32) {
          uint4 o;
          o.x = (uint32_t)nbk_f32_to_bf16(v[0]) | ((uint32_t)nbk_f32_to_bf16(v[1]) << 16);
          o.y = (uint32_t)nbk_f32_to_bf16(v[2]) | ((uint32_t)nbk_f32_to_bf16(v[3]) << 16);
          o.z = (uint32_t)nbk_f32_to_bf16(v[4]) | ((uint32_t)nbk_f32_to_bf16(v[5]) << 16);
          o.w = (uint32_t)nbk_f32_to_bf16(v[6]) | ((uint32_t)nbk_f32_to_bf16(v[7]) << 16);
          if (g.c_stream) {
            const u32x4 ov = {o.x, o.y, o.z, o.w};
            __builtin_nontemporal_store(ov, (u32x4*)((uint16_t*)g.C + idx));
          } else {
            *(uint4*)((uint16_t*)g.C + idx) = o;
          }
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
    };
    if constexpr (EPI == 2) {
#pragma unroll
      for (int pass = 0; pass < NP; ++pass) one_pass(pass, rpre[i][pass]);
    } else if constexpr (EPI == 4) {
#pragma unroll
      for (int pass = 0; pass < NP; ++pass) one_pass(pass, pre[i * NP + pass]);
    } else {
#pragma unroll 1
      for (int pass = 0; pass < NP; ++pass) one_pass(pass, make_uint4(0u, 0u, 0u, 0u));
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // slab reads done before the next tile row overwrites it
  });
}

// 32x32 MFMA blocks: D[i][j] lives in lane (j, (i / 4) % 2), register (i / 8) * 4 + i % 4.
template <int TM, int TN, int WN, bool FAST, int EPI>
__device__ __forceinline__ void gemm_epilogue(f32x16 (&acc)[TM][TN], const GemmArgs& g, int64_t m0,
                                              int64_t n0, int wm, int wn, int64_t c_off, int wave,
                                              int lane, const uint4* pre = nullptr) {
  const int li = lane & 31, kg = lane >> 5;
  gemm_epilogue_bands<TM, WN, FAST, EPI>(
      [&](auto ti, float* slab) {
        constexpr int i = decltype(ti)::value;
        static_for<TN>([&](auto tj) {
          constexpr int j = decltype(tj)::value;
          const f32x16 a = acc[i][j];
#pragma unroll
          for (int r = 0; r < 16; ++r)
            slab[((r >> 2) * 8 + kg * 4 + (r & 3)) * (WN + 4) + j * 32 + li] = a[r];
        });
      },
      g, m0, n0, wm, wn, c_off, wave, lane, pre);
}

// 16x16 MFMA blocks: D[i][j] lives in lane (j, i / 4), register i % 4; a band is two block rows.
// (Storing straight from the registers, with the product transposed so that a lane holds four
// consecutive columns, was measured: the 32-byte row pieces it writes make the epilogue slower
// than the slab round trip with its whole 128-byte lines.)
template <int TM, int TN, int WN, bool FAST, int EPI>
__device__ __forceinline__ void gemm_epilogue(f32x4 (&acc)[TM][TN], const GemmArgs& g, int64_t m0,
                                              int64_t n0, int wm, int wn, int64_t c_off, int wave,
                                              int lane) {
  static_assert(TM % 2 == 0, "block rows per wave tile");
  const int p = lane & 15, q = lane >> 4;
  gemm_epilogue_bands<TM / 2, WN, FAST, EPI>(
      [&](auto ti, float* slab) {
        constexpr int i = decltype(ti)::value;
        static_for<2 * TN>([&](auto tb) {
          constexpr int ib = decltype(tb)::value / TN, j = decltype(tb)::value % TN;
          const f32x4 a = acc[2 * i + ib][j];
#pragma unroll
          for (int r = 0; r < 4; ++r) slab[(ib * 16 + 4 * q + r) * (WN + 4) + j * 16 + p] = a[r];
        });
      },
      g, m0, n0, wm, wn, c_off, wave, lane);
}

// NW waves: 4 as 2 x 2, or 8 as 2 x 4 (two waves per SIMD, each with half the accumulators:
// they cover each other's waits at the price of 1.5 x the LDS fragment traffic).
template <int BM, int BN, bool A_KC, bool B_KC, bool EPI, int NW, bool B_Q = false>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_kernel(const GemmArgs g) {
  constexpr int NT = NW * 64, WGN = NW / 2;
  // B_Q: B holds NF4 codes (one byte per weight, addressed like a dense B) and g.b_scales the
  // block scales; the tile loader dequantises on the way into LDS
  __shared__ float nf4_table[B_Q ? 16 : 1];
  if (B_Q) {
    if (threadIdx.x < 16) nf4_table[threadIdx.x] = nbk_nf4_levels[threadIdx.x];
    __syncthreads();
  }
  constexpr int WM = BM / 2, WN = BN / WGN;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int CA = TileGeom<BM, A_KC>::CHUNKS, CB = TileGeom<BN, B_KC>::CHUNKS;
  constexpr int TILE_CHUNKS = CA + CB;
  constexpr int PA = TileGeom<BM, A_KC>::PITCH * 16, PB = TileGeom<BN, B_KC>::PITCH * 16;  // bytes
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

  TileLoader<BM, A_KC, NT> la;
  TileLoader<BN, B_KC, NT> lb;
  const int64_t nk = (g.K + 63) / 64;
  // A is rows = m; for the loader a K-contiguous operand has (rs = row stride, k unit),
  // a row-contiguous one has (cs = k stride, row unit).
  la.load(A, g.a_rs, g.a_cs, m0, g.M, 0, g.K, g.a_vec);
  if constexpr (B_Q) lb.load_nf4((const uint8_t*)g.B, g.b_scales, g.b_block, nf4_table, g.b_cs, g.b_rs, n0, g.N, 0, g.K);
  else lb.load(B, g.b_cs, g.b_rs, n0, g.N, 0, g.K, g.b_vec);
  la.store(gemm_lds);
  lb.store(gemm_lds + CA);
  __syncthreads();

  // Fragment addresses.  swz(row, ks * 2 + kg) = (row * 8 | t) ^ (ks * 2) with
  // t = kg ^ (row % 8) ^ (row / 8 % 8): only a constant XOR moves with ks.
  // A k-major operand needs one byte offset per wave: lane p of group q = lane / 16 points at
  // k-row 8 * (q / 2) + p / 4, rows 16 * (q % 2) + 4 * (p % 4) of the wave's first tile; the
  // tile row, the k-step and the second half of the fragment are constant offsets.
  int a_addr[TM], b_addr[TN];
  const int tr_k = 8 * (lane >> 5) + ((lane & 15) >> 2), tr_r = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int a_tr = tr_k * PA + (wm + tr_r) * 2, b_tr = CA * 16 + tr_k * PB + (wn + tr_r) * 2;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = wm + i * 32 + li;
    a_addr[i] = row * 8 + (kg ^ (row & 7) ^ ((row >> 3) & 7));
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = wn + j * 32 + li;
    b_addr[j] = CA + row * 8 + (kg ^ (row & 7) ^ ((row >> 3) & 7));
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
      if constexpr (A_KC) {
        const u32x4 u = tile[a_addr[R] ^ sel];
        fa[SET][R] = *(const bf16x8*)&u;
      } else {
        const char* p = (const char*)tile + a_tr + (R * 64 + ks * 16 * PA);
        const s16x4 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * PA);
        const s16x8 u = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        fa[SET][R] = *(const bf16x8*)&u;
      }
    } else {
      if constexpr (B_KC) {
        const u32x4 u = tile[b_addr[R - TM] ^ sel];
        fb[SET][R - TM] = *(const bf16x8*)&u;
      } else {
        const char* p = (const char*)tile + b_tr + ((R - TM) * 64 + ks * 16 * PB);
        const s16x4 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * PB);
        const s16x8 u = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        fb[SET][R - TM] = *(const bf16x8*)&u;
      }
    }
  };
  // LDS read instructions of fragment r in the order above: a k-major operand takes two
  auto frag_reads = [](int r0) constexpr {
    const int r = r0 == 0 ? 0 : (r0 <= TN ? TM + r0 - 1 : r0 - TN);
    return r < TM ? (A_KC ? 1 : 2) : (B_KC ? 1 : 2);
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
      __builtin_amdgcn_sched_group_barrier(0x100, frag_reads(decltype(r)::value), 0);  // DS read
      if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x008, n, 0);  // MFMAs
    });
    __builtin_amdgcn_sched_barrier(0);  // later stages' work (and its waits) stays behind
  };

  static_for<NFRAG>([&](auto r) { read_frag(std::integral_constant<int, 0>{}, r, gemm_lds, 0); });
  {
    const int64_t k1 = nk > 1 ? 64 : 0;  // a single-tile problem re-reads tile 0 (never stored)
    la.load(A, g.a_rs, g.a_cs, m0, g.M, k1, g.K, g.a_vec);
    if constexpr (B_Q) lb.load_nf4((const uint8_t*)g.B, g.b_scales, g.b_block, nf4_table, g.b_cs, g.b_rs, n0, g.N, k1, g.K);
    else lb.load(B, g.b_cs, g.b_rs, n0, g.N, k1, g.K, g.b_vec);
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
      using LA = TileLoader<BM, A_KC, NT>;
      using LB = TileLoader<BN, B_KC, NT>;
      constexpr int NPA = LA::NPIECE, NP = LA::NPIECE + LB::NPIECE;
      constexpr int PER = (NP + NFRAG - 1) / NFRAG;
      static_for<NFRAG>([&](auto r) {
        read_frag(S1{}, r, cur, 3);
        static_for<PER>([&](auto e) {
          constexpr int P = decltype(r)::value * PER + decltype(e)::value;
          if constexpr (P < NPA) la.template store_piece<P>(nxt);
          else if constexpr (P < NP) lb.template store_piece<P - NPA>(nxt + CA);
        });
      });
      static_for<NMFMA>([&](auto q) { mfma(S0{}, q); });
      static_for<NFRAG>([&](auto r) {
        constexpr int n = share(NMFMA, NFRAG, decltype(r)::value);
        __builtin_amdgcn_sched_group_barrier(0x100, frag_reads(decltype(r)::value), 0);  // DS read
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
      if constexpr (B_Q) lb.load_nf4((const uint8_t*)g.B, g.b_scales, g.b_block, nf4_table, g.b_cs, g.b_rs, n0, g.N, k2, g.K);
      else lb.load(B, g.b_cs, g.b_rs, n0, g.N, k2, g.K, g.b_vec);
    }
    static_for<NMFMA / 2>([&](auto q) { mfma(S1{}, q); });
    {
      constexpr int NL = TileLoader<BM, A_KC, NT>::NREG + TileLoader<BN, B_KC, NT>::NREG;
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
      __builtin_amdgcn_sched_group_barrier(0x100, frag_reads(decltype(r)::value), 0);
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

  gemm_epilogue<TM, TN, WN, false, EPI ? 2 : 0>(acc, g, m0, n0, wm, wn, c_off, wave, lane);
}

// ------------------------------------------------------------- bf16, direct-to-LDS loads
// The hot form (16-byte-aligned operands, K % 64 == 0): tiles go from global memory into LDS
// without passing through registers (global_load_lds_dwordx4: lane l of a wave deposits its
// 16 bytes at a wave-uniform LDS base + 16 l), so that the fragment reads are the only LDS
// instructions of the K loop and the lanes hold no staging registers.  Because the LDS side
// of such a load is linear in the lane, both layouts are unpadded and XOR-swizzled, and the
// swizzle is applied to the global address each lane fetches from:
//   K-contiguous operand   [row][8 chunks]: chunk c of row r sits at c ^ dl_kc_xor(r) (below);
//   row-contiguous operand [64 k][ROWS / 8 chunks]: chunk c of k-row k sits at
//     c ^ 2 * T[k % 4], T = {0, 3, 6, 5}, which sends the eight 32-byte segments that half a
//     wave touches in one transposing read to eight different bank groups.
// ds_read_b128 serves 16 lanes per cycle, and not neighbouring ones: lanes {0-3, 12-15, 20-23,
// 24-27} share a cycle, lanes {4-11, 16-19, 28-31} the next, and the same again 32 lanes up
// (measured with the bank-conflict counter, two lanes at a time).  The 16 chunks of such a group
// have to fall into 16 different 16-byte slots of the 256-byte bank window.
//   32 x 32 x 16 fragments (lane = row % 32, one chunk per half-wave): rows {0-3, 12-15, 20-23,
//     24-27} of a block at one chunk: c ^ (r % 8) ^ (r / 8 % 2) does it;
//   16 x 16 x 32 fragments (lane = row % 16 + 16 * chunk): rows {0-3, 12-15} at chunk c together
//     with rows {4-11} at chunk c ^ 1: the row pairs e = r / 2 % 8 of the first set go to
//     {0..3}, those of the second to {4..7}, so that c and c ^ 1 never meet.
template <bool MI16>
__device__ __forceinline__ int dl_kc_xor(int row) {
  if constexpr (MI16) {
    const int e = (row >> 1) & 7;
    return ((((e >> 1) ^ (e >> 2)) & 1) << 2) | (((e >> 2) & 1) << 1) | (e & 1);
  } else {
    return (row & 7) ^ ((row >> 3) & 1);
  }
}
__device__ __forceinline__ int dl_seg_xor(int k) { return (k & 3) ^ (((k & 3) << 1) & 7); }
// The 16x16x32 form reads k-rows k .. k + 3 and k + 8 .. k + 11 of one 32-byte segment in
// half a wave: bit 3 of k joins the swizzle.
template <bool MI16>
__device__ __forceinline__ int dl_seg_xor_of(int k) {
  return MI16 ? dl_seg_xor(k) ^ ((k >> 3) & 1) : dl_seg_xor(k);
}

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

template <int ROWS, bool KC, int NW, bool MI16 = false>
struct DirectLoader {
  // ROWS * 8 chunks, 64 per wave instruction, dealt to the waves in consecutive runs
  static constexpr int N = ROWS / (8 * NW);
  static constexpr int NC = ROWS / 8;
  static_assert(N >= 1 && N % 2 == 0, "instructions per wave");
  int voff[N];         // byte offset of this lane's chunk from the tile's first element
  const char* base;    // operand + tile row offset (wave-uniform)
  int64_t kstep;       // bytes between consecutive K tiles (wave-uniform)
  int first;           // first instruction of this wave

  __device__ __forceinline__ void init(const uint16_t* op, int64_t rs, int64_t cs, int64_t row0,
                                       int64_t rows_total, int wave, int lane) {
    first = wave * N;
    if (KC) {
      base = (const char*)(op + row0 * rs);
      kstep = 128;
      const int64_t last = rows_total - 1 - row0;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const int row = (first + j) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ dl_kc_xor<MI16>(row);
        const int64_t r = row < last ? row : last;
        voff[j] = (int)(r * rs * 2 + c * 16);
      }
    } else {
      base = (const char*)(op + row0);
      kstep = 128 * cs;
      const int64_t last = rows_total - 8 - row0;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const int l = (first + j) * 64 + lane;
        const int k = l / NC, c = (l % NC) ^ (dl_seg_xor_of<MI16>(k) << 1);
        const int64_t r = c * 8 < last ? c * 8 : last;
        voff[j] = (int)(k * cs * 2 + r * 2);
      }
    }
  }
  // One K tile of a second, shallower operand (only k < kvalid of the tile's 64 k-rows exist),
  // laid out in `region` like any other tile: a lane whose chunk lies beyond kvalid writes zeros
  // to its LDS slot instead of fetching.  Keeps no state; (rs, cs) as for init.
  __device__ __forceinline__ static void issue_tail(u32x4* region, const uint16_t* op, int64_t rs,
                                                    int64_t cs, int64_t row0, int64_t rows_total,
                                                    int kvalid, int wave, int lane) {
    const int first_ = wave * N;
    static_for<N>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      const char* src;
      bool there;
      if (KC) {
        const int64_t last = rows_total - 1 - row0;
        const int row = (first_ + j) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ dl_kc_xor<MI16>(row);
        const int64_t r = row < last ? row : last;
        src = (const char*)(op + row0 * rs) + (r * rs * 2 + c * 16);
        there = c * 8 < kvalid;
      } else {
        const int64_t last = rows_total - 8 - row0;
        const int l = (first_ + j) * 64 + lane;
        const int k = l / NC, c = (l % NC) ^ (dl_seg_xor_of<MI16>(k) << 1);
        const int64_t r = c * 8 < last ? c * 8 : last;
        src = (const char*)(op + row0) + (k * cs * 2 + r * 2);
        there = k < kvalid;
      }
      if (there)
        __builtin_amdgcn_global_load_lds((glb_void_t*)src, (lds_void_t*)(region + (first_ + j) * 64),
                                         16, 0, 0);
      else
        region[(first_ + j) * 64 + lane] = (u32x4)(0u);
    });
  }
  // start the copy of K tile `kt` into `region` (this operand's part of a tile buffer)
  __device__ __forceinline__ const char* tile_src(int64_t kt) const { return base + kt * kstep; }
  template <int J>
  __device__ __forceinline__ void issue_one(u32x4* region, const char* src) const {
    __builtin_amdgcn_global_load_lds((glb_void_t*)(src + voff[J]),
                                     (lds_void_t*)(region + (first + J) * 64), 16, 0, 0);
  }
  __device__ __forceinline__ void issue(u32x4* region, int64_t kt) const {
    const char* src = tile_src(kt);
    static_for<N>([&](auto j) { issue_one<decltype(j)::value>(region, src); });
  }
};

// MI16: the matrix instruction is v_mfma_f32_16x16x32_bf16 (blocks of 16 x 16, 32 deep) instead
// of v_mfma_f32_32x32x16_bf16 (32 x 32, 16 deep).  Same LDS traffic and register budget; the
// 16 x 16 form does the same arithmetic for about a tenth less power, and these products run at
// the power limit (the clock under MFMA load settles where the limit puts it), so it is the
// faster one with two waves per SIMD to keep its shorter instructions back to back.
// KSS: k-steps (one MFMA deep) per fragment set.  A step of KSS k-steps is multiplied out of one
// set while the other is filled for the next step; small wave tiles take 2, so that a read has
// more than a handful of MFMAs to land.
// COLSUM: the launch also leaves sum_k B[k][n] (the bias gradient beside a weight gradient
// x^T dy, which reads dy anyway): the waves that hold the first block row of the first tile row
// multiply a fragment of ones into one more accumulator per block column, from the B fragments
// that are in registers for the product -- no byte is read twice.
template <int BM, int BN, bool A_KC, bool B_KC, int EPI, int NW, int KSS, bool MI16, bool COLSUM = false>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_dl_kernel(const GemmArgs g) {
  constexpr int WGN = NW / 2;
  constexpr int WM = BM / 2, WN = BN / WGN;  // wave tile
  constexpr int FM = MI16 ? 16 : 32;          // rows / columns of an MFMA block
  constexpr int KQ = MI16 ? 32 : 16;          // depth of one MFMA
  constexpr int TM = WM / FM, TN = WN / FM;
  constexpr int CA = BM * 8, TILE_CHUNKS = (BM + BN) * 8;
  int tm_i, tn_i;
  gemm_tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tm_i, tn_i);
  const int64_t m0 = (int64_t)tm_i * BM, n0 = (int64_t)tn_i * BN;
  const int64_t bo = (int64_t)blockIdx.y / g.batch_inner, bi = (int64_t)blockIdx.y % g.batch_inner;
  const uint16_t* A = (const uint16_t*)g.A + bo * g.a_bs + bi * g.a_bs2;
  const uint16_t* B = (const uint16_t*)g.B + bo * g.b_bs + bi * g.b_bs2;
  const int64_t c_off = bo * g.c_bs + bi * g.c_bs2;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = (wave / WGN) * WM, wn = (wave % WGN) * WN;
  const int li = lane & 31, kg = lane >> 5;

  using Acc = std::conditional_t<MI16, f32x4, f32x16>;
  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (Acc)(0.f);

  static_assert(!COLSUM || MI16, "column sums ride on the 16 x 16 x 32 instruction");
  f32x4 cs[COLSUM ? TN : 1];
  bool do_cs = false;
  if constexpr (COLSUM) {
#pragma unroll
    for (int j = 0; j < TN; ++j) cs[j] = (f32x4)(0.f);
    do_cs = tm_i == 0 && wm == 0;  // (uniform over the wave)
  }

  using LA = DirectLoader<BM, A_KC, NW, MI16>;
  using LB = DirectLoader<BN, B_KC, NW, MI16>;
  LA la;
  LB lb;
  // K tiles of the launch: the shallow pairs (one tile each; their offsets are dead before the
  // loop's are made), then A and B, then the deep pairs, which share the loop's lane offsets and
  // differ in the wave-uniform base only.  src_a(t) / src_b(t): where tile t starts in memory.
  // (tile numbers are 32-bit: the scalar unit compares those, 64-bit ones go through vector registers)
  const int ns = g.n_shallow;
  const int e0 = ns + (int)(g.K / 64);                                   // first tile past A and B
  const int e1 = e0 + (g.n_deep > 0 ? (int)(g.deep[0].K / 64) : 0);      // ... past the first deep pair
  const int nk = e1 + (g.n_deep > 1 ? (int)(g.deep[1].K / 64) : 0);
  if (ns > 0) {
    const auto& t0 = g.shallow[0];
    LA::issue_tail(gemm_lds, (const uint16_t*)t0.A, t0.a_rs, t0.a_cs, m0, g.M, (int)t0.K, wave, lane);
    LB::issue_tail(gemm_lds + CA, (const uint16_t*)t0.B, t0.b_cs, t0.b_rs, n0, g.N, (int)t0.K, wave, lane);
  }
  if (ns > 1) {
    const auto& t1 = g.shallow[1];
    LA::issue_tail(gemm_lds + TILE_CHUNKS, (const uint16_t*)t1.A, t1.a_rs, t1.a_cs, m0, g.M, (int)t1.K,
                   wave, lane);
    LB::issue_tail(gemm_lds + TILE_CHUNKS + CA, (const uint16_t*)t1.B, t1.b_cs, t1.b_rs, n0, g.N,
                   (int)t1.K, wave, lane);
  }
  la.init(A, g.a_rs, g.a_cs, m0, g.M, wave, lane);
  lb.init(B, g.b_cs, g.b_rs, n0, g.N, wave, lane);
  // base of every run of tiles, moved back by the tiles before it, so that tile t of the launch
  // is at base + t * kstep whichever run it belongs to (wave-uniform values, held in scalar
  // registers as 64-bit integers: the K loop has no vector register to spare)
  auto uniform = [](const char* p) {
    const uint64_t b = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  const uint64_t a_run0 = uniform(la.base - ns * la.kstep), b_run0 = uniform(lb.base - ns * lb.kstep);
  uint64_t a_run1 = a_run0, b_run1 = b_run0, a_run2 = a_run0, b_run2 = b_run0;
  if (g.n_deep > 0) {
    a_run1 = uniform(la.base + ((const char*)g.deep[0].A - (const char*)A) - (int64_t)e0 * la.kstep);
    b_run1 = uniform(lb.base + ((const char*)g.deep[0].B - (const char*)B) - (int64_t)e0 * lb.kstep);
  }
  if (g.n_deep > 1) {
    a_run2 = uniform(la.base + ((const char*)g.deep[1].A - (const char*)A) - (int64_t)e1 * la.kstep);
    b_run2 = uniform(lb.base + ((const char*)g.deep[1].B - (const char*)B) - (int64_t)e1 * lb.kstep);
  }
  const int64_t a_kstep = la.kstep, b_kstep = lb.kstep;
#define GEMM_SRC_A(t) ((const char*)(((t) < e0 ? a_run0 : ((t) < e1 ? a_run1 : a_run2)) + (uint64_t)((int64_t)(t) * a_kstep)))
#define GEMM_SRC_B(t) ((const char*)(((t) < e0 ? b_run0 : ((t) < e1 ? b_run1 : b_run2)) + (uint64_t)((int64_t)(t) * b_kstep)))
  if (ns == 0) {
    const char* sa = GEMM_SRC_A(0);
    const char* sb = GEMM_SRC_B(0);
    static_for<LA::N>([&](auto j) { la.template issue_one<decltype(j)::value>(gemm_lds, sa); });
    static_for<LB::N>([&](auto j) { lb.template issue_one<decltype(j)::value>(gemm_lds + CA, sb); });
  }

  // Fragment addresses, one per block row / column of the wave tile.  32 x 32 x 16:
  //   K-contiguous: byte address 16 ((row * 8 | t) ^ (2 ks)), t = kg ^ (row % 8) ^ (row / 8 % 2);
  //   row-contiguous: byte address of this lane's 8 bytes in the transposing read of k-step 0,
  //     first half; the k-step and the half are constant offsets.  Lane p of group q = lane / 16
  //     points at k-row 8 (q / 2) + p / 4, rows 16 (q % 2) + 4 (p % 4) .. + 4 of the block.
  // 16 x 16 x 32 (lane p of group q holds k = 8 q .. + 8 of row p):
  //   K-contiguous: 16 ((row * 8 | t) ^ (4 ks)), t = q ^ dl_kc_xor<true>(row);
  //   row-contiguous: k-row 8 q + p / 4, rows 4 (p % 4) .. + 4 of the block.
  int a_addr[TM], b_addr[TN];
  if constexpr (MI16) {
    const int p = lane & 15, q = lane >> 4;
    const int kl = 8 * q + (p >> 2), sx = dl_seg_xor_of<true>(kl);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm + i * 16 + p;
      if (A_KC) a_addr[i] = (row * 8 + (q ^ dl_kc_xor<true>(row))) * 16;
      else a_addr[i] = kl * (BM * 2) + ((((wm >> 4) + i) ^ sx) * 32) + 8 * (p & 3);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wn + j * 16 + p;
      if (B_KC) b_addr[j] = (CA + row * 8 + (q ^ dl_kc_xor<true>(row))) * 16;
      else b_addr[j] = CA * 16 + kl * (BN * 2) + ((((wn >> 4) + j) ^ sx) * 32) + 8 * (p & 3);
    }
  } else {
    const int p = lane & 15, q = lane >> 4;
    const int kl = 8 * (q >> 1) + (p >> 2), sx = dl_seg_xor(p >> 2);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm + i * 32 + li;
      if (A_KC) a_addr[i] = (row * 8 + (kg ^ dl_kc_xor<false>(row))) * 16;
      else a_addr[i] = kl * (BM * 2) + ((((wm >> 4) + 2 * i + (q & 1)) ^ sx) * 32) + 8 * (p & 3);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wn + j * 32 + li;
      if (B_KC) b_addr[j] = (CA + row * 8 + (kg ^ dl_kc_xor<false>(row))) * 16;
      else
        b_addr[j] = CA * 16 + kl * (BN * 2) + ((((wn >> 4) + 2 * j + (q & 1)) ^ sx) * 32) +
                    8 * (p & 3);
    }
  }

  bf16x8 fa[2][KSS * TM], fb[2][KSS * TN];
  constexpr int NSTEP = 64 / KQ / KSS;
  static_assert(NSTEP >= 2 && NSTEP % 2 == 0, "steps per tile");
  constexpr int NFRAG = KSS * (TM + TN), NMFMA = KSS * TM * TN;  // per step
  // read fragment r of step `step` from `tile` into set SET; order of use by the MFMAs
  // (k-step by k-step, row-major over the wave's blocks): A0, every B, A1, A2 ...
  auto read_frag = [&](auto set, auto r, const u32x4* tile, int step) {
    constexpr int SET = decltype(set)::value;
    constexpr int KL = decltype(r)::value / (TM + TN), R0 = decltype(r)::value % (TM + TN);
    constexpr int R = R0 == 0 ? 0 : (R0 <= TN ? TM + R0 - 1 : R0 - TN);
    const int ks = step * KSS + KL;
    if constexpr (R < TM) {
      if constexpr (A_KC) {
        int sel = ks * (KQ * 2);
        asm volatile("" : "+s"(sel));  // recomputed at every read: hoisted variants would spill
        fa[SET][KL * TM + R] = lds_read_b128(lds_addr(tile) + (a_addr[R] ^ sel));
      } else {
        const uint32_t p = lds_addr(tile) + a_addr[R];
        fa[SET][KL * TM + R] = lds_read_tr_pair(p, ks * KQ * (BM * 2), (ks * KQ + 4) * (BM * 2));
      }
    } else {
      if constexpr (B_KC) {
        int sel = ks * (KQ * 2);
        asm volatile("" : "+s"(sel));
        fb[SET][KL * TN + R - TM] = lds_read_b128(lds_addr(tile) + (b_addr[R - TM] ^ sel));
      } else {
        const uint32_t p = lds_addr(tile) + b_addr[R - TM];
        fb[SET][KL * TN + R - TM] = lds_read_tr_pair(p, ks * KQ * (BN * 2), (ks * KQ + 4) * (BN * 2));
      }
    }
  };
  // The compiler does not see the fragment reads (inline assembly): before the MFMAs of a
  // k-step may touch a fragment set, wait for LDS by hand, with the set's registers as
  // operands of the wait so that no MFMA can be moved in front of it.
  auto frags_ready = [&](auto set) {
    constexpr int SET = decltype(set)::value;
    __builtin_amdgcn_sched_barrier(0);
    lds_wait_for(fa[SET]);
    lds_wait_for(fb[SET]);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto mfma = [&](auto set, auto q) {
    constexpr int SET = decltype(set)::value, Q = decltype(q)::value;
    constexpr int kl = Q / (TM * TN), i = Q % (TM * TN) / TN, j = Q % TN;
    if constexpr (MI16)
      acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[SET][kl * TM + i], fb[SET][kl * TN + j],
                                                          acc[i][j], 0, 0, 0);
    else
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[SET][kl * TM + i], fb[SET][kl * TN + j],
                                                          acc[i][j], 0, 0, 0);
  };
  // column sums of the step whose B fragments are in set SET (still whole: reads fill the other)
  auto colsum_step = [&](auto set) {
    if constexpr (COLSUM) {
      constexpr int SET = decltype(set)::value;
      if (do_cs) {
        const uint32_t one2 = 0x3f803f80u;  // two bf16 ones
        const u32x4 ones4 = {one2, one2, one2, one2};
        const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
#pragma unroll
        for (int kl = 0; kl < KSS; ++kl)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            cs[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, fb[SET][kl * TN + j], cs[j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // step on fragment set SET while set 1 - SET is filled for step `step_next` of `tile`
  auto stage = [&](auto set, const u32x4* tile, int step_next) {
    constexpr int SET = decltype(set)::value;
    frags_ready(set);
    // the reads go out between the MFMAs of the first half (pinned: the scheduler would batch
    // them), so that they have the second half to land
    constexpr int SPREAD = NMFMA / 2;
    static_for<NMFMA>([&](auto q) {
      constexpr int Q = decltype(q)::value;
      static_for<NFRAG>([&](auto r) {
        if constexpr (decltype(r)::value * SPREAD / NFRAG == Q)
          read_frag(std::integral_constant<int, 1 - SET>{}, r, tile, step_next);
      });
      mfma(set, q);
      if constexpr (Q < SPREAD) __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_sched_barrier(0);
    colsum_step(set);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  // a workgroup barrier behind which every wave's copies have landed
  auto tile_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's copies are in LDS
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    __builtin_amdgcn_sched_barrier(0);
  };

  // Two tile buffers.  Tile kt + 1 is on its way while tile kt is multiplied; the barrier that
  // ends tile kt (in the middle of its last step, whose fragments are in registers by then)
  // frees its buffer for tile kt + 2, whose copies are started right behind that barrier and
  // have the whole of tile kt + 1 to land.
  tile_barrier();
  static_for<NFRAG>([&](auto r) { read_frag(S0{}, r, gemm_lds, 0); });
  if (nk > 1 && ns < 2) {
    const char* sa = GEMM_SRC_A(1);
    const char* sb = GEMM_SRC_B(1);
    static_for<LA::N>([&](auto j) { la.template issue_one<decltype(j)::value>(gemm_lds + TILE_CHUNKS, sa); });
    static_for<LB::N>([&](auto j) { lb.template issue_one<decltype(j)::value>(gemm_lds + TILE_CHUNKS + CA, sb); });
  }
  for (int kt = 0; kt + 1 < nk; ++kt) {
    u32x4* cur = gemm_lds + (kt & 1) * TILE_CHUNKS;
    const u32x4* nxt = gemm_lds + ((kt + 1) & 1) * TILE_CHUNKS;
    static_for<NSTEP - 1>([&](auto st) {
      constexpr int ST = decltype(st)::value;
      stage(std::integral_constant<int, ST & 1>{}, cur, ST + 1);
    });
    frags_ready(S1{});  // the last step (NSTEP is even) is on set 1
    static_for<NMFMA / 2>([&](auto q) { mfma(S1{}, q); });
    tile_barrier();
    {
      // Behind the barrier: the first fragments of tile kt + 1, the copies of tile kt + 2 and
      // the second half of the MFMAs, dealt out evenly and pinned in this order (the copies
      // and the reads both touch LDS, so the scheduler would otherwise leave the MFMAs last).
      // (the last pass has no tile kt + 2: it fetches tile nk - 1 again, into a buffer that
      // is not read any more, which keeps this block free of branches)
      constexpr int NL = LA::N + LB::N, H = NMFMA / 2;
      const int k2 = kt + 2 < nk ? kt + 2 : nk - 1;
      const char* src_a2 = GEMM_SRC_A(k2);
      const char* src_b2 = GEMM_SRC_B(k2);
      static_for<H>([&](auto q) {
        constexpr int Q = decltype(q)::value;
        static_for<NFRAG>([&](auto r) {
          constexpr int R = decltype(r)::value;
          if constexpr (R >= NFRAG * Q / H && R < NFRAG * (Q + 1) / H) read_frag(S0{}, r, nxt, 0);
        });
        static_for<NL>([&](auto l) {
          constexpr int L = decltype(l)::value;
          if constexpr (L >= NL * Q / H && L < NL * (Q + 1) / H) {
            if constexpr (L < LA::N) la.template issue_one<L>(cur, src_a2);
            else lb.template issue_one<L - LA::N>(cur + CA, src_b2);
          }
        });
        mfma(S1{}, std::integral_constant<int, Q + H>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    }
    __builtin_amdgcn_sched_barrier(0);
    colsum_step(S1{});
  }
  {
    const u32x4* cur = gemm_lds + ((nk - 1) & 1) * TILE_CHUNKS;
    static_for<NSTEP - 1>([&](auto st) {
      constexpr int ST = decltype(st)::value;
      stage(std::integral_constant<int, ST & 1>{}, cur, ST + 1);
    });
    frags_ready(S1{});
    static_for<NMFMA>([&](auto q) { mfma(S1{}, q); });
    colsum_step(S1{});
  }
  if constexpr (COLSUM) {
    // every row of a block holds the same sums: lanes 0..15 have row 0 of their column
    if (do_cs && lane < 16) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int64_t col = n0 + wn + j * 16 + lane;
        if (col < g.N) {
          const int64_t at = (int64_t)blockIdx.y * g.N + col;
          if (g.dtype_c == NBK_F32) ((float*)g.colsum)[at] = cs[j][0];
          else ((uint16_t*)g.colsum)[at] = nbk_f32_to_bf16(cs[j][0]);
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): no copy may land in a slab
  __syncthreads();  // the epilogue reuses the tile buffers as per-wave slabs
  gemm_epilogue<TM, TN, WN, true, EPI>(acc, g, m0, n0, wm, wn, c_off, wave, lane);
#undef GEMM_SRC_A
#undef GEMM_SRC_B
}

// ------------------------------------------------------------------- bf16, K <= 16
// C = alpha * A @ B (+ residual) with a contraction of at most 16 (the "up" product of a
// low-rank adapter): one MFMA deep, all memory traffic.  No K loop and no operand tiles in
// LDS: every lane reads its 8 k-values of an A row / a B column straight from global memory
// into the MFMA fragment, and the tile leaves through the shared epilogue.
template <bool B_KC, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_k_kernel(const GemmArgs g) {
  constexpr int TM = 2, TN = 2, WN = 64;
  int tm_i, tn_i;
  gemm_tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tm_i, tn_i);
  const int64_t m0 = (int64_t)tm_i * 128, n0 = (int64_t)tn_i * 128;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int li = lane & 31, kg = lane >> 5;
  const uint16_t* A = (const uint16_t*)g.A;
  const uint16_t* B = (const uint16_t*)g.B;
  // 8 k-values from k0 = 8 kg on, zero past K; rows / columns past the edge are clamped
  // (their products are never stored)
  auto frag8 = [&](const uint16_t* p, int64_t stride, bool vec) {
    const int k0 = 8 * kg;
    u32x4 u = {0u, 0u, 0u, 0u};
    if (vec && k0 + 8 <= g.K) {
      u = *(const u32x4*)(p + k0);
    } else {
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) h[e] = k0 + e < g.K ? p[(k0 + e) * stride] : 0u;
      u.x = h[0] | (h[1] << 16); u.y = h[2] | (h[3] << 16);
      u.z = h[4] | (h[5] << 16); u.w = h[6] | (h[7] << 16);
    }
    return *(const bf16x8*)&u;
  };
  // The two 32-row bands of a wave's tile are worked off one after the other (not unrolled), so
  // that one band's accumulators, residual pieces and epilogue registers are all a lane holds:
  // four workgroups then fit a CU, and the 1024 tiles of an 8192 x 2048 result are resident at
  // once instead of leaving a quarter of them to a second, mostly empty round.
  // (EPI 4: the residual is on its way before the operands are, one memory latency for both)
  bf16x8 fb[TN];
  uint4 pre[WN / 16];
  u32x4 b_piece = {0u, 0u, 0u, 0u};
  if (!B_KC && g.b_vec) {
    const int k = threadIdx.x >> 4;
    const int64_t col = n0 + (threadIdx.x & 15) * 8;
    if (k < g.K && col + 8 <= g.N) b_piece = *(const u32x4*)(B + (int64_t)k * g.b_rs + col);
  }
  if constexpr (EPI == 4) gemm_residual_prefetch<1, WN>(g, m0, n0, wm, wn, lane, pre);
  if (!B_KC && g.b_vec) {
    // B given as [K][N] with whole 16-byte pieces of its rows readable: the workgroup's 16 x 128
    // piece goes to LDS k-major (one coalesced 16-byte load per lane, zeros past K and N; it was
    // requested above, ahead of the first band's residual) and
    // the fragments come out through the transposing read -- instead of eight strided 2-byte
    // loads per lane and column block.
    char* bst = (char*)gemm_lds + 4 * 32 * (64 + 4) * sizeof(float);
    *(u32x4*)(bst + (threadIdx.x >> 4) * 256 + (threadIdx.x & 15) * 16) = b_piece;
    __syncthreads();
    const int p = lane & 15, q = lane >> 4;
    const char* tr = bst + (8 * (q >> 1) + (p >> 2)) * 256 + (wn + 16 * (q & 1) + 4 * (p & 3)) * 2;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const s16x4 lo = lds_read_tr(tr + j * 64), hi = lds_read_tr(tr + j * 64 + 4 * 256);
      const s16x8 u = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      fb[j] = *(const bf16x8*)&u;
    }
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int64_t col = n0 + wn + j * 32 + li;
      col = col < g.N ? col : g.N - 1;
      fb[j] = B_KC ? frag8(B + col * g.b_cs, 1, g.b_vec) : frag8(B + col, g.b_rs, false);
    }
  }
#pragma unroll 1
  for (int i = 0; i < TM; ++i) {
    if (EPI == 4 && i > 0) gemm_residual_prefetch<1, WN>(g, m0, n0, wm + i * 32, wn, lane, pre);
    int64_t row = m0 + wm + i * 32 + li;
    row = row < g.M ? row : g.M - 1;
    const bf16x8 fa = frag8(A + row * g.a_rs, 1, g.a_vec);
    f32x16 acc[1][TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[j], (f32x16)(0.f), 0, 0, 0);
    gemm_epilogue<1, TN, WN, true, EPI>(acc, g, m0, n0, wm + i * 32, wn, 0, wave, lane,
                                        EPI == 4 ? pre : nullptr);
  }
}

// ------------------------------------------------------------------- bf16, N <= 32
// C[M x N] = alpha * A[M x K] @ B[K x N] with at most 32 columns (the "down" product of a
// low-rank adapter and its transpose in the backward pass): A is read once and that is all the
// traffic there is.  One workgroup per 32 rows of A; its eight waves split K, each reads its
// part of the rows straight from global memory into MFMA fragments (one 32 x 32 accumulator
// tile; columns past N hold whatever the clamped or padded reads give and are never stored:
// a column of B only reaches the same column of C), and the eight partial tiles are added
// through LDS.
//   B_KC:  B given as [N][K] (K contiguous): fragments come straight from global memory too.
//   !B_KC: B given as [K][N] (N contiguous, N % 8 == 0): every wave stages its K range in LDS
//          k-major and reads fragments through the transposing read.
extern __shared__ __align__(16) u32x4 skinny_lds[];

constexpr int SKN_WAVES = 8;

template <bool B_KC>
__global__ __launch_bounds__(SKN_WAVES * 64) void gemm_skinny_n_kernel(const GemmArgs g,
                                                                        int pitch_chunks) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 31, kg = lane >> 5;
  const uint16_t* A = (const uint16_t*)g.A;
  const uint16_t* B = (const uint16_t*)g.B;
  const int64_t row0 = (int64_t)blockIdx.x * 32;
  // this wave's 64-wide K chunks
  const int chunks = (int)(g.K >> 6);
  const int per = (chunks + SKN_WAVES - 1) / SKN_WAVES;
  const int c_begin = wave * per;
  const int c_end = c_begin + per < chunks ? c_begin + per : chunks;
  float* red = (float*)skinny_lds;                                   // [waves][16 regs][64 lanes]
  char* stage = (char*)(skinny_lds + SKN_WAVES * 16 * 64 / 4);        // behind the reduction area
  const int pitch = pitch_chunks * 16;                                // bytes per staged k-row
  const char* tr_ptr = nullptr;
  const uint16_t* bp = nullptr;
  if (B_KC) {
    const int64_t col = li < g.N ? li : g.N - 1;
    bp = B + col * g.b_cs + 8 * kg;
  } else {
    // (rows [64 c_begin, 64 c_end) of B are staged below, behind the first requests for A)
    // lane p of group q = lane / 16: k-row 8 (q / 2) + p / 4, columns 16 (q % 2) + 4 (p % 4) .. + 4
    // (every lane of a group takes part in the exchange, also those that point at padding)
    const int p = lane & 15, q = lane >> 4;
    const int col0 = 16 * (q & 1) + 4 * (p & 3);
    tr_ptr = stage + (8 * (q >> 1) + (p >> 2)) * pitch + col0 * 2;
  }
  f32x16 acc = (f32x16)(0.f);
  // A streams through a 4 KB slab per wave (the bytes that later hold this wave's partial tile):
  // a 32-row x 64-k chunk arrives in four fully coalesced loads (eight lanes per 128-byte row
  // piece; fetching the 32-byte pieces of 32 rows that an MFMA fragment consists of straight
  // from memory runs at a quarter of that rate), is written to the slab swizzled and read back
  // as fragments.  The slab belongs to one wave, whose LDS accesses execute in order, so no
  // workgroup barrier is involved.  Three chunks are in flight in registers.
  u32x4* slab = (u32x4*)(red + wave * 16 * 64);
  const int lrow = lane >> 3, lch = lane & 7;
  const uint16_t* arow_p[4];
  int w_at[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int r = p * 8 + lrow;
    const int64_t gr = row0 + r < g.M ? row0 + r : g.M - 1;
    arow_p[p] = A + gr * g.a_rs + 8 * lch;
    w_at[p] = r * 8 + (lch ^ dl_kc_xor<false>(r));
  }
  const int r_at = li * 8, r_x = dl_kc_xor<false>(li);
  constexpr int AHEAD = 3;
  u32x4 an[AHEAD][4], bn[AHEAD][4];
  auto fetch = [&](auto slot, int c) {
    constexpr int J = decltype(slot)::value;
    const int64_t k0 = (int64_t)c * 64;
#pragma unroll
    for (int p = 0; p < 4; ++p) an[J][p] = *(const u32x4*)(arow_p[p] + k0);
    if (B_KC) {
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) bn[J][s4] = *(const u32x4*)(bp + k0 + 16 * s4);
    }
  };
  static_for<AHEAD>([&](auto j) {
    if (c_begin + decltype(j)::value < c_end) fetch(j, c_begin + decltype(j)::value);
  });
  if (!B_KC) {
    // stage rows [64 c_begin, 64 c_end) of B; a k-row holds N / 8 chunks (pitch_chunks >= that);
    // four pieces per lane are on their way at a time
    const int nch = (int)(g.N >> 3);
    const int total = (c_end - c_begin) * 64 * nch;
    for (int t0 = 0; t0 < total; t0 += 256) {
      u32x4 piece[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * 64 + lane;
        const int k = t / nch, c = t - k * nch;
        const int64_t gk = (int64_t)c_begin * 64 + k;
        if (t < total) piece[u] = *(const u32x4*)(B + gk * g.b_rs + c * 8);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * 64 + lane;
        const int k = t / nch, c = t - k * nch;
        const int64_t gk = (int64_t)c_begin * 64 + k;
        if (t < total) *(u32x4*)(stage + (size_t)gk * pitch + c * 16) = piece[u];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  for (int c = c_begin; c < c_end; c += AHEAD) {
    static_for<AHEAD>([&](auto j) {
      constexpr int J = decltype(j)::value;
      const int cc = c + J;
      if (cc < c_end) {  // (uniform over the wave)
        const int64_t k0 = (int64_t)cc * 64;
#pragma unroll
        for (int p = 0; p < 4; ++p) slab[w_at[p]] = an[J][p];
        bf16x8 fa[4], fb[4];
        if (B_KC) {
#pragma unroll
          for (int s4 = 0; s4 < 4; ++s4) fb[s4] = *(const bf16x8*)&bn[J][s4];
        } else {
#pragma unroll
          for (int s4 = 0; s4 < 4; ++s4) {
            const char* a0 = tr_ptr + (k0 + 16 * s4) * pitch;
            const s16x4 lo = lds_read_tr(a0), hi = lds_read_tr(a0 + 4 * pitch);
            const s16x8 u = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            fb[s4] = *(const bf16x8*)&u;
          }
        }
        if (cc + AHEAD < c_end) fetch(j, cc + AHEAD);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
          const u32x4 u = slab[r_at + ((2 * s4 + kg) ^ r_x)];
          fa[s4] = *(const bf16x8*)&u;
        }
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[s4], fb[s4], acc, 0, 0, 0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
    });
  }
  // (the slab is this wave's part of the reduction area: its last fragments are in registers)
#pragma unroll
  for (int r = 0; r < 16; ++r) red[(wave * 16 + r) * 64 + lane] = acc[r];
  __syncthreads();
  if (wave != 0) return;
  const int64_t col = li;
  if (col >= g.N) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SKN_WAVES; ++w) v += red[(w * 16 + r) * 64 + lane];
    const int64_t row = row0 + 8 * (r >> 2) + 4 * kg + (r & 3);
    if (row < g.M) nbk_store_from_f32(g.C, row * g.ldc + col, g.dtype_c, v * g.alpha);
  }
}

// ---------------------------------------------------------------------------- fp32
// 128 x 128 x 16 tile, LDS k-major ([k][rows], rows padded by 4 floats).
template <bool A_KC, bool B_KC, bool B_Q = false>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmArgs g) {
  constexpr int BM = 128, BN = 128, BK = 16, LD = 128 + 4;
  __shared__ float As[2][BK][LD];
  __shared__ float Bs[2][BK][LD];
  __shared__ float nf4_table[B_Q ? 16 : 1];  // B_Q: B holds NF4 codes, g.b_scales the block scales
  if (B_Q) {
    if (threadIdx.x < 16) nf4_table[threadIdx.x] = nbk_nf4_levels[threadIdx.x];
    __syncthreads();
  }
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
  // B from NF4 codes: the same eight elements per lane, dequantised
  auto load_b = [&](int64_t k0, float* r) {
    if constexpr (B_Q) {
      if (B_KC) {
        const int row = tid >> 1, kk = (tid & 1) * 8;
        const int64_t gr = n0 + row, gk = k0 + kk;
        nf4_load8((const uint8_t*)g.B, g.b_scales, g.b_block, nf4_table, gr * g.b_cs + gk,
                  gr < g.N ? g.K - gk : 0, r);
      } else {
        const int kk = tid >> 4, rr = (tid & 15) * 8;
        const int64_t gk = k0 + kk, gr = n0 + rr;
        nf4_load8((const uint8_t*)g.B, g.b_scales, g.b_block, nf4_table, gk * g.b_rs + gr,
                  gk < g.K ? g.N - gr : 0, r);
      }
    } else {
      load_tile(B, g.b_cs, g.b_rs, n0, g.N, k0, B_KC, g.b_vec, r);
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
  load_b(0, rb);
  store_tile(As[0], A_KC, ra);
  store_tile(Bs[0], B_KC, rb);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      load_tile(A, g.a_rs, g.a_cs, m0, g.M, (kt + 1) * BK, A_KC, g.a_vec, ra);
      load_b((kt + 1) * BK, rb);
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
        const int64_t idx = c_off + row * g.ldc + col;
        float v, dv;
        if (g.C2) {
          gemm_act_pair<false>(acc[i][j][r] * g.alpha + bv, g.act, v, dv);
          ((float*)g.C2)[idx] = dv;
        } else {
          v = gemm_act(acc[i][j][r] * g.alpha + bv, g.act);
        }
        if (g.residual) v = g.res_mul ? v * ((const float*)g.residual)[idx] : v + ((const float*)g.residual)[idx];
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
    const int64_t idx = c_off + row * g.ldc + col;
    const float x = v * g.alpha + (g.bias ? ((const float*)g.bias)[col] : 0.f);
    if (g.C2) {
      float dv;
      gemm_act_pair<false>(x, g.act, v, dv);
      ((float*)g.C2)[idx] = dv;
    } else {
      v = gemm_act(x, g.act);
    }
    if (g.residual) v = g.res_mul ? v * ((const float*)g.residual)[idx] : v + ((const float*)g.residual)[idx];
    C[idx] = v;
  }
}

// ------------------------------------------------------------------------- dispatch
template <int BM, int BN, int NW = 4>
static int launch_bf16(const GemmArgs& a, bool akc, bool bkc, int64_t batch, hipStream_t st) {
  GemmArgs g = a;
  g.tiles_m = (int)((a.M + BM - 1) / BM);
  g.tiles_n = (int)((a.N + BN - 1) / BN);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
  const size_t pipe_of[2][2] = {
      {2 * (size_t)(TileGeom<BM, false>::CHUNKS + TileGeom<BN, false>::CHUNKS) * 16,
       2 * (size_t)(TileGeom<BM, false>::CHUNKS + TileGeom<BN, true>::CHUNKS) * 16},
      {2 * (size_t)(TileGeom<BM, true>::CHUNKS + TileGeom<BN, false>::CHUNKS) * 16,
       2 * (size_t)(TileGeom<BM, true>::CHUNKS + TileGeom<BN, true>::CHUNKS) * 16}};
  const size_t pipe = pipe_of[akc][bkc];
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
    auto kern = gemm_bf16_kernel<BM, BN, AK, BK_, EP, NW>;                              \
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

template <int BM, int BN, int NW, int KSS, bool MI16>
static int launch_bf16_dl(const GemmArgs& a, bool akc, bool bkc, int64_t batch, hipStream_t st) {
  GemmArgs g = a;
  g.tiles_m = (int)((a.M + BM - 1) / BM);
  g.tiles_n = (int)((a.N + BN - 1) / BN);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
  const size_t pipe = 2 * (size_t)(BM + BN) * 8 * 16;
  const size_t slabs = NW * 32 * (size_t)(BN / (NW / 2) + 4) * sizeof(float);
  const size_t lds = pipe > slabs ? pipe : slabs;
  const int epi = (a.residual != nullptr || a.act != NBK_ACT_NONE) ? 2 : (a.bias != nullptr ? 1 : 0);
#define NBK_LAUNCH_DL(AK, BK_, EP)                                                            \
  do {                                                                                        \
    auto kern = gemm_bf16_dl_kernel<BM, BN, AK, BK_, EP, NW, KSS, MI16>;                      \
    static bool attr_set = false; /* idempotent, so a race only repeats the call */          \
    if (!attr_set) {                                                                          \
      NBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                  (int)lds));                                                 \
      attr_set = true;                                                                        \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, st, g);                                \
  } while (0)
#define NBK_LAUNCH_DL2(AK, BK_)                                                               \
  do {                                                                                        \
    if (epi == 2) NBK_LAUNCH_DL(AK, BK_, 2);                                                  \
    else if (epi == 1) NBK_LAUNCH_DL(AK, BK_, 1);                                             \
    else NBK_LAUNCH_DL(AK, BK_, 0);                                                           \
  } while (0)
  if (akc && bkc) NBK_LAUNCH_DL2(true, true);
  else if (akc && !bkc) NBK_LAUNCH_DL2(true, false);
  else if (!akc && bkc) NBK_LAUNCH_DL2(false, true);
  else NBK_LAUNCH_DL2(false, false);
#undef NBK_LAUNCH_DL
#undef NBK_LAUNCH_DL2
  return nbk_check_launch("gemm_bf16_dl_kernel");
}

// The same launch with the column sums of B as a second result (both operands row-contiguous,
// no epilogue: the weight gradient x^T dy beside the bias gradient).
template <int BM, int BN, int NW>
static int launch_bf16_dl_colsum(const GemmArgs& a, int64_t batch, hipStream_t st) {
  GemmArgs g = a;
  g.tiles_m = (int)((a.M + BM - 1) / BM);
  g.tiles_n = (int)((a.N + BN - 1) / BN);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
  const size_t pipe = 2 * (size_t)(BM + BN) * 8 * 16;
  const size_t slabs = NW * 32 * (size_t)(BN / (NW / 2) + 4) * sizeof(float);
  const size_t lds = pipe > slabs ? pipe : slabs;
  auto kern = gemm_bf16_dl_kernel<BM, BN, false, false, 0, NW, 1, true, true>;
  static bool attr_set = false; /* idempotent, so a race only repeats the call */
  if (!attr_set) {
    NBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, st, g);
  return nbk_check_launch("gemm_bf16_dl_kernel (column sums)");
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
  GemmArgs a = {};
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
  // A result beyond the 256 MiB last-level cache does not survive until its consumer runs: it is
  // streamed (non-temporal stores), which leaves the cache to the operands.  Smaller results are
  // stored normally: measured inside the decoder step, streaming them takes as much from the
  // kernels that read them next as it gives the product.
  a.c_stream = d->M * d->N * d->batch * (d->dtype_c == NBK_F32 ? 4 : 2) > (256ll << 20) ? 1 : 0;
  NBK_REQUIRE(d->aux_op == NBK_AUX_NONE || d->aux_op == NBK_AUX_ACT_GRAD, "gemm: aux_op %d", d->aux_op);
  NBK_REQUIRE((d->aux_op == NBK_AUX_NONE) == (d->C_aux == nullptr),
              "gemm: C_aux and aux_op go together");
  NBK_REQUIRE(d->aux_op == NBK_AUX_NONE || (d->act != NBK_ACT_NONE && d->residual == nullptr),
              "gemm: the derivative of the activation needs an activation and no residual");
  a.C2 = d->C_aux;
  NBK_REQUIRE(d->residual_op == NBK_RES_ADD || d->residual_op == NBK_RES_MUL,
              "gemm: residual_op %d", d->residual_op);
  a.res_mul = d->residual_op == NBK_RES_MUL;
  a.colsum = d->colsum;
  // K-contiguous when the stride along k is 1 (ties: a single row / column counts as K-contiguous)
  const bool akc = d->a_cs == 1;
  const bool bkc = d->b_rs == 1;
  NBK_REQUIRE(d->n_terms >= 0 && d->n_terms <= NBK_GEMM_MAX_TERMS, "gemm: n_terms %d", d->n_terms);
  const bool tail = d->n_terms > 0;
  if (tail) {
    NBK_REQUIRE(d->dtype_ab == NBK_BF16 && d->batch == 1 && d->colsum == nullptr,
                "gemm: more operand pairs go with one bf16 product without column sums");
    for (int i = 0; i < d->n_terms; ++i) {
      const nbk_gemm_term& t = d->term[i];
      NBK_REQUIRE(t.A && t.B && t.K > 0, "gemm: term %d is empty", i);
      NBK_REQUIRE(t.a_rs == 1 || t.a_cs == 1, "gemm: A of term %d needs a unit stride", i);
      NBK_REQUIRE(t.b_rs == 1 || t.b_cs == 1, "gemm: B of term %d needs a unit stride", i);
    }
  }
  const int esz = d->dtype_ab == NBK_F32 ? 4 : 2;
  auto vec_ok = [&](const void* p, int64_t other_stride, int64_t bs, int64_t bs2) {
    const int64_t q = 16 / esz;
    return ((uintptr_t)p % 16 == 0) && (other_stride % q == 0) && (bs % q == 0) && (bs2 % q == 0);
  };
  a.a_vec = vec_ok(d->A, akc ? d->a_rs : d->a_cs, d->a_bs, a.a_bs2);
  a.b_vec = vec_ok(d->B, bkc ? d->b_cs : d->b_rs, d->b_bs, a.b_bs2);
  // (checked before any kernel is chosen: no path may take the product and drop the sums)
  NBK_REQUIRE(d->colsum == nullptr || (d->dtype_ab == NBK_BF16 && !akc && !bkc),
              "gemm: column sums need bf16 operands that are both row-contiguous (a_rs == b_cs == 1)");
  if (!tail && d->dtype_ab == NBK_BF16 && d->N <= 32 && d->M >= 1024 && d->K >= 256 && d->K % 64 == 0 &&
      akc && a.a_vec && d->batch == 1 && d->bias == nullptr && d->residual == nullptr &&
      d->act == NBK_ACT_NONE && (bkc ? (bool)a.b_vec : (d->b_cs == 1 && d->N % 8 == 0 && a.b_vec))) {
    // 32 rows per workgroup, K split over its eight waves
    const int pitch_chunks = d->N <= 16 ? 2 : 4;
    const size_t red = SKN_WAVES * 16 * 64 * sizeof(float);
    const size_t stage = bkc ? 0 : (size_t)d->K * pitch_chunks * 16 + 64;
    if (red + stage <= 160 * 1024 - 512 && (d->M + 31) / 32 <= 0x7fffffff) {
      dim3 grid((unsigned)((d->M + 31) / 32));
      if (bkc) {
        hipLaunchKernelGGL((gemm_skinny_n_kernel<true>), grid, dim3(SKN_WAVES * 64), red, st, a,
                           pitch_chunks);
      } else {
        static bool attr_set = false; /* idempotent, so a race only repeats the call */
        if (!attr_set) {
          NBK_HIP(hipFuncSetAttribute((const void*)gemm_skinny_n_kernel<false>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
          attr_set = true;
        }
        hipLaunchKernelGGL((gemm_skinny_n_kernel<false>), grid, dim3(SKN_WAVES * 64), red + stage, st, a,
                           pitch_chunks);
      }
      return nbk_check_launch("gemm_skinny_n_kernel");
    }
  }
  if (!tail && d->dtype_ab == NBK_BF16 && d->K <= 16 && akc && d->batch == 1 && d->N % 8 == 0 &&
      d->ldc % 8 == 0 && ((uintptr_t)d->C & 15) == 0 && ((uintptr_t)d->residual & 15) == 0 &&
      (d->K == 16 ? a.a_vec : d->K == 8 && (d->a_rs % 8 == 0) && ((uintptr_t)d->A & 15) == 0)) {
    // (the vector path reads whole 16-byte pieces of A rows: K = 16 or 8)
    a.a_vec = 1;
    // (K-contiguous B: whole fragments from memory; row-contiguous B: whole row pieces into LDS)
    a.b_vec = bkc ? (d->K == 16 ? a.b_vec : (d->b_cs % 8 == 0) && ((uintptr_t)d->B & 15) == 0)
                  : (d->b_cs == 1 && d->b_rs % 8 == 0 && ((uintptr_t)d->B & 15) == 0);
    a.tiles_m = (int)((d->M + 127) / 128);
    a.tiles_n = (int)((d->N + 127) / 128);
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n));
    const size_t lds = 4 * 32 * (size_t)(64 + 4) * sizeof(float) + 16 * 256;  // slabs + a B piece
    // 0 plain; 3 a bias and / or an added residual (the adapter's update on top of the base
    // product: all memory traffic, so the lean epilogue that keeps four waves per SIMD); 2 the rest
    const bool any = a.bias != nullptr || a.residual != nullptr || a.act != NBK_ACT_NONE;
    // (4: the same with the residual requested before the operands -- bf16 results only)
    const int epi = !any ? 0 : ((a.act == NBK_ACT_NONE && a.C2 == nullptr && !a.res_mul)
                                    ? (a.residual != nullptr && d->dtype_c == NBK_BF16 ? 4 : 3) : 2);
#define NBK_LAUNCH_SKK(BK_)                                                                        \
  do {                                                                                             \
    if (epi == 0) hipLaunchKernelGGL((gemm_skinny_k_kernel<BK_, 0>), grid, dim3(256), lds, st, a); \
    else if (epi == 4) hipLaunchKernelGGL((gemm_skinny_k_kernel<BK_, 4>), grid, dim3(256), lds, st, a); \
    else if (epi == 3) hipLaunchKernelGGL((gemm_skinny_k_kernel<BK_, 3>), grid, dim3(256), lds, st, a); \
    else hipLaunchKernelGGL((gemm_skinny_k_kernel<BK_, 2>), grid, dim3(256), lds, st, a);         \
  } while (0)
    if (bkc) NBK_LAUNCH_SKK(true);
    else NBK_LAUNCH_SKK(false);
#undef NBK_LAUNCH_SKK
    return nbk_check_launch("gemm_skinny_k_kernel");
  }
  if (d->dtype_ab == NBK_BF16) {
    // (the direct kernel keeps per-lane byte offsets within a tile in 32 bits: 256 rows or
    // 64 k-rows times the stride)
    const int64_t a_stride = akc ? d->a_rs : d->a_cs, b_stride = bkc ? d->b_cs : d->b_rs;
    const bool fast = a.a_vec && a.b_vec && (d->K % 64 == 0) && (akc || d->M % 8 == 0) &&
                      (bkc || d->N % 8 == 0) && d->M >= 8 && d->N >= 8 &&
                      a_stride >= 0 && b_stride >= 0 && a_stride < (1 << 22) && b_stride < (1 << 22);
    if (tail) {
      // In the accumulator of the direct-to-LDS kernels when every pair is laid out like A and B
      // and 16-byte aligned: shallow pairs (one K tile each, at most two) and deep pairs with
      // exactly the strides of A and B (at most two); otherwise one product after the other,
      // each adding itself to the result so far (plain products only: an epilogue would have to
      // wait for the last one).
      bool inside = fast && d->M >= 128 && d->N >= 128;
      a.n_shallow = 0;
      a.n_deep = 0;
      for (int i = 0; inside && i < d->n_terms; ++i) {
        const nbk_gemm_term& t = d->term[i];
        const bool tkc_a = t.a_cs == 1, tkc_b = t.b_rs == 1;
        const int64_t sa = tkc_a ? t.a_rs : t.a_cs, sb = tkc_b ? t.b_cs : t.b_rs;
        if (tkc_a != akc || tkc_b != bkc || ((uintptr_t)t.A & 15) || ((uintptr_t)t.B & 15) || sa % 8 ||
            sb % 8 || sa < 0 || sb < 0 || sa >= (1 << 22) || sb >= (1 << 22)) {
          inside = false;
        } else if (t.K <= 64 && t.K % 8 == 0 && a.n_shallow < 2) {
          GemmArgs::Shallow& sh = a.shallow[a.n_shallow++];
          sh.A = t.A; sh.B = t.B; sh.K = t.K;
          sh.a_rs = t.a_rs; sh.a_cs = t.a_cs; sh.b_rs = t.b_rs; sh.b_cs = t.b_cs;
        } else if (t.K % 64 == 0 && a.n_deep < 2 && t.a_rs == d->a_rs && t.a_cs == d->a_cs &&
                   t.b_rs == d->b_rs && t.b_cs == d->b_cs) {
          GemmArgs::Deep& dp = a.deep[a.n_deep++];
          dp.A = t.A; dp.B = t.B; dp.K = t.K;
        } else {
          inside = false;
        }
      }
      if (!inside) {
        NBK_REQUIRE(d->bias == nullptr && d->residual == nullptr && d->act == NBK_ACT_NONE &&
                        d->C_aux == nullptr && d->alpha == 1.f,
                    "gemm: operand pairs outside the direct kernels' conditions go with a plain "
                    "product only");
        nbk_gemm_desc one = *d;
        one.n_terms = 0;
        int rc = nbk_gemm(&one, stream);
        for (int i = 0; rc == NBK_OK && i < d->n_terms; ++i) {
          const nbk_gemm_term& t = d->term[i];
          one.A = t.A; one.B = t.B; one.K = t.K;
          one.a_rs = t.a_rs; one.a_cs = t.a_cs; one.b_rs = t.b_rs; one.b_cs = t.b_cs;
          one.residual = d->C;  // (every kernel reads a residual element in the lane that writes it)
          one.residual_op = NBK_RES_ADD;
          rc = nbk_gemm(&one, stream);
        }
        return rc;
      }
    }
    if (d->colsum != nullptr) {
      NBK_REQUIRE(fast && !akc && !bkc && d->bias == nullptr &&
                      d->residual == nullptr && d->act == NBK_ACT_NONE && d->alpha == 1.f,
                  "gemm: column sums go with a plain bf16 product of two row-contiguous, 16-byte "
                  "aligned operands (K %% 64 == 0, M %% 8 == 0, N %% 8 == 0)");
      return launch_bf16_dl_colsum<128, 128, 4>(a, d->batch, st);
    }
    if (!fast) return launch_bf16<128, 128>(a, akc, bkc, d->batch, st);
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
      return launch_bf16_dl<256, 256, 8, 1, true>(a, akc, bkc, d->batch, st);
    // (a 256 x 128 tile was measured and is no faster than 128 x 128 on mid-sized problems:
    // with one workgroup per CU a short K loop is bound by load latency, and two co-resident
    // 128 x 128 workgroups hide it better)
    // (the 16 x 16 x 32 instruction is 3-8 % faster on every shape and layout of the big tile; on
    // this one it gains 4-9 % with a row-contiguous operand and loses 5-10 % with two K-contiguous)
    return !(akc && bkc) ? launch_bf16_dl<128, 128, 4, 1, true>(a, akc, bkc, d->batch, st)
                         : launch_bf16_dl<128, 128, 4, 1, false>(a, akc, bkc, d->batch, st);
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

// ------------------------------------------------------------------ NF4-coded weights
extern "C" int nbk_gemm_nf4(const nbk_gemm_nf4_desc* d, void* stream) {
  NBK_REQUIRE(d != nullptr, "gemm_nf4: null descriptor");
  NBK_REQUIRE(d->A && d->codes && d->scales && d->C, "gemm_nf4: null pointer");
  NBK_REQUIRE(d->M > 0 && d->w_rows > 0 && d->w_cols > 0, "gemm_nf4: empty problem");
  NBK_REQUIRE(d->dtype == NBK_BF16 || d->dtype == NBK_F32, "gemm_nf4: dtype %d", d->dtype);
  NBK_REQUIRE(d->block > 0 && d->block % 8 == 0 && d->w_cols % 8 == 0,
              "gemm_nf4: the block length (%d) and the weight's width (%lld) must be multiples of 8",
              d->block, (long long)d->w_cols);
  NBK_REQUIRE(((uintptr_t)d->codes & 7) == 0, "gemm_nf4: codes must be 8-byte aligned");
  // C = A @ W (K = rows of W, N = its columns) or A @ W^T (K = columns of W, N = its rows)
  const int64_t K = d->transpose_w ? d->w_cols : d->w_rows;
  const int64_t N = d->transpose_w ? d->w_rows : d->w_cols;
  NBK_REQUIRE(d->lda >= K && d->ldc >= N, "gemm_nf4: leading dimension too small");
  GemmArgs a = {};
  a.A = d->A; a.B = d->codes; a.C = d->C;
  a.M = d->M; a.N = N; a.K = K;
  a.a_rs = d->lda; a.a_cs = 1;
  // the element (k, n) of the B operand is code k * b_rs + n * b_cs of the flattened weight
  a.b_rs = d->transpose_w ? 1 : d->w_cols;
  a.b_cs = d->transpose_w ? d->w_cols : 1;
  a.ldc = d->ldc; a.batch_inner = 1;
  a.dtype_c = d->dtype; a.act = NBK_ACT_NONE; a.alpha = d->alpha;
  a.b_scales = (const float*)d->scales; a.b_block = d->block;
  a.a_vec = ((uintptr_t)d->A % 16 == 0) && (d->lda % (d->dtype == NBK_F32 ? 4 : 8) == 0);
  a.b_vec = 0;
  a.tiles_m = (int)((a.M + 127) / 128);
  a.tiles_n = (int)((a.N + 127) / 128);
  NBK_REQUIRE((int64_t)a.tiles_m * a.tiles_n <= 0x7fffffffLL, "gemm_nf4: launch too large");
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), 1);
  hipStream_t st = (hipStream_t)stream;
  const bool bkc = d->transpose_w != 0;
  if (d->dtype == NBK_F32) {
    if (bkc) hipLaunchKernelGGL((gemm_f32_kernel<true, true, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_f32_kernel<true, false, true>), grid, dim3(256), 0, st, a);
    return nbk_check_launch("gemm_f32_kernel (nf4)");
  }
  const size_t pipe = 2 * (size_t)(TileGeom<128, true>::CHUNKS +
                                   (bkc ? TileGeom<128, true>::CHUNKS : TileGeom<128, false>::CHUNKS)) * 16;
  const size_t slabs = 4 * 32 * (size_t)(64 + 4) * sizeof(float);
  const size_t lds = pipe > slabs ? pipe : slabs;
#define NBK_LAUNCH_NF4(BK_)                                                                   \
  do {                                                                                        \
    auto kern = gemm_bf16_kernel<128, 128, true, BK_, false, 4, true>;                        \
    static bool attr_set = false; /* idempotent, so a race only repeats the call */          \
    if (!attr_set) {                                                                          \
      NBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                  (int)lds));                                                 \
      attr_set = true;                                                                        \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, a);                                    \
  } while (0)
  if (bkc) NBK_LAUNCH_NF4(true);
  else NBK_LAUNCH_NF4(false);
#undef NBK_LAUNCH_NF4
  return nbk_check_launch("gemm_bf16_kernel (nf4)");
}
