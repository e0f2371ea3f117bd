// Fused scaled-dot-product attention for gfx950, bf16 in / fp32 accumulate.
//
//   forward : O = softmax(mask(Q K^T * scale)) V,  LSE = log-sum-exp of every score row
//   backward: dQ, dK, dV from (Q, K, V, O, LSE, dO) with the probabilities recomputed
//
// The S x S score matrix never reaches memory.  Tensors are [B, S, H, hd] in any
// strides with a unit stride along hd (heads are read in place), hd = 64 or 128,
// S a multiple of 128.
//
// Register layouts of v_mfma_f32_32x32x16_bf16 (lane l, li = l % 32, h = l / 32):
//   A: lane holds A[row li][k = 8h .. 8h+7]      B: lane holds B[k = 8h .. 8h+7][col li]
//   D: register r holds D[row (r/4)*8 + 4h + r%4][col li]
// All three kernels compute the scores TRANSPOSED with respect to the tensor the wave
// owns in registers: the owned rows (queries in the forward and dQ kernels, keys in
// the dK/dV kernel) sit on the MFMA's column side, one per lane, so that
//   * a softmax row lives in one lane pair (li, li + 32): row max and sum are
//     register reductions plus one exchange between the two halves;
//   * the probabilities (or dS) leave the first MFMA in exactly the layout the second
//     MFMA wants for its B operand: registers 8t .. 8t+7 of a 32-row tile are k-slots
//     8h .. 8h+7 of the t-th 16-wide k-step, if slot 8h + i stands for row
//     16t + 4h + i (i < 4) and 16t + 8 + 4h + (i - 4) (i >= 4).  The A operand of that
//     second MFMA is read from a transposed LDS tile with the same permutation: two
//     8-byte reads at columns 16t + 4h and 16t + 8 + 4h.
// LDS tiles:
//   row-major  [64 rows][hd]      16-byte chunks XOR-swizzled by the row so that the 16-byte
//                                  fragment reads of 16 consecutive rows hit distinct banks
//   transposed [hd rows][64 cols]  row pitch 68 elements: the 8-byte reads of 32
//                                  consecutive rows fall on distinct banks per half
// The forward kernel, the dQ kernel and the dK/dV kernel for 128-wide heads keep no transposed
// tiles: they take the A operand of the second MFMA out of the row-major tile with
// ds_read_b64_tr_b16 (the swizzle at_sw serves both kinds of read).  The forward kernel's tiles
// go from memory into LDS directly (global_load_lds: no staging registers, which lets four
// waves per SIMD run with 64-wide heads).
#include "nbk_common.h"
#include <mutex>

#include <utility>

typedef __bf16 at_bf16x8 __attribute__((ext_vector_type(8)));
typedef float at_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t at_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t at_u32x2 __attribute__((ext_vector_type(2)));

template <typename F, int... I>
__device__ __forceinline__ void at_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void at_static_for(F&& f) {
  at_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

struct AttnTensor {
  const uint16_t* p;
  int64_t sb, ss, sh;  // element strides of batch, sequence, head; hd is contiguous
};

struct AttnArgs {
  AttnTensor q, k, v, o, dout, dq, dk, dv;
  AttnTensor o_lo;  // optional: what rounding O to bf16 cut off, itself as bf16 (p == nullptr: none)
  float* lse;    // [B, H, S]
  float* delta;  // [B, H, S]: rowsum(dO * O), backward only
  int32_t B, H, S;
  int32_t causal;
  float scale;
};

constexpr int AT_TP = 68;  // pitch (elements) of a transposed tile row

__device__ __forceinline__ float at_neg_big() { return -1.0e30f; }

typedef float at_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 at_bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t at_pack2(float a, float b) {
  const at_f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, at_bf16x2));
}

// 64 x HD tile -> LDS, row-major swizzled.  256 lanes, 16 bytes each per pass.
template <int HD>
struct AtRowTile {
  static constexpr int NCH = HD / 8;             // 16-byte chunks per row
  static constexpr int NREG = 64 * NCH / 256;    // passes (2 for hd 64, 4 for hd 128)
  at_u32x4 reg[NREG];
  // Chunk swizzle of a row: the LDS has 64 banks, so one ds_read_b128 serves 16 lanes per
  // cycle; the 16 rows they read must land on 16 distinct 16-byte slots of the 256-byte window.
  static __device__ __forceinline__ int sw(int row) {
    if constexpr (NCH == 8) return (row & 7) ^ ((row >> 3) & 1);  // 128-byte rows: two per window
    else return row & 15;
  }
  __device__ __forceinline__ void load(const uint16_t* base, int64_t row_stride, int row0) {
#pragma unroll
    for (int s = 0; s < NREG; ++s) {
      const int t = threadIdx.x + s * 256;
      const int row = t / NCH, c = t % NCH;
      reg[s] = *(const at_u32x4*)(base + (int64_t)(row0 + row) * row_stride + c * 8);
    }
  }
  __device__ __forceinline__ void store(at_u32x4* lds) const {
#pragma unroll
    for (int s = 0; s < NREG; ++s) {
      const int t = threadIdx.x + s * 256;
      const int row = t / NCH, c = t % NCH;
      lds[row * NCH + (c ^ sw(row))] = reg[s];
    }
  }
  // fragment: 8 consecutive k (chunk) of `row`
  static __device__ __forceinline__ at_bf16x8 frag(const at_u32x4* lds, int row, int chunk) {
    const at_u32x4 u = lds[row * NCH + (chunk ^ sw(row))];
    return __builtin_bit_cast(at_bf16x8, u);
  }
};

// 64 x HD tile -> LDS transposed ([HD][64], pitch AT_TP).  Every lane transposes one block of
// KPB rows x 8 columns (KPB = 2 for hd 64, 4 for hd 128, so that 256 lanes cover the tile):
// KPB loads of 16 bytes in, 8 stores of KPB elements out.  Lane -> block: four neighbouring
// lanes read 64 contiguous bytes of one row, and the stores of a wave spread over all banks.
template <int HD>
struct AtTransTile {
  static constexpr int KPB = HD / 32;
  static constexpr int NKB = 64 / KPB;  // row blocks
  at_u32x4 reg[KPB];
  static __device__ __forceinline__ void block_of(int& kb, int& db) {
    const int t = threadIdx.x;
    kb = (t >> 2) % NKB;
    db = (t & 3) + 4 * (t / (4 * NKB));
  }
  __device__ __forceinline__ void load(const uint16_t* base, int64_t row_stride, int row0) {
    int kb, db;
    block_of(kb, db);
#pragma unroll
    for (int r = 0; r < KPB; ++r)
      reg[r] = *(const at_u32x4*)(base + (int64_t)(row0 + kb * KPB + r) * row_stride + db * 8);
  }
  __device__ __forceinline__ void store(uint16_t* lds) const {
    int kb, db;
    block_of(kb, db);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // column j of the block: element j of each of the KPB rows
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      uint16_t* dst = lds + (db * 8 + j) * AT_TP + kb * KPB;
      if constexpr (KPB == 2) {
        *(uint32_t*)dst = __builtin_amdgcn_perm(reg[1][j >> 1], reg[0][j >> 1], sel);
      } else {
        at_u32x2 w;
        w.x = __builtin_amdgcn_perm(reg[1][j >> 1], reg[0][j >> 1], sel);
        w.y = __builtin_amdgcn_perm(reg[3][j >> 1], reg[2][j >> 1], sel);
        *(at_u32x2*)dst = w;
      }
    }
  }
  // A fragment of the second MFMA: row d, k-slots of the t-th 16-wide step of 32-row tile kt2
  static __device__ __forceinline__ at_bf16x8 frag(const uint16_t* lds, int d, int kt2, int t, int h) {
    const uint16_t* p = lds + d * AT_TP + kt2 * 32 + t * 16 + 4 * h;
    const at_u32x2 a = *(const at_u32x2*)p;
    const at_u32x2 b = *(const at_u32x2*)(p + 8);
    const at_u32x4 u = {a.x, a.y, b.x, b.y};
    return __builtin_bit_cast(at_bf16x8, u);
  }
};

// B fragment of the second MFMA from the registers of a transposed score tile
__device__ __forceinline__ at_bf16x8 at_regs_frag(const at_f32x16& s, int t) {
  at_u32x4 u;
  if (t == 0) {
    u.x = at_pack2(s[0], s[1]); u.y = at_pack2(s[2], s[3]);
    u.z = at_pack2(s[4], s[5]); u.w = at_pack2(s[6], s[7]);
  } else {
    u.x = at_pack2(s[8], s[9]); u.y = at_pack2(s[10], s[11]);
    u.z = at_pack2(s[12], s[13]); u.w = at_pack2(s[14], s[15]);
  }
  return __builtin_bit_cast(at_bf16x8, u);
}

__device__ __forceinline__ float at_xhalf(float v) { return __shfl_xor(v, 32, 64); }

// acc + the sum of eight packed bf16 values
__device__ __forceinline__ float at_sum_bf16x8(at_bf16x8 v, float acc) {
  // (written as the instruction itself: __builtin_amdgcn_fdot2_f32_bf16 in an unrolled loop over
  // the elements of a vector came out of hipcc 7.2 as four reads of the first element)
  const at_u32x4 u = __builtin_bit_cast(at_u32x4, v);
  const uint32_t ones = 0x3f803f80u;  // two bf16 ones
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = u[i];
    asm("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(acc) : "v"(ones), "v"(w));
  }
  return acc;
}

// Swizzle of the [rows][16 chunks] tiles that are read both by rows and through the transposing
// LDS read (the kernels for 128-wide heads; the layout is described at the dK / dV kernel).
template <int NCH>
__device__ __forceinline__ int at_sw(int row) {
  if constexpr (NCH == 16) return ((row & 3) << 2) | ((row >> 2) & 3);
  // 128-byte rows, two per 256-byte window: the row's parity picks the half, bits 1..3 the slot
  else return (((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1);
}

typedef __attribute__((address_space(3))) void at_lds_void;
typedef __attribute__((address_space(1))) const void at_glb_void;
typedef short at_s16x4 __attribute__((ext_vector_type(4)));
typedef short at_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) at_s16x4 at_lds_s16x4;

__device__ __forceinline__ at_bf16x8 at_tr_pair(const unsigned char* lo, const unsigned char* hi) {
  const at_s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((at_lds_s16x4*)lo);
  const at_s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((at_lds_s16x4*)hi);
  const at_s16x8 u = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(at_bf16x8, u);
}


// ------------------------------------------------------------------------------ forward
// Grid: (B * H, S / 128).  Wave w owns queries q0 + 32w .. + 31 (one per lane pair).
//
// The softmax runs in base 2 on t = score * scale * log2(e).  The running maximum m of a
// row is only raised when some row of the wave has outgrown it by more than AT_SLACK (a
// wave-uniform decision): until then exp2(t - m) <= 2^AT_SLACK, which fp32 sums and bf16
// probabilities hold without loss, and the accumulators need no rescaling.
constexpr float AT_SLACK = 8.0f;
constexpr float AT_LOG2E = 1.4426950408889634f;
constexpr float AT_LN2 = 0.6931471805599453f;

template <int HD>
__global__ __launch_bounds__(256, HD == 64 ? 4 : 2) void attn_fwd_kernel(const AttnArgs g) {
  constexpr int KSTEPS = HD / 16, DT = HD / 32, NCH = HD / 8;
  constexpr int TILE = 64 * HD * 2, STAGE = 2 * TILE;
  extern __shared__ __align__(16) unsigned char at_lds[];
  auto k_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE); };
  auto v_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE + TILE); };

  // Grid (B * H, tiles): workgroups are handed out along x first, so every (batch, head) runs
  // its longest causal rows before any runs a shorter one, and the tail of the launch consists
  // of the shortest workgroups.
  const int bh = blockIdx.x, b = bh / g.H, hh = bh % g.H;
  const int qt = (int)gridDim.y - 1 - (int)blockIdx.y;
  const int q0 = qt * 128;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 31, h = lane >> 5;
  const uint16_t* Q = g.q.p + (int64_t)b * g.q.sb + (int64_t)hh * g.q.sh;
  const uint16_t* K = g.k.p + (int64_t)b * g.k.sb + (int64_t)hh * g.k.sh;
  const uint16_t* V = g.v.p + (int64_t)b * g.v.sb + (int64_t)hh * g.v.sh;
  const int wq0 = q0 + wave * 32;  // first query of the wave
  const int my_q = wq0 + li;
  const float c = g.scale * AT_LOG2E;

  // the wave's queries as B fragments of the score MFMA
  at_bf16x8 qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const at_u32x4 u = *(const at_u32x4*)(Q + (int64_t)my_q * g.q.ss + s * 16 + h * 8);
    qf[s] = __builtin_bit_cast(at_bf16x8, u);
  }

  at_f32x16 o_acc[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o_acc[d] = (at_f32x16)(0.f);
  float m_i = at_neg_big(), l_i = 0.f;
  // The output is normalised by the sum of the probabilities as the matrix cores saw them
  // (rounded to bf16), so that it is an exact convex combination of the values: a part common to
  // all values then passes through unchanged, which the backward pass's dP - delta relies on.
  // That sum (l_r) is taken from the packed bf16 pairs on their way to the second product, one
  // v_dot2c_f32_bf16 against a pair of ones each; l_i, the sum before rounding, goes into the
  // log-sum-exp, with which the probabilities that the backward pass recomputes sum to one too.
  float l_r = 0.f;

  const int n_tiles = g.causal ? (q0 + 128) / 64 : g.S / 64;
  // K and V tiles go from memory into LDS without passing through registers: a wave instruction
  // deposits 64 x 16 bytes in a row (four rows of a 128-wide tile, eight of a 64-wide one), so
  // the swizzle is applied to the address each lane fetches from.
  constexpr int PER_WAVE = 64 * NCH / 64 / 4;  // instructions per wave and tile
  int src_off_k[PER_WAVE], src_off_v[PER_WAVE];  // element offsets of this lane's chunks in a tile
#pragma unroll
  for (int j = 0; j < PER_WAVE; ++j) {
    const int slot = (wave * PER_WAVE + j) * 64 + lane, row = slot / NCH, c = (slot % NCH) ^ at_sw<NCH>(row);
    src_off_k[j] = row * (int)g.k.ss + c * 8;
    src_off_v[j] = row * (int)g.v.ss + c * 8;
  }
  auto request = [&](int kt, int buf) {
    const uint16_t* ks = K + (int64_t)kt * 64 * g.k.ss;
    const uint16_t* vs = V + (int64_t)kt * 64 * g.v.ss;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      __builtin_amdgcn_global_load_lds((at_glb_void*)(ks + src_off_k[j]),
                                       (at_lds_void*)(k_tile(buf) + (wave * PER_WAVE + j) * 64), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((at_glb_void*)(vs + src_off_v[j]),
                                       (at_lds_void*)(v_tile(buf) + (wave * PER_WAVE + j) * 64), 16, 0, 0);
    }
  };
  // a workgroup barrier behind which every wave's copies have landed
  auto tile_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  };
  auto frag = [&](const at_u32x4* tile, int row, int chunk) {
    return __builtin_bit_cast(at_bf16x8, tile[row * NCH + (chunk ^ at_sw<NCH>(row))]);
  };
  int tr_lo, tr_hi, tr_x_lo, tr_x_hi;  // the transposing read of V, as the dQ kernel reads K
  {
    const int p = lane & 15, G = lane >> 4;
    const int kl = 4 * (G >> 1) + (p >> 2);
    const int d0 = 16 * (G & 1) + 4 * (p & 3);
    tr_x_lo = (d0 >> 3) ^ at_sw<NCH>(kl);
    tr_x_hi = (d0 >> 3) ^ at_sw<NCH>(kl + 8);
    tr_lo = kl * (HD * 2) + (d0 & 7) * 2;
    tr_hi = (kl + 8) * (HD * 2) + (d0 & 7) * 2;
  }
  auto tr_frag = [&](const at_u32x4* tile, int dd, int k16) {
    const unsigned char* base = (const unsigned char*)tile + k16 * 16 * (HD * 2);
    return at_tr_pair(base + tr_lo + ((tr_x_lo ^ (dd << 2)) << 4), base + tr_hi + ((tr_x_hi ^ (dd << 2)) << 4));
  };
  request(0, 0);
  tile_barrier();
  for (int kt = 0; kt < n_tiles; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < n_tiles;
    if (more) request(kt + 1, cur ^ 1);
    const at_u32x4* Ks = k_tile(cur);
    const at_u32x4* Vs = v_tile(cur);
    const int k0 = kt * 64;
    auto tile = [&](auto masked) {
      constexpr bool MASK = decltype(masked)::value;
      // transposed scores: rows = keys (two 32-row tiles), columns = the wave's queries
      at_f32x16 st[2];
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2) {
        // all fragments of the 32 keys are requested before the first MFMA waits for one
        at_bf16x8 kfr[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) kfr[s] = frag(Ks, kt2 * 32 + li, 2 * s + h);
        __builtin_amdgcn_sched_barrier(0);  // keeps the scheduler from sinking each read to its MFMA
        at_f32x16 acc = (at_f32x16)(0.f);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[s], qf[s], acc, 0, 0, 0);
        st[kt2] = acc;
      }
      float mx = at_neg_big();
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (MASK) {
            const int key = k0 + kt2 * 32 + (r >> 2) * 8 + 4 * h + (r & 3);
            if (key > my_q) st[kt2][r] = at_neg_big();
          }
          mx = fmaxf(mx, st[kt2][r]);
        }
      mx = fmaxf(mx, at_xhalf(mx)) * c;
      if (__any(mx - m_i > AT_SLACK)) {
        const float m_new = fmaxf(m_i, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
        l_i *= alpha;
        m_i = m_new;
#pragma unroll
        for (int d = 0; d < DT; ++d) o_acc[d] *= alpha;
        l_r *= alpha;
      }
      float sum = 0.f;
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kt2][r], c, -m_i));
          st[kt2][r] = p;
          sum += p;
        }
      l_i += sum;  // each half of the lane pair keeps the sum of its own keys
      // O^T[d, q] += V^T[d, key] P^T[key, q]
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const at_bf16x8 pf = at_regs_frag(st[kt2], t);
#pragma unroll
          for (int d = 0; d < DT; ++d)
            o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Vs, d, 2 * kt2 + t), pf, o_acc[d], 0, 0, 0);
          l_r = at_sum_bf16x8(pf, l_r);
        }
    };
    // keys of this tile against the wave's queries: all visible, some, or none
    if (!g.causal || k0 + 63 <= wq0) tile(std::false_type{});
    else if (k0 <= wq0 + 31) tile(std::true_type{});
    tile_barrier();
  }
  // normalise and write: register r of tile d is O[my_q][32 d + (r/4)*8 + 4h + r%4]
  l_i += at_xhalf(l_i);
  l_r += at_xhalf(l_r);
  const float inv = 1.0f / l_r;
  uint16_t* O = (uint16_t*)g.o.p + (int64_t)b * g.o.sb + (int64_t)hh * g.o.sh + (int64_t)my_q * g.o.ss;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      at_u32x2 w;
      w.x = at_pack2(o_acc[d][gq * 4 + 0] * inv, o_acc[d][gq * 4 + 1] * inv);
      w.y = at_pack2(o_acc[d][gq * 4 + 2] * inv, o_acc[d][gq * 4 + 3] * inv);
      *(at_u32x2*)(O + d * 32 + gq * 8 + 4 * h) = w;
    }
  if (g.o_lo.p != nullptr) {
    // The backward pass needs delta = rowsum(dO * O) to more digits than bf16 O has (dS is
    // P * (dP - delta), and with many keys of similar value dP - delta cancels almost
    // everything): the part of O that the rounding above cut off goes out as a second bf16 tensor.
    uint16_t* OL = (uint16_t*)g.o_lo.p + (int64_t)b * g.o_lo.sb + (int64_t)hh * g.o_lo.sh + (int64_t)my_q * g.o_lo.ss;
    auto rest = [&](float x) { return x - __uint_as_float((uint32_t)nbk_f32_to_bf16(x) << 16); };
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        at_u32x2 w;
        w.x = at_pack2(rest(o_acc[d][gq * 4 + 0] * inv), rest(o_acc[d][gq * 4 + 1] * inv));
        w.y = at_pack2(rest(o_acc[d][gq * 4 + 2] * inv), rest(o_acc[d][gq * 4 + 3] * inv));
        *(at_u32x2*)(OL + d * 32 + gq * 8 + 4 * h) = w;
      }
  }
  if (h == 0) g.lse[((int64_t)b * g.H + hh) * g.S + my_q] = m_i * AT_LN2 + __logf(l_i);
}


// ------------------------------------------------------------------------------ backward
// dK, dV.  Grid: (B * H, S / 128).  Wave w owns keys k0 + 32w .. + 31 (one per lane pair)
// and walks the query tiles that can see them.
//   S[q, key]  = Q K^T          (A: Q tile rows, B: the wave's K fragments)
//   P          = exp(S * scale - LSE[q])   (as exp2, with LSE staged in base-2 units)
//   dV^T[d,key] += dO^T[d, q] P[q, key]        (A: transposed dO tile, B: P registers)
//   dP[q, key] = dO V^T         (A: dO tile rows, B: the wave's V fragments)
//   dS         = P * (dP - delta[q])
//   dK^T[d,key] += Q^T[d, q] dS[q, key]         (A: transposed Q tile, B: dS registers; * scale at the end)
template <int HD>
__global__ __launch_bounds__(256) void attn_bwd_kv_kernel(const AttnArgs g) {
  using RowT = AtRowTile<HD>;
  using TrT = AtTransTile<HD>;
  constexpr int KSTEPS = HD / 16, DT = HD / 32;
  constexpr int ROW_BYTES = 64 * HD * 2, TR_BYTES = HD * AT_TP * 2;
  constexpr int STAGE = 2 * ROW_BYTES + 2 * TR_BYTES + 2 * 64 * 4;
  extern __shared__ __align__(16) unsigned char at_lds[];
  auto q_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE); };
  auto do_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE + ROW_BYTES); };
  auto qt_tile = [&](int buf) { return (uint16_t*)(at_lds + buf * STAGE + 2 * ROW_BYTES); };
  auto dot_tile = [&](int buf) { return (uint16_t*)(at_lds + buf * STAGE + 2 * ROW_BYTES + TR_BYTES); };
  auto lse_tile = [&](int buf) { return (float*)(at_lds + buf * STAGE + 2 * ROW_BYTES + 2 * TR_BYTES); };

  const int bh = blockIdx.x, b = bh / g.H, hh = bh % g.H;
  const int k0 = blockIdx.y * 128;  // the first key tiles see the most queries
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 31, h = lane >> 5;
  const uint16_t* Q = g.q.p + (int64_t)b * g.q.sb + (int64_t)hh * g.q.sh;
  const uint16_t* K = g.k.p + (int64_t)b * g.k.sb + (int64_t)hh * g.k.sh;
  const uint16_t* V = g.v.p + (int64_t)b * g.v.sb + (int64_t)hh * g.v.sh;
  const uint16_t* DO = g.dout.p + (int64_t)b * g.dout.sb + (int64_t)hh * g.dout.sh;
  const float* LSE = g.lse + ((int64_t)b * g.H + hh) * g.S;
  const float* DEL = g.delta + ((int64_t)b * g.H + hh) * g.S;
  const int my_k = k0 + wave * 32 + li;

  at_bf16x8 kf[KSTEPS], vf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const at_u32x4 uk = *(const at_u32x4*)(K + (int64_t)my_k * g.k.ss + s * 16 + h * 8);
    const at_u32x4 uv = *(const at_u32x4*)(V + (int64_t)my_k * g.v.ss + s * 16 + h * 8);
    kf[s] = __builtin_bit_cast(at_bf16x8, uk);
    vf[s] = __builtin_bit_cast(at_bf16x8, uv);
  }
  at_f32x16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) {
    dk_acc[d] = (at_f32x16)(0.f);
    dv_acc[d] = (at_f32x16)(0.f);
  }

  const int first = g.causal ? k0 / 64 : 0;  // first query tile that sees key k0
  const int n_tiles = g.S / 64;
  RowT ql, dol;
  TrT qtl, dotl;
  float lreg = 0.f;  // lanes 0..63: LSE, 64..127: delta of the tile's queries
  auto load_all = [&](int qt) {
    ql.load(Q, g.q.ss, qt * 64);
    dol.load(DO, g.dout.ss, qt * 64);
    qtl.load(Q, g.q.ss, qt * 64);
    dotl.load(DO, g.dout.ss, qt * 64);
    if (threadIdx.x < 64) lreg = LSE[qt * 64 + threadIdx.x] * AT_LOG2E;
    else if (threadIdx.x < 128) lreg = DEL[qt * 64 + threadIdx.x - 64];
  };
  auto store_all = [&](int buf) {
    ql.store(q_tile(buf));
    dol.store(do_tile(buf));
    qtl.store(qt_tile(buf));
    dotl.store(dot_tile(buf));
    if (threadIdx.x < 128) lse_tile(buf)[threadIdx.x] = lreg;
  };
  const int wk0 = k0 + wave * 32;  // first key of the wave
  const float c = g.scale * AT_LOG2E;
  load_all(first);
  store_all(0);
  __syncthreads();
  for (int qt = first; qt < n_tiles; ++qt) {
    const int cur = (qt - first) & 1;
    const bool more = qt + 1 < n_tiles;
    if (more) load_all(qt + 1);
    const at_u32x4* Qs = q_tile(cur);
    const at_u32x4* DOs = do_tile(cur);
    const uint16_t* QTs = qt_tile(cur);
    const uint16_t* DOTs = dot_tile(cur);
    const float* Ls = lse_tile(cur);
    const int q0 = qt * 64;
    auto subtile = [&](auto masked, int qt2) {
      constexpr bool MASK = decltype(masked)::value;
      at_f32x16 s_acc = (at_f32x16)(0.f), dp_acc = (at_f32x16)(0.f);
#pragma unroll
      for (int s = 0; s < KSTEPS; s += 4) {
        // fragments of four k-steps are requested before the first MFMA waits for one
        at_bf16x8 qfr[4], dfr[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          qfr[u] = RowT::frag(Qs, qt2 * 32 + li, 2 * (s + u) + h);
          dfr[u] = RowT::frag(DOs, qt2 * 32 + li, 2 * (s + u) + h);
        }
        __builtin_amdgcn_sched_barrier(0);  // keeps the scheduler from sinking each read to its MFMA
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[u], kf[s + u], s_acc, 0, 0, 0);
          dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dfr[u], vf[s + u], dp_acc, 0, 0, 0);
        }
      }
      // rows of these tiles are queries: register r is query q0 + 32 qt2 + (r/4)*8 + 4h + r%4
      at_f32x16 p, ds;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int qb = qt2 * 32 + gq * 8 + 4 * h;
        const float4 l4 = *(const float4*)(Ls + qb);
        const float4 d4 = *(const float4*)(Ls + 64 + qb);
        const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = gq * 4 + e;
          float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[r], c, -lv[e]));
          if (MASK && my_k > q0 + qb + e) pv = 0.f;
          p[r] = pv;
          ds[r] = pv * (dp_acc[r] - dv[e]);
        }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const at_bf16x8 pf = at_regs_frag(p, t), dsf = at_regs_frag(ds, t);
#pragma unroll
        for (int d = 0; d < DT; ++d) {
          dv_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TrT::frag(DOTs, d * 32 + li, qt2, t, h), pf,
                                                              dv_acc[d], 0, 0, 0);
          dk_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TrT::frag(QTs, d * 32 + li, qt2, t, h), dsf,
                                                              dk_acc[d], 0, 0, 0);
        }
      }
    };
#pragma unroll
    for (int qt2 = 0; qt2 < 2; ++qt2) {
      const int sq0 = q0 + qt2 * 32;  // queries sq0 .. sq0 + 31 against keys wk0 .. wk0 + 31
      if (!g.causal || wk0 + 31 <= sq0) subtile(std::false_type{}, qt2);
      else if (wk0 <= sq0 + 31) subtile(std::true_type{}, qt2);
    }
    if (more) store_all(cur ^ 1);
    __syncthreads();
  }
  uint16_t* DK = (uint16_t*)g.dk.p + (int64_t)b * g.dk.sb + (int64_t)hh * g.dk.sh + (int64_t)my_k * g.dk.ss;
  uint16_t* DV = (uint16_t*)g.dv.p + (int64_t)b * g.dv.sb + (int64_t)hh * g.dv.sh + (int64_t)my_k * g.dv.ss;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      at_u32x2 wk, wv;
      wk.x = at_pack2(dk_acc[d][gq * 4 + 0] * g.scale, dk_acc[d][gq * 4 + 1] * g.scale);
      wk.y = at_pack2(dk_acc[d][gq * 4 + 2] * g.scale, dk_acc[d][gq * 4 + 3] * g.scale);
      wv.x = at_pack2(dv_acc[d][gq * 4 + 0], dv_acc[d][gq * 4 + 1]);
      wv.y = at_pack2(dv_acc[d][gq * 4 + 2], dv_acc[d][gq * 4 + 3]);
      *(at_u32x2*)(DK + d * 32 + gq * 8 + 4 * h) = wk;
      *(at_u32x2*)(DV + d * 32 + gq * 8 + 4 * h) = wv;
    }
}

// dK, dV for 128-wide heads, eight waves.  The four-wave form above keeps 376 registers per lane,
// so a wave is alone on its SIMD and its matrix, LDS and exp phases run one after the other.
// Here the 128 keys of a workgroup are owned by wave pairs: wave w works on keys
// k0 + 32 (w % 4) .. + 31 and on the query half w / 4 of every 64-query tile, with its own
// partial dK^T / dV^T accumulators (the halves meet in LDS at the end).  To fit two waves on a
// SIMD (256 registers each)
//   * K and V sit in LDS for the whole kernel (row-major, swizzled) instead of in registers;
//   * there are no transposed tile copies: the A operand of dV^T += dO^T P and dK^T += Q^T dS is
//     read out of the row-major tile with the transposing LDS read (ds_read_b64_tr_b16: lane i
//     of a 16-lane group receives four consecutive k of row i from a k-major tile, which is what
//     a [query][d] tile is for these products), with the k-slot permutation of the P registers.
// Tile layout [rows][16 chunks of 16 bytes]: chunk c of row r sits at c ^ sw(r),
// sw(r) = 4 (r % 4) + (r / 4) % 4.  Sixteen consecutive rows send one chunk to sixteen different
// 16-byte slots (the fragment reads of 16 lanes), and four consecutive rows send a 64-byte piece
// to four different 64-byte windows (the transposing read of half a wave).
template <int HD>
__global__ __launch_bounds__(512) void attn_bwd_kv8_kernel(const AttnArgs g) {
  constexpr int KSTEPS = HD / 16, DT = HD / 32, NCH = HD / 8;
  constexpr int TILE = 64 * HD * 2;    // a 64-row tile
  constexpr int KV = 128 * HD * 2;     // the workgroup's K (or V) rows
  constexpr int STAGE = 2 * TILE + 2 * 64 * 4;
  extern __shared__ __align__(16) unsigned char at_lds[];
  at_u32x4* Ks = (at_u32x4*)at_lds;
  at_u32x4* Vs = (at_u32x4*)(at_lds + KV);
  auto q_tile = [&](int buf) { return (at_u32x4*)(at_lds + 2 * KV + buf * STAGE); };
  auto do_tile = [&](int buf) { return (at_u32x4*)(at_lds + 2 * KV + buf * STAGE + TILE); };
  auto lse_tile = [&](int buf) { return (float*)(at_lds + 2 * KV + buf * STAGE + 2 * TILE); };

  const int bh = blockIdx.x, b = bh / g.H, hh = bh % g.H;
  const int k0 = blockIdx.y * 128;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, h = lane >> 5;
  const int kw = wave & 3, qh = wave >> 2;
  const uint16_t* Q = g.q.p + (int64_t)b * g.q.sb + (int64_t)hh * g.q.sh;
  const uint16_t* K = g.k.p + (int64_t)b * g.k.sb + (int64_t)hh * g.k.sh;
  const uint16_t* V = g.v.p + (int64_t)b * g.v.sb + (int64_t)hh * g.v.sh;
  const uint16_t* DO = g.dout.p + (int64_t)b * g.dout.sb + (int64_t)hh * g.dout.sh;
  const float* LSE = g.lse + ((int64_t)b * g.H + hh) * g.S;
  const float* DEL = g.delta + ((int64_t)b * g.H + hh) * g.S;
  const int my_k = k0 + kw * 32 + li;

  // K and V rows of the workgroup -> LDS (512 lanes, 16 bytes each)
#pragma unroll
  for (int s = 0; s < 128 * NCH / 512; ++s) {
    const int t = tid + s * 512, row = t / NCH, c = t % NCH;
    Ks[row * NCH + (c ^ at_sw<NCH>(row))] = *(const at_u32x4*)(K + (int64_t)(k0 + row) * g.k.ss + c * 8);
    Vs[row * NCH + (c ^ at_sw<NCH>(row))] = *(const at_u32x4*)(V + (int64_t)(k0 + row) * g.v.ss + c * 8);
  }

  at_f32x16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) {
    dk_acc[d] = (at_f32x16)(0.f);
    dv_acc[d] = (at_f32x16)(0.f);
  }

  const int first = g.causal ? k0 / 64 : 0;  // first query tile that sees key k0
  const int n_tiles = g.S / 64;
  constexpr int TP = 64 * NCH / 512;  // passes over a 64-row tile
  at_u32x4 qreg[TP], doreg[TP];
  float lreg = 0.f;  // lanes 0..63: LSE, 64..127: delta of the tile's queries
  auto load_all = [&](int qt) {
#pragma unroll
    for (int s = 0; s < TP; ++s) {
      const int t = tid + s * 512, row = t / NCH, c = t % NCH;
      qreg[s] = *(const at_u32x4*)(Q + (int64_t)(qt * 64 + row) * g.q.ss + c * 8);
      doreg[s] = *(const at_u32x4*)(DO + (int64_t)(qt * 64 + row) * g.dout.ss + c * 8);
    }
    if (tid < 64) lreg = LSE[qt * 64 + tid] * AT_LOG2E;
    else if (tid < 128) lreg = DEL[qt * 64 + tid - 64];
  };
  auto store_all = [&](int buf) {
    at_u32x4* qd = q_tile(buf);
    at_u32x4* dd = do_tile(buf);
#pragma unroll
    for (int s = 0; s < TP; ++s) {
      const int t = tid + s * 512, row = t / NCH, c = t % NCH;
      qd[row * NCH + (c ^ at_sw<NCH>(row))] = qreg[s];
      dd[row * NCH + (c ^ at_sw<NCH>(row))] = doreg[s];
    }
    if (tid < 128) lse_tile(buf)[tid] = lreg;
  };
  // row fragment: 8 consecutive d (chunk) of `row`
  auto frag = [&](const at_u32x4* tile, int row, int chunk) {
    return __builtin_bit_cast(at_bf16x8, tile[row * NCH + (chunk ^ at_sw<NCH>(row))]);
  };
  // Transposed fragments.  Lane p of group G = lane / 16 points at query 4 (G / 2) + p / 4 (+ 8 for
  // the second half of the k-slots) of a 16-query step and at d = 16 (G % 2) + 4 (p % 4) .. + 4 of
  // a 32-wide d block: byte offsets of both halves inside a tile, the d block and the 16-query
  // step left out (the block flips bits 2-3 of the chunk index, the step adds whole rows).
  int tr_lo, tr_hi, tr_x_lo, tr_x_hi;
  {
    const int p = lane & 15, G = lane >> 4;
    const int ql = 4 * (G >> 1) + (p >> 2);
    const int d0 = 16 * (G & 1) + 4 * (p & 3);
    tr_x_lo = (d0 >> 3) ^ at_sw<NCH>(ql);
    tr_x_hi = (d0 >> 3) ^ at_sw<NCH>(ql + 8);
    tr_lo = ql * (HD * 2) + (d0 & 7) * 2;
    tr_hi = (ql + 8) * (HD * 2) + (d0 & 7) * 2;
  }
  auto tr_frag = [&](const at_u32x4* tile, int dd, int q16) {
    const unsigned char* base = (const unsigned char*)tile + q16 * 16 * (HD * 2);
    return at_tr_pair(base + tr_lo + ((tr_x_lo ^ (dd << 2)) << 4), base + tr_hi + ((tr_x_hi ^ (dd << 2)) << 4));
  };

  const int wk0 = k0 + kw * 32;  // first key of the wave
  const float c = g.scale * AT_LOG2E;
  load_all(first);
  store_all(0);
  __syncthreads();
  for (int qt = first; qt < n_tiles; ++qt) {
    const int cur = (qt - first) & 1;
    const bool more = qt + 1 < n_tiles;
    if (more) load_all(qt + 1);
    const at_u32x4* Qs = q_tile(cur);
    const at_u32x4* DOs = do_tile(cur);
    const float* Ls = lse_tile(cur);
    const int sq0 = qt * 64 + qh * 32;  // queries sq0 .. sq0 + 31 against keys wk0 .. wk0 + 31
    auto subtile = [&](auto masked) {
      constexpr bool MASK = decltype(masked)::value;
      at_f32x16 s_acc = (at_f32x16)(0.f), dp_acc = (at_f32x16)(0.f);
#pragma unroll
      for (int s = 0; s < KSTEPS; s += 2) {
        at_bf16x8 qfr[2], kfr[2], dfr[2], vfr[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          qfr[u] = frag(Qs, qh * 32 + li, 2 * (s + u) + h);
          kfr[u] = frag(Ks, kw * 32 + li, 2 * (s + u) + h);
          dfr[u] = frag(DOs, qh * 32 + li, 2 * (s + u) + h);
          vfr[u] = frag(Vs, kw * 32 + li, 2 * (s + u) + h);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[u], kfr[u], s_acc, 0, 0, 0);
          dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dfr[u], vfr[u], dp_acc, 0, 0, 0);
        }
      }
      // rows of these tiles are queries: register r is query sq0 + (r/4)*8 + 4h + r%4
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int qb = qh * 32 + gq * 8 + 4 * h;
        const float4 l4 = *(const float4*)(Ls + qb);
        const float4 d4 = *(const float4*)(Ls + 64 + qb);
        const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = gq * 4 + e;
          float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[r], c, -lv[e]));
          if (MASK && my_k > qt * 64 + qb + e) pv = 0.f;
          s_acc[r] = pv;                          // P in place of S
          dp_acc[r] = pv * (dp_acc[r] - dv[e]);   // dS in place of dP
        }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const at_bf16x8 pf = at_regs_frag(s_acc, t), dsf = at_regs_frag(dp_acc, t);
#pragma unroll
        for (int d = 0; d < DT; ++d) {
          dv_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(DOs, d, 2 * qh + t), pf, dv_acc[d], 0, 0, 0);
          dk_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Qs, d, 2 * qh + t), dsf, dk_acc[d], 0, 0, 0);
        }
      }
    };
    if (!g.causal || wk0 + 31 <= sq0) subtile(std::false_type{});
    else if (wk0 <= sq0 + 31) subtile(std::true_type{});
    if (more) store_all(cur ^ 1);
    __syncthreads();
  }
  // the two query halves of a key group meet: the upper half hands its sums over through LDS
  // (16 bytes per lane and piece, lanes side by side), the lower half adds them and writes
  float4* xch = (float4*)at_lds + (size_t)kw * (2 * DT * 4 * 64) + lane;
  if (qh == 1) {
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        xch[((0 * DT + d) * 4 + gq) * 64] = make_float4(dk_acc[d][gq * 4], dk_acc[d][gq * 4 + 1], dk_acc[d][gq * 4 + 2], dk_acc[d][gq * 4 + 3]);
        xch[((1 * DT + d) * 4 + gq) * 64] = make_float4(dv_acc[d][gq * 4], dv_acc[d][gq * 4 + 1], dv_acc[d][gq * 4 + 2], dv_acc[d][gq * 4 + 3]);
      }
  }
  __syncthreads();
  if (qh == 1) return;
  uint16_t* DK = (uint16_t*)g.dk.p + (int64_t)b * g.dk.sb + (int64_t)hh * g.dk.sh + (int64_t)my_k * g.dk.ss;
  uint16_t* DV = (uint16_t*)g.dv.p + (int64_t)b * g.dv.sb + (int64_t)hh * g.dv.sh + (int64_t)my_k * g.dv.ss;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const float4 ok = xch[((0 * DT + d) * 4 + gq) * 64], ov = xch[((1 * DT + d) * 4 + gq) * 64];
      at_u32x2 wk, wv;
      wk.x = at_pack2((dk_acc[d][gq * 4 + 0] + ok.x) * g.scale, (dk_acc[d][gq * 4 + 1] + ok.y) * g.scale);
      wk.y = at_pack2((dk_acc[d][gq * 4 + 2] + ok.z) * g.scale, (dk_acc[d][gq * 4 + 3] + ok.w) * g.scale);
      wv.x = at_pack2(dv_acc[d][gq * 4 + 0] + ov.x, dv_acc[d][gq * 4 + 1] + ov.y);
      wv.y = at_pack2(dv_acc[d][gq * 4 + 2] + ov.z, dv_acc[d][gq * 4 + 3] + ov.w);
      *(at_u32x2*)(DK + d * 32 + gq * 8 + 4 * h) = wk;
      *(at_u32x2*)(DV + d * 32 + gq * 8 + 4 * h) = wv;
    }
}

// dQ.  Grid: (B * H, S / 128).  Wave w owns queries q0 + 32w .. + 31 and walks the key tiles.
//   S^T[key, q]  = K Q^T                (A: K tile rows, B: the wave's Q fragments)
//   P^T          = exp(S^T * scale - LSE[q])
//   dP^T[key, q] = V dO^T               (A: V tile rows, B: the wave's dO fragments)
//   dS^T         = P^T * (dP^T - delta[q])
//   dQ^T[d, q]  += K^T[d, key] dS^T[key, q]   (A: K tile through the transposing read, B: dS^T registers; * scale at the end)
// There is no transposed copy of K: the A operand of the last product comes out of the row-major
// K tile through the transposing LDS read, in the layout of the eight-wave dK / dV kernel above.
// Two stages of K and V (32 KB each with 128-wide heads) fit twice on a CU.
template <int HD>
__global__ __launch_bounds__(256, 2) void attn_bwd_q_tr_kernel(const AttnArgs g) {
  constexpr int KSTEPS = HD / 16, DT = HD / 32, NCH = HD / 8;
  constexpr int TILE = 64 * HD * 2, STAGE = 2 * TILE;
  extern __shared__ __align__(16) unsigned char at_lds[];
  auto k_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE); };
  auto v_tile = [&](int buf) { return (at_u32x4*)(at_lds + buf * STAGE + TILE); };

  const int bh = blockIdx.x, b = bh / g.H, hh = bh % g.H;
  const int qt = (int)gridDim.y - 1 - (int)blockIdx.y;
  const int q0 = qt * 128;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, h = lane >> 5;
  const uint16_t* Q = g.q.p + (int64_t)b * g.q.sb + (int64_t)hh * g.q.sh;
  const uint16_t* K = g.k.p + (int64_t)b * g.k.sb + (int64_t)hh * g.k.sh;
  const uint16_t* V = g.v.p + (int64_t)b * g.v.sb + (int64_t)hh * g.v.sh;
  const uint16_t* DO = g.dout.p + (int64_t)b * g.dout.sb + (int64_t)hh * g.dout.sh;
  const int my_q = q0 + wave * 32 + li;
  const float my_lse = g.lse[((int64_t)b * g.H + hh) * g.S + my_q] * AT_LOG2E;
  const int wq0 = q0 + wave * 32;  // first query of the wave
  const float c = g.scale * AT_LOG2E;

  at_f32x16 dq_acc[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) dq_acc[d] = (at_f32x16)(0.f);

  const int n_tiles = g.causal ? (q0 + 128) / 64 : g.S / 64;
  constexpr int TP = 64 * NCH / 256;  // passes over a 64-row tile
  at_u32x4 kreg[TP], vreg[TP];
  auto load_all = [&](int kt) {
#pragma unroll
    for (int s = 0; s < TP; ++s) {
      const int t = tid + s * 256, row = t / NCH, ch = t % NCH;
      kreg[s] = *(const at_u32x4*)(K + (int64_t)(kt * 64 + row) * g.k.ss + ch * 8);
      vreg[s] = *(const at_u32x4*)(V + (int64_t)(kt * 64 + row) * g.v.ss + ch * 8);
    }
  };
  auto store_all = [&](int buf) {
    at_u32x4* kd = k_tile(buf);
    at_u32x4* vd = v_tile(buf);
#pragma unroll
    for (int s = 0; s < TP; ++s) {
      const int t = tid + s * 256, row = t / NCH, ch = t % NCH;
      kd[row * NCH + (ch ^ at_sw<NCH>(row))] = kreg[s];
      vd[row * NCH + (ch ^ at_sw<NCH>(row))] = vreg[s];
    }
  };
  auto frag = [&](const at_u32x4* tile, int row, int chunk) {
    return __builtin_bit_cast(at_bf16x8, tile[row * NCH + (chunk ^ at_sw<NCH>(row))]);
  };
  int tr_lo, tr_hi, tr_x_lo, tr_x_hi;  // as in the dK / dV kernel, keys in the place of queries
  {
    const int p = lane & 15, G = lane >> 4;
    const int kl = 4 * (G >> 1) + (p >> 2);
    const int d0 = 16 * (G & 1) + 4 * (p & 3);
    tr_x_lo = (d0 >> 3) ^ at_sw<NCH>(kl);
    tr_x_hi = (d0 >> 3) ^ at_sw<NCH>(kl + 8);
    tr_lo = kl * (HD * 2) + (d0 & 7) * 2;
    tr_hi = (kl + 8) * (HD * 2) + (d0 & 7) * 2;
  }
  auto tr_frag = [&](const at_u32x4* tile, int dd, int k16) {
    const unsigned char* base = (const unsigned char*)tile + k16 * 16 * (HD * 2);
    return at_tr_pair(base + tr_lo + ((tr_x_lo ^ (dd << 2)) << 4), base + tr_hi + ((tr_x_hi ^ (dd << 2)) << 4));
  };

  // delta[q] = sum_d dO[q, d] O[q, d] comes out of the dO fragments this kernel loads anyway and
  // the matching pieces of O (a lane pair holds one row); it is left in g.delta for the dK / dV
  // kernel, which runs after this one.
  // With the forward pass's second tensor (what bf16 O lost) the sum runs over O to about 16
  // bits: a delta off by 2^-9 of |dO| |O| would be a visible share of dP - delta wherever the
  // keys a query sees have values with a large common part.
  // Order of the requests: the first K / V tile, then Q and dO, then O and its remainder -- the
  // tile is waited for first (to go to LDS), and the pieces of O, which only delta needs, are
  // still on their way while the tile is stored and the workgroup meets at the barrier.
  const uint16_t* O = g.o.p + (int64_t)b * g.o.sb + (int64_t)hh * g.o.sh;
  const uint16_t* OL = g.o_lo.p == nullptr ? nullptr
                                           : g.o_lo.p + (int64_t)b * g.o_lo.sb + (int64_t)hh * g.o_lo.sh;
  at_bf16x8 qf[KSTEPS], dof[KSTEPS];
  at_u32x4 uo[KSTEPS], ul[KSTEPS];
  load_all(0);
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const at_u32x4 uq = *(const at_u32x4*)(Q + (int64_t)my_q * g.q.ss + s * 16 + h * 8);
    const at_u32x4 ud = *(const at_u32x4*)(DO + (int64_t)my_q * g.dout.ss + s * 16 + h * 8);
    qf[s] = __builtin_bit_cast(at_bf16x8, uq);
    dof[s] = __builtin_bit_cast(at_bf16x8, ud);
  }
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    uo[s] = *(const at_u32x4*)(O + (int64_t)my_q * g.o.ss + s * 16 + h * 8);
    ul[s] = (at_u32x4){0u, 0u, 0u, 0u};
    if (OL != nullptr) ul[s] = *(const at_u32x4*)(OL + (int64_t)my_q * g.o_lo.ss + s * 16 + h * 8);
  }
  store_all(0);
  __syncthreads();
  float my_delta = 0.f;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const at_u32x4 ud = __builtin_bit_cast(at_u32x4, dof[s]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      my_delta += (__uint_as_float(uo[s][e] << 16) + __uint_as_float(ul[s][e] << 16)) * __uint_as_float(ud[e] << 16);
      my_delta += (__uint_as_float(uo[s][e] & 0xffff0000u) + __uint_as_float(ul[s][e] & 0xffff0000u)) *
                  __uint_as_float(ud[e] & 0xffff0000u);
    }
  }
  my_delta += at_xhalf(my_delta);
  if (h == 0) g.delta[((int64_t)b * g.H + hh) * g.S + my_q] = my_delta;
  for (int kt = 0; kt < n_tiles; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < n_tiles;
    if (more) load_all(kt + 1);
    const at_u32x4* Ks = k_tile(cur);
    const at_u32x4* Vs = v_tile(cur);
    const int k0 = kt * 64;
    auto subtile = [&](auto masked, int kt2) {
      constexpr bool MASK = decltype(masked)::value;
      at_f32x16 s_acc = (at_f32x16)(0.f), dp_acc = (at_f32x16)(0.f);
#pragma unroll
      for (int s = 0; s < KSTEPS; s += 2) {
        at_bf16x8 kfr[2], vfr[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          kfr[u] = frag(Ks, kt2 * 32 + li, 2 * (s + u) + h);
          vfr[u] = frag(Vs, kt2 * 32 + li, 2 * (s + u) + h);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[u], qf[s + u], s_acc, 0, 0, 0);
          dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[u], dof[s + u], dp_acc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[r], c, -my_lse));
        if (MASK) {
          const int key = k0 + kt2 * 32 + (r >> 2) * 8 + 4 * h + (r & 3);
          if (key > my_q) pv = 0.f;
        }
        dp_acc[r] = pv * (dp_acc[r] - my_delta);  // dS^T in place of dP^T
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const at_bf16x8 dsf = at_regs_frag(dp_acc, t);
#pragma unroll
        for (int d = 0; d < DT; ++d)
          dq_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Ks, d, 2 * kt2 + t), dsf, dq_acc[d], 0, 0, 0);
      }
    };
#pragma unroll
    for (int kt2 = 0; kt2 < 2; ++kt2) {
      const int sk0 = k0 + kt2 * 32;  // keys sk0 .. sk0 + 31 against queries wq0 .. wq0 + 31
      if (!g.causal || sk0 + 31 <= wq0) subtile(std::false_type{}, kt2);
      else if (sk0 <= wq0 + 31) subtile(std::true_type{}, kt2);
    }
    if (more) store_all(cur ^ 1);
    __syncthreads();
  }
  uint16_t* DQ = (uint16_t*)g.dq.p + (int64_t)b * g.dq.sb + (int64_t)hh * g.dq.sh + (int64_t)my_q * g.dq.ss;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      at_u32x2 w;
      w.x = at_pack2(dq_acc[d][gq * 4 + 0] * g.scale, dq_acc[d][gq * 4 + 1] * g.scale);
      w.y = at_pack2(dq_acc[d][gq * 4 + 2] * g.scale, dq_acc[d][gq * 4 + 3] * g.scale);
      *(at_u32x2*)(DQ + d * 32 + gq * 8 + 4 * h) = w;
    }
}

// ------------------------------------------------------------------------------ host
static int attn_tensor(const nbk_attn_tensor* t, const char* what, AttnTensor* out, bool need) {
  if (!need && (t == nullptr || t->ptr == nullptr)) {
    out->p = nullptr;
    out->sb = out->ss = out->sh = 0;
    return NBK_OK;
  }
  NBK_REQUIRE(t != nullptr && t->ptr != nullptr, "attention: null tensor %s", what);
  NBK_REQUIRE(((uintptr_t)t->ptr & 15) == 0, "attention: %s is not 16-byte aligned", what);
  NBK_REQUIRE(t->sb >= 0 && t->ss > 0 && t->sh > 0 && t->sb % 8 == 0 && t->ss % 8 == 0 && t->sh % 8 == 0,
              "attention: strides of %s (%lld, %lld, %lld) must be positive multiples of 8 elements",
              what, (long long)t->sb, (long long)t->ss, (long long)t->sh);
  out->p = (const uint16_t*)t->ptr;
  out->sb = t->sb; out->ss = t->ss; out->sh = t->sh;
  return NBK_OK;
}

static int attn_common(const nbk_attn_desc* d, AttnArgs* a) {
  NBK_REQUIRE(d != nullptr, "attention: null descriptor");
  NBK_REQUIRE(d->dtype == NBK_BF16, "attention: only bf16 is implemented (dtype %d)", d->dtype);
  NBK_REQUIRE(d->hd == 64 || d->hd == 128, "attention: head size %lld must be 64 or 128", (long long)d->hd);
  NBK_REQUIRE(d->B > 0 && d->H > 0 && d->S > 0 && d->S % 128 == 0,
              "attention: B %lld, H %lld, S %lld (S must be a positive multiple of 128)",
              (long long)d->B, (long long)d->H, (long long)d->S);
  NBK_REQUIRE(d->B * d->H <= 0x7fffffffLL && d->S / 128 <= 65535, "attention: extent beyond the grid limits");
  a->B = (int32_t)d->B; a->H = (int32_t)d->H; a->S = (int32_t)d->S;
  a->causal = d->causal ? 1 : 0;
  a->scale = d->scale;
  return NBK_OK;
}

template <typename Kern>
static int attn_set_lds(Kern kern, size_t bytes) {
  if (bytes > 64 * 1024)
    NBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return NBK_OK;
}

extern "C" int nbk_attention_fwd(const nbk_attn_desc* d, const nbk_attn_tensor* q, const nbk_attn_tensor* k,
                                 const nbk_attn_tensor* v, const nbk_attn_tensor* o,
                                 const nbk_attn_tensor* o_lo, void* lse, void* stream) {
  AttnArgs a = {};
  int rc = attn_common(d, &a);
  if (rc) return rc;
  if ((rc = attn_tensor(q, "q", &a.q, true)) || (rc = attn_tensor(k, "k", &a.k, true)) ||
      (rc = attn_tensor(v, "v", &a.v, true)) || (rc = attn_tensor(o, "o", &a.o, true)) ||
      (rc = attn_tensor(o_lo, "o_lo", &a.o_lo, false)))
    return rc;
  NBK_REQUIRE(lse != nullptr, "attention: null lse");
  a.lse = (float*)lse;
  const dim3 grid((unsigned)(d->B * d->H), (unsigned)(d->S / 128));
  hipStream_t st = (hipStream_t)stream;
  // two stages of a row-major K and V tile each
  const size_t lds = 2 * 2 * 64 * (size_t)d->hd * 2;
  if (d->hd == 64) {
    if ((rc = attn_set_lds(attn_fwd_kernel<64>, lds))) return rc;
    hipLaunchKernelGGL(attn_fwd_kernel<64>, grid, dim3(256), lds, st, a);
  } else {
    if ((rc = attn_set_lds(attn_fwd_kernel<128>, lds))) return rc;
    hipLaunchKernelGGL(attn_fwd_kernel<128>, grid, dim3(256), lds, st, a);
  }
  return nbk_check_launch("attn_fwd_kernel");
}

extern "C" int64_t nbk_attention_bwd_workspace(const nbk_attn_desc* d) {
  if (d == nullptr || d->B <= 0 || d->H <= 0 || d->S <= 0) return -1;
  return d->B * d->H * d->S * (int64_t)sizeof(float);
}

// Launches of the backward pass once the arguments are checked; `delta` is B * H * S floats of
// device scratch (one per score row).
static int attn_bwd_launch(const nbk_attn_desc* d, AttnArgs& a, float* delta, hipStream_t st) {
  int rc;
  a.delta = delta;
  const dim3 grid((unsigned)(d->B * d->H), (unsigned)(d->S / 128));
  if (d->hd == 64) {
    // (the eight-wave dK / dV form was measured on this head size too: 70 against 68 us on the
    // transformer block's shape, so 64-wide heads keep the four-wave kernel, which fits twice on a CU)
    // (the dQ kernel first: it leaves delta, the row sums of dO * O, for the dK / dV kernel)
    const size_t lds_kv = 2 * (2 * 64 * 64 * 2 + 2 * 64 * AT_TP * 2 + 2 * 64 * 4);
    const size_t lds_qtr = 2 * (2 * 64 * 64 * 2);
    if ((rc = attn_set_lds(attn_bwd_kv_kernel<64>, lds_kv))) return rc;
    hipLaunchKernelGGL(attn_bwd_q_tr_kernel<64>, grid, dim3(256), lds_qtr, st, a);
    hipLaunchKernelGGL(attn_bwd_kv_kernel<64>, grid, dim3(256), lds_kv, st, a);
  } else {
    const size_t lds_kv8 = 2 * (128 * 128 * 2) + 2 * (2 * 64 * 128 * 2 + 2 * 64 * 4);
    const size_t lds_qtr = 2 * (2 * 64 * 128 * 2);
    if ((rc = attn_set_lds(attn_bwd_kv8_kernel<128>, lds_kv8))) return rc;
    hipLaunchKernelGGL(attn_bwd_q_tr_kernel<128>, grid, dim3(256), lds_qtr, st, a);
    hipLaunchKernelGGL(attn_bwd_kv8_kernel<128>, grid, dim3(512), lds_kv8, st, a);
  }
  return nbk_check_launch("attn_bwd kernels");
}

static int attn_bwd_args(const nbk_attn_desc* d, const nbk_attn_tensor* q, const nbk_attn_tensor* k,
                         const nbk_attn_tensor* v, const nbk_attn_tensor* o,
                         const nbk_attn_tensor* o_lo, const void* lse,
                         const nbk_attn_tensor* dout, const nbk_attn_tensor* dq,
                         const nbk_attn_tensor* dk, const nbk_attn_tensor* dv, AttnArgs* a) {
  int rc = attn_common(d, a);
  if (rc) return rc;
  if ((rc = attn_tensor(q, "q", &a->q, true)) || (rc = attn_tensor(k, "k", &a->k, true)) ||
      (rc = attn_tensor(v, "v", &a->v, true)) || (rc = attn_tensor(o, "o", &a->o, true)) ||
      (rc = attn_tensor(o_lo, "o_lo", &a->o_lo, false)) ||
      (rc = attn_tensor(dout, "dout", &a->dout, true)) || (rc = attn_tensor(dq, "dq", &a->dq, true)) ||
      (rc = attn_tensor(dk, "dk", &a->dk, true)) || (rc = attn_tensor(dv, "dv", &a->dv, true)))
    return rc;
  NBK_REQUIRE(lse != nullptr, "attention: null lse");
  a->lse = (float*)lse;
  return NBK_OK;
}

extern "C" int nbk_attention_bwd(const nbk_attn_desc* d, const nbk_attn_tensor* q, const nbk_attn_tensor* k,
                                 const nbk_attn_tensor* v, const nbk_attn_tensor* o,
                                 const nbk_attn_tensor* o_lo, const void* lse,
                                 const nbk_attn_tensor* dout, const nbk_attn_tensor* dq,
                                 const nbk_attn_tensor* dk, const nbk_attn_tensor* dv, void* workspace,
                                 int64_t workspace_bytes, void* stream) {
  AttnArgs a = {};
  int rc = attn_bwd_args(d, q, k, v, o, o_lo, lse, dout, dq, dk, dv, &a);
  if (rc) return rc;
  NBK_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 15) == 0 &&
                  workspace_bytes >= nbk_attention_bwd_workspace(d),
              "attention: backward needs %lld bytes of 16-byte aligned workspace",
              (long long)nbk_attention_bwd_workspace(d));
  return attn_bwd_launch(d, a, (float*)workspace, (hipStream_t)stream);
}

// ---- the backward pass for callers that cannot allocate ------------------------------------
// Scratch of the library's own: one float per score row, NBK_ATTN_STATIC_ROWS of them, in a
// file-scope device array (every GPU the library runs on holds its own copy, 4 MiB, until the
// process ends).  In host code the array's name is only a handle: the device address is asked
// for once per device and kept.
static __device__ __align__(256) float attn_scratch[NBK_ATTN_STATIC_ROWS];
#define NBK_MAX_DEVICES 64
static float* g_attn_scratch_ptr[NBK_MAX_DEVICES] = {};
static std::mutex g_attn_scratch_mu;

// The address of this device's copy of the scratch array (the device must be current).
static int attn_scratch_for_current_device(float** out) {
  int dev = -1;
  NBK_HIP(hipGetDevice(&dev));
  NBK_REQUIRE(dev >= 0 && dev < NBK_MAX_DEVICES, "attention: device ordinal %d beyond %d", dev,
              NBK_MAX_DEVICES);
  std::lock_guard<std::mutex> lk(g_attn_scratch_mu);
  if (g_attn_scratch_ptr[dev] == nullptr) {
    float* ptr = nullptr;
    NBK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(attn_scratch)));
    NBK_REQUIRE(ptr != nullptr, "attention: no device address for the scratch array");
    g_attn_scratch_ptr[dev] = ptr;
  }
  *out = g_attn_scratch_ptr[dev];
  return NBK_OK;
}

// Called by nbk_init with the chosen device current.
int nbk_attention_static_setup(void) {
  float* ptr;
  return attn_scratch_for_current_device(&ptr);
}

extern "C" int nbk_attention_bwd_static(const nbk_attn_desc* d, const nbk_attn_tensor* q,
                                        const nbk_attn_tensor* k, const nbk_attn_tensor* v,
                                        const nbk_attn_tensor* o, const nbk_attn_tensor* o_lo,
                                        const void* lse,
                                        const nbk_attn_tensor* dout, const nbk_attn_tensor* dq,
                                        const nbk_attn_tensor* dk, const nbk_attn_tensor* dv,
                                        void* stream) {
  AttnArgs a = {};
  int rc = attn_bwd_args(d, q, k, v, o, o_lo, lse, dout, dq, dk, dv, &a);
  if (rc) return rc;
  const int64_t rows = d->B * d->H * d->S;
  NBK_REQUIRE(rows <= NBK_ATTN_STATIC_ROWS,
              "attention: B * H * S = %lld score rows exceed the %d rows of built-in scratch; use "
              "nbk_attention_bwd with a workspace",
              (long long)rows, NBK_ATTN_STATIC_ROWS);
  float* delta = nullptr;
  if ((rc = attn_scratch_for_current_device(&delta))) return rc;
  // every row of the scratch that the dK / dV kernel reads is written first by the dQ kernel of
  // this call, so nothing has to be cleared between calls
  return attn_bwd_launch(d, a, delta, (hipStream_t)stream);
}

