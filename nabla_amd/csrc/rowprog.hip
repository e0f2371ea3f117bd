// Row-program interpreter: fused elementwise chains and last-axis reductions.
//
// Two launch shapes share one instruction interpreter:
//   * flat  (has_reduce = 0): one lane per 4-column chunk of the rows x C
//     domain, no cross-lane traffic;
//   * block (has_reduce = 1): one workgroup per row.  Lanes sweep the row in
//     4-column chunks (coalesced 16-byte accesses), partial results are
//     combined with 64-wide wavefront shuffles and an LDS tree across the
//     waves of the group.  Rows that are read in more than one phase can be
//     pre-loaded into LDS so HBM sees them once.
//
// Registers live in VGPRs: the 16 vector registers are four 16-wide vectors
// (one per chunk component) indexed with a wave-uniform index, which the
// compiler turns into VGPR-relative moves instead of scratch memory.
#include "nbk_common.h"
#include "rowprog_device.h"
#include "rowprog_spec.h"
#include <stddef.h>
#include <mutex>
#include <unordered_map>

typedef float vf16 __attribute__((ext_vector_type(16)));
typedef float vf4 __attribute__((ext_vector_type(4)));

struct RpRegs {
  vf16 x, y, z, w;  // vector registers 0..15, by chunk component
  vf16 s;           // per-row scalar registers 16..31
  vf4 acc;          // reduction accumulators
};

__device__ __forceinline__ float4 rp_read(const RpRegs& R, int i) {
  if (i < NBK_RP_NVEC) {
    return make_float4(R.x[i], R.y[i], R.z[i], R.w[i]);
  }
  float s = R.s[i - NBK_RP_NVEC];
  return make_float4(s, s, s, s);
}
__device__ __forceinline__ void rp_write(RpRegs& R, int i, float4 v) {
  R.x[i] = v.x; R.y[i] = v.y; R.z[i] = v.z; R.w[i] = v.w;
}

// readfirstlane returns a SIGNED int: widening it directly to 64 bits would
// sign-extend and corrupt the high half of a pointer, so go through uint32_t.
__device__ __forceinline__ uint32_t rp_sgpr(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ uint64_t rp_sgpr64(uint2 v) {
  return (uint64_t)rp_sgpr(v.x) | ((uint64_t)rp_sgpr(v.y) << 32);
}

__device__ __forceinline__ nbk_operand rp_operand(const nbk_rowprog& S, int i, int n_lead);

__host__ __device__ __forceinline__ bool rp_is_unary(int op) {
  return (op >= NBK_OP_MOV && op < NBK_OP_ADD) || op == NBK_OP_DGELU || op == NBK_OP_SIN ||
         op == NBK_OP_COS || (op >= NBK_OP_INEG && op <= NBK_OP_INEZ);
}
__host__ __device__ __forceinline__ bool rp_is_binary(int op) {
  return (op >= NBK_OP_ADD && op < NBK_OP_WHERE) || (op >= NBK_OP_IADD && op <= NBK_OP_ILE);
}
__host__ __device__ __forceinline__ bool rp_is_ew(int op) {
  return rp_is_unary(op) || rp_is_binary(op) || op == NBK_OP_WHERE || op == NBK_OP_FMA;
}

// One body instruction on one chunk.
template <typename IDX>
__device__ __forceinline__ void rp_exec_body(const nbk_rowprog& P, const nbk_ins in, RpRegs& R,
                                             const IDX* lead_idx, int64_t col, int valid,
                                             const float* stage, int64_t c_pad, int n_lead) {
  const int op = in.op;
  if (rp_is_binary(op)) {
    float4 a = rp_read(R, in.a), b = rp_read(R, in.b), r;
    switch (op) {  // the hot ones without a per-component switch
      case NBK_OP_ADD: r = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); break;
      case NBK_OP_SUB: r = make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w); break;
      case NBK_OP_MUL: r = make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); break;
      default:
        r = make_float4(rp_binary(op, a.x, b.x), rp_binary(op, a.y, b.y),
                        rp_binary(op, a.z, b.z), rp_binary(op, a.w, b.w));
    }
    rp_write(R, in.dst, r);
  } else if (rp_is_unary(op)) {
    float4 a = rp_read(R, in.a);
    float4 r = make_float4(rp_unary(op, a.x), rp_unary(op, a.y), rp_unary(op, a.z),
                           rp_unary(op, a.w));
    rp_write(R, in.dst, r);
  } else if (op == NBK_OP_LDG) {
    const nbk_operand o = rp_operand(P, in.a, n_lead);
    float4 r;
    if (o.stage_slot >= 0 && stage != nullptr) {
      r = *(const float4*)(stage + o.stage_slot * c_pad + col);
    } else {
      r = rp_load4(o, rp_row_offset(o, lead_idx, n_lead), col, valid);
    }
    rp_write(R, in.dst, r);
  } else if (op == NBK_OP_STG) {
    const nbk_operand o = rp_operand(P, in.dst, n_lead);
    rp_store4(o, rp_row_offset(o, lead_idx, n_lead), col, valid, rp_read(R, in.a));
  } else if (op == NBK_OP_ACC) {
    float4 a = rp_read(R, in.a);
    const int kind = in.b;
    float v = R.acc[in.dst];
    if (valid > 0) v = rp_combine(v, a.x, kind);
    if (valid > 1) v = rp_combine(v, a.y, kind);
    if (valid > 2) v = rp_combine(v, a.z, kind);
    if (valid > 3) v = rp_combine(v, a.w, kind);
    R.acc[in.dst] = v;
  } else if (op == NBK_OP_WHERE) {
    float4 c = rp_read(R, in.a), a = rp_read(R, in.b), b = rp_read(R, in.c);
    rp_write(R, in.dst, rp_where4(c, a, b));
  } else if (op == NBK_OP_FMA) {
    float4 a = rp_read(R, in.a), b = rp_read(R, in.b), c = rp_read(R, in.c);
    rp_write(R, in.dst, make_float4(fmaf(a.x, b.x, c.x), fmaf(a.y, b.y, c.y),
                                    fmaf(a.z, b.z, c.z), fmaf(a.w, b.w, c.w)));
  } else if (op == NBK_OP_COLIDX) {
    rp_write(R, in.dst, rp_colidx4(col, in.a != 0));
  }
}

// Prologue (per-row, scalar-register) instruction.  Returns through R.
template <typename IDX>
__device__ __forceinline__ void rp_exec_scalar(const nbk_rowprog& P, const nbk_ins in, RpRegs& R,
                                               const IDX* lead_idx, bool writer, float* red_buf,
                                               int n_lead) {
  const int op = in.op;
  const int d = in.dst - NBK_RP_NVEC;
  if (op == NBK_OP_IMM) {
    R.s[d] = __uint_as_float(rp_sgpr(__float_as_uint(P.imm[in.a])));
  } else if (op == NBK_OP_LDR) {
    const nbk_operand o = rp_operand(P, in.a, n_lead);
    R.s[d] = rp_load1(o.ptr, rp_row_offset(o, lead_idx, n_lead), o.dtype);
  } else if (op == NBK_OP_STR) {
    const nbk_operand o = rp_operand(P, in.dst, n_lead);
    if (writer) {
      rp_store1(o.ptr, rp_row_offset(o, lead_idx, n_lead), o.dtype, R.s[in.a - NBK_RP_NVEC]);
    }
  } else if (op == NBK_OP_LEADIDX) {
    const int k = in.a;
    const int li = (int)(k == 0 ? lead_idx[0] : k == 1 ? lead_idx[1] : k == 2 ? lead_idx[2] : lead_idx[3]);
    R.s[d] = in.b != 0 ? rp_ibits(li) : (float)li;
  } else if (op == NBK_OP_ACCINIT) {
    R.acc[in.dst] = rp_identity(in.a);
  } else if (op == NBK_OP_RED) {
    R.s[d] = rp_block_reduce(R.acc[in.a], in.b, red_buf);
  } else if (rp_is_binary(op)) {
    R.s[d] = rp_binary(op, R.s[in.a - NBK_RP_NVEC], R.s[in.b - NBK_RP_NVEC]);
  } else if (rp_is_unary(op)) {
    R.s[d] = rp_unary(op, R.s[in.a - NBK_RP_NVEC]);
  } else if (op == NBK_OP_WHERE) {
    R.s[d] = rp_where(R.s[in.a - NBK_RP_NVEC], R.s[in.b - NBK_RP_NVEC], R.s[in.c - NBK_RP_NVEC]);
  } else if (op == NBK_OP_FMA) {
    R.s[d] = fmaf(R.s[in.a - NBK_RP_NVEC], R.s[in.b - NBK_RP_NVEC], R.s[in.c - NBK_RP_NVEC]);
  }
}

// ---------------------------------------------------------------- program staging
// Kernel arguments live in uncached memory: a scalar load from them costs a full
// memory round trip, far too slow for an instruction stream that is re-read for
// every chunk.  Each workgroup therefore copies the program into LDS once and
// then walks rows persistently; the interpreter fetches instructions and operand
// descriptors from LDS and turns them into scalars with readfirstlane.
#define RP_WORDS ((int)(sizeof(nbk_rowprog) / 4))
static_assert(sizeof(nbk_rowprog) % 4 == 0, "program is copied word by word");
static_assert(sizeof(nbk_operand) % 8 == 0 && offsetof(nbk_rowprog, operand) % 8 == 0 &&
                  offsetof(nbk_operand, col_stride) % 8 == 0 && offsetof(nbk_operand, vec_ok) % 8 == 0,
              "operand descriptors are read from LDS with 8-byte accesses");
static_assert(sizeof(nbk_ins) == 8 && offsetof(nbk_rowprog, ins) % 8 == 0,
              "instructions are read from LDS with 8-byte accesses");

__device__ __forceinline__ void rp_copy_program(const nbk_rowprog& P, uint32_t* dst) {
  const uint32_t* src = reinterpret_cast<const uint32_t*>(&P);
  for (int i = threadIdx.x; i < RP_WORDS; i += blockDim.x) dst[i] = src[i];
  __syncthreads();
}

__device__ __forceinline__ nbk_ins rp_fetch(const nbk_rowprog& S, int q) {
  const uint2 u = *reinterpret_cast<const uint2*>(&S.ins[q]);
  const uint32_t lo = rp_sgpr(u.x);
  const uint32_t hi = rp_sgpr(u.y);
  nbk_ins in;
  in.op = lo & 0xff; in.dst = (lo >> 8) & 0xff; in.a = (lo >> 16) & 0xff; in.b = lo >> 24;
  in.c = hi & 0xff; in.pad = 0; in.aux = (uint16_t)(hi >> 16);
  return in;
}

// Scalar copy of one operand descriptor out of LDS.
__device__ __forceinline__ nbk_operand rp_operand(const nbk_rowprog& S, int i, int n_lead) {
  const nbk_operand& o = S.operand[i];
  nbk_operand r;
  r.ptr = reinterpret_cast<void*>(rp_sgpr64(*reinterpret_cast<const uint2*>(&o.ptr)));
  // descriptors are 56 bytes apart, so only 8-byte alignment is guaranteed here
  const uint2 t0 = *reinterpret_cast<const uint2*>(&o.col_stride);
  const uint2 t1 = *reinterpret_cast<const uint2*>(&o.vec_ok);
  r.col_stride = (int32_t)rp_sgpr(t0.x);
  r.dtype = (int32_t)rp_sgpr(t0.y);
  r.vec_ok = (int32_t)rp_sgpr(t1.x);
  r.stage_slot = (int32_t)rp_sgpr(t1.y);
  // the host zero-fills strides beyond n_lead
  (void)n_lead;
#pragma unroll
  for (int k = 0; k < NBK_RP_MAX_LEAD; ++k) {
    r.lead_stride[k] = (int64_t)rp_sgpr64(*reinterpret_cast<const uint2*>(&o.lead_stride[k]));
  }
  return r;
}

// ---------------------------------------------------------------- block mode
extern __shared__ __align__(16) float rp_stage_lds[];

__global__ __launch_bounds__(512) void rp_block_kernel(const nbk_rowprog P, int64_t rows) {
  __shared__ float red_buf[16];
  __shared__ __align__(16) uint32_t prog_lds[RP_WORDS];
  rp_copy_program(P, prog_lds);
  const nbk_rowprog& S = *reinterpret_cast<const nbk_rowprog*>(prog_lds);
  RpRegs R;
  R.acc = (vf4)(0.f);
  const int64_t C = P.C;
  const int64_t c_pad = (C + 3) & ~(int64_t)3;
  const int64_t n_chunks = c_pad >> 2;
  const int n_lead = P.n_lead;
  const int n_ins = P.n_ins;
  const int n_operands = P.n_operands;
  const int n_stage = P.n_stage;
  int64_t lead_dim[NBK_RP_MAX_LEAD];
#pragma unroll
  for (int k = 0; k < NBK_RP_MAX_LEAD; ++k) lead_dim[k] = P.lead_dim[k];
  const float* stage = n_stage > 0 ? rp_stage_lds : nullptr;
  const bool writer = threadIdx.x == 0;

  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    // decompose the row index over the leading dims (wave-uniform)
    // unused leading dims have extent 1, so the same three divisions serve every n_lead
    int64_t lead_idx[NBK_RP_MAX_LEAD];
    {
      int64_t rem = row, q;
      q = rem / lead_dim[3]; lead_idx[3] = rem - q * lead_dim[3]; rem = q;
      q = rem / lead_dim[2]; lead_idx[2] = rem - q * lead_dim[2]; rem = q;
      q = rem / lead_dim[1]; lead_idx[1] = rem - q * lead_dim[1]; rem = q;
      lead_idx[0] = rem;
    }

    // pre-load staged operands: every lane stages exactly the chunks it will
    // later read back, so no barrier is needed between the two.
    if (n_stage > 0) {
      for (int oi = 0; oi < n_operands; ++oi) {
        const nbk_operand o = rp_operand(S, oi, n_lead);
        if (o.stage_slot < 0) continue;
        rp_stage_row(o, rp_row_offset(o, lead_idx, n_lead), rp_stage_lds + o.stage_slot * c_pad, C,
                     n_chunks);
      }
    }

    int pc = 0;
    while (pc < n_ins) {
      const nbk_ins in = rp_fetch(S, pc);
      if (in.op == NBK_OP_HALT) break;
      if (in.op == NBK_OP_BODY) {
        const int b0 = pc + 1, b1 = pc + 1 + in.aux;
        for (int64_t ch = threadIdx.x; ch < n_chunks; ch += blockDim.x) {
          const int64_t col = ch << 2;
          const int64_t left = C - col;
          const int valid = left >= 4 ? 4 : (int)left;
          nbk_ins nxt = rp_fetch(S, b0);
#pragma unroll 1
          for (int q = b0; q < b1; ++q) {
            const nbk_ins cur = nxt;
            if (q + 1 < b1) nxt = rp_fetch(S, q + 1);  // fetch ahead of the decode
            rp_exec_body(S, cur, R, lead_idx, col, valid, stage, c_pad, n_lead);
          }
        }
        pc = b1;
      } else {
        rp_exec_scalar(S, in, R, lead_idx, writer, red_buf, n_lead);
        ++pc;
      }
    }
    // rows reuse the staging buffer and red_buf; RED already ends with a barrier,
    // the staging area is private per lane, so no extra barrier is needed here
  }
}

// ----------------------------------------------------------------- flat mode
__global__ __launch_bounds__(256) void rp_flat_kernel(const nbk_rowprog P, uint32_t cpr,
                                                      uint64_t total_chunks) {
  __shared__ __align__(16) uint32_t prog_lds[RP_WORDS];
  rp_copy_program(P, prog_lds);
  const nbk_rowprog& S = *reinterpret_cast<const nbk_rowprog*>(prog_lds);
  RpRegs R;
  R.acc = (vf4)(0.f);
  const int n_lead = P.n_lead;
  const int n_ins = P.n_ins;
  const int64_t C = P.C;
  uint32_t lead_dim[NBK_RP_MAX_LEAD];
#pragma unroll
  for (int k = 0; k < NBK_RP_MAX_LEAD; ++k) lead_dim[k] = (uint32_t)P.lead_dim[k];
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t g = (uint64_t)blockIdx.x * 256u + threadIdx.x; g < total_chunks; g += stride) {
    uint32_t row, cc;
    if (cpr == 1) { row = (uint32_t)g; cc = 0; }
    else if (total_chunks <= cpr) { row = 0; cc = (uint32_t)g; }
    else { row = (uint32_t)(g / cpr); cc = (uint32_t)(g - (uint64_t)row * cpr); }
    uint32_t lead_idx[NBK_RP_MAX_LEAD] = {0, 0, 0, 0};
    if (n_lead > 0) {
      uint32_t rem = row, q;
      q = rem / lead_dim[3]; lead_idx[3] = rem - q * lead_dim[3]; rem = q;
      q = rem / lead_dim[2]; lead_idx[2] = rem - q * lead_dim[2]; rem = q;
      q = rem / lead_dim[1]; lead_idx[1] = rem - q * lead_dim[1]; rem = q;
      lead_idx[0] = rem;
    }
    const int64_t col = (int64_t)cc << 2;
    const int64_t left = C - col;
    const int valid = left >= 4 ? 4 : (int)left;
    int pc = 0;
    while (pc < n_ins) {
      const nbk_ins in = rp_fetch(S, pc);
      if (in.op == NBK_OP_HALT) break;
      if (in.op == NBK_OP_BODY) {
        const int b1 = pc + 1 + in.aux;
        nbk_ins nxt = rp_fetch(S, pc + 1);
#pragma unroll 1
        for (int q = pc + 1; q < b1; ++q) {
          const nbk_ins cur = nxt;
          if (q + 1 < b1) nxt = rp_fetch(S, q + 1);
          rp_exec_body(S, cur, R, lead_idx, col, valid, nullptr, 0, n_lead);
        }
        pc = b1;
      } else {
        // one lane per row writes row scalars: the lane that owns chunk 0
        rp_exec_scalar(S, in, R, lead_idx, cc == 0, nullptr, n_lead);
        ++pc;
      }
    }
  }
}

// ------------------------------------------------------------------ host side
static int rp_validate(const nbk_rowprog* p) {
  NBK_REQUIRE(p != nullptr, "rowprog: null program");
  NBK_REQUIRE(p->n_lead >= 0 && p->n_lead <= NBK_RP_MAX_LEAD, "rowprog: n_lead %d out of range",
              p->n_lead);
  NBK_REQUIRE(p->n_operands >= 0 && p->n_operands <= NBK_RP_MAX_OPERANDS,
              "rowprog: %d operands exceed the limit %d", p->n_operands, NBK_RP_MAX_OPERANDS);
  NBK_REQUIRE(p->n_ins > 0 && p->n_ins <= NBK_RP_MAX_INS, "rowprog: %d instructions (limit %d)",
              p->n_ins, NBK_RP_MAX_INS);
  NBK_REQUIRE(p->n_imm >= 0 && p->n_imm <= NBK_RP_MAX_IMM, "rowprog: %d immediates (limit %d)",
              p->n_imm, NBK_RP_MAX_IMM);
  NBK_REQUIRE(p->C > 0, "rowprog: row length %lld", (long long)p->C);
  for (int k = 0; k < p->n_lead; ++k)
    NBK_REQUIRE(p->lead_dim[k] > 0, "rowprog: leading dim %d is %lld", k,
                (long long)p->lead_dim[k]);
  for (int i = 0; i < p->n_operands; ++i) {
    const nbk_operand& o = p->operand[i];
    NBK_REQUIRE(o.ptr != nullptr, "rowprog: operand %d has a null pointer", i);
    NBK_REQUIRE(nbk_dtype_size(o.dtype) > 0, "rowprog: operand %d has dtype %d", i, o.dtype);
    NBK_REQUIRE(o.stage_slot < NBK_RP_MAX_STAGE, "rowprog: operand %d stage slot %d", i,
                o.stage_slot);
    if (o.vec_ok) {
      NBK_REQUIRE(o.col_stride == 1, "rowprog: operand %d vec_ok needs unit column stride", i);
      const int64_t a = 4 * nbk_dtype_size(o.dtype);
      NBK_REQUIRE(((uintptr_t)o.ptr % (uintptr_t)a) == 0,
                  "rowprog: operand %d pointer not aligned for 4-wide access", i);
      for (int k = 0; k < p->n_lead; ++k)
        NBK_REQUIRE(o.lead_stride[k] % 4 == 0,
                    "rowprog: operand %d lead stride %d not a multiple of 4", i, k);
    }
  }
  // instruction stream: register / operand indices in range, bodies closed
  int pc = 0;
  bool halted = false;
  while (pc < p->n_ins) {
    const nbk_ins in = p->ins[pc];
    if (in.op == NBK_OP_HALT) { halted = true; break; }
    if (in.op == NBK_OP_BODY) {
      NBK_REQUIRE(pc + 1 + in.aux <= p->n_ins, "rowprog: body at %d runs past the end", pc);
      for (int q = pc + 1; q < pc + 1 + in.aux; ++q) {
        const nbk_ins b = p->ins[q];
        const int op = b.op;
        if (op == NBK_OP_LDG) {
          NBK_REQUIRE(b.a < p->n_operands && b.dst < NBK_RP_NVEC, "rowprog: bad LDG at %d", q);
        } else if (op == NBK_OP_STG) {
          NBK_REQUIRE(b.dst < p->n_operands && b.a < 32, "rowprog: bad STG at %d", q);
        } else if (op == NBK_OP_ACC) {
          NBK_REQUIRE(p->has_reduce && b.dst < NBK_RP_NACC && b.a < 32 && b.b <= NBK_RED_MIN,
                      "rowprog: bad ACC at %d", q);
        } else if (op == NBK_OP_COLIDX) {
          NBK_REQUIRE(b.dst < NBK_RP_NVEC, "rowprog: bad COLIDX at %d", q);
        } else if (rp_is_ew(op)) {
          NBK_REQUIRE(b.dst < NBK_RP_NVEC && b.a < 32 && b.b < 32 && b.c < 32,
                      "rowprog: bad register at %d", q);
        } else {
          NBK_REQUIRE(false, "rowprog: opcode %d not allowed in a body (at %d)", op, q);
        }
      }
      pc += 1 + in.aux;
      continue;
    }
    const int op = in.op;
    const bool sreg_dst = in.dst >= NBK_RP_NVEC && in.dst < 32;
    if (op == NBK_OP_IMM) {
      NBK_REQUIRE(sreg_dst && in.a < p->n_imm, "rowprog: bad IMM at %d", pc);
    } else if (op == NBK_OP_LDR) {
      NBK_REQUIRE(sreg_dst && in.a < p->n_operands, "rowprog: bad LDR at %d", pc);
    } else if (op == NBK_OP_STR) {
      NBK_REQUIRE(in.dst < p->n_operands && in.a >= NBK_RP_NVEC && in.a < 32,
                  "rowprog: bad STR at %d", pc);
    } else if (op == NBK_OP_LEADIDX) {
      NBK_REQUIRE(sreg_dst && in.a < p->n_lead, "rowprog: bad LEADIDX at %d", pc);
    } else if (op == NBK_OP_ACCINIT) {
      NBK_REQUIRE(in.dst < NBK_RP_NACC && in.a <= NBK_RED_MIN, "rowprog: bad ACCINIT at %d", pc);
    } else if (op == NBK_OP_RED) {
      NBK_REQUIRE(p->has_reduce && sreg_dst && in.a < NBK_RP_NACC && in.b <= NBK_RED_MIN,
                  "rowprog: bad RED at %d", pc);
    } else if (rp_is_ew(op)) {
      NBK_REQUIRE(sreg_dst && in.a >= NBK_RP_NVEC && in.a < 32, "rowprog: bad scalar op at %d",
                  pc);
      if (!rp_is_unary(op))
        NBK_REQUIRE(in.b >= NBK_RP_NVEC && in.b < 32, "rowprog: bad scalar op at %d", pc);
      if (op == NBK_OP_WHERE || op == NBK_OP_FMA)
        NBK_REQUIRE(in.c >= NBK_RP_NVEC && in.c < 32, "rowprog: bad scalar op at %d", pc);
    } else {
      NBK_REQUIRE(false, "rowprog: opcode %d not allowed in a prologue (at %d)", op, pc);
    }
    ++pc;
  }
  NBK_REQUIRE(halted, "rowprog: program has no HALT");
  return NBK_OK;
}

// ---- specialised kernels -------------------------------------------------------
// FNV-1a over the canonical bytes of a program (same bytes as program_bytes() in
// nabla_amd/backend/specialize.py): header, per-operand (dtype, stride class,
// vec_ok, stage slot), instructions, immediates.  Extents and addresses are not
// part of it -- a specialised kernel serves every size.
static uint64_t rp_program_hash(const nbk_rowprog* p) {
  uint64_t h = 0xCBF29CE484222325ULL;
  auto eat = [&](const void* data, size_t n) {
    const uint8_t* b = (const uint8_t*)data;
    for (size_t i = 0; i < n; ++i) h = (h ^ b[i]) * 0x100000001B3ULL;
  };
  const uint8_t head[6] = {(uint8_t)(p->has_reduce ? 1 : 0), (uint8_t)p->n_operands,
                           (uint8_t)(p->n_ins & 0xff), (uint8_t)(p->n_ins >> 8),
                           (uint8_t)p->n_imm, (uint8_t)p->n_stage};
  eat(head, 6);
  for (int i = 0; i < p->n_operands; ++i) {
    const nbk_operand& o = p->operand[i];
    const uint8_t ob[4] = {(uint8_t)o.dtype,
                           (uint8_t)(o.col_stride == 0 ? 0 : (o.col_stride == 1 ? 1 : 2)),
                           (uint8_t)(o.vec_ok ? 1 : 0), (uint8_t)(int8_t)o.stage_slot};
    eat(ob, 4);
  }
  for (int i = 0; i < p->n_ins; ++i) {
    const nbk_ins& in = p->ins[i];
    const uint8_t ib[8] = {in.op, in.dst, in.a, in.b, in.c, 0, (uint8_t)(in.aux & 0xff),
                           (uint8_t)(in.aux >> 8)};
    eat(ib, 8);
  }
  eat(p->imm, sizeof(float) * (size_t)p->n_imm);
  return h;
}

struct RpSpec {
  const void* kernel[5];
  const void* kernel_full[5];
  const void* kernel_stream[5];
  const void* kernel_flat;
  const void* kernel_stage16;
  const rp_hand_entry* hand;
  int block_mode;
  bool lds_attr_set;
  bool lds16_attr_set;
};
static std::mutex g_spec_mu;
static std::unordered_map<uint64_t, RpSpec>* g_specs = nullptr;

static RpSpec* rp_find_spec(uint64_t h) {
  std::lock_guard<std::mutex> lk(g_spec_mu);
  if (!g_specs) {
    g_specs = new std::unordered_map<uint64_t, RpSpec>();
    const rp_spec_entry* tabs[NBK_RP_SPEC_FILES] = {rp_spec_table_0, rp_spec_table_1,
                                                   rp_spec_table_2, rp_spec_table_3};
    const int counts[NBK_RP_SPEC_FILES] = {rp_spec_count_0, rp_spec_count_1, rp_spec_count_2,
                                           rp_spec_count_3};
    for (int t = 0; t < NBK_RP_SPEC_FILES; ++t)
      for (int i = 0; i < counts[t]; ++i)
      {
        RpSpec e;
        for (int k = 0; k < 5; ++k) {
          e.kernel[k] = tabs[t][i].kernel[k];
          e.kernel_full[k] = tabs[t][i].kernel_full[k];
          e.kernel_stream[k] = tabs[t][i].kernel_stream[k];
        }
        e.kernel_flat = tabs[t][i].kernel_flat;
        e.kernel_stage16 = tabs[t][i].kernel_stage16;
        e.block_mode = tabs[t][i].block_mode;
        e.lds_attr_set = false;
        e.lds16_attr_set = false;
        e.hand = nullptr;
        (*g_specs)[tabs[t][i].hash] = e;
      }
    // (a hand-scheduled kernel stands beside generated ones, which take the launches it declines)
    for (int i = 0; i < rp_hand_count; ++i) {
      auto it = g_specs->find(rp_hand_table[i].hash);
      if (it != g_specs->end()) it->second.hand = &rp_hand_table[i];
    }
  }
  auto it = g_specs->find(h);
  return it == g_specs->end() ? nullptr : &it->second;
}

// Resident workgroups per CU of a kernel at a block size (no dynamic LDS); cached.
static int rp_occupancy(const void* fn, int block, int* out) {
  static std::mutex mu;
  static std::unordered_map<uint64_t, int>* cache = nullptr;
  const uint64_t key = (uint64_t)(uintptr_t)fn ^ ((uint64_t)block << 48);
  std::lock_guard<std::mutex> lk(mu);
  if (!cache) cache = new std::unordered_map<uint64_t, int>();
  auto it = cache->find(key);
  if (it == cache->end()) {
    int n = 0;
    NBK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, block, 0));
    if (n < 1) n = 1;
    it = cache->emplace(key, n).first;
  }
  *out = it->second;
  return NBK_OK;
}

// 1: interpreter only (debug / comparison); read once.
static bool rp_specs_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("NBK_ROWPROG_INTERPRET");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

// 1: generated kernels only (comparison of a hand-scheduled kernel with them); read once.
static bool rp_hand_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("NBK_ROWPROG_HAND");
    v = (e && e[0] == '0') ? 1 : 0;
  }
  return v == 1;
}

extern "C" int nbk_rowprog_is_specialized(const nbk_rowprog* prog) {
  if (rp_validate(prog) != NBK_OK || rp_specs_disabled()) return 0;
  RpSpec* spec = rp_find_spec(rp_program_hash(prog));
  if (!spec) return 0;
  return (spec->hand && !rp_hand_disabled() && spec->hand->fits(prog)) ? 2 : 1;
}

extern "C" uint64_t nbk_rowprog_hash(const nbk_rowprog* prog) {
  if (rp_validate(prog) != NBK_OK) return 0;
  return rp_program_hash(prog);
}

extern "C" int nbk_rowprog_launch(const nbk_rowprog* prog, void* stream) {
  int rc = rp_validate(prog);
  if (rc != NBK_OK) return rc;
  // normalised copy: unused leading dims get extent 1 and stride 0 so the kernels
  // can index all four unconditionally
  nbk_rowprog norm = *prog;
  for (int k = norm.n_lead; k < NBK_RP_MAX_LEAD; ++k) {
    norm.lead_dim[k] = 1;
    for (int i = 0; i < norm.n_operands; ++i) norm.operand[i].lead_stride[k] = 0;
  }
  const nbk_rowprog* p = &norm;
  RpSpec* spec = (rp_specs_disabled() || prog->reserved == 1) ? nullptr
                                                               : rp_find_spec(rp_program_hash(prog));
  if (spec && spec->block_mode != (p->has_reduce ? 1 : 0)) spec = nullptr;
  hipStream_t st = (hipStream_t)stream;
  int64_t rows = 1;
  for (int k = 0; k < p->n_lead; ++k) rows *= p->lead_dim[k];
  if (p->has_reduce) {
    const int block = p->block;
    NBK_REQUIRE(block >= 64 && block <= 512 && (block & (block - 1)) == 0,
                "rowprog: workgroup size %d must be a power of two in [64, 512]", block);
    NBK_REQUIRE(rows <= 0x7fffffffLL, "rowprog: %lld rows exceed the grid limit", (long long)rows);
    const int64_t c_pad = (p->C + 3) & ~(int64_t)3;
    size_t lds = (size_t)p->n_stage * (size_t)c_pad * sizeof(float);
    NBK_REQUIRE(p->n_stage >= 0 && p->n_stage <= NBK_RP_MAX_STAGE, "rowprog: n_stage %d",
                p->n_stage);
    NBK_REQUIRE(lds <= 64 * 1024, "rowprog: staging %zu bytes of LDS exceeds 64 KiB", lds);
    if (lds > 32 * 1024) {
      // static (program copy) + dynamic (staging) LDS exceeds the 64 KiB default cap
      static bool attr_set = false;  // idempotent, a race only repeats the call
      if (!attr_set) {
        NBK_HIP(hipFuncSetAttribute((const void*)rp_block_kernel,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
        attr_set = true;
      }
    }
    // persistent workgroups: enough to fill every CU at this block size / LDS use
    const int per_cu = lds > 48 * 1024 ? 2 : (block >= 512 ? 2 : (block >= 256 ? 4 : 8));
    int64_t grid = (int64_t)nbk_num_cus() * per_cu;
    if (grid > rows) grid = rows;
    if (spec) {
      int64_t rows_arg = rows;
      void* args[2] = {(void*)p, (void*)&rows_arg};
      if (spec->hand && !rp_hand_disabled() && spec->hand->fits(p)) {
        int64_t bytes = 0;
        for (int i = 0; i < p->n_operands; ++i)
          if (p->operand[i].col_stride != 0)
            bytes += rows * p->C * (int64_t)nbk_dtype_size(p->operand[i].dtype);
        const void* fn = bytes > (256ll << 20) ? spec->hand->kernel_stream : spec->hand->kernel;
        int per_cu = 0;
        { const int orc = rp_occupancy(fn, spec->hand->block, &per_cu); if (orc != NBK_OK) return orc; }
        int64_t g2 = (int64_t)nbk_num_cus() * per_cu;
        if (g2 > rows) g2 = rows;
        NBK_HIP(hipLaunchKernel(fn, dim3((unsigned)g2), dim3(spec->hand->block), args, 0, st));
        return NBK_OK;
      }
      // register-resident form: lanes own ceil(chunks / block) chunks each
      const int64_t n_chunks = c_pad >> 2;
      const int64_t need = (n_chunks + block - 1) / block;
      int slot = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 3 : need <= 8 ? 4 : 0;
      if (slot && spec->kernel[slot]) {
        static const int cpt_of[5] = {0, 1, 2, 4, 8};
        const bool full = p->C == (int64_t)4 * cpt_of[slot] * block && spec->kernel_full[slot];
        const void* fn = spec->kernel[slot];
        if (full) {
          // bytes of the row-shaped operands; beyond the 256 MiB last-level cache nothing
          // written here survives until a consumer runs, so stream it
          int64_t bytes = 0;
          for (int i = 0; i < p->n_operands; ++i)
            if (p->operand[i].col_stride != 0)
              bytes += rows * p->C * (int64_t)nbk_dtype_size(p->operand[i].dtype);
          fn = (bytes > (256ll << 20) && spec->kernel_stream[slot]) ? spec->kernel_stream[slot]
                                                                    : spec->kernel_full[slot];
        }
        // persistent workgroups, exactly as many as are resident at once: the program
        // descriptor is read from kernel-argument memory once per workgroup, not once per
        // row, and no second partial wave of workgroups trails behind the first
        int per_cu = 0;
        { const int orc = rp_occupancy(fn, block, &per_cu); if (orc != NBK_OK) return orc; }
        int64_t g2 = (int64_t)nbk_num_cus() * per_cu;
        if (g2 > rows) g2 = rows;
        NBK_HIP(hipLaunchKernel(fn, dim3((unsigned)g2), dim3(block), args, 0, st));
        return NBK_OK;
      }
      if (spec->kernel_stage16 && p->n_stage == 0 && (p->C & 3) == 0 && c_pad * 2 <= 64000) {
        // a long 16-bit row that several phases read: one copy in LDS as stored, two
        // workgroups per CU so that one row's traffic overlaps the other's arithmetic
        if (!spec->lds16_attr_set) {
          NBK_HIP(hipFuncSetAttribute(spec->kernel_stage16, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      64 * 1024));
          spec->lds16_attr_set = true;
        }
        int64_t g2 = (int64_t)nbk_num_cus() * 2;
        if (g2 > rows) g2 = rows;
        NBK_HIP(hipLaunchKernel(spec->kernel_stage16, dim3((unsigned)g2), dim3(block), args,
                                (size_t)c_pad * 2, st));
        return NBK_OK;
      }
      if (lds > 32 * 1024 && !spec->lds_attr_set) {
        NBK_HIP(hipFuncSetAttribute(spec->kernel[0], hipFuncAttributeMaxDynamicSharedMemorySize,
                                    64 * 1024));
        spec->lds_attr_set = true;
      }
      NBK_HIP(hipLaunchKernel(spec->kernel[0], dim3((unsigned)grid), dim3(block), args, lds, st));
      return NBK_OK;
    }
    hipLaunchKernelGGL(rp_block_kernel, dim3((unsigned)grid), dim3(block), lds, st, *p, rows);
    return nbk_check_launch("rp_block_kernel");
  }
  NBK_REQUIRE(rows <= 0xffffffffLL, "rowprog: %lld rows exceed 2^32", (long long)rows);
  for (int k = 0; k < p->n_lead; ++k)
    NBK_REQUIRE(p->lead_dim[k] <= 0xffffffffLL, "rowprog: leading dim too large");
  const uint64_t cpr = (uint64_t)((p->C + 3) >> 2);
  NBK_REQUIRE(cpr <= 0xffffffffULL, "rowprog: row too long for a flat launch");
  const uint64_t total = (uint64_t)rows * cpr;
  uint64_t blocks = (total + 255) / 256;
  const uint64_t cap = (uint64_t)nbk_num_cus() * 8;
  if (blocks > cap) blocks = cap;
  if (spec) {
    uint32_t cpr_arg = (uint32_t)cpr;
    uint64_t total_arg = total;
    void* args[3] = {(void*)p, (void*)&cpr_arg, (void*)&total_arg};
    const void* fn = (rows == 1 && spec->kernel_flat) ? spec->kernel_flat : spec->kernel[0];
    NBK_HIP(hipLaunchKernel(fn, dim3((unsigned)blocks), dim3(256), args, 0, st));
    return NBK_OK;
  }
  hipLaunchKernelGGL(rp_flat_kernel, dim3((unsigned)blocks), dim3(256), 0, st, *p, (uint32_t)cpr,
                     total);
  return nbk_check_launch("rp_flat_kernel");
}
