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
#include <stddef.h>

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

__device__ __forceinline__ float rp_combine(float a, float b, int kind) {
  if (kind == NBK_RED_SUM) return a + b;
  if (kind == NBK_RED_MAX) return fmaxf(a, b);
  return fminf(a, b);
}
__device__ __forceinline__ float rp_identity(int kind) {
  if (kind == NBK_RED_SUM) return 0.0f;
  if (kind == NBK_RED_MAX) return -INFINITY;
  return INFINITY;
}

// ---- chunk load / store ----------------------------------------------------
__device__ __forceinline__ float4 rp_load4(const nbk_operand& o, int64_t off, int64_t col,
                                           int valid) {
  const int dt = o.dtype;
  const int64_t cs = o.col_stride;
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  if (o.vec_ok && valid == 4) {
    const int64_t e = off + col;
    if (dt == NBK_F32) {
      r = *(const float4*)((const float*)o.ptr + e);
    } else if (dt == NBK_BF16) {
      uint2 u = *(const uint2*)((const uint16_t*)o.ptr + e);
      r.x = __uint_as_float(u.x << 16);
      r.y = __uint_as_float(u.x & 0xffff0000u);
      r.z = __uint_as_float(u.y << 16);
      r.w = __uint_as_float(u.y & 0xffff0000u);
    } else if (dt == NBK_F16) {
      const __half* h = (const __half*)o.ptr + e;
      uint2 u = *(const uint2*)h;
      __half2 a = *(__half2*)&u.x, b = *(__half2*)&u.y;
      float2 fa = __half22float2(a), fb = __half22float2(b);
      r = make_float4(fa.x, fa.y, fb.x, fb.y);
    } else if (dt == NBK_I32) {
      int4 u = *(const int4*)((const int32_t*)o.ptr + e);
      r = make_float4((float)u.x, (float)u.y, (float)u.z, (float)u.w);
    } else if (dt == NBK_I64) {
      const int64_t* p = (const int64_t*)o.ptr + e;
      longlong2 u0 = *(const longlong2*)p, u1 = *(const longlong2*)(p + 2);
      r = make_float4((float)u0.x, (float)u0.y, (float)u1.x, (float)u1.y);
    } else {
      uint32_t u = *(const uint32_t*)((const uint8_t*)o.ptr + e);
      r = make_float4((float)(u & 0xff), (float)((u >> 8) & 0xff), (float)((u >> 16) & 0xff),
                      (float)(u >> 24));
    }
    return r;
  }
  const int64_t e0 = off + col * cs;
  if (valid > 0) r.x = nbk_load_as_f32(o.ptr, e0, dt);
  if (cs == 0) {
    r.y = r.z = r.w = r.x;
    return r;
  }
  if (valid > 1) r.y = nbk_load_as_f32(o.ptr, e0 + cs, dt);
  if (valid > 2) r.z = nbk_load_as_f32(o.ptr, e0 + 2 * cs, dt);
  if (valid > 3) r.w = nbk_load_as_f32(o.ptr, e0 + 3 * cs, dt);
  return r;
}

__device__ __forceinline__ void rp_store4(const nbk_operand& o, int64_t off, int64_t col,
                                          int valid, float4 v) {
  const int dt = o.dtype;
  const int64_t cs = o.col_stride;
  if (o.vec_ok && valid == 4) {
    const int64_t e = off + col;
    if (dt == NBK_F32) {
      *(float4*)((float*)o.ptr + e) = v;
    } else if (dt == NBK_BF16) {
      uint2 u;
      u.x = (uint32_t)nbk_f32_to_bf16(v.x) | ((uint32_t)nbk_f32_to_bf16(v.y) << 16);
      u.y = (uint32_t)nbk_f32_to_bf16(v.z) | ((uint32_t)nbk_f32_to_bf16(v.w) << 16);
      *(uint2*)((uint16_t*)o.ptr + e) = u;
    } else if (dt == NBK_F16) {
      __half2 a = __floats2half2_rn(v.x, v.y), b = __floats2half2_rn(v.z, v.w);
      uint2 u;
      u.x = *(uint32_t*)&a;
      u.y = *(uint32_t*)&b;
      *(uint2*)((__half*)o.ptr + e) = u;
    } else if (dt == NBK_I32) {
      *(int4*)((int32_t*)o.ptr + e) = make_int4((int)v.x, (int)v.y, (int)v.z, (int)v.w);
    } else if (dt == NBK_I64) {
      int64_t* p = (int64_t*)o.ptr + e;
      p[0] = (int64_t)v.x; p[1] = (int64_t)v.y; p[2] = (int64_t)v.z; p[3] = (int64_t)v.w;
    } else {
      uint32_t u = (uint32_t)(v.x != 0.f) | ((uint32_t)(v.y != 0.f) << 8) |
                   ((uint32_t)(v.z != 0.f) << 16) | ((uint32_t)(v.w != 0.f) << 24);
      *(uint32_t*)((uint8_t*)o.ptr + e) = u;
    }
    return;
  }
  const int64_t e0 = off + col * cs;
  if (valid > 0) nbk_store_from_f32(o.ptr, e0, dt, v.x);
  if (valid > 1) nbk_store_from_f32(o.ptr, e0 + cs, dt, v.y);
  if (valid > 2) nbk_store_from_f32(o.ptr, e0 + 2 * cs, dt, v.z);
  if (valid > 3) nbk_store_from_f32(o.ptr, e0 + 3 * cs, dt, v.w);
}

// ---- elementwise functions --------------------------------------------------


__device__ __forceinline__ float rp_unary(int op, float a) {
  switch (op) {
    case NBK_OP_MOV: return a;
    case NBK_OP_NEG: return -a;
    case NBK_OP_RELU: return fmaxf(a, 0.0f);
    case NBK_OP_EXP: return expf(a);
    case NBK_OP_LOG: return logf(a);
    case NBK_OP_SQRT: return sqrtf(a);
    case NBK_OP_RSQRT: return 1.0f / sqrtf(a);
    case NBK_OP_ERF: return erff(a);
    case NBK_OP_GELU: return 0.5f * a * (1.0f + erff(a * 0.70710678118654752440f));
    case NBK_OP_TANH: return tanhf(a);
    case NBK_OP_SIGMOID: return 1.0f / (1.0f + expf(-a));
    case NBK_OP_ABS: return fabsf(a);
    case NBK_OP_RBF16: return nbk_bf16_to_f32(nbk_f32_to_bf16(a));
    case NBK_OP_NOT: return a != 0.0f ? 0.0f : 1.0f;
    case NBK_OP_TRUNC: return truncf(a);
    case NBK_OP_NEZ: return a != 0.0f ? 1.0f : 0.0f;
    default: return a;
  }
}
__device__ __forceinline__ float rp_binary(int op, float a, float b) {
  switch (op) {
    case NBK_OP_ADD: return a + b;
    case NBK_OP_SUB: return a - b;
    case NBK_OP_MUL: return a * b;
    case NBK_OP_DIV: return a / b;
    case NBK_OP_MAX: return fmaxf(a, b);
    case NBK_OP_MIN: return fminf(a, b);
    case NBK_OP_GT: return a > b ? 1.0f : 0.0f;
    case NBK_OP_GE: return a >= b ? 1.0f : 0.0f;
    case NBK_OP_EQ: return a == b ? 1.0f : 0.0f;
    case NBK_OP_NE: return a != b ? 1.0f : 0.0f;
    case NBK_OP_LT: return a < b ? 1.0f : 0.0f;
    case NBK_OP_LE: return a <= b ? 1.0f : 0.0f;
    case NBK_OP_POW: return powf(a, b);
    case NBK_OP_AND: return (a != 0.0f && b != 0.0f) ? 1.0f : 0.0f;
    case NBK_OP_OR: return (a != 0.0f || b != 0.0f) ? 1.0f : 0.0f;
    default: return a;
  }
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

// Offset of the current row inside one operand.  Strides and indices beyond
// n_lead are zero, so all four terms can be added unconditionally (constant
// indices keep both arrays in registers).
template <typename IDX>
__device__ __forceinline__ int64_t rp_row_offset(const nbk_operand& o, const IDX* lead_idx,
                                                 int n_lead) {
  (void)n_lead;
  return (int64_t)lead_idx[0] * o.lead_stride[0] + (int64_t)lead_idx[1] * o.lead_stride[1] +
         (int64_t)lead_idx[2] * o.lead_stride[2] + (int64_t)lead_idx[3] * o.lead_stride[3];
}

// One body instruction on one chunk.
template <typename IDX>
__device__ __forceinline__ void rp_exec_body(const nbk_rowprog& P, const nbk_ins in, RpRegs& R,
                                             const IDX* lead_idx, int64_t col, int valid,
                                             const float* stage, int64_t c_pad, int n_lead) {
  const int op = in.op;
  if (op >= NBK_OP_ADD && op < NBK_OP_WHERE) {
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
  } else if (op >= NBK_OP_MOV && op < NBK_OP_ADD) {
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
    rp_write(R, in.dst, make_float4(c.x != 0.f ? a.x : b.x, c.y != 0.f ? a.y : b.y,
                                    c.z != 0.f ? a.z : b.z, c.w != 0.f ? a.w : b.w));
  } else if (op == NBK_OP_FMA) {
    float4 a = rp_read(R, in.a), b = rp_read(R, in.b), c = rp_read(R, in.c);
    rp_write(R, in.dst, make_float4(fmaf(a.x, b.x, c.x), fmaf(a.y, b.y, c.y),
                                    fmaf(a.z, b.z, c.z), fmaf(a.w, b.w, c.w)));
  } else if (op == NBK_OP_COLIDX) {
    float c0 = (float)col;
    rp_write(R, in.dst, make_float4(c0, c0 + 1.f, c0 + 2.f, c0 + 3.f));
  }
}

// Block-wide reduction of one float: wavefront shuffles, then an LDS tree.
__device__ __forceinline__ float rp_block_reduce(float v, int kind, float* red_buf) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = rp_combine(v, __shfl_xor(v, off, 64), kind);
  const int nw = blockDim.x >> 6;
  if (nw == 1) return v;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) red_buf[w] = v;
  __syncthreads();
  float r = red_buf[0];
  for (int i = 1; i < nw; ++i) r = rp_combine(r, red_buf[i], kind);
  __syncthreads();
  return r;
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
    R.s[d] = nbk_load_as_f32(o.ptr, rp_row_offset(o, lead_idx, n_lead), o.dtype);
  } else if (op == NBK_OP_STR) {
    const nbk_operand o = rp_operand(P, in.dst, n_lead);
    if (writer) {
      nbk_store_from_f32(o.ptr, rp_row_offset(o, lead_idx, n_lead), o.dtype,
                         R.s[in.a - NBK_RP_NVEC]);
    }
  } else if (op == NBK_OP_LEADIDX) {
    const int k = in.a;
    R.s[d] = (float)(k == 0 ? lead_idx[0] : k == 1 ? lead_idx[1] : k == 2 ? lead_idx[2] : lead_idx[3]);
  } else if (op == NBK_OP_ACCINIT) {
    R.acc[in.dst] = rp_identity(in.a);
  } else if (op == NBK_OP_RED) {
    R.s[d] = rp_block_reduce(R.acc[in.a], in.b, red_buf);
  } else if (op >= NBK_OP_ADD && op < NBK_OP_WHERE) {
    R.s[d] = rp_binary(op, R.s[in.a - NBK_RP_NVEC], R.s[in.b - NBK_RP_NVEC]);
  } else if (op >= NBK_OP_MOV && op < NBK_OP_ADD) {
    R.s[d] = rp_unary(op, R.s[in.a - NBK_RP_NVEC]);
  } else if (op == NBK_OP_WHERE) {
    R.s[d] = R.s[in.a - NBK_RP_NVEC] != 0.f ? R.s[in.b - NBK_RP_NVEC] : R.s[in.c - NBK_RP_NVEC];
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
        const int64_t off = rp_row_offset(o, lead_idx, n_lead);
        float* dst = rp_stage_lds + o.stage_slot * c_pad;
        if (o.vec_ok && o.dtype == NBK_F32 && (C & 3) == 0) {
          const float4* src = (const float4*)((const float*)o.ptr + off);
          int64_t ch = threadIdx.x;
          const int64_t bd = blockDim.x;
          // four independent 16-byte loads in flight per lane
          for (; ch + 3 * bd < n_chunks; ch += 4 * bd) {
            const float4 v0 = src[ch], v1 = src[ch + bd], v2 = src[ch + 2 * bd],
                         v3 = src[ch + 3 * bd];
            ((float4*)dst)[ch] = v0;
            ((float4*)dst)[ch + bd] = v1;
            ((float4*)dst)[ch + 2 * bd] = v2;
            ((float4*)dst)[ch + 3 * bd] = v3;
          }
          for (; ch < n_chunks; ch += bd) ((float4*)dst)[ch] = src[ch];
        } else {
          for (int64_t ch = threadIdx.x; ch < n_chunks; ch += blockDim.x) {
            const int64_t col = ch << 2;
            const int64_t left = C - col;
            ((float4*)dst)[ch] = rp_load4(o, off, col, left >= 4 ? 4 : (int)left);
          }
        }
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
        } else if (op >= NBK_OP_MOV && op <= NBK_OP_FMA) {
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
    } else if (op >= NBK_OP_MOV && op <= NBK_OP_FMA) {
      NBK_REQUIRE(sreg_dst && in.a >= NBK_RP_NVEC && in.a < 32, "rowprog: bad scalar op at %d",
                  pc);
      if (op >= NBK_OP_ADD)
        NBK_REQUIRE(in.b >= NBK_RP_NVEC && in.b < 32, "rowprog: bad scalar op at %d", pc);
      if (op >= NBK_OP_WHERE)
        NBK_REQUIRE(in.c >= NBK_RP_NVEC && in.c < 32, "rowprog: bad scalar op at %d", pc);
    } else {
      NBK_REQUIRE(false, "rowprog: opcode %d not allowed in a prologue (at %d)", op, pc);
    }
    ++pc;
  }
  NBK_REQUIRE(halted, "rowprog: program has no HALT");
  return NBK_OK;
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
  hipLaunchKernelGGL(rp_flat_kernel, dim3((unsigned)blocks), dim3(256), 0, st, *p, (uint32_t)cpr,
                     total);
  return nbk_check_launch("rp_flat_kernel");
}
