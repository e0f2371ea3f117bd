// Device helpers shared by the row-program interpreter and the specialised
// row kernels: typed 4-column loads / stores, the elementwise functions, the
// row-offset arithmetic and the block-wide reduction.
#pragma once
#include "nbk_common.h"

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
// Streaming forms for launches whose operands exceed the last-level cache: the
// non-temporal hint keeps lines that are touched once from displacing others.
typedef float rp_vf4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 rp_load4_stream(const float* p) {
  rp_vf4 v = __builtin_nontemporal_load((const rp_vf4*)p);
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void rp_store4_stream(float* p, float4 r) {
  rp_vf4 v = {r.x, r.y, r.z, r.w};
  __builtin_nontemporal_store(v, (rp_vf4*)p);
}

// Registers are 32 bits wide and typed by the program, not by the hardware: a value of an
// integer tensor (int32, int64) is held as a two's-complement int32 in the register's bits and
// computed with the integer instructions, so integers are exact over the whole int32 range
// (an int64 operand is read saturated to the int32 range and written sign-extended: the lowering
// keeps int64 tensors in these programs only where they are compared with an index or constant
// strictly inside that range, which saturation leaves exact, and sends every other operation
// on int64 values to the 64-bit elementwise kernel);
// everything else -- floats, and bool / uint8 as 0.0, 1.0, ... -- is held as fp32.
__device__ __forceinline__ float rp_ibits(int v) { return __int_as_float(v); }
__device__ __forceinline__ int rp_int(float v) { return __float_as_int(v); }

__device__ __forceinline__ int rp_sat32(int64_t v) {
  return v > 2147483647LL ? 2147483647 : (v < -2147483648LL ? (int)(-2147483647 - 1) : (int)v);
}
__device__ __forceinline__ float rp_load1(const void* p, int64_t i, int dt) {
  if (dt == NBK_I32) return rp_ibits(((const int32_t*)p)[i]);
  if (dt == NBK_I64) return rp_ibits(rp_sat32(((const int64_t*)p)[i]));
  return nbk_load_as_f32(p, i, dt);
}
__device__ __forceinline__ void rp_store1(void* p, int64_t i, int dt, float v) {
  if (dt == NBK_I32) ((int32_t*)p)[i] = rp_int(v);
  else if (dt == NBK_I64) ((int64_t*)p)[i] = (int64_t)rp_int(v);
  else nbk_store_from_f32(p, i, dt, v);
}

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
      r = *(const float4*)((const int32_t*)o.ptr + e);  // the bits as they are
    } else if (dt == NBK_I64) {
      const int64_t* p = (const int64_t*)o.ptr + e;
      longlong2 u0 = *(const longlong2*)p, u1 = *(const longlong2*)(p + 2);
      r = make_float4(rp_ibits(rp_sat32(u0.x)), rp_ibits(rp_sat32(u0.y)), rp_ibits(rp_sat32(u1.x)),
                      rp_ibits(rp_sat32(u1.y)));
    } else {
      uint32_t u = *(const uint32_t*)((const uint8_t*)o.ptr + e);
      r = make_float4((float)(u & 0xff), (float)((u >> 8) & 0xff), (float)((u >> 16) & 0xff),
                      (float)(u >> 24));
    }
    return r;
  }
  const int64_t e0 = off + col * cs;
  if (valid > 0) r.x = rp_load1(o.ptr, e0, dt);
  if (cs == 0) {
    r.y = r.z = r.w = r.x;
    return r;
  }
  if (valid > 1) r.y = rp_load1(o.ptr, e0 + cs, dt);
  if (valid > 2) r.z = rp_load1(o.ptr, e0 + 2 * cs, dt);
  if (valid > 3) r.w = rp_load1(o.ptr, e0 + 3 * cs, dt);
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
      *(float4*)((int32_t*)o.ptr + e) = v;
    } else if (dt == NBK_I64) {
      longlong2* p = (longlong2*)((int64_t*)o.ptr + e);
      p[0] = make_longlong2((int64_t)rp_int(v.x), (int64_t)rp_int(v.y));
      p[1] = make_longlong2((int64_t)rp_int(v.z), (int64_t)rp_int(v.w));
    } else {
      uint32_t u = (uint32_t)(v.x != 0.f) | ((uint32_t)(v.y != 0.f) << 8) |
                   ((uint32_t)(v.z != 0.f) << 16) | ((uint32_t)(v.w != 0.f) << 24);
      *(uint32_t*)((uint8_t*)o.ptr + e) = u;
    }
    return;
  }
  const int64_t e0 = off + col * cs;
  if (valid > 0) rp_store1(o.ptr, e0, dt, v.x);
  if (valid > 1) rp_store1(o.ptr, e0 + cs, dt, v.y);
  if (valid > 2) rp_store1(o.ptr, e0 + 2 * cs, dt, v.z);
  if (valid > 3) rp_store1(o.ptr, e0 + 3 * cs, dt, v.w);
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
    case NBK_OP_DGELU:  // Phi(a) + a * phi(a)
      return 0.5f * (1.0f + erff(a * 0.70710678118654752440f)) +
             a * 0.39894228040143267794f * expf(-0.5f * a * a);
    case NBK_OP_TANH: return tanhf(a);
    case NBK_OP_SIN: return sinf(a);
    case NBK_OP_COS: return cosf(a);
    case NBK_OP_SIGMOID: return 1.0f / (1.0f + expf(-a));
    case NBK_OP_ABS: return fabsf(a);
    case NBK_OP_RBF16: return nbk_bf16_to_f32(nbk_f32_to_bf16(a));
    case NBK_OP_NOT: return a != 0.0f ? 0.0f : 1.0f;
    case NBK_OP_TRUNC: return truncf(a);
    case NBK_OP_NEZ: return a != 0.0f ? 1.0f : 0.0f;
    // integer registers
    case NBK_OP_INEG: return rp_ibits(-rp_int(a));
    case NBK_OP_IABS: return rp_ibits(rp_int(a) < 0 ? -rp_int(a) : rp_int(a));
    case NBK_OP_IRELU: return rp_ibits(rp_int(a) > 0 ? rp_int(a) : 0);
    case NBK_OP_I2F: return (float)rp_int(a);
    case NBK_OP_F2I: return rp_ibits((int)a);
    case NBK_OP_INEZ: return rp_int(a) != 0 ? 1.0f : 0.0f;
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
    // integer registers (wrap-around arithmetic; comparisons give a float 0 / 1)
    case NBK_OP_IADD: return rp_ibits((int)((uint32_t)rp_int(a) + (uint32_t)rp_int(b)));
    case NBK_OP_ISUB: return rp_ibits((int)((uint32_t)rp_int(a) - (uint32_t)rp_int(b)));
    case NBK_OP_IMUL: return rp_ibits((int)((uint32_t)rp_int(a) * (uint32_t)rp_int(b)));
    case NBK_OP_IMAX: return rp_ibits(rp_int(a) > rp_int(b) ? rp_int(a) : rp_int(b));
    case NBK_OP_IMIN: return rp_ibits(rp_int(a) < rp_int(b) ? rp_int(a) : rp_int(b));
    case NBK_OP_IGT: return rp_int(a) > rp_int(b) ? 1.0f : 0.0f;
    case NBK_OP_IGE: return rp_int(a) >= rp_int(b) ? 1.0f : 0.0f;
    case NBK_OP_IEQ: return rp_int(a) == rp_int(b) ? 1.0f : 0.0f;
    case NBK_OP_INE: return rp_int(a) != rp_int(b) ? 1.0f : 0.0f;
    case NBK_OP_ILT: return rp_int(a) < rp_int(b) ? 1.0f : 0.0f;
    case NBK_OP_ILE: return rp_int(a) <= rp_int(b) ? 1.0f : 0.0f;
    default: return a;
  }
}

// Reduced-precision forms for programs whose every stored tensor is a 16-bit float:
// hardware exp2 / log2 / rcp / rsq (about 1e-6 relative) and a five-term erf (1.5e-7
// absolute, Abramowitz & Stegun 7.1.26) are far inside the 4e-3 of a bf16 result, and
// they take a fifth of the instructions of the correctly rounded library routines,
// which is what bounds these kernels once their traffic is halved by the 16-bit I/O.
// e = exp(-x^2), passed in so that a caller that needs it anyway computes it once
__device__ __forceinline__ float rp_fast_erf_with(float x, float e) { return nbk_fast_erf_with(x, e); }
__device__ __forceinline__ float rp_fast_erf(float x) { return rp_fast_erf_with(x, __expf(-x * x)); }
// GELU for 16-bit results without erf: x Phi(x) = max(x, 0) - |x| Q(|x|) with the upper tail
// Q(t) = 1 - Phi(t) = 2^p(t), p a degree-7 fit of log2 Q on [0, 8] (relative error of the result
// below 1e-4 for |x| <= 8, also far out in the negative tail where Q is all there is; beyond 8
// the tail is held at Q(8) = 6e-16).  Eleven instructions, one of them transcendental, against
// sixteen and two for the erf form: the GELU kernels of 16-bit steps are bound by the vector ALU.
__device__ __forceinline__ float rp_fast_gelu(float x) {
  const float t = fminf(fabsf(x), 8.0f);
  float p = -1.2768182e-06f;
  p = fmaf(p, t, 4.8467238e-05f);
  p = fmaf(p, t, -8.0841628e-04f);
  p = fmaf(p, t, 7.9395650e-03f);
  p = fmaf(p, t, -5.2579608e-02f);
  p = fmaf(p, t, -4.6011573e-01f);
  p = fmaf(p, t, -1.1504445f);
  p = fmaf(p, t, -1.0000888f);
  return fmaf(-t, __builtin_amdgcn_exp2f(p), fmaxf(x, 0.0f));
}
__device__ __forceinline__ float rp_unary_lowp(int op, float a) {
  switch (op) {
    case NBK_OP_EXP: return __expf(a);
    case NBK_OP_LOG: return __logf(a);
    case NBK_OP_SQRT: return __builtin_amdgcn_sqrtf(a);
    case NBK_OP_RSQRT: return __builtin_amdgcn_rsqf(a);
    case NBK_OP_ERF: return rp_fast_erf(a);
    case NBK_OP_GELU: return rp_fast_gelu(a);
    case NBK_OP_DGELU: {
      // the same exp(-a^2 / 2) serves the erf approximation and the density, and a GELU of
      // the same value in the same kernel shares all of it after common-subexpression removal
      const float z = a * 0.70710678118654752440f;
      const float e = __expf(-z * z);
      return 0.5f * (1.0f + rp_fast_erf_with(z, e)) + a * 0.39894228040143267794f * e;
    }
    case NBK_OP_SIGMOID: return __builtin_amdgcn_rcpf(1.0f + __expf(-a));
    default: return rp_unary(op, a);
  }
}
__device__ __forceinline__ float rp_binary_lowp(int op, float a, float b) {
  if (op == NBK_OP_DIV) return a * __builtin_amdgcn_rcpf(b);
  return rp_binary(op, a, b);
}

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

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the
// wave's outstanding global loads and stores; the reductions below exchange data
// through LDS alone, and the pipelined row kernels want their next row's loads to
// stay in flight across them.
__device__ __forceinline__ void rp_lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Cross-lane step: combine every lane's value with the value the DPP control word
// selects; lanes the row mask excludes (or that select an invalid lane) take part
// with the identity.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float rp_dpp_step(float v, int kind) {
  const int ident = __float_as_int(rp_identity(kind));
  const int t = __builtin_amdgcn_update_dpp(ident, __float_as_int(v), CTRL, ROW_MASK, 0xf, false);
  return rp_combine(v, __int_as_float(t), kind);
}

// Reduction over the 64 lanes of a wavefront on the VALU's data-parallel-primitive
// path (no LDS round trips).  Every lane must be active.  Returns the wave's total,
// uniform across the wave.
__device__ __forceinline__ float rp_wave_reduce(float v, int kind) {
  v = rp_dpp_step<0xB1, 0xf>(v, kind);   // quad_perm [1,0,3,2]: lane ^ 1
  v = rp_dpp_step<0x4E, 0xf>(v, kind);   // quad_perm [2,3,0,1]: lane ^ 2
  v = rp_dpp_step<0x141, 0xf>(v, kind);  // row_half_mirror: the other quad of each 8
  v = rp_dpp_step<0x140, 0xf>(v, kind);  // row_mirror: the other half of each row of 16
  v = rp_dpp_step<0x142, 0xa>(v, kind);  // row_bcast15 into rows 1 and 3
  v = rp_dpp_step<0x143, 0xc>(v, kind);  // row_bcast31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Total over the first eight lanes (one partial per wave of the workgroup), uniform.
__device__ __forceinline__ float rp_reduce8(float v, int kind) {
  v = rp_dpp_step<0xB1, 0xf>(v, kind);
  v = rp_dpp_step<0x4E, 0xf>(v, kind);
  v = rp_dpp_step<0x141, 0xf>(v, kind);
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

// Block-wide reduction of one float: DPP within each wave, then one partial per
// wave through LDS.  Two barriers: safe to call back to back on the same buffer.
__device__ __forceinline__ float rp_block_reduce(float v, int kind, float* red_buf) {
  v = rp_wave_reduce(v, kind);
  const int nw = blockDim.x >> 6;
  if (nw == 1) return v;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) red_buf[w] = v;
  rp_lds_barrier();
  float r = rp_reduce8(lane < nw ? red_buf[lane] : rp_identity(kind), kind);
  rp_lds_barrier();
  return r;
}

// The same with ONE barrier per call.  ``red2`` holds two banks of 32 floats and
// ``phase`` counts the calls of the workgroup: consecutive calls use different banks,
// and a bank is rewritten only after the barrier of the call in between, which every
// wave reaches after it has read that bank.  Up to four values (slot k of a bank
// holds the partials of value k) share the barrier.
__device__ __forceinline__ void rp_block_reduce_n(float* v, const int* kind, int n, float* red2,
                                                  int& phase) {
  for (int k = 0; k < n; ++k) v[k] = rp_wave_reduce(v[k], kind[k]);
  const int nw = blockDim.x >> 6;
  if (nw == 1) return;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  float* bank = red2 + ((phase & 1) << 5);
  ++phase;
  if (lane == 0)
    for (int k = 0; k < n; ++k) bank[k * 8 + w] = v[k];
  rp_lds_barrier();
  for (int k = 0; k < n; ++k)
    v[k] = rp_reduce8(lane < nw ? bank[k * 8 + lane] : rp_identity(kind[k]), kind[k]);
}

// Row index -> indices of the (up to four) leading dimensions; rows < 2^31.
__device__ __forceinline__ void rp_decompose_row(uint32_t row, int n_lead, uint32_t d1, uint32_t d2,
                                                 uint32_t d3, uint32_t* li) {
  if (n_lead <= 1) {
    li[0] = row; li[1] = 0; li[2] = 0; li[3] = 0;
    return;
  }
  uint32_t rem = row, q;
  q = rem / d3; li[3] = rem - q * d3; rem = q;
  q = rem / d2; li[2] = rem - q * d2; rem = q;
  q = rem / d1; li[1] = rem - q * d1; rem = q;
  li[0] = rem;
}


// ---- helpers of the specialised (straight-line) row kernels ---------------------
__device__ __forceinline__ float4 rp_splat(float s) { return make_float4(s, s, s, s); }

template <int OP, bool LOWP = false>
__device__ __forceinline__ float4 rp_un4(float4 a) {
  if (LOWP)
    return make_float4(rp_unary_lowp(OP, a.x), rp_unary_lowp(OP, a.y), rp_unary_lowp(OP, a.z),
                       rp_unary_lowp(OP, a.w));
  return make_float4(rp_unary(OP, a.x), rp_unary(OP, a.y), rp_unary(OP, a.z), rp_unary(OP, a.w));
}
template <int OP, bool LOWP = false>
__device__ __forceinline__ float4 rp_bin4(float4 a, float4 b) {
  if (LOWP)
    return make_float4(rp_binary_lowp(OP, a.x, b.x), rp_binary_lowp(OP, a.y, b.y),
                       rp_binary_lowp(OP, a.z, b.z), rp_binary_lowp(OP, a.w, b.w));
  return make_float4(rp_binary(OP, a.x, b.x), rp_binary(OP, a.y, b.y), rp_binary(OP, a.z, b.z),
                     rp_binary(OP, a.w, b.w));
}
// The choice moves register bits, whatever they hold.
__device__ __forceinline__ float rp_where(float c, float a, float b) {
  return rp_ibits(c != 0.f ? rp_int(a) : rp_int(b));
}
__device__ __forceinline__ float4 rp_where4(float4 c, float4 a, float4 b) {
  return make_float4(rp_where(c.x, a.x, b.x), rp_where(c.y, a.y, b.y), rp_where(c.z, a.z, b.z),
                     rp_where(c.w, a.w, b.w));
}
// Column indices col .. col + 3 as floats or, for an integer register, as int32.
__device__ __forceinline__ float4 rp_colidx4(int64_t col, bool as_int) {
  if (as_int) {
    const int c0 = (int)col;
    return make_float4(rp_ibits(c0), rp_ibits(c0 + 1), rp_ibits(c0 + 2), rp_ibits(c0 + 3));
  }
  const float c0 = (float)col;
  return make_float4(c0, c0 + 1.f, c0 + 2.f, c0 + 3.f);
}
__device__ __forceinline__ float4 rp_fma4(float4 a, float4 b, float4 c) {
  return make_float4(fmaf(a.x, b.x, c.x), fmaf(a.y, b.y, c.y), fmaf(a.z, b.z, c.z),
                     fmaf(a.w, b.w, c.w));
}
__device__ __forceinline__ float rp_acc4(float acc, float4 a, int kind, int valid) {
  if (valid > 0) acc = rp_combine(acc, a.x, kind);
  if (valid > 1) acc = rp_combine(acc, a.y, kind);
  if (valid > 2) acc = rp_combine(acc, a.z, kind);
  if (valid > 3) acc = rp_combine(acc, a.w, kind);
  return acc;
}

// Copy one row of a 16-bit operand (unit column stride, C % 4 == 0) into LDS as it is stored.
// A lane copies the 4-element chunks it reads back later (chunk index = lane + j * workgroup
// size), so no barrier separates staging from use; eight loads are in flight per lane.
__device__ __forceinline__ void rp_stage_row16(const nbk_operand& o, int64_t off, uint2* dst,
                                               int64_t n_chunks) {
  const uint16_t* base = (const uint16_t*)o.ptr + off;
  const int64_t bd = blockDim.x;
  int64_t ch = threadIdx.x;
  if ((((uintptr_t)base) & 7) == 0) {
    const uint2* src = (const uint2*)base;
    for (; ch + 7 * bd < n_chunks; ch += 8 * bd) {
      uint2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[ch + u * bd];
#pragma unroll
      for (int u = 0; u < 8; ++u) dst[ch + u * bd] = v[u];
    }
    for (; ch < n_chunks; ch += bd) dst[ch] = src[ch];
  } else {
    for (; ch < n_chunks; ch += bd) {
      const uint16_t* q = base + (ch << 2);
      dst[ch] = make_uint2((uint32_t)q[0] | ((uint32_t)q[1] << 16), (uint32_t)q[2] | ((uint32_t)q[3] << 16));
    }
  }
}
// Four elements of a row staged by rp_stage_row16, as registers.
__device__ __forceinline__ float4 rp_staged16(const uint2* stage, int64_t col, int dt) {
  const uint2 u = stage[col >> 2];
  if (dt == NBK_BF16)
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  __half2 a = *(const __half2*)&u.x, b = *(const __half2*)&u.y;
  const float2 fa = __half22float2(a), fb = __half22float2(b);
  return make_float4(fa.x, fa.y, fb.x, fb.y);
}

// Copy one row of an operand into LDS as fp32.  Every lane stages exactly the
// chunks it reads back later (chunk index = lane + j * workgroup size), so no
// barrier separates staging from use.
__device__ __forceinline__ void rp_stage_row(const nbk_operand& o, int64_t off, float* dst,
                                             int64_t C, int64_t n_chunks) {
  if (o.vec_ok && o.dtype == NBK_F32 && (C & 3) == 0) {
    const float4* src = (const float4*)((const float*)o.ptr + off);
    int64_t ch = threadIdx.x;
    const int64_t bd = blockDim.x;
    // four independent 16-byte loads in flight per lane
    for (; ch + 3 * bd < n_chunks; ch += 4 * bd) {
      const float4 v0 = src[ch], v1 = src[ch + bd], v2 = src[ch + 2 * bd], v3 = src[ch + 3 * bd];
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
