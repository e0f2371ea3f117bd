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


// ---- helpers of the specialised (straight-line) row kernels ---------------------
__device__ __forceinline__ float4 rp_splat(float s) { return make_float4(s, s, s, s); }

template <int OP>
__device__ __forceinline__ float4 rp_un4(float4 a) {
  return make_float4(rp_unary(OP, a.x), rp_unary(OP, a.y), rp_unary(OP, a.z), rp_unary(OP, a.w));
}
template <int OP>
__device__ __forceinline__ float4 rp_bin4(float4 a, float4 b) {
  return make_float4(rp_binary(OP, a.x, b.x), rp_binary(OP, a.y, b.y), rp_binary(OP, a.z, b.z),
                     rp_binary(OP, a.w, b.w));
}
__device__ __forceinline__ float4 rp_where4(float4 c, float4 a, float4 b) {
  return make_float4(c.x != 0.f ? a.x : b.x, c.y != 0.f ? a.y : b.y, c.z != 0.f ? a.z : b.z,
                     c.w != 0.f ? a.w : b.w);
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
