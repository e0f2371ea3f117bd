// Shared helpers for the libnbk translation units (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <stdlib.h>
#include "nbk.h"

// ---- error reporting (thread-local message, C ABI status codes) ----------
void nbk_set_error(const char* fmt, ...);
// Compute units of the current device (256 on MI355X); set by nbk_init, lazily otherwise.
int nbk_num_cus(void);
// Looks up the device address of the attention kernels' built-in scratch for the current
// device (attention.hip); nbk_init calls it right after selecting the device.
int nbk_attention_static_setup(void);

#define NBK_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) {                        \
      nbk_set_error(__VA_ARGS__);         \
      return NBK_ERR_INVALID;             \
    }                                     \
  } while (0)

#define NBK_HIP(call)                                                     \
  do {                                                                    \
    hipError_t e_ = (call);                                               \
    if (e_ != hipSuccess) {                                               \
      nbk_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                    __FILE__, __LINE__);                                  \
      return NBK_ERR_LAUNCH;                                              \
    }                                                                     \
  } while (0)

static inline int nbk_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    nbk_set_error("launch of %s failed: %s", what, hipGetErrorString(e));
    return NBK_ERR_LAUNCH;
  }
  return NBK_OK;
}

static inline int nbk_dtype_size(int dt) {
  switch (dt) {
    case NBK_F32: return 4;
    case NBK_BF16: return 2;
    case NBK_F16: return 2;
    case NBK_I32: return 4;
    case NBK_I64: return 8;
    case NBK_U8: return 1;
    default: return 0;
  }
}

// ---- device-side scalar conversions ---------------------------------------
#ifdef __HIPCC__
__device__ __forceinline__ float nbk_bf16_to_f32(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}
// round-to-nearest-even, NaN kept quiet: one hardware conversion (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t nbk_f32_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}
// Five-term erf (Abramowitz & Stegun 7.1.26, 1.5e-7 absolute) on hardware rcp; e = exp(-x^2) is
// passed in so that a caller that needs it anyway computes it once.  For results that are
// stored as 16-bit floats.
__device__ __forceinline__ float nbk_fast_erf_with(float x, float e) {
  const float ax = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, ax, 1.0f));
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float r = fmaf(-p * t, e, 1.0f);
  return copysignf(r, x);
}
__device__ __forceinline__ float nbk_load_as_f32(const void* p, int64_t i, int dt) {
  switch (dt) {
    case NBK_F32: return ((const float*)p)[i];
    case NBK_BF16: return nbk_bf16_to_f32(((const uint16_t*)p)[i]);
    case NBK_F16: return __half2float(((const __half*)p)[i]);
    case NBK_I32: return (float)((const int32_t*)p)[i];
    case NBK_I64: return (float)((const int64_t*)p)[i];
    default: return (float)((const uint8_t*)p)[i];
  }
}
__device__ __forceinline__ void nbk_store_from_f32(void* p, int64_t i, int dt, float v) {
  switch (dt) {
    case NBK_F32: ((float*)p)[i] = v; break;
    case NBK_BF16: ((uint16_t*)p)[i] = nbk_f32_to_bf16(v); break;
    case NBK_F16: ((__half*)p)[i] = __float2half(v); break;
    case NBK_I32: ((int32_t*)p)[i] = (int32_t)v; break;
    case NBK_I64: ((int64_t*)p)[i] = (int64_t)v; break;
    default: ((uint8_t*)p)[i] = (uint8_t)(v != 0.0f); break;
  }
}
#endif
