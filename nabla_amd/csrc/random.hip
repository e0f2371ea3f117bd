// Device random numbers: Philox4x32-10 (Salmon et al., SC'11), counter-based.
//
// Nothing is carried from element to element: element i of a tensor takes word i % 4 of the
// block whose counter is (i / 4 low, i / 4 high, stream, run) under the key (seed low, seed
// high).  `stream` tells the random tensors of one step apart, `run` counts the steps; seed and
// run live in device memory (two int64 the caller owns) so that a recorded launch sequence
// draws new numbers on every replay: nbk_rng_advance, a one-lane kernel at the end of the
// step, bumps the run counter.  One lane produces one block = four consecutive elements.
#include "nbk_common.h"

namespace {

struct Philox {
  uint32_t c[4];
};

__device__ __forceinline__ Philox philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    if (r) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
  }
  Philox out;
  out.c[0] = c0; out.c[1] = c1; out.c[2] = c2; out.c[3] = c3;
  return out;
}

__device__ __forceinline__ float unit_float(uint32_t w) { return (float)(w >> 8) * 5.9604644775390625e-8f; }

__global__ __launch_bounds__(256) void random_kernel(void* __restrict__ out, int dtype, int64_t n,
                                                     int mode, float a, float b,
                                                     const int64_t* __restrict__ state,
                                                     uint32_t stream) {
  const uint64_t seed = (uint64_t)state[0];
  const uint32_t run = (uint32_t)state[1];
  const int64_t blocks = (n + 3) >> 2;
  for (int64_t blk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; blk < blocks;
       blk += (int64_t)gridDim.x * blockDim.x) {
    const Philox r = philox4x32_10((uint32_t)blk, (uint32_t)((uint64_t)blk >> 32), stream, run,
                                   (uint32_t)seed, (uint32_t)(seed >> 32));
    float v[4];
    if (mode == NBK_RANDOM_UNIFORM) {
#pragma unroll
      for (int e = 0; e < 4; ++e)  // (product and sum rounded separately, never contracted)
        v[e] = __fadd_rn(a, __fmul_rn(b - a, unit_float(r.c[e])));
    } else if (mode == NBK_RANDOM_KEEP) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = unit_float(r.c[e]) > a ? 1.0f : 0.0f;
    } else {  // Box-Muller, one pair of words per pair of values
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float u1 = ((float)(r.c[2 * h] >> 8) + 1.0f) * 5.9604644775390625e-8f;
        const float u2 = unit_float(r.c[2 * h + 1]);
        const float rad = sqrtf(-2.0f * logf(u1));
        float sn, cs;
        sincosf(6.28318530717958647692f * u2, &sn, &cs);
        v[2 * h] = a + b * rad * cs;
        v[2 * h + 1] = a + b * rad * sn;
      }
    }
    const int64_t i0 = blk << 2;
    if (dtype == NBK_F32 && i0 + 4 <= n) {
      *(float4*)((float*)out + i0) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < n) nbk_store_from_f32(out, i0 + e, dtype, v[e]);
    }
  }
}

__global__ void rng_advance_kernel(int64_t* state) {
  if (threadIdx.x == 0 && blockIdx.x == 0) state[1] += 1;
}

}  // namespace

extern "C" int nbk_random(void* out, int32_t dtype, int64_t n, int32_t mode, float a, float b,
                          const int64_t* state, uint32_t stream_id, void* stream) {
  NBK_REQUIRE(out && state, "random: null pointer");
  NBK_REQUIRE(n > 0, "random: %lld elements", (long long)n);
  NBK_REQUIRE(mode >= NBK_RANDOM_UNIFORM && mode <= NBK_RANDOM_KEEP, "random: mode %d", mode);
  NBK_REQUIRE(dtype == NBK_F32 || dtype == NBK_BF16 || dtype == NBK_F16 ||
                  (mode == NBK_RANDOM_KEEP && dtype == NBK_U8),
              "random: dtype %d for mode %d", dtype, mode);
  NBK_REQUIRE(((uintptr_t)out & 15) == 0 || dtype != NBK_F32, "random: fp32 output must be 16-byte aligned");
  const int64_t blocks = (n + 3) >> 2;
  int64_t grid = (blocks + 255) / 256;
  const int64_t cap = (int64_t)nbk_num_cus() * 16;
  if (grid > cap) grid = cap;
  hipLaunchKernelGGL(random_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, out, dtype,
                     n, mode, a, b, state, stream_id);
  return nbk_check_launch("random_kernel");
}

extern "C" int nbk_rng_advance(int64_t* state, void* stream) {
  NBK_REQUIRE(state != nullptr, "rng_advance: null pointer");
  hipLaunchKernelGGL(rng_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, state);
  return nbk_check_launch("rng_advance_kernel");
}
