// Integer / index kernels: gather along an axis and first-extremum argmax.
// Both are exact: gather copies bits, argmax compares in the input's own type
// widened to fp32 (exact for f32 / bf16 / f16) and returns int64 positions.
#include "nbk_common.h"

template <typename T, typename IDX>
__global__ __launch_bounds__(256) void gather_kernel(const T* __restrict__ table,
                                                     const IDX* __restrict__ idx,
                                                     T* __restrict__ out, int64_t outer,
                                                     int64_t axis_len, int64_t n_idx,
                                                     int64_t inner, int32_t* status) {
  // one workgroup per (outer, index) pair; lanes sweep `inner`
  const int64_t pair = blockIdx.x;
  const int64_t o = pair / n_idx, j = pair - o * n_idx;
  int64_t i = (int64_t)idx[j];
  if (i < 0) i += axis_len;
  if (i < 0 || i >= axis_len) {
    if (threadIdx.x == 0) atomicExch(status, 1);
    return;
  }
  const T* src = table + (o * axis_len + i) * inner;
  T* dst = out + (o * n_idx + j) * inner;
  const int bytes_per = sizeof(T);
  if ((inner * bytes_per) % 16 == 0 && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0)) {
    const int64_t n16 = inner * bytes_per / 16;
    const uint4* s4 = (const uint4*)src;
    uint4* d4 = (uint4*)dst;
    for (int64_t c = threadIdx.x; c < n16; c += 256) d4[c] = s4[c];
  } else {
    for (int64_t c = threadIdx.x; c < inner; c += 256) dst[c] = src[c];
  }
}

extern "C" int nbk_gather(const void* table, const void* idx, void* out, int32_t dtype,
                          int32_t idx_dtype, int64_t outer, int64_t axis_len, int64_t n_idx,
                          int64_t inner, int32_t* status, void* stream) {
  NBK_REQUIRE(table && idx && out && status, "gather: null pointer");
  NBK_REQUIRE(outer > 0 && axis_len > 0 && n_idx > 0 && inner > 0, "gather: empty extent");
  NBK_REQUIRE(idx_dtype == NBK_I32 || idx_dtype == NBK_I64, "gather: index dtype %d", idx_dtype);
  const int es = nbk_dtype_size(dtype);
  NBK_REQUIRE(es > 0, "gather: bad dtype %d", dtype);
  NBK_REQUIRE(outer * n_idx <= 0x7fffffffLL, "gather: too many rows");
  dim3 grid((unsigned)(outer * n_idx));
  hipStream_t st = (hipStream_t)stream;
#define NBK_GATHER(T)                                                                            \
  do {                                                                                           \
    if (idx_dtype == NBK_I64)                                                                    \
      hipLaunchKernelGGL((gather_kernel<T, int64_t>), grid, dim3(256), 0, st, (const T*)table,   \
                         (const int64_t*)idx, (T*)out, outer, axis_len, n_idx, inner, status);   \
    else                                                                                         \
      hipLaunchKernelGGL((gather_kernel<T, int32_t>), grid, dim3(256), 0, st, (const T*)table,   \
                         (const int32_t*)idx, (T*)out, outer, axis_len, n_idx, inner, status);   \
  } while (0)
  if (es == 4) NBK_GATHER(uint32_t);
  else if (es == 2) NBK_GATHER(uint16_t);
  else if (es == 8) NBK_GATHER(uint64_t);
  else NBK_GATHER(uint8_t);
#undef NBK_GATHER
  return nbk_check_launch("gather_kernel");
}

// ---- scatter: out[o, idx[j], :] = upd[o, j, :] on top of what `out` already holds -----------
// Rows named twice are decided in advance: `winner[r]` is the largest position j with
// idx[j] == r (numpy's assignment rule: the last write wins), found with an atomic maximum;
// only that position writes, so the result does not depend on scheduling.
__global__ __launch_bounds__(256) void scatter_init_kernel(int32_t* winner, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) winner[i] = -1;
}

template <typename IDX>
__global__ __launch_bounds__(256) void scatter_mark_kernel(const IDX* __restrict__ idx,
                                                           int32_t* __restrict__ winner,
                                                           int64_t axis_len, int64_t n_idx,
                                                           int32_t* status) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n_idx) return;
  int64_t i = (int64_t)idx[j];
  if (i < 0) i += axis_len;
  if (i < 0 || i >= axis_len) {
    atomicExch(status, 1);
    return;
  }
  atomicMax(&winner[i], (int32_t)j);
}

template <typename T, typename IDX>
__global__ __launch_bounds__(256) void scatter_write_kernel(const T* __restrict__ upd,
                                                            const IDX* __restrict__ idx,
                                                            T* __restrict__ out,
                                                            const int32_t* __restrict__ winner,
                                                            int64_t axis_len, int64_t n_idx,
                                                            int64_t inner) {
  const int64_t pair = blockIdx.x;
  const int64_t o = pair / n_idx, j = pair - o * n_idx;
  int64_t i = (int64_t)idx[j];
  if (i < 0) i += axis_len;
  if (i < 0 || i >= axis_len || winner[i] != (int32_t)j) return;
  const T* src = upd + (o * n_idx + j) * inner;
  T* dst = out + (o * axis_len + i) * inner;
  const int bytes_per = sizeof(T);
  if ((inner * bytes_per) % 16 == 0 && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0)) {
    const int64_t n16 = inner * bytes_per / 16;
    const uint4* s4 = (const uint4*)src;
    uint4* d4 = (uint4*)dst;
    for (int64_t c = threadIdx.x; c < n16; c += 256) d4[c] = s4[c];
  } else {
    for (int64_t c = threadIdx.x; c < inner; c += 256) dst[c] = src[c];
  }
}

extern "C" int nbk_scatter(const void* idx, const void* upd, void* out, int32_t dtype,
                           int32_t idx_dtype, int64_t outer, int64_t axis_len, int64_t n_idx,
                           int64_t inner, int32_t* winner, int32_t* status, void* stream) {
  NBK_REQUIRE(idx && upd && out && winner && status, "scatter: null pointer");
  NBK_REQUIRE(outer > 0 && axis_len > 0 && n_idx > 0 && inner > 0, "scatter: empty extent");
  NBK_REQUIRE(idx_dtype == NBK_I32 || idx_dtype == NBK_I64, "scatter: index dtype %d", idx_dtype);
  const int es = nbk_dtype_size(dtype);
  NBK_REQUIRE(es > 0, "scatter: bad dtype %d", dtype);
  NBK_REQUIRE(outer * n_idx <= 0x7fffffffLL && n_idx <= 0x7fffffffLL, "scatter: too many rows");
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(scatter_init_kernel, dim3((unsigned)((axis_len + 255) / 256)), dim3(256), 0, st,
                     winner, axis_len);
  const dim3 mgrid((unsigned)((n_idx + 255) / 256));
  if (idx_dtype == NBK_I64)
    hipLaunchKernelGGL((scatter_mark_kernel<int64_t>), mgrid, dim3(256), 0, st, (const int64_t*)idx,
                       winner, axis_len, n_idx, status);
  else
    hipLaunchKernelGGL((scatter_mark_kernel<int32_t>), mgrid, dim3(256), 0, st, (const int32_t*)idx,
                       winner, axis_len, n_idx, status);
  const dim3 grid((unsigned)(outer * n_idx));
#define NBK_SCATTER(T)                                                                           \
  do {                                                                                           \
    if (idx_dtype == NBK_I64)                                                                    \
      hipLaunchKernelGGL((scatter_write_kernel<T, int64_t>), grid, dim3(256), 0, st,             \
                         (const T*)upd, (const int64_t*)idx, (T*)out, winner, axis_len, n_idx,   \
                         inner);                                                                 \
    else                                                                                         \
      hipLaunchKernelGGL((scatter_write_kernel<T, int32_t>), grid, dim3(256), 0, st,             \
                         (const T*)upd, (const int32_t*)idx, (T*)out, winner, axis_len, n_idx,   \
                         inner);                                                                 \
  } while (0)
  if (es == 4) NBK_SCATTER(uint32_t);
  else if (es == 2) NBK_SCATTER(uint16_t);
  else if (es == 8) NBK_SCATTER(uint64_t);
  else NBK_SCATTER(uint8_t);
#undef NBK_SCATTER
  return nbk_check_launch("scatter kernels");
}

// One wave per row.  Ties resolve to the lowest index.
__global__ __launch_bounds__(256) void argmax_rows_kernel(const void* __restrict__ in,
                                                          int64_t* __restrict__ out, int dt,
                                                          int64_t rows, int64_t C, int want_min) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float best = want_min ? INFINITY : -INFINITY;
  int64_t bi = 0x7fffffffffffffffLL;
  bool any_nan = false;
  for (int64_t c = lane; c < C; c += 64) {
    float v = nbk_load_as_f32(in, row * C + c, dt);
    if (v != v) {  // NaN wins, first one (numpy / torch convention)
      if (!any_nan) { any_nan = true; bi = c; }
      continue;
    }
    if (any_nan) continue;
    const bool better = want_min ? (v < best) : (v > best);
    if (better || bi == 0x7fffffffffffffffLL) { best = v; bi = c; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    float ob = __shfl_xor(best, off, 64);
    int64_t oi = __shfl_xor(bi, off, 64);
    int on = __shfl_xor((int)any_nan, off, 64);
    bool take;
    if (on != (int)any_nan) take = on;           // the side that saw a NaN wins
    else if (any_nan) take = oi < bi;            // both NaN: lowest index
    else if (oi == 0x7fffffffffffffffLL) take = false;
    else if (bi == 0x7fffffffffffffffLL) take = true;
    else if (ob == best) take = oi < bi;
    else take = want_min ? (ob < best) : (ob > best);
    if (take) { best = ob; bi = oi; any_nan = on; }
  }
  if (lane == 0) out[row] = bi;
}

extern "C" int nbk_argmax_rows(const void* in, int64_t* out, int32_t dtype, int64_t rows,
                               int64_t C, int32_t want_min, void* stream) {
  NBK_REQUIRE(in && out, "argmax: null pointer");
  NBK_REQUIRE(rows > 0 && C > 0, "argmax: empty extent");
  NBK_REQUIRE(dtype == NBK_F32 || dtype == NBK_BF16 || dtype == NBK_F16 || dtype == NBK_I32,
              "argmax: dtype %d is not supported", dtype);
  const int64_t blocks = (rows + 3) / 4;
  NBK_REQUIRE(blocks <= 0x7fffffffLL, "argmax: too many rows");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     (hipStream_t)stream, in, out, dtype, rows, C, want_min);
  return nbk_check_launch("argmax_rows_kernel");
}
