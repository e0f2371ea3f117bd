// Integer / index kernels: gather along an axis and first-extremum argmax.
// Both are exact: gather copies bits, argmax compares in the input's own type
// widened to fp32 (exact for f32 / bf16 / f16) and returns int64 positions.
#include "nbk_common.h"
#include <type_traits>

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

// One wave per row.  Ties resolve to the lowest index.  Floating-point inputs compare as fp32
// (exact for f32 / bf16 / f16), integer inputs as int64 (exact for int32 / int64).
template <bool INTEGER>
__global__ __launch_bounds__(256) void argmax_rows_kernel(const void* __restrict__ in,
                                                          int64_t* __restrict__ out, int dt,
                                                          int64_t rows, int64_t C, int want_min) {
  using V = typename std::conditional<INTEGER, int64_t, float>::type;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  V best = 0;
  int64_t bi = 0x7fffffffffffffffLL;
  bool any_nan = false;
  for (int64_t c = lane; c < C; c += 64) {
    V v;
    if constexpr (INTEGER) {
      v = dt == NBK_I64 ? ((const int64_t*)in)[row * C + c] : (int64_t)((const int32_t*)in)[row * C + c];
    } else {
      v = nbk_load_as_f32(in, row * C + c, dt);
      if (v != v) {  // NaN wins, first one (numpy / torch convention)
        if (!any_nan) { any_nan = true; bi = c; }
        continue;
      }
      if (any_nan) continue;
    }
    const bool better = want_min ? (v < best) : (v > best);
    if (better || bi == 0x7fffffffffffffffLL) { best = v; bi = c; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    V ob = __shfl_xor(best, off, 64);
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
  NBK_REQUIRE(dtype == NBK_F32 || dtype == NBK_BF16 || dtype == NBK_F16 || dtype == NBK_I32 ||
                  dtype == NBK_I64, "argmax: dtype %d is not supported", dtype);
  const int64_t blocks = (rows + 3) / 4;
  NBK_REQUIRE(blocks <= 0x7fffffffLL, "argmax: too many rows");
  if (dtype == NBK_I32 || dtype == NBK_I64)
    hipLaunchKernelGGL(argmax_rows_kernel<true>, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, in, out, dtype, rows, C, want_min);
  else
    hipLaunchKernelGGL(argmax_rows_kernel<false>, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, in, out, dtype, rows, C, want_min);
  return nbk_check_launch("argmax_rows_kernel");
}

// ---- elementwise arithmetic on 64-bit integers -------------------------------------------
// Fused row programs hold integers in 32-bit registers; whatever computes on int64 values or
// produces them runs here instead, one operation per launch, exact over the whole int64 range
// (sums, differences and products wrap modulo 2^64 as numpy's do).
struct Ew64Args {
  int32_t op, rank, n_in, out_dt;
  int64_t n;
  int64_t shape[NBK_MAX_RANK];
  int64_t out_stride[NBK_MAX_RANK];
  const void* in[3];
  int32_t in_dt[3];
  int32_t is_imm[3];
  int64_t imm[3];
  int64_t stride[3][NBK_MAX_RANK];
  void* out;
};

__device__ __forceinline__ int64_t ew64_from_float(float x) {
  if (x != x) return 0;
  x = truncf(x);
  if (x >= 9223372036854775807.0f) return INT64_MAX;
  if (x <= -9223372036854775808.0f) return INT64_MIN;
  return (int64_t)x;
}
__device__ __forceinline__ int64_t ew64_load(const void* p, int64_t i, int dt) {
  switch (dt) {
    case NBK_I64: return ((const int64_t*)p)[i];
    case NBK_I32: return (int64_t)((const int32_t*)p)[i];
    case NBK_U8: return (int64_t)((const uint8_t*)p)[i];
    default: return ew64_from_float(nbk_load_as_f32(p, i, dt));
  }
}
__device__ __forceinline__ int64_t ew64_pow(int64_t b, int64_t e) {
  if (e < 0) return b == 1 ? 1 : (b == -1 ? ((e & 1) ? -1 : 1) : 0);
  uint64_t r = 1, x = (uint64_t)b;
  while (e) {
    if (e & 1) r *= x;
    x *= x;
    e >>= 1;
  }
  return (int64_t)r;
}
__device__ __forceinline__ int64_t ew64_apply(int op, int64_t a, int64_t b, int64_t c) {
  const uint64_t ua = (uint64_t)a, ub = (uint64_t)b;
  switch (op) {
    case NBK_OP_MOV: case NBK_OP_TRUNC: return a;
    case NBK_OP_NEG: return (int64_t)(0 - ua);
    case NBK_OP_ABS: return a < 0 ? (int64_t)(0 - ua) : a;
    case NBK_OP_RELU: return a > 0 ? a : 0;
    case NBK_OP_NOT: return a == 0;
    case NBK_OP_NEZ: return a != 0;
    case NBK_OP_ADD: return (int64_t)(ua + ub);
    case NBK_OP_SUB: return (int64_t)(ua - ub);
    case NBK_OP_MUL: return (int64_t)(ua * ub);
    case NBK_OP_DIV:  // toward zero, as the 32-bit registers of the fused kernels divide
      return b == 0 ? 0 : ((a == INT64_MIN && b == -1) ? INT64_MIN : a / b);
    case NBK_OP_MAX: return a > b ? a : b;
    case NBK_OP_MIN: return a < b ? a : b;
    case NBK_OP_GT: return a > b;
    case NBK_OP_GE: return a >= b;
    case NBK_OP_EQ: return a == b;
    case NBK_OP_NE: return a != b;
    case NBK_OP_LT: return a < b;
    case NBK_OP_LE: return a <= b;
    case NBK_OP_POW: return ew64_pow(a, b);
    case NBK_OP_AND: return (a != 0) & (b != 0);
    case NBK_OP_OR: return (a != 0) | (b != 0);
    case NBK_OP_WHERE: return a != 0 ? b : c;
    case NBK_OP_FMA: return (int64_t)(ua * ub + (uint64_t)c);
    default: return 0;
  }
}

__global__ __launch_bounds__(256) void ew_int64_kernel(const Ew64Args A) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < A.n; g += stride) {
    int64_t rem = g, oo = 0, off[3] = {0, 0, 0};
    for (int d = A.rank - 1; d >= 0; --d) {
      const int64_t q = rem / A.shape[d], i = rem - q * A.shape[d];
      rem = q;
      oo += i * A.out_stride[d];
      for (int k = 0; k < A.n_in; ++k) off[k] += i * A.stride[k][d];
    }
    int64_t v[3] = {0, 0, 0};
    for (int k = 0; k < A.n_in; ++k)
      v[k] = A.is_imm[k] ? A.imm[k] : ew64_load(A.in[k], off[k], A.in_dt[k]);
    const int64_t r = ew64_apply(A.op, v[0], v[1], v[2]);
    switch (A.out_dt) {
      case NBK_I64: ((int64_t*)A.out)[oo] = r; break;
      case NBK_I32: ((int32_t*)A.out)[oo] = (int32_t)r; break;
      case NBK_U8: ((uint8_t*)A.out)[oo] = (uint8_t)(r != 0); break;
      default: nbk_store_from_f32(A.out, oo, A.out_dt, (float)r); break;
    }
  }
}

extern "C" int nbk_ew_int64(int32_t op, const nbk_tensor* in, const int64_t* imm, int32_t n_in,
                            const nbk_tensor* out, void* stream) {
  NBK_REQUIRE(in && out, "ew_int64: null pointer");
  NBK_REQUIRE(n_in >= 1 && n_in <= 3, "ew_int64: %d operands", n_in);
  const bool known =
      op == NBK_OP_MOV || op == NBK_OP_TRUNC || op == NBK_OP_NEG || op == NBK_OP_ABS ||
      op == NBK_OP_RELU || op == NBK_OP_NOT || op == NBK_OP_NEZ || (op >= NBK_OP_ADD && op <= NBK_OP_OR) ||
      op == NBK_OP_WHERE || op == NBK_OP_FMA;
  NBK_REQUIRE(known, "ew_int64: operation %d has no 64-bit integer form", op);
  const int want = (op == NBK_OP_WHERE || op == NBK_OP_FMA) ? 3 : (op >= NBK_OP_ADD && op <= NBK_OP_OR) ? 2 : 1;
  NBK_REQUIRE(n_in == want, "ew_int64: operation %d takes %d operands, got %d", op, want, n_in);
  NBK_REQUIRE(out->rank >= 0 && out->rank <= NBK_MAX_RANK, "ew_int64: rank %d", out->rank);
  NBK_REQUIRE(nbk_dtype_size(out->dtype) > 0, "ew_int64: bad result dtype %d", out->dtype);
  Ew64Args A{};
  A.op = op;
  A.rank = out->rank;
  A.n_in = n_in;
  A.out_dt = out->dtype;
  A.out = out->ptr;
  A.n = 1;
  for (int d = 0; d < out->rank; ++d) {
    NBK_REQUIRE(out->shape[d] >= 0, "ew_int64: negative extent");
    A.shape[d] = out->shape[d];
    A.out_stride[d] = out->stride[d];
    A.n *= out->shape[d];
  }
  if (A.n == 0) return NBK_OK;  // (nothing to compute: an empty result may come without memory)
  NBK_REQUIRE(out->ptr != nullptr, "ew_int64: null result pointer");
  for (int k = 0; k < n_in; ++k) {
    if (in[k].ptr == nullptr) {
      NBK_REQUIRE(imm != nullptr, "ew_int64: operand %d has neither memory nor an immediate", k);
      A.is_imm[k] = 1;
      A.imm[k] = imm[k];
      continue;
    }
    NBK_REQUIRE(nbk_dtype_size(in[k].dtype) > 0, "ew_int64: bad dtype %d of operand %d", in[k].dtype, k);
    NBK_REQUIRE(in[k].rank == out->rank, "ew_int64: operand %d has rank %d, the result %d", k,
                in[k].rank, out->rank);
    A.in[k] = in[k].ptr;
    A.in_dt[k] = in[k].dtype;
    for (int d = 0; d < out->rank; ++d) {
      NBK_REQUIRE(in[k].shape[d] == out->shape[d], "ew_int64: operand %d differs from the result along axis %d", k, d);
      A.stride[k][d] = in[k].stride[d];
    }
  }
  int64_t blocks = (A.n + 255) / 256;
  const int64_t cap = (int64_t)nbk_num_cus() * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(ew_int64_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, A);
  return nbk_check_launch("ew_int64_kernel");
}
