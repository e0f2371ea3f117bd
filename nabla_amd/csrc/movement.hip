// Data-movement kernels: strided copy (materialise a view), fill, and the
// reduction over a middle axis.
#include "nbk_common.h"

struct CopyDesc {
  int rank;
  int64_t shape[NBK_MAX_RANK];
  int64_t sstride[NBK_MAX_RANK];
  int64_t dstride[NBK_MAX_RANK];
};

// Generic path: one lane per element, index decomposed innermost-first.
template <typename T_SRC, typename T_DST, bool CONVERT>
__global__ __launch_bounds__(256) void copy_strided_kernel(const void* __restrict__ src,
                                                           void* __restrict__ dst, CopyDesc d,
                                                           int64_t total, int dts, int dtd) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    int64_t rem = i, so = 0, dof = 0;
    for (int k = d.rank - 1; k >= 0; --k) {
      int64_t q = rem / d.shape[k];
      int64_t r = rem - q * d.shape[k];
      so += r * d.sstride[k];
      dof += r * d.dstride[k];
      rem = q;
    }
    if (CONVERT) {
      nbk_store_from_f32(dst, dof, dtd, nbk_load_as_f32(src, so, dts));
    } else {
      ((T_DST*)dst)[dof] = ((const T_SRC*)src)[so];
    }
  }
}

// 2-D transpose-style tile through LDS for the case where the source is
// unit-stride along some axis other than the last: both sides stay coalesced.
template <typename T>
__global__ __launch_bounds__(256) void copy_tile_kernel(const T* __restrict__ src,
                                                        T* __restrict__ dst, CopyDesc d,
                                                        int ax_s /* src-contiguous axis */) {
  // tile over (ax_s, last); the remaining axes are enumerated by blockIdx.z
  __shared__ T tile[64][65];
  const int last = d.rank - 1;
  const int64_t n_s = d.shape[ax_s], n_l = d.shape[last];
  int64_t rem = blockIdx.z, so = 0, dof = 0;
  for (int k = d.rank - 1; k >= 0; --k) {
    if (k == ax_s || k == last) continue;
    int64_t q = rem / d.shape[k];
    int64_t r = rem - q * d.shape[k];
    so += r * d.sstride[k];
    dof += r * d.dstride[k];
    rem = q;
  }
  const int64_t s0 = (int64_t)blockIdx.y * 64, l0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  // read: lanes run along ax_s (unit stride in src)
  for (int j = ty; j < 64; j += 4) {
    int64_t s = s0 + tx, l = l0 + j;
    if (s < n_s && l < n_l) tile[j][tx] = src[so + s * d.sstride[ax_s] + l * d.sstride[last]];
  }
  __syncthreads();
  // write: lanes run along the last axis (unit stride in dst)
  for (int j = ty; j < 64; j += 4) {
    int64_t s = s0 + j, l = l0 + tx;
    if (s < n_s && l < n_l) dst[dof + s * d.dstride[ax_s] + l * d.dstride[last]] = tile[tx][j];
  }
}

extern "C" int nbk_copy_strided(const void* src, void* dst, int32_t dts, int32_t dtd, int32_t rank,
                                const int64_t* shape, const int64_t* sstride,
                                const int64_t* dstride, void* stream) {
  NBK_REQUIRE(src && dst, "copy_strided: null pointer");
  NBK_REQUIRE(rank >= 0 && rank <= NBK_MAX_RANK, "copy_strided: rank %d exceeds %d", rank,
              NBK_MAX_RANK);
  NBK_REQUIRE(nbk_dtype_size(dts) > 0 && nbk_dtype_size(dtd) > 0, "copy_strided: bad dtype");
  CopyDesc d;
  d.rank = rank;
  int64_t total = 1;
  for (int k = 0; k < rank; ++k) {
    NBK_REQUIRE(shape[k] >= 0, "copy_strided: negative extent");
    d.shape[k] = shape[k];
    d.sstride[k] = sstride[k];
    d.dstride[k] = dstride[k];
    total *= shape[k];
  }
  if (total == 0) return NBK_OK;
  hipStream_t st = (hipStream_t)stream;
  const int es = nbk_dtype_size(dts);
  if (dts == dtd && rank >= 2 && d.dstride[rank - 1] == 1 && d.sstride[rank - 1] != 1 &&
      (es == 4 || es == 2)) {
    int ax = -1;
    for (int k = rank - 2; k >= 0; --k)
      if (d.sstride[k] == 1 && d.shape[k] >= 16) { ax = k; break; }
    if (ax >= 0 && d.shape[rank - 1] >= 16) {
      int64_t nz = total / (d.shape[ax] * d.shape[rank - 1]);
      int64_t gx = (d.shape[rank - 1] + 63) / 64, gy = (d.shape[ax] + 63) / 64;
      if (nz <= 65535 && gy <= 65535) {
        dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)nz);
        if (es == 4)
          hipLaunchKernelGGL(copy_tile_kernel<uint32_t>, grid, dim3(256), 0, st,
                             (const uint32_t*)src, (uint32_t*)dst, d, ax);
        else
          hipLaunchKernelGGL(copy_tile_kernel<uint16_t>, grid, dim3(256), 0, st,
                             (const uint16_t*)src, (uint16_t*)dst, d, ax);
        return nbk_check_launch("copy_tile_kernel");
      }
    }
  }
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1 << 20) blocks = 1 << 20;
  dim3 grid((unsigned)blocks);
  if (dts != dtd) {
    hipLaunchKernelGGL((copy_strided_kernel<float, float, true>), grid, dim3(256), 0, st, src, dst,
                       d, total, dts, dtd);
  } else if (es == 4) {
    hipLaunchKernelGGL((copy_strided_kernel<uint32_t, uint32_t, false>), grid, dim3(256), 0, st,
                       src, dst, d, total, dts, dtd);
  } else if (es == 2) {
    hipLaunchKernelGGL((copy_strided_kernel<uint16_t, uint16_t, false>), grid, dim3(256), 0, st,
                       src, dst, d, total, dts, dtd);
  } else if (es == 8) {
    hipLaunchKernelGGL((copy_strided_kernel<uint64_t, uint64_t, false>), grid, dim3(256), 0, st,
                       src, dst, d, total, dts, dtd);
  } else {
    hipLaunchKernelGGL((copy_strided_kernel<uint8_t, uint8_t, false>), grid, dim3(256), 0, st, src,
                       dst, d, total, dts, dtd);
  }
  return nbk_check_launch("copy_strided_kernel");
}

// ---- fill -------------------------------------------------------------------
__global__ __launch_bounds__(256) void fill_kernel(void* dst, int dt, int64_t n, float v,
                                                   int64_t iv) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    if (dt == NBK_I64) ((int64_t*)dst)[i] = iv;
    else if (dt == NBK_I32) ((int32_t*)dst)[i] = (int32_t)iv;
    else nbk_store_from_f32(dst, i, dt, v);
  }
}
extern "C" int nbk_fill(void* dst, int32_t dtype, int64_t n, double value, void* stream) {
  NBK_REQUIRE(dst || n == 0, "fill: null pointer");
  NBK_REQUIRE(nbk_dtype_size(dtype) > 0, "fill: bad dtype %d", dtype);
  if (n <= 0) return NBK_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, dst,
                     dtype, n, (float)value, (int64_t)value);
  return nbk_check_launch("fill_kernel");
}

// ---- reduction over a middle axis ---------------------------------------------
// in [outer, red, inner] -> out [outer, inner].  Lanes run along `inner`
// (coalesced); each workgroup owns a 64-column strip and splits `red` over its
// four waves, then combines the four partials through LDS.  (A long axis over few
// columns is cut into slices by the caller: two launches, fp32 partials in between.)
__device__ __forceinline__ float red_comb(float a, float b, int kind) {
  return kind == NBK_RED_SUM ? a + b : (kind == NBK_RED_MAX ? fmaxf(a, b) : fminf(a, b));
}
__device__ __forceinline__ void reduce_mid_body(const void* __restrict__ in, void* __restrict__ out,
                                                int dti, int dto, int64_t red, int64_t inner,
                                                int kind, int64_t bx, int64_t o) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t col = bx * 64 + lane;
  float acc = kind == NBK_RED_SUM ? 0.f : (kind == NBK_RED_MAX ? -INFINITY : INFINITY);
  if (col < inner) {
    const int64_t base = o * red * inner + col;
    // four accumulators; sixteen loads in flight while the axis is long enough (a short axis
    // over few columns is pure latency: every round trip saved shows), then four
    float a0 = acc, a1 = acc, a2 = acc, a3 = acc;
    int64_t r = w;
    for (; r + 60 < red; r += 64) {
      float v[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) v[q] = nbk_load_as_f32(in, base + (r + 4 * q) * inner, dti);
#pragma unroll
      for (int q = 0; q < 16; q += 4) {
        a0 = red_comb(a0, v[q], kind); a1 = red_comb(a1, v[q + 1], kind);
        a2 = red_comb(a2, v[q + 2], kind); a3 = red_comb(a3, v[q + 3], kind);
      }
    }
    for (; r + 12 < red; r += 16) {
      float v0 = nbk_load_as_f32(in, base + r * inner, dti);
      float v1 = nbk_load_as_f32(in, base + (r + 4) * inner, dti);
      float v2 = nbk_load_as_f32(in, base + (r + 8) * inner, dti);
      float v3 = nbk_load_as_f32(in, base + (r + 12) * inner, dti);
      a0 = red_comb(a0, v0, kind); a1 = red_comb(a1, v1, kind);
      a2 = red_comb(a2, v2, kind); a3 = red_comb(a3, v3, kind);
    }
    for (; r < red; r += 4) a0 = red_comb(a0, nbk_load_as_f32(in, base + r * inner, dti), kind);
    acc = red_comb(red_comb(a0, a1, kind), red_comb(a2, a3, kind), kind);
  }
  part[w][lane] = acc;
  __syncthreads();
  if (w == 0 && col < inner) {
    float v = red_comb(red_comb(part[0][lane], part[1][lane], kind),
                       red_comb(part[2][lane], part[3][lane], kind), kind);
    nbk_store_from_f32(out, o * inner + col, dto, v);
  }
}
__global__ __launch_bounds__(256) void reduce_mid_kernel(const void* __restrict__ in,
                                                         void* __restrict__ out, int dti, int dto,
                                                         int64_t red, int64_t inner, int kind) {
  reduce_mid_body(in, out, dti, dto, red, inner, kind, blockIdx.x, blockIdx.y);
}

// Vector form: a lane owns VEC consecutive columns (16 bytes of input per row), a
// workgroup 64 * VEC columns; its four waves take every fourth row and keep up to
// sixteen row loads in flight each.  T is the input element (uint16_t = bf16, float).
template <typename T, int VEC>
__device__ __forceinline__ void reduce_mid_vec_body(const T* __restrict__ in, void* __restrict__ out,
                                                    int dto, int64_t red, int64_t inner, int kind,
                                                    int64_t bx, int64_t o, int wc) {
  // The four waves stand wc (1, 2 or 4) side by side along the row and 4 / wc deep along the
  // reduced axis: a wide row is read in long contiguous runs, and a short reduced axis (the
  // partial sums of a split product) still keeps every wave busy.
  __shared__ float part[4][64][VEC + 1];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wcid = w % wc, wr = w / wc, WR = 4 / wc;
  const int64_t col = ((bx * wc + wcid) * 64 + lane) * VEC;
  const float ident = kind == NBK_RED_SUM ? 0.f : (kind == NBK_RED_MAX ? -INFINITY : INFINITY);
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = ident;
  if (col < inner) {
    const T* base = in + o * red * inner + col;
    auto unpack = [&](const uint4 u, float* v) {
      if (sizeof(T) == 2) {
        v[0] = __uint_as_float(u.x << 16); v[1] = __uint_as_float(u.x & 0xffff0000u);
        v[2] = __uint_as_float(u.y << 16); v[3] = __uint_as_float(u.y & 0xffff0000u);
        v[4 % VEC] = __uint_as_float(u.z << 16); v[5 % VEC] = __uint_as_float(u.z & 0xffff0000u);
        v[6 % VEC] = __uint_as_float(u.w << 16); v[7 % VEC] = __uint_as_float(u.w & 0xffff0000u);
      } else {
        v[0] = __uint_as_float(u.x); v[1] = __uint_as_float(u.y);
        v[2] = __uint_as_float(u.z); v[3] = __uint_as_float(u.w);
      }
    };
    auto load = [&](int64_t r, float* v) { unpack(*(const uint4*)(base + r * inner), v); };
    int64_t r = wr;
    for (; r + 15 * WR < red; r += 16 * WR) {  // sixteen rows in flight, kept packed until added
      uint4 raw[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) raw[q] = *(const uint4*)(base + (r + WR * q) * inner);
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        float v[VEC];
        unpack(raw[q], v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = red_comb(acc[e], v[e], kind);
      }
    }
    for (; r + 7 * WR < red; r += 8 * WR) {
      float v[8][VEC];
#pragma unroll
      for (int q = 0; q < 8; ++q) load(r + WR * q, v[q]);
#pragma unroll
      for (int q = 0; q < 8; ++q)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = red_comb(acc[e], v[q][e], kind);
    }
    for (; r < red; r += WR) {
      float v[VEC];
      load(r, v);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = red_comb(acc[e], v[e], kind);
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) part[w][lane][e] = acc[e];
  __syncthreads();
  if (wr == 0 && col < inner) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = part[wcid][lane][e];
      for (int k = 1; k < WR; ++k) v = red_comb(v, part[k * wc + wcid][lane][e], kind);
      nbk_store_from_f32(out, o * inner + col + e, dto, v);
    }
  }
}
// A few rows of a long fp32 row (the partial products of a GEMM split along K): one 16-byte piece
// per lane and row, as above, is too little work per lane and leaves two loads in flight.  Here a
// lane sums FEW_CPL pieces of the row, two rows of all of them requested at once, and stores
// whole pieces.  Same order of summation as above (row 0 first), so the same results.
constexpr int FEW_CPL = 4;
__device__ __forceinline__ void reduce_few_rows_body(const float* __restrict__ in, void* __restrict__ out,
                                                     int dto, int64_t red, int64_t inner, int kind,
                                                     int64_t bx, int64_t o) {
  const int64_t chunks = inner >> 2;
  const float4* base = (const float4*)(in + o * red * inner);
  const float ident = kind == NBK_RED_SUM ? 0.f : (kind == NBK_RED_MAX ? -INFINITY : INFINITY);
  int64_t c[FEW_CPL];
  float4 acc[FEW_CPL];
#pragma unroll
  for (int j = 0; j < FEW_CPL; ++j) {
    c[j] = bx * (256 * FEW_CPL) + j * 256 + threadIdx.x;
    acc[j] = make_float4(ident, ident, ident, ident);
  }
  auto add = [&](float4& a, const float4 v) {
    a.x = red_comb(a.x, v.x, kind); a.y = red_comb(a.y, v.y, kind);
    a.z = red_comb(a.z, v.z, kind); a.w = red_comb(a.w, v.w, kind);
  };
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  int64_t r = 0;
  for (; r + 1 < red; r += 2) {
    float4 v0[FEW_CPL], v1[FEW_CPL];
#pragma unroll
    for (int j = 0; j < FEW_CPL; ++j) {
      v0[j] = c[j] < chunks ? base[r * chunks + c[j]] : zero;
      v1[j] = c[j] < chunks ? base[(r + 1) * chunks + c[j]] : zero;
    }
#pragma unroll
    for (int j = 0; j < FEW_CPL; ++j) { add(acc[j], v0[j]); add(acc[j], v1[j]); }
  }
  if (r < red) {
#pragma unroll
    for (int j = 0; j < FEW_CPL; ++j) add(acc[j], c[j] < chunks ? base[r * chunks + c[j]] : zero);
  }
#pragma unroll
  for (int j = 0; j < FEW_CPL; ++j) {
    if (c[j] >= chunks) continue;
    const int64_t at = o * chunks + c[j];  // in pieces of four elements
    if (dto == NBK_F32) {
      ((float4*)out)[at] = acc[j];
    } else if (dto == NBK_BF16) {
      uint2 u;
      u.x = (uint32_t)nbk_f32_to_bf16(acc[j].x) | ((uint32_t)nbk_f32_to_bf16(acc[j].y) << 16);
      u.y = (uint32_t)nbk_f32_to_bf16(acc[j].z) | ((uint32_t)nbk_f32_to_bf16(acc[j].w) << 16);
      ((uint2*)out)[at] = u;
    } else {
      nbk_store_from_f32(out, at * 4 + 0, dto, acc[j].x); nbk_store_from_f32(out, at * 4 + 1, dto, acc[j].y);
      nbk_store_from_f32(out, at * 4 + 2, dto, acc[j].z); nbk_store_from_f32(out, at * 4 + 3, dto, acc[j].w);
    }
  }
}
// what a reduction must look like for the body above
static bool reduce_few_rows_fits(const void* in, const void* out, int dti, int64_t red, int64_t inner) {
  return dti == NBK_F32 && red <= 8 && inner % 4 == 0 && inner >= 65536 &&
         ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0;
}
__global__ __launch_bounds__(256) void reduce_few_rows_kernel(const float* __restrict__ in,
                                                              void* __restrict__ out, int dto, int64_t red,
                                                              int64_t inner, int kind) {
  reduce_few_rows_body(in, out, dto, red, inner, kind, blockIdx.x, blockIdx.y);
}

// Integer tensors: exact, with a 64-bit accumulator.  The same [outer, red, inner] layout and
// strip of 64 columns per workgroup as above; the four waves split `red` and meet in LDS.
__device__ __forceinline__ int64_t red_comb_i(int64_t a, int64_t b, int kind) {
  return kind == NBK_RED_SUM ? a + b : (kind == NBK_RED_MAX ? (a > b ? a : b) : (a < b ? a : b));
}
__device__ __forceinline__ int64_t load_as_i64(const void* p, int64_t i, int dt) {
  return dt == NBK_I64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}
__global__ __launch_bounds__(256) void reduce_mid_int_kernel(const void* __restrict__ in,
                                                             void* __restrict__ out, int dti, int dto,
                                                             int64_t red, int64_t inner, int kind) {
  __shared__ int64_t part[4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t col = (int64_t)blockIdx.x * 64 + lane, o = blockIdx.y;
  int64_t acc = kind == NBK_RED_SUM ? 0 : (kind == NBK_RED_MAX ? INT64_MIN : INT64_MAX);
  if (col < inner) {
    const int64_t base = o * red * inner + col;
    for (int64_t r = w; r < red; r += 4) acc = red_comb_i(acc, load_as_i64(in, base + r * inner, dti), kind);
  }
  part[w][lane] = acc;
  __syncthreads();
  if (w == 0 && col < inner) {
    const int64_t v = red_comb_i(red_comb_i(part[0][lane], part[1][lane], kind),
                                 red_comb_i(part[2][lane], part[3][lane], kind), kind);
    const int64_t at = o * inner + col;
    if (dto == NBK_I64) ((int64_t*)out)[at] = v;
    else if (dto == NBK_I32) ((int32_t*)out)[at] = (int32_t)v;
    else nbk_store_from_f32(out, at, dto, (float)v);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void reduce_mid_vec_kernel(const T* __restrict__ in,
                                                             void* __restrict__ out, int dto,
                                                             int64_t red, int64_t inner, int kind,
                                                             int wc) {
  reduce_mid_vec_body<T, VEC>(in, out, dto, red, inner, kind, blockIdx.x, blockIdx.y, wc);
}

// Several independent reductions in one launch (the column sums behind the bias and norm
// gradients of a step are many, small and ready at the same time: one launch instead of one
// each).  A workgroup finds its task from the running block counts and runs the same body.
struct ReduceBatchArgs {
  int32_t n;
  int32_t first_block[NBK_REDUCE_BATCH_MAX + 1];
  int32_t blocks_x[NBK_REDUCE_BATCH_MAX];
  int32_t mode[NBK_REDUCE_BATCH_MAX];  // 0: element-wise, 1: bf16 x 8, 2: fp32 x 4, 3: few fp32 rows
  int32_t wc[NBK_REDUCE_BATCH_MAX];    // waves side by side along the row (vector modes)
  nbk_reduce_task t[NBK_REDUCE_BATCH_MAX];
};

__global__ __launch_bounds__(256) void reduce_batch_kernel(const ReduceBatchArgs B) {
  int i = 0;
  while (i + 1 < B.n && (int)blockIdx.x >= B.first_block[i + 1]) ++i;
  const nbk_reduce_task& t = B.t[i];
  const int lb = (int)blockIdx.x - B.first_block[i];
  const int64_t bx = lb % B.blocks_x[i], o = lb / B.blocks_x[i];
  if (B.mode[i] == 1)
    reduce_mid_vec_body<uint16_t, 8>((const uint16_t*)t.in, t.out, t.dtype_out, t.red, t.inner, t.kind, bx, o, B.wc[i]);
  else if (B.mode[i] == 2)
    reduce_mid_vec_body<float, 4>((const float*)t.in, t.out, t.dtype_out, t.red, t.inner, t.kind, bx, o, B.wc[i]);
  else if (B.mode[i] == 3)
    reduce_few_rows_body((const float*)t.in, t.out, t.dtype_out, t.red, t.inner, t.kind, bx, o);
  else
    reduce_mid_body(t.in, t.out, t.dtype_in, t.dtype_out, t.red, t.inner, t.kind, bx, o);
}

// Waves side by side for a row of `chunks` 16-byte pieces: as many as the row fills.  (A
// function of the row alone: the order of summation, and so the result, does not depend on
// how reductions are grouped into launches.)
static int reduce_waves_across(int64_t chunks) { return chunks >= 256 ? 4 : (chunks >= 128 ? 2 : 1); }

static int reduce_mid_slab(const void* in, void* out, int32_t dti, int32_t dto, int64_t outer,
                           int64_t red, int64_t inner, int32_t kind, void* stream);

extern "C" int nbk_reduce_mid(const void* in, void* out, int32_t dti, int32_t dto, int64_t outer,
                              int64_t red, int64_t inner, int32_t kind, void* stream) {
  NBK_REQUIRE(in && out, "reduce_mid: null pointer");
  NBK_REQUIRE(outer > 0 && red > 0 && inner > 0, "reduce_mid: empty extent");
  NBK_REQUIRE(kind >= NBK_RED_SUM && kind <= NBK_RED_MIN, "reduce_mid: kind %d", kind);
  NBK_REQUIRE(nbk_dtype_size(dti) > 0 && nbk_dtype_size(dto) > 0, "reduce_mid: bad dtype");
  // `outer` rides on the grid's second dimension (65535 at most): longer ones go in slabs
  const int64_t kSlab = 65535;
  for (int64_t o0 = 0; o0 < outer; o0 += kSlab) {
    const int64_t n = outer - o0 < kSlab ? outer - o0 : kSlab;
    const int rc = reduce_mid_slab((const char*)in + o0 * red * inner * nbk_dtype_size(dti),
                                   (char*)out + o0 * inner * nbk_dtype_size(dto), dti, dto, n, red,
                                   inner, kind, stream);
    if (rc != NBK_OK) return rc;
  }
  return NBK_OK;
}

static int reduce_mid_slab(const void* in, void* out, int32_t dti, int32_t dto, int64_t outer,
                           int64_t red, int64_t inner, int32_t kind, void* stream) {
  if (dti == NBK_I32 || dti == NBK_I64) {
    dim3 grid((unsigned)((inner + 63) / 64), (unsigned)outer);
    hipLaunchKernelGGL(reduce_mid_int_kernel, grid, dim3(256), 0, (hipStream_t)stream, in, out, dti,
                       dto, red, inner, kind);
    return nbk_check_launch("reduce_mid_int_kernel");
  }
  const bool aligned = ((uintptr_t)in & 15) == 0;
  if (reduce_few_rows_fits(in, out, dti, red, inner)) {
    dim3 grid((unsigned)((inner / 4 + 256 * FEW_CPL - 1) / (256 * FEW_CPL)), (unsigned)outer);
    hipLaunchKernelGGL(reduce_few_rows_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const float*)in,
                       out, dto, red, inner, kind);
    return nbk_check_launch("reduce_few_rows_kernel");
  }
  if (dti == NBK_BF16 && inner % 8 == 0 && aligned) {
    const int wc = reduce_waves_across(inner / 8);
    dim3 grid((unsigned)((inner / 8 + 64 * wc - 1) / (64 * wc)), (unsigned)outer);
    hipLaunchKernelGGL((reduce_mid_vec_kernel<uint16_t, 8>), grid, dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)in, out, dto, red, inner, kind, wc);
    return nbk_check_launch("reduce_mid_vec_kernel");
  }
  if (dti == NBK_F32 && inner % 4 == 0 && aligned) {
    const int wc = reduce_waves_across(inner / 4);
    dim3 grid((unsigned)((inner / 4 + 64 * wc - 1) / (64 * wc)), (unsigned)outer);
    hipLaunchKernelGGL((reduce_mid_vec_kernel<float, 4>), grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)in, out, dto, red, inner, kind, wc);
    return nbk_check_launch("reduce_mid_vec_kernel");
  }
  dim3 grid((unsigned)((inner + 63) / 64), (unsigned)outer);
  hipLaunchKernelGGL(reduce_mid_kernel, grid, dim3(256), 0, (hipStream_t)stream, in, out, dti, dto,
                     red, inner, kind);
  return nbk_check_launch("reduce_mid_kernel");
}

extern "C" int nbk_reduce_mid_batch(const nbk_reduce_task* tasks, int32_t n, void* stream) {
  NBK_REQUIRE(tasks != nullptr && n > 0, "reduce_mid_batch: no tasks");
  for (int32_t i = 0; i < n; ++i)
    if (tasks[i].dtype_in == NBK_I32 || tasks[i].dtype_in == NBK_I64) {
      // integer tensors take the exact kernel, one launch each; the float ones share launches
      int32_t n_float = 0;
      nbk_reduce_task rest[NBK_REDUCE_BATCH_MAX];
      for (int32_t j = 0; j < n; ++j) {
        const nbk_reduce_task& t = tasks[j];
        if (t.dtype_in == NBK_I32 || t.dtype_in == NBK_I64) {
          const int rc = nbk_reduce_mid(t.in, t.out, t.dtype_in, t.dtype_out, t.outer, t.red, t.inner,
                                        t.kind, stream);
          if (rc != NBK_OK) return rc;
        } else {
          rest[n_float++] = t;
          if (n_float == NBK_REDUCE_BATCH_MAX) {
            const int rc = nbk_reduce_mid_batch(rest, n_float, stream);
            if (rc != NBK_OK) return rc;
            n_float = 0;
          }
        }
      }
      return n_float > 0 ? nbk_reduce_mid_batch(rest, n_float, stream) : NBK_OK;
    }
  for (int32_t base = 0; base < n; base += NBK_REDUCE_BATCH_MAX) {
    ReduceBatchArgs B;
    B.n = n - base < NBK_REDUCE_BATCH_MAX ? n - base : NBK_REDUCE_BATCH_MAX;
    int64_t blocks = 0;
    for (int i = 0; i < B.n; ++i) {
      const nbk_reduce_task& t = tasks[base + i];
      NBK_REQUIRE(t.in && t.out, "reduce_mid_batch: task %d: null pointer", base + i);
      NBK_REQUIRE(t.outer > 0 && t.red > 0 && t.inner > 0, "reduce_mid_batch: task %d: empty extent", base + i);
      NBK_REQUIRE(t.kind >= NBK_RED_SUM && t.kind <= NBK_RED_MIN, "reduce_mid_batch: task %d: kind %d", base + i, t.kind);
      NBK_REQUIRE(nbk_dtype_size(t.dtype_in) > 0 && nbk_dtype_size(t.dtype_out) > 0,
                  "reduce_mid_batch: task %d: bad dtype", base + i);
      const bool aligned = ((uintptr_t)t.in & 15) == 0;
      int vec = 1;
      B.mode[i] = 0;
      if (t.dtype_in == NBK_BF16 && t.inner % 8 == 0 && aligned) { B.mode[i] = 1; vec = 8; }
      else if (t.dtype_in == NBK_F32 && t.inner % 4 == 0 && aligned) { B.mode[i] = 2; vec = 4; }
      B.wc[i] = vec > 1 ? reduce_waves_across(t.inner / vec) : 1;
      int64_t bx = (t.inner / vec + 64 * B.wc[i] - 1) / (64 * B.wc[i]);
      if (reduce_few_rows_fits(t.in, t.out, t.dtype_in, t.red, t.inner)) {
        B.mode[i] = 3;
        bx = (t.inner / 4 + 256 * FEW_CPL - 1) / (256 * FEW_CPL);
      }
      B.blocks_x[i] = (int32_t)bx;
      B.first_block[i] = (int32_t)blocks;
      blocks += bx * t.outer;
      NBK_REQUIRE(blocks <= 0x7fffffffLL, "reduce_mid_batch: launch too large");
      B.t[i] = t;
    }
    B.first_block[B.n] = (int32_t)blocks;
    hipLaunchKernelGGL(reduce_batch_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, B);
  }
  return nbk_check_launch("reduce_batch_kernel");
}
